// Generalised advantage estimation (reverse scan over the response) and masked whitening.
//
// Replaces compute_gae_advantage_return (siirl/dag_worker/core_algos.py:229-276) and masked_mean / masked_var /
// masked_whiten (siirl/utils/model_utils/torch_functional.py:154-206).
//
// The scan is the reference's recurrence, evaluated per row in the same float32 operation order (this file is
// compiled with -ffp-contract=off, so no multiply-add is fused and the un-whitened advantages and the returns
// are bit-identical to the reference's):
//   delta = r_t + gamma * V_next - V_t ;  cand = delta + (gamma * lam) * A_next
//   V_next <- V_t * m_t + (1 - m_t) * V_next ;  A_next <- cand * m_t + (1 - m_t) * A_next ;  A_t = A_next
// A workgroup is one wave that owns 16 rows and walks them right to left in tiles of 128 columns: the tile's
// rewards, values and mask are fetched with 16-byte loads (coalesced, four rows per wave instruction) into
// registers while the previous tile is being scanned, pass through LDS, lanes 0-15 each walk one row of the tile
// (the recurrence is sequential: ~12 dependent-ish float operations per token), and the results leave row-wise
// again.  Rows are independent, so waves never synchronise with each other; 16 rows per wave gives B / 16 waves
// (343 at B = 5488) to spread over the chip, each bound by the latency of its own chain.
#include "common.hpp"
#include "loss_token.hpp"

namespace siirl {
namespace {

constexpr int kRows = 16, kCols = 128;
constexpr int kPitch = kCols + 4;  // floats: rows stay 16-byte aligned and the 16 scanning lanes, each reading 16
                                   // bytes of its own row at the same column, cover all 64 banks exactly once
constexpr int kChunks = kRows * kCols / 4 / kWave;  // 16-byte chunks (4 tokens) per lane per tile: 8

constexpr int kNStat = 3;

// One pass gathers, in double, S1 = sum m * d, S2 = sum m * d^2 and S0 = sum m over the tokens with m != 0
// (S0 over all), d = x - K for a pivot K near the data (the first value; 0 for the advantages of the scan above).
// From these the float32 mean the reference computes, mean = float(K * S0 + S1) / (S0 + 1e-8), and the sum of
// squared deviations about that rounded mean, S2 - 2 (mean - K) S1 + (mean - K)^2 S0, follow exactly as if a
// second pass had been made; the pivot keeps the subtraction well conditioned.
__device__ __forceinline__ void stat_add(double (&s)[kNStat], float x, float m, double K) {
  if (m != 0.f) {
    const double d = (double)x - K, md = (double)m * d;
    s[0] += md;
    s[1] += md * d;
  }
  s[2] += (double)m;
}
__device__ __forceinline__ double pivot_of(const float* v) {
  if (v == nullptr) return 0.0;
  const float k = v[0];
  return (k - k == 0.f) ? (double)k : 0.0;  // a non-finite first value (padding) is no pivot
}

// mask layouts with a vector path; anything else (and unaligned or odd-length rows) takes the scalar kernel
enum { MK_I64 = 0, MK_B32 = 1, MK_U8 = 2 };

__device__ __forceinline__ void gae_step(float r, float v, float m, float gamma, float gamma_lam, float& nv,
                                         float& lg) {
  const float delta = (r + gamma * nv) - v;
  const float cand = delta + gamma_lam * lg;
  const float om = 1.f - m;
  nv = v * m + om * nv;
  lg = cand * m + om * lg;
}

// One token of the scan composed onto the affine map (nv, lg) -> (a00 nv + b0, a10 nv + a11 lg + b1) of the
// tokens to its right (nv' never depends on lg, so that entry of the matrix stays zero and is not kept).
struct GaeMap {
  float a00, a10, a11, b0, b1;
};
__device__ __forceinline__ void gae_compose(float r, float v, float m, float gamma, float gamma_lam, GaeMap& g) {
  const float om = 1.f - m, mg = m * gamma, k = om + m * gamma_lam;
  const float a10 = mg * g.a00 + k * g.a10;
  const float b1 = (mg * g.b0 + k * g.b1) + m * (r - v);
  g.a11 = k * g.a11;
  g.a00 = om * g.a00;
  g.b0 = om * g.b0 + m * v;
  g.a10 = a10;
  g.b1 = b1;
}

enum { MODE_SCAN = 0, MODE_COMPOSE = 1 };

// MODE_SCAN: the recurrence itself, from the state `init` gives each row (zero when null).  MODE_COMPOSE: no output
// per token; each row's tokens are folded into one GaeMap written to `maps`.  With rows that are chunks of the real
// rows (B = rows x chunks, L = chunk length: chunks of a row are adjacent in memory) a compose pass, a carry over
// the chunk maps and a scan pass evaluate the recurrence with a dependent chain of one chunk instead of one row.
template <int MK, bool F32MASK, int MODE>
__global__ __launch_bounds__(kWave) void gae_scan_vec_kernel(const float* __restrict__ rewards,
                                                              const float* __restrict__ values,
                                                              const void* __restrict__ mask, int64_t B, int64_t L,
                                                              float gamma, float gamma_lam, float* __restrict__ adv,
                                                              float* __restrict__ ret, double* __restrict__ part,
                                                              const float* __restrict__ init,
                                                              float* __restrict__ maps) {
  __shared__ __align__(16) float s_r[kRows * kPitch], s_v[kRows * kPitch], s_m[kRows * kPitch], s_a[kRows * kPitch];
  const int lane = threadIdx.x;
  const int64_t row0 = (int64_t)blockIdx.x * kRows;
  const int nrows = (int)((B - row0) < kRows ? (B - row0) : kRows);
  // chunk q = lane + 64 * k of a tile: row q / 32, columns 4 * (q % 32) .. + 3
  u32x4 pr[kChunks], pv[kChunks], pm[kChunks][MK == MK_I64 ? 2 : 1];
  auto issue = [&](int64_t c0) {
#pragma unroll
    for (int k = 0; k < kChunks; ++k) {
      const int q = lane + kWave * k, rr = q / (kCols / 4);
      const int64_t col = c0 + 4 * (q % (kCols / 4));
      pr[k] = pv[k] = pm[k][0] = pm[k][MK == MK_I64 ? 1 : 0] = u32x4{0u, 0u, 0u, 0u};  // slots past the edges
      if (rr < nrows && col < L) {
        const int64_t idx = (row0 + rr) * L + col;
        pr[k] = *reinterpret_cast<const u32x4*>(rewards + idx);
        pv[k] = *reinterpret_cast<const u32x4*>(values + idx);
        if (MK == MK_I64) {
          pm[k][0] = reinterpret_cast<const u32x4*>((const int64_t*)mask + idx)[0];
          pm[k][MK == MK_I64 ? 1 : 0] = reinterpret_cast<const u32x4*>((const int64_t*)mask + idx)[1];
        } else if (MK == MK_B32) {
          pm[k][0] = *reinterpret_cast<const u32x4*>((const uint32_t*)mask + idx);
        } else {
          pm[k][0] = u32x4{*reinterpret_cast<const uint32_t*>((const uint8_t*)mask + idx), 0u, 0u, 0u};
        }
      }
    }
  };
  auto commit = [&]() {  // registers -> LDS, mask converted to float
#pragma unroll
    for (int k = 0; k < kChunks; ++k) {
      const int q = lane + kWave * k, rr = q / (kCols / 4), o = rr * kPitch + 4 * (q % (kCols / 4));
      *reinterpret_cast<u32x4*>(s_r + o) = pr[k];
      *reinterpret_cast<u32x4*>(s_v + o) = pv[k];
      float4 m;
      if (MK == MK_I64) {
        const u32x4 a = pm[k][0], b = pm[k][MK == MK_I64 ? 1 : 0];
        // values that fit 32 bits (every mask in practice) convert with one instruction each
        const bool wide = ((int32_t)a.y != ((int32_t)a.x >> 31)) | ((int32_t)a.w != ((int32_t)a.z >> 31)) |
                          ((int32_t)b.y != ((int32_t)b.x >> 31)) | ((int32_t)b.w != ((int32_t)b.z >> 31));
        if (__builtin_amdgcn_ballot_w64(wide) == 0) {
          m = make_float4((float)(int32_t)a.x, (float)(int32_t)a.z, (float)(int32_t)b.x, (float)(int32_t)b.z);
        } else {
          m.x = (float)(int64_t)(((uint64_t)a.y << 32) | a.x);
          m.y = (float)(int64_t)(((uint64_t)a.w << 32) | a.z);
          m.z = (float)(int64_t)(((uint64_t)b.y << 32) | b.x);
          m.w = (float)(int64_t)(((uint64_t)b.w << 32) | b.z);
        }
      } else if (MK == MK_B32) {
        const u32x4 a = pm[k][0];
        if (F32MASK) m = make_float4(u2f(a.x), u2f(a.y), u2f(a.z), u2f(a.w));
        else m = make_float4((float)(int32_t)a.x, (float)(int32_t)a.y, (float)(int32_t)a.z, (float)(int32_t)a.w);
      } else {
        const uint32_t u = pm[k][0].x;
        m = make_float4((float)(u & 0xffu), (float)((u >> 8) & 0xffu), (float)((u >> 16) & 0xffu), (float)(u >> 24));
      }
      *reinterpret_cast<float4*>(s_m + o) = m;
    }
  };
  float nv = 0.f, lg = 0.f;
  if (MODE == MODE_SCAN && init != nullptr && lane < nrows) {
    nv = init[2 * (row0 + lane)];
    lg = init[2 * (row0 + lane) + 1];
  }
  GaeMap gm{1.f, 0.f, 1.f, 0.f, 0.f};
  double st[kNStat] = {0.0, 0.0, 0.0};  // whitening statistics of this wave's advantages (pivot 0)
  const int64_t c_last = (L - 1) / kCols * kCols;
  issue(c_last);
  for (int64_t c0 = c_last; c0 >= 0; c0 -= kCols) {
    const int ncols = (int)((L - c0) < kCols ? (L - c0) : kCols);  // a multiple of 4
    commit();  // waits for this tile's loads
    if (c0 > 0) issue(c0 - kCols);  // in flight while this tile is scanned
    __syncthreads();
    if (lane < nrows) {
      const float* r4 = s_r + lane * kPitch;
      const float* v4 = s_v + lane * kPitch;
      const float* m4 = s_m + lane * kPitch;
      // the LDS reads of the next four tokens are issued before the current four are walked
      float4 r = *reinterpret_cast<const float4*>(r4 + ncols - 4), v = *reinterpret_cast<const float4*>(v4 + ncols - 4),
             m = *reinterpret_cast<const float4*>(m4 + ncols - 4);
      for (int cc = ncols - 4; cc >= 0; cc -= 4) {
        const int nx = cc >= 4 ? cc - 4 : 0;
        const float4 rn = *reinterpret_cast<const float4*>(r4 + nx), vn = *reinterpret_cast<const float4*>(v4 + nx),
                     mn = *reinterpret_cast<const float4*>(m4 + nx);
        if (MODE == MODE_SCAN) {
          float4 a;
          gae_step(r.w, v.w, m.w, gamma, gamma_lam, nv, lg); a.w = lg;
          gae_step(r.z, v.z, m.z, gamma, gamma_lam, nv, lg); a.z = lg;
          gae_step(r.y, v.y, m.y, gamma, gamma_lam, nv, lg); a.y = lg;
          gae_step(r.x, v.x, m.x, gamma, gamma_lam, nv, lg); a.x = lg;
          *reinterpret_cast<float4*>(s_a + lane * kPitch + cc) = a;
        } else {
          gae_compose(r.w, v.w, m.w, gamma, gamma_lam, gm);
          gae_compose(r.z, v.z, m.z, gamma, gamma_lam, gm);
          gae_compose(r.y, v.y, m.y, gamma, gamma_lam, gm);
          gae_compose(r.x, v.x, m.x, gamma, gamma_lam, gm);
        }
        r = rn; v = vn; m = mn;
      }
    }
    __syncthreads();
    if (MODE == MODE_SCAN) {
#pragma unroll
    for (int k = 0; k < kChunks; ++k) {
      const int q = lane + kWave * k, rr = q / (kCols / 4), ch = q % (kCols / 4);
      const int64_t col = c0 + 4 * ch;
      if (rr < nrows && col < L) {
        const int64_t idx = (row0 + rr) * L + col;
        const float4 a = *reinterpret_cast<const float4*>(s_a + rr * kPitch + 4 * ch);
        const float4 v = *reinterpret_cast<const float4*>(s_v + rr * kPitch + 4 * ch);
        *reinterpret_cast<float4*>(adv + idx) = a;
        *reinterpret_cast<float4*>(ret + idx) = make_float4(a.x + v.x, a.y + v.y, a.z + v.z, a.w + v.w);
        if (part) {
          const float4 m = *reinterpret_cast<const float4*>(s_m + rr * kPitch + 4 * ch);
          stat_add(st, a.x, m.x, 0.0);
          stat_add(st, a.y, m.y, 0.0);
          stat_add(st, a.z, m.z, 0.0);
          stat_add(st, a.w, m.w, 0.0);
        }
      }
    }
    }
    __syncthreads();  // the next commit overwrites s_v / s_a
  }
  if (MODE == MODE_COMPOSE) {
    if (lane < nrows) {
      float* o = maps + 5 * (row0 + lane);
      o[0] = gm.a00; o[1] = gm.a10; o[2] = gm.a11; o[3] = gm.b0; o[4] = gm.b1;
    }
    return;
  }
  if (part) {
#pragma unroll
    for (int k = 0; k < kNStat; ++k) {
      const double t = wave_sum(st[k]);
      if (lane == 0) part[kNStat * blockIdx.x + k] = t;
    }
  }
}

// State entering each chunk: chunk C - 1 of a row starts from zero, chunk c from chunk c + 1's map applied to the
// state that entered chunk c + 1.  One thread per row.
__global__ __launch_bounds__(256) void gae_carry_kernel(const float* __restrict__ maps, int64_t B, int chunks,
                                                        float* __restrict__ init) {
  const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (b >= B) return;
  float nv = 0.f, lg = 0.f;
  for (int c = chunks - 1; c >= 0; --c) {
    const int64_t r = b * chunks + c;
    init[2 * r] = nv;
    init[2 * r + 1] = lg;
    const float* g = maps + 5 * r;
    const float nnv = g[0] * nv + g[3];
    lg = (g[1] * nv + g[2] * lg) + g[4];
    nv = nnv;
  }
}

// Scalar variant for rows that are not 16-byte aligned, lengths that are not a multiple of 4, or other mask
// dtypes: same tiling, element-wise loads and stores, no prefetch.
__global__ __launch_bounds__(kWave) void gae_scan_kernel(const float* __restrict__ rewards,
                                                         const float* __restrict__ values, const void* mask,
                                                         int mask_dtype, int64_t B, int64_t L, float gamma,
                                                         float gamma_lam, float* __restrict__ adv,
                                                         float* __restrict__ ret) {
  __shared__ float s_r[kRows * kPitch], s_v[kRows * kPitch], s_m[kRows * kPitch], s_a[kRows * kPitch];
  const int lane = threadIdx.x;
  const int64_t row0 = (int64_t)blockIdx.x * kRows;
  const int nrows = (int)((B - row0) < kRows ? (B - row0) : kRows);
  float nv = 0.f, lg = 0.f;
  for (int64_t c0 = (L - 1) / kCols * kCols; c0 >= 0; c0 -= kCols) {
    const int ncols = (int)((L - c0) < kCols ? (L - c0) : kCols);
    __syncthreads();
    for (int rr = 0; rr < nrows; ++rr)
      for (int cc = lane; cc < ncols; cc += kWave) {
        const int64_t idx = (row0 + rr) * L + c0 + cc;
        s_r[rr * kPitch + cc] = rewards[idx];
        s_v[rr * kPitch + cc] = values[idx];
        s_m[rr * kPitch + cc] = load_mask(mask, mask_dtype, idx);
      }
    __syncthreads();
    if (lane < nrows)
      for (int cc = ncols - 1; cc >= 0; --cc) {
        gae_step(s_r[lane * kPitch + cc], s_v[lane * kPitch + cc], s_m[lane * kPitch + cc], gamma, gamma_lam, nv, lg);
        s_a[lane * kPitch + cc] = lg;
      }
    __syncthreads();
    for (int rr = 0; rr < nrows; ++rr)
      for (int cc = lane; cc < ncols; cc += kWave) {
        const int64_t idx = (row0 + rr) * L + c0 + cc;
        const float a = s_a[rr * kPitch + cc];
        adv[idx] = a;
        ret[idx] = a + s_v[rr * kPitch + cc];
      }
  }
}

// ---------------------------------------------------------------------------- masked whitening

constexpr int kThreads = 256;
constexpr int kMaxParts = 8192;
__global__ __launch_bounds__(kThreads) void whiten_stats_kernel(const float* __restrict__ v, const void* mask,
                                                                int mask_dtype, int64_t n, int vec,
                                                                double* __restrict__ part) {
  const double K = pivot_of(v);
  double s[kNStat] = {0.0, 0.0, 0.0};
  const int64_t nq = (n + 3) / 4;
  for (int64_t q = (int64_t)blockIdx.x * kThreads + threadIdx.x; q < nq; q += (int64_t)gridDim.x * kThreads) {
    const int64_t i0 = 4 * q;
    const int nv = (int)((n - i0) < 4 ? (n - i0) : 4);
    const tok::Quad m4 = tok::load_mask_quad(mask, mask_dtype, i0, vec != 0, nv);
    const tok::Quad x4 = tok::load_quad(v, i0, vec != 0, nv, 0.f);
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (e < nv) stat_add(s, x4.v[e], m4.v[e], K);
  }
  __shared__ double sh[kThreads / kWave + 1];
#pragma unroll
  for (int k = 0; k < kNStat; ++k) {
    const double t = block_sum(s[k], sh);
    if (threadIdx.x == 0) part[kNStat * blockIdx.x + k] = t;
  }
}

// stats = { mean, var, mask sum }: var is masked_mean of the squared deviations about the float32 mean, times the
// float32 quotient n / (n - 1) when unbiased.
__global__ __launch_bounds__(kThreads) void whiten_finish_kernel(const double* __restrict__ part, int nparts,
                                                                 const float* __restrict__ pivot_src, int unbiased,
                                                                 float* __restrict__ stats) {
  double s[kNStat] = {0.0, 0.0, 0.0};
  for (int i = threadIdx.x; i < nparts; i += kThreads)
#pragma unroll
    for (int k = 0; k < kNStat; ++k) s[k] += part[kNStat * i + k];
  __shared__ double sh[kThreads / kWave + 1];
#pragma unroll
  for (int k = 0; k < kNStat; ++k) s[k] = block_sum(s[k], sh);
  if (threadIdx.x != 0) return;
  const double K = pivot_of(pivot_src);
  const float n = (float)s[2];
  const float mean = (float)(K * s[2] + s[0]) / (n + 1e-8f);
  const double dl = (double)mean - K;
  const float var = (float)(s[1] - 2.0 * dl * s[0] + dl * dl * s[2]) / (n + 1e-8f);
  stats[0] = mean;
  stats[1] = unbiased ? var * (n / (n - 1.f)) : var;
  stats[2] = n;
}

__global__ __launch_bounds__(kThreads) void whiten_apply_kernel(const float* __restrict__ v, int64_t n, int vec,
                                                                const float* __restrict__ stats, int shift_mean,
                                                                float* __restrict__ out) {
  const float mean = stats[0];
  const float scale = 1.f / sqrtf(stats[1] + 1e-8f);
  const int64_t nq = (n + 3) / 4;
  for (int64_t q = (int64_t)blockIdx.x * kThreads + threadIdx.x; q < nq; q += (int64_t)gridDim.x * kThreads) {
    const int64_t i0 = 4 * q;
    const int nv = (int)((n - i0) < 4 ? (n - i0) : 4);
    tok::Quad x4 = tok::load_quad(v, i0, vec != 0, nv, 0.f);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float w = (x4.v[e] - mean) * scale;
      if (!shift_mean) w += mean;
      x4.v[e] = w;
    }
    tok::store_quad(out, i0, vec != 0, nv, x4);
  }
}

int check_mask(int dt) {
  SIIRL_REQUIRE(dt == SIIRL_U8 || dt == SIIRL_I64 || dt == SIIRL_I32 || dt == SIIRL_F32 || dt == SIIRL_BF16 ||
                    dt == SIIRL_F16, "mask dtype %d not supported", dt);
  return SIIRL_OK;
}

constexpr size_t kWhitenWs = (size_t)kMaxParts * kNStat * sizeof(double);

int check_whiten_ws(const void* ws, size_t ws_bytes) {
  if (ws == nullptr || ws_bytes < kWhitenWs)
    return fail(SIIRL_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", ws_bytes, kWhitenWs);
  SIIRL_REQUIRE(((uintptr_t)ws & 7) == 0, "workspace must be 8-byte aligned");
  return SIIRL_OK;
}

// `parts_ready` > 0: the statistics partials (pivot 0) are already in the workspace, that many of them
int run_whiten(const float* values, const void* mask, int mask_dtype, int64_t n, int shift_mean, float* out,
               float* stats3, void* ws, int parts_ready, hipStream_t st) {
  double* part = (double*)ws;
  const int mask_es = (int)dtype_size(mask_dtype);
  const bool vec = n % 4 == 0 && (((uintptr_t)values | (uintptr_t)out) & 15) == 0 &&
                   ((uintptr_t)mask % (size_t)(mask_es * 4 < 16 ? mask_es * 4 : 16)) == 0;
  int nparts = parts_ready;
  if (nparts <= 0) {
    const int64_t want = (n + kThreads * 16 - 1) / (kThreads * 16);
    nparts = (int)(want < 1 ? 1 : (want > kMaxParts ? kMaxParts : want));
    whiten_stats_kernel<<<dim3(nparts), dim3(kThreads), 0, st>>>(values, mask, mask_dtype, n, vec ? 1 : 0, part);
    SIIRL_LAUNCH_CHECK("whiten_stats_kernel");
  }
  whiten_finish_kernel<<<1, dim3(kThreads), 0, st>>>(part, nparts, parts_ready > 0 ? nullptr : values, 1, stats3);
  SIIRL_LAUNCH_CHECK("whiten_finish_kernel");
  const int64_t nq = (n + 3) / 4;
  const unsigned blocks = (unsigned)((nq + kThreads - 1) / kThreads < 8192 ? (nq + kThreads - 1) / kThreads : 8192);
  whiten_apply_kernel<<<dim3(blocks), dim3(kThreads), 0, st>>>(values, n, vec ? 1 : 0, stats3, shift_mean, out);
  SIIRL_LAUNCH_CHECK("whiten_apply_kernel");
  return SIIRL_OK;
}

}  // namespace
}  // namespace siirl

using namespace siirl;

extern "C" size_t siirl_whiten_workspace_bytes(void) { return kWhitenWs; }

extern "C" int siirl_masked_whiten(const float* values, const void* mask, int mask_dtype, int64_t n, int shift_mean,
                                   float* out, float* stats3, void* workspace, size_t workspace_bytes,
                                   siirl_stream_t stream) {
  SIIRL_REQUIRE(n >= 1, "n=%lld must be positive", (long long)n);
  if (int rc = check_mask(mask_dtype)) return rc;
  SIIRL_REQUIRE(values && mask && out && stats3, "NULL operand");
  if (int rc = check_whiten_ws(workspace, workspace_bytes)) return rc;
  return run_whiten(values, mask, mask_dtype, n, shift_mean, out, stats3, workspace, 0, (hipStream_t)stream);
}

// chunks per row of the chunked scan: the largest of 16, 8, 4, 2 that leaves chunks of at least 256 tokens whose
// length is a multiple of 4; 1 = the plain scan
static int gae_chunks(int64_t L) {
  for (int c = 16; c >= 2; c /= 2)
    if (L % (4 * c) == 0 && L / c >= 256) return c;
  return 1;
}
constexpr int kGaeMaxChunks = 16;
static size_t gae_ws_bytes(int64_t B) {
  return kWhitenWs + (size_t)B * kGaeMaxChunks * (5 + 2) * sizeof(float) + 256;
}

extern "C" size_t siirl_gae_workspace_bytes(int64_t B, int64_t L) {
  (void)L;
  return B < 1 ? 0 : gae_ws_bytes(B);
}

template <int MK, bool F32MASK>
static int launch_gae_vec(const float* rewards, const float* values, const void* mask, int64_t B, int64_t L, float g,
                          float gl, float* adv, float* ret, void* ws, int chunks, int* parts_ready, hipStream_t st) {
  const int64_t rows = B * chunks, len = L / chunks;
  const dim3 grid((unsigned)((rows + kRows - 1) / kRows)), block(kWave);
  // the scan leaves its whitening statistics in the workspace, one partial per workgroup, when they fit
  const bool fused_stats = grid.x <= (unsigned)kMaxParts;
  double* part = fused_stats ? (double*)ws : nullptr;
  *parts_ready = fused_stats ? (int)grid.x : 0;
  const float* init = nullptr;
  if (chunks > 1) {
    float* maps = reinterpret_cast<float*>((char*)ws + kWhitenWs);
    float* ini = maps + (size_t)rows * 5;
    gae_scan_vec_kernel<MK, F32MASK, MODE_COMPOSE><<<grid, block, 0, st>>>(rewards, values, mask, rows, len, g, gl, nullptr,
                                                                        nullptr, nullptr, nullptr, maps);
    SIIRL_LAUNCH_CHECK("gae_scan_vec_kernel<compose>");
    gae_carry_kernel<<<dim3((unsigned)((B + 255) / 256)), dim3(256), 0, st>>>(maps, B, chunks, ini);
    SIIRL_LAUNCH_CHECK("gae_carry_kernel");
    init = ini;
  }
  gae_scan_vec_kernel<MK, F32MASK, MODE_SCAN><<<grid, block, 0, st>>>(rewards, values, mask, rows, len, g, gl, adv, ret,
                                                                   part, init, nullptr);
  SIIRL_LAUNCH_CHECK("gae_scan_vec_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_gae_advantage_return(const float* token_level_rewards, const float* values, const void* mask,
                                          int mask_dtype, int64_t B, int64_t L, double gamma, double lam,
                                          float* advantages, float* returns, float* stats3, void* workspace,
                                          size_t workspace_bytes, int order, siirl_stream_t stream) {
  SIIRL_REQUIRE(B >= 1 && L >= 1 && B <= (1LL << 32), "B=%lld L=%lld out of range", (long long)B, (long long)L);
  if (int rc = check_mask(mask_dtype)) return rc;
  SIIRL_REQUIRE(token_level_rewards && values && mask && advantages && returns && stats3, "NULL operand");
  SIIRL_REQUIRE(advantages != returns, "advantages and returns must be different buffers");
  SIIRL_REQUIRE(order == SIIRL_GAE_EXACT_ORDER || order == SIIRL_GAE_CHUNKED, "unknown scan order %d", order);
  if (workspace == nullptr || workspace_bytes < gae_ws_bytes(B))
    return fail(SIIRL_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes,
                gae_ws_bytes(B));
  SIIRL_REQUIRE(((uintptr_t)workspace & 7) == 0, "workspace must be 8-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const float g = (float)gamma, gl = (float)(gamma * lam);
  const uintptr_t bases = (uintptr_t)token_level_rewards | (uintptr_t)values | (uintptr_t)advantages | (uintptr_t)returns;
  const bool vec = L % 4 == 0 && (bases & 15) == 0;
  const int chunks = order == SIIRL_GAE_CHUNKED ? gae_chunks(L) : 1;
  int parts_ready = 0;
  int rc = SIIRL_OK;
  if (vec && mask_dtype == SIIRL_I64 && ((uintptr_t)mask & 15) == 0)
    rc = launch_gae_vec<MK_I64, false>(token_level_rewards, values, mask, B, L, g, gl, advantages, returns, workspace, chunks,
                                       &parts_ready, st);
  else if (vec && mask_dtype == SIIRL_F32 && ((uintptr_t)mask & 15) == 0)
    rc = launch_gae_vec<MK_B32, true>(token_level_rewards, values, mask, B, L, g, gl, advantages, returns, workspace, chunks,
                                      &parts_ready, st);
  else if (vec && mask_dtype == SIIRL_I32 && ((uintptr_t)mask & 15) == 0)
    rc = launch_gae_vec<MK_B32, false>(token_level_rewards, values, mask, B, L, g, gl, advantages, returns, workspace, chunks,
                                       &parts_ready, st);
  else if (vec && mask_dtype == SIIRL_U8 && ((uintptr_t)mask & 3) == 0)
    rc = launch_gae_vec<MK_U8, false>(token_level_rewards, values, mask, B, L, g, gl, advantages, returns, workspace, chunks,
                                      &parts_ready, st);
  else {  // the scalar kernel walks whole rows in the reference's order, whatever `order` asks for
    gae_scan_kernel<<<dim3((unsigned)((B + kRows - 1) / kRows)), dim3(kWave), 0, st>>>(
        token_level_rewards, values, mask, mask_dtype, B, L, g, gl, advantages, returns);
    SIIRL_LAUNCH_CHECK("gae_scan_kernel");
  }
  if (rc) return rc;
  return run_whiten(advantages, mask, mask_dtype, B * L, 1, advantages, stats3, workspace, parts_ready, st);
}
