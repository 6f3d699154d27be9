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
// A workgroup is one wave that owns 64 rows: 64 x 64 tiles are loaded row-wise (coalesced) into LDS, each lane
// walks its own row of the tile right to left, and the results leave through LDS row-wise again.
#include "common.hpp"

namespace siirl {
namespace {

constexpr int kRows = 64, kCols = 64, kPad = kCols + 1;  // 65-float rows: lanes walking a column hit distinct banks

__global__ __launch_bounds__(kRows) void gae_scan_kernel(const float* __restrict__ rewards,
                                                         const float* __restrict__ values, const void* mask,
                                                         int mask_dtype, int64_t B, int64_t L, float gamma,
                                                         float gamma_lam, float* __restrict__ adv,
                                                         float* __restrict__ ret) {
  __shared__ float s_r[kRows * kPad], s_v[kRows * kPad], s_m[kRows * kPad], s_a[kRows * kPad];
  const int lane = threadIdx.x;
  const int64_t row0 = (int64_t)blockIdx.x * kRows;
  const int nrows = (int)((B - row0) < kRows ? (B - row0) : kRows);
  float nv = 0.f, lg = 0.f;
  for (int64_t c0 = (L - 1) / kCols * kCols; c0 >= 0; c0 -= kCols) {
    const int ncols = (int)((L - c0) < kCols ? (L - c0) : kCols);
    __syncthreads();
    if (lane < ncols)
      for (int rr = 0; rr < nrows; ++rr) {
        const int64_t idx = (row0 + rr) * L + c0 + lane;
        s_r[rr * kPad + lane] = rewards[idx];
        s_v[rr * kPad + lane] = values[idx];
        s_m[rr * kPad + lane] = load_mask(mask, mask_dtype, idx);
      }
    __syncthreads();
    if (lane < nrows)
      for (int cc = ncols - 1; cc >= 0; --cc) {
        const float r = s_r[lane * kPad + cc], v = s_v[lane * kPad + cc], m = s_m[lane * kPad + cc];
        const float delta = (r + gamma * nv) - v;
        const float cand = delta + gamma_lam * lg;
        const float om = 1.f - m;
        nv = v * m + om * nv;
        lg = cand * m + om * lg;
        s_a[lane * kPad + cc] = lg;
      }
    __syncthreads();
    if (lane < ncols)
      for (int rr = 0; rr < nrows; ++rr) {
        const int64_t idx = (row0 + rr) * L + c0 + lane;
        const float a = s_a[rr * kPad + lane];
        adv[idx] = a;
        ret[idx] = a + s_v[rr * kPad + lane];
      }
  }
}

// ---------------------------------------------------------------------------- masked whitening

constexpr int kThreads = 256;
constexpr int kMaxParts = 1024;

// part[wg] = { sum where(m, f(v), 0) * m, sum m } in double; f(v) = v (SQDEV false) or (v - mean)^2 with the
// float32 mean in stats[0] (SQDEV true)
template <bool SQDEV>
__global__ __launch_bounds__(kThreads) void whiten_partials_kernel(const float* __restrict__ v, const void* mask,
                                                                   int mask_dtype, int64_t n,
                                                                   const float* __restrict__ stats,
                                                                   double* __restrict__ part) {
  const float mean = SQDEV ? stats[0] : 0.f;
  double sv = 0.0, sm = 0.0;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads) {
    const float m = load_mask(mask, mask_dtype, i);
    float x = v[i];
    if (SQDEV) {
      const float c = x - mean;
      x = c * c;
    }
    sv += m != 0.f ? (double)(x * m) : 0.0;
    sm += (double)m;
  }
  __shared__ double sh[kThreads / kWave + 1];
  sv = block_sum(sv, sh);
  sm = block_sum(sm, sh);
  if (threadIdx.x == 0) {
    part[2 * blockIdx.x] = sv;
    part[2 * blockIdx.x + 1] = sm;
  }
}

// stats = { mean, var, mask sum }.  Pass 1 writes the mean and the mask sum, pass 2 the variance:
// masked_mean of the squared deviations times the float32 quotient n / (n - 1) when unbiased.
__global__ __launch_bounds__(kThreads) void whiten_finish_kernel(const double* __restrict__ part, int nparts, int pass,
                                                                 int unbiased, float* __restrict__ stats) {
  double sv = 0.0, sm = 0.0;
  for (int i = threadIdx.x; i < nparts; i += kThreads) {
    sv += part[2 * i];
    sm += part[2 * i + 1];
  }
  __shared__ double sh[kThreads / kWave + 1];
  sv = block_sum(sv, sh);
  sm = block_sum(sm, sh);
  if (threadIdx.x != 0) return;
  const float n = (float)sm;
  const float mm = (float)sv / (n + 1e-8f);
  if (pass == 1) {
    stats[0] = mm;
    stats[2] = n;
  } else {
    stats[1] = unbiased ? mm * (n / (n - 1.f)) : mm;
  }
}

__global__ __launch_bounds__(kThreads) void whiten_apply_kernel(const float* __restrict__ v, int64_t n,
                                                                const float* __restrict__ stats, int shift_mean,
                                                                float* __restrict__ out) {
  const float mean = stats[0];
  const float scale = 1.f / sqrtf(stats[1] + 1e-8f);
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads) {
    float w = (v[i] - mean) * scale;
    if (!shift_mean) w += mean;
    out[i] = w;
  }
}

int check_mask(int dt) {
  SIIRL_REQUIRE(dt == SIIRL_U8 || dt == SIIRL_I64 || dt == SIIRL_I32 || dt == SIIRL_F32 || dt == SIIRL_BF16 ||
                    dt == SIIRL_F16, "mask dtype %d not supported", dt);
  return SIIRL_OK;
}

constexpr size_t kWhitenWs = (size_t)kMaxParts * 2 * sizeof(double);

int run_whiten(const float* values, const void* mask, int mask_dtype, int64_t n, int shift_mean, float* out,
               float* stats3, void* ws, size_t ws_bytes, hipStream_t st) {
  if (ws == nullptr || ws_bytes < kWhitenWs)
    return fail(SIIRL_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", ws_bytes, kWhitenWs);
  SIIRL_REQUIRE(((uintptr_t)ws & 7) == 0, "workspace must be 8-byte aligned");
  double* part = (double*)ws;
  const int64_t want = (n + kThreads * 8 - 1) / (kThreads * 8);
  const int nparts = (int)(want < 1 ? 1 : (want > kMaxParts ? kMaxParts : want));
  whiten_partials_kernel<false><<<dim3(nparts), dim3(kThreads), 0, st>>>(values, mask, mask_dtype, n, stats3, part);
  SIIRL_LAUNCH_CHECK("whiten_partials_kernel<mean>");
  whiten_finish_kernel<<<1, dim3(kThreads), 0, st>>>(part, nparts, 1, 1, stats3);
  SIIRL_LAUNCH_CHECK("whiten_finish_kernel");
  whiten_partials_kernel<true><<<dim3(nparts), dim3(kThreads), 0, st>>>(values, mask, mask_dtype, n, stats3, part);
  SIIRL_LAUNCH_CHECK("whiten_partials_kernel<var>");
  whiten_finish_kernel<<<1, dim3(kThreads), 0, st>>>(part, nparts, 2, 1, stats3);
  SIIRL_LAUNCH_CHECK("whiten_finish_kernel");
  const unsigned blocks = (unsigned)((n + kThreads - 1) / kThreads < 8192 ? (n + kThreads - 1) / kThreads : 8192);
  whiten_apply_kernel<<<dim3(blocks), dim3(kThreads), 0, st>>>(values, n, stats3, shift_mean, out);
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
  return run_whiten(values, mask, mask_dtype, n, shift_mean, out, stats3, workspace, workspace_bytes,
                    (hipStream_t)stream);
}

extern "C" int siirl_gae_advantage_return(const float* token_level_rewards, const float* values, const void* mask,
                                          int mask_dtype, int64_t B, int64_t L, double gamma, double lam,
                                          float* advantages, float* returns, float* stats3, void* workspace,
                                          size_t workspace_bytes, siirl_stream_t stream) {
  SIIRL_REQUIRE(B >= 1 && L >= 1 && B <= (1LL << 36), "B=%lld L=%lld out of range", (long long)B, (long long)L);
  if (int rc = check_mask(mask_dtype)) return rc;
  SIIRL_REQUIRE(token_level_rewards && values && mask && advantages && returns && stats3, "NULL operand");
  SIIRL_REQUIRE(advantages != returns, "advantages and returns must be different buffers");
  hipStream_t st = (hipStream_t)stream;
  gae_scan_kernel<<<dim3((unsigned)((B + kRows - 1) / kRows)), dim3(kRows), 0, st>>>(
      token_level_rewards, values, mask, mask_dtype, B, L, (float)gamma, (float)(gamma * lam), advantages, returns);
  SIIRL_LAUNCH_CHECK("gae_scan_kernel");
  return run_whiten(advantages, mask, mask_dtype, B * L, 1, advantages, stats3, workspace, workspace_bytes, st);
}
