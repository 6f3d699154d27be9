// Log-prob and entropy from logits[T, V]: forward (one read of the row) and backward (one read of the
// row, one write of the gradient).  HBM-bound streaming kernels for gfx950; one workgroup per row.
//
// Replaces logprobs_from_logits / entropy_from_logits and their autograd backward:
//   siirl/utils/model_utils/torch_functional.py:56-116,128-143
//   siirl/utils/experimental/torch_functional.py:49-62 (closed form of the gradient)
//
// Forward keeps, per lane, an online-softmax state in base-2 arithmetic
//     mx = running max of raw x,   s = sum 2^{(x - mx) k},   t = sum x * 2^{(x - mx) k},   k = log2(e)/T
// so that each element costs one fma, one v_exp_f32 and two accumulations; the running max is
// refreshed once per UNROLL 16-byte loads (v_max3 chains), the rescale is a rarely-taken branch.
// States are merged across the wave with shuffles and across waves through LDS.
#include "common.hpp"

#include <type_traits>
#include "loss_token.hpp"

namespace siirl {
namespace {

// A label equal to this value is ignored: log-prob 0 and no gradient through it.  It is the default ignore_index of
// flash-attn's cross_entropy_loss, which the reference's logprobs_from_logits dispatches to when flash-attn is
// installed (siirl/utils/model_utils/torch_functional.py:73-90).  Any other label outside [0, V) yields NaN.
constexpr int64_t kIgnoreIndex = -100;
// A label equal to this value says that nothing of the row is wanted (a prompt token of a packed batch: the actor
// keeps the response slice of the log-probs only, siirl/engine/actor/dp_actor.py:228-231): the forward writes zeros
// for the row without reading it, the backward writes a zero gradient whatever the upstream gradients hold.
constexpr int64_t kSkipRow = SIIRL_LABEL_SKIP_ROW;

// Tuning knobs.  Measured on MI355X at T=32768, V=152064, bf16: non-temporal loads are worth 12% on the
// forward (a pure read stream); on the backward (read + write) the hints are within run-to-run noise;
// 256 threads with 4 loads in flight per lane beat 512/1024 threads and deeper unrolling on both.
// A flat (dense-stream) forward with per-chunk partials and a merge kernel was tried and is slower than one
// workgroup per row (1.60-1.72 ms against 1.49 ms): the per-workgroup reduction costs more than the DRAM
// locality returns on a pure read stream.  The flat backward below, which has no reduction, is 17% faster.
#ifndef SIIRL_LPE_FWD_THREADS
#define SIIRL_LPE_FWD_THREADS 256
#endif
#ifndef SIIRL_LPE_FWD_UNROLL
#define SIIRL_LPE_FWD_UNROLL 4
#endif
#ifndef SIIRL_LPE_FWD_NT_LOAD
#define SIIRL_LPE_FWD_NT_LOAD 1
#endif
#ifndef SIIRL_LPE_BWD_THREADS
#define SIIRL_LPE_BWD_THREADS 256
#endif
#ifndef SIIRL_LPE_BWD_UNROLL
#define SIIRL_LPE_BWD_UNROLL 4
#endif
#ifndef SIIRL_LPE_BWD_NT_LOAD
#define SIIRL_LPE_BWD_NT_LOAD 1
#endif
#ifndef SIIRL_LPE_BWD_FLAT
#define SIIRL_LPE_BWD_FLAT 1
#endif
#ifndef SIIRL_LPE_BWD_NT_STORE
#define SIIRL_LPE_BWD_NT_STORE 1
#endif
constexpr int kFwdThreads = SIIRL_LPE_FWD_THREADS;  // waves per row = threads / 64
constexpr int kFwdUnroll = SIIRL_LPE_FWD_UNROLL;    // 16-byte loads in flight per lane
constexpr int kBwdThreads = SIIRL_LPE_BWD_THREADS;
constexpr int kBwdUnroll = SIIRL_LPE_BWD_UNROLL;

template <bool NT>
__device__ __forceinline__ u32x4 ld16(const u32x4* p) {
  if constexpr (NT) return __builtin_nontemporal_load(p);
  else return *p;
}
template <bool NT>
__device__ __forceinline__ void st16(u32x4 v, u32x4* p) {
  if constexpr (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}

// ------------------------------------------------------------------ element traits (16-byte vectors)

struct ElemBF16 {
  using elem_t = uint16_t;
  static constexpr int VEC = 8;
  static __device__ __forceinline__ void unpack(const u32x4& r, float* v) {
    v[0] = bf16_lo(r.x); v[1] = bf16_hi(r.x); v[2] = bf16_lo(r.y); v[3] = bf16_hi(r.y);
    v[4] = bf16_lo(r.z); v[5] = bf16_hi(r.z); v[6] = bf16_lo(r.w); v[7] = bf16_hi(r.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float* v) {
    return mk4(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7]));
  }
  static __device__ __forceinline__ float load1(const elem_t* p) { return u2f(((uint32_t)*p) << 16); }
  static __device__ __forceinline__ void store1(elem_t* p, float f) { *p = (elem_t)(pack_bf16(f, 0.f) & 0xffffu); }
};

struct ElemF16 {
  using elem_t = uint16_t;
  static constexpr int VEC = 8;
  static __device__ __forceinline__ void unpack(const u32x4& r, float* v) {
    v[0] = f16_lo(r.x); v[1] = f16_hi(r.x); v[2] = f16_lo(r.y); v[3] = f16_hi(r.y);
    v[4] = f16_lo(r.z); v[5] = f16_hi(r.z); v[6] = f16_lo(r.w); v[7] = f16_hi(r.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float* v) {
    return mk4(pack_f16(v[0], v[1]), pack_f16(v[2], v[3]), pack_f16(v[4], v[5]), pack_f16(v[6], v[7]));
  }
  static __device__ __forceinline__ float load1(const elem_t* p) { return f16_lo((uint32_t)*p); }
  static __device__ __forceinline__ void store1(elem_t* p, float f) { *p = (elem_t)(pack_f16(f, 0.f) & 0xffffu); }
};

struct ElemF32 {
  using elem_t = float;
  static constexpr int VEC = 4;
  static __device__ __forceinline__ void unpack(const u32x4& r, float* v) {
    v[0] = u2f(r.x); v[1] = u2f(r.y); v[2] = u2f(r.z); v[3] = u2f(r.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float* v) {
    return mk4(f2u(v[0]), f2u(v[1]), f2u(v[2]), f2u(v[3]));
  }
  static __device__ __forceinline__ float load1(const elem_t* p) { return *p; }
  static __device__ __forceinline__ void store1(elem_t* p, float f) { *p = f; }
};

// A row is split into [0, head) scalars up to the first 16-byte boundary, nvec 16-byte vectors, and
// the scalars left over.  When the source and destination rows do not share their alignment the
// whole row is scalar (head = V).
template <class E>
struct RowSplit {
  int head, nvec, tail0;
  __device__ __forceinline__ RowSplit(const void* a, const void* b, int V) {
    const uintptr_t pa = (uintptr_t)a, pb = b ? (uintptr_t)b : pa;
    constexpr int ES = sizeof(typename E::elem_t);
    int h = (int)(((16u - (unsigned)(pa & 15u)) & 15u) / ES);
    if ((pa & 15u) != (pb & 15u)) h = V;
    head = h < V ? h : V;
    nvec = (V - head) / E::VEC;
    tail0 = head + nvec * E::VEC;
  }
};

// ----------------------------------------------------------------------------------- forward

struct SoftState {
  float mx, s, t;
};

__device__ __forceinline__ void merge(SoftState& a, float omx, float os, float ot, float k) {
  const float M = fmaxf(a.mx, omx);
  const float fa = fast_exp2((a.mx - M) * k), fb = fast_exp2((omx - M) * k);
  a.s = a.s * fa + os * fb;
  a.t = a.t * fa + ot * fb;
  a.mx = M;
}

template <bool ENT>
__device__ __forceinline__ void absorb1(SoftState& st, float v, float k) {
  if (v > st.mx) {
    const float sc = fast_exp2((st.mx - v) * k);
    st.s *= sc;
    st.t *= sc;
    st.mx = v;
  }
  const float e = fast_exp2((v - st.mx) * k);
  st.s += e;
  if (ENT) st.t = fmaf(v, e, st.t);
}

template <class E, bool ENT, int N>
__device__ __forceinline__ void absorb_vecs(SoftState& st, const u32x4* buf, float k) {
  float v[N][E::VEC];
#pragma unroll
  for (int u = 0; u < N; ++u) E::unpack(buf[u], v[u]);
  float cm = v[0][0];
#pragma unroll
  for (int u = 0; u < N; ++u)
#pragma unroll
    for (int j = 0; j < E::VEC; ++j) cm = fmaxf(cm, v[u][j]);
  if (cm > st.mx) {
    const float sc = fast_exp2((st.mx - cm) * k);
    st.s *= sc;
    st.t *= sc;
    st.mx = cm;
  }
  const float nmk = -st.mx * k;
  float s = st.s, t = st.t;
#pragma unroll
  for (int u = 0; u < N; ++u)
#pragma unroll
    for (int j = 0; j < E::VEC; ++j) {
      const float e = fast_exp2(fmaf(v[u][j], k, nmk));
      s += e;
      if (ENT) t = fmaf(v[u][j], e, t);
    }
  st.s = s;
  st.t = t;
}

// NT: the row is streamed with non-temporal loads (worth 12 % when the logits are many times the memory-side cache);
// without them a tensor that fits that cache is still there when the backward reads it again.
template <class E, bool ENT, bool NT>
__global__ __launch_bounds__(kFwdThreads) void lpe_fwd_kernel(const typename E::elem_t* __restrict__ logits,
                                                           int64_t row_stride, int V,
                                                           const int64_t* __restrict__ labels, float inv_T,
                                                           float* __restrict__ logprob, float* __restrict__ entropy,
                                                           float* __restrict__ lse_out, float* __restrict__ ex_out) {
  using elem_t = typename E::elem_t;
  const int64_t row = blockIdx.x;
  const elem_t* __restrict__ x = logits + row * row_stride;
  const int tid = threadIdx.x;
  if (labels != nullptr && labels[row] == kSkipRow) {  // (uniform over the workgroup: no barrier is left behind)
    if (tid == 0) {
      lse_out[row] = 0.f;
      if (ENT) {
        ex_out[row] = 0.f;
        entropy[row] = 0.f;
      }
      if (logprob != nullptr) logprob[row] = 0.f;
    }
    return;
  }
  const float k = inv_T * kLog2e;
  const RowSplit<E> sp(x, nullptr, V);

  SoftState st{-1e30f, 0.f, 0.f};

  for (int i = tid; i < sp.head; i += kFwdThreads) absorb1<ENT>(st, E::load1(x + i), k);
  for (int i = sp.tail0 + tid; i < V; i += kFwdThreads) absorb1<ENT>(st, E::load1(x + i), k);

  const u32x4* __restrict__ xv = reinterpret_cast<const u32x4*>(x + sp.head);
  constexpr int kTile = kFwdThreads * kFwdUnroll;
  const int nfull = sp.nvec / kTile * kTile;
  for (int base = 0; base < nfull; base += kTile) {
    u32x4 buf[kFwdUnroll];
#pragma unroll
    for (int u = 0; u < kFwdUnroll; ++u) buf[u] = ld16<NT>(xv + base + u * kFwdThreads + tid);
    absorb_vecs<E, ENT, kFwdUnroll>(st, buf, k);
  }
  for (int i = nfull + tid; i < sp.nvec; i += kFwdThreads) {
    u32x4 b = ld16<NT>(xv + i);
    absorb_vecs<E, ENT, 1>(st, &b, k);
  }

  // wave merge
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const float omx = __shfl_xor(st.mx, o, kWave);
    const float os = __shfl_xor(st.s, o, kWave);
    const float ot = __shfl_xor(st.t, o, kWave);
    merge(st, omx, os, ot, k);
  }
  __shared__ float sm[3 * (kFwdThreads / kWave)];
  const int lane = tid & (kWave - 1), wid = tid / kWave;
  if (lane == 0) {
    sm[wid * 3 + 0] = st.mx;
    sm[wid * 3 + 1] = st.s;
    sm[wid * 3 + 2] = st.t;
  }
  __syncthreads();
  if (tid == 0) {
#pragma unroll
    for (int w = 1; w < kFwdThreads / kWave; ++w) merge(st, sm[w * 3], sm[w * 3 + 1], sm[w * 3 + 2], k);
    const float lse = st.mx * inv_T + logf(st.s);
    lse_out[row] = lse;
    if (ENT) {
      const float exv = inv_T * (st.t / st.s);
      ex_out[row] = exv;
      entropy[row] = lse - exv;
    }
    if (logprob != nullptr) {
      const int64_t y = labels[row];
      float lp = y == kIgnoreIndex ? 0.f : __builtin_nanf("");
      if (y >= 0 && y < (int64_t)V) lp = E::load1(x + y) * inv_T - lse;
      logprob[row] = lp;
    }
  }
}

// ----------------------------------------------------------------------------------- backward

struct BwdCoef {
  float k, nl, c0, c1;
};

template <bool HAS_ENT>
__device__ __forceinline__ float grad1(float x, const BwdCoef& c) {
  const float p = fast_exp2(fmaf(x, c.k, c.nl));
  return HAS_ENT ? p * fmaf(x, c.c1, c.c0) : p * c.c0;
}

template <class E, bool HAS_ENT>
__global__ __launch_bounds__(kBwdThreads) void lpe_bwd_kernel(const typename E::elem_t* logits, int64_t row_stride,
                                                           int V, const int64_t* __restrict__ labels, float inv_T,
                                                           const float* __restrict__ lse,
                                                           const float* __restrict__ ex,
                                                           const float* __restrict__ g_lp,
                                                           const float* __restrict__ g_ent,
                                                           typename E::elem_t* dlogits, int64_t d_stride,
                                                           uint32_t flags) {
  using elem_t = typename E::elem_t;
  const int64_t row = blockIdx.x;
  const elem_t* x = logits + row * row_stride;
  elem_t* d = dlogits + row * d_stride;
  const int tid = threadIdx.x;
  const RowSplit<E> sp(x, d, V);

  const bool skipped = labels != nullptr && labels[row] == kSkipRow;
  const float g1 = (g_lp && labels[row] != kIgnoreIndex) ? g_lp[row] : 0.f;
  const float g2 = HAS_ENT ? g_ent[row] : 0.f;
  const u32x4* xv = reinterpret_cast<const u32x4*>(x + sp.head);
  u32x4* dv = reinterpret_cast<u32x4*>(d + sp.head);

  if (skipped || ((flags & SIIRL_BWD_SKIP_ZERO_ROWS) && g1 == 0.f && g2 == 0.f)) {
    for (int i = tid; i < sp.head; i += kBwdThreads) E::store1(d + i, 0.f);
    for (int i = sp.tail0 + tid; i < V; i += kBwdThreads) E::store1(d + i, 0.f);
    const u32x4 z = u32x4{0u, 0u, 0u, 0u};
    for (int i = tid; i < sp.nvec; i += kBwdThreads) st16<SIIRL_LPE_BWD_NT_STORE>(z, dv + i);
    return;
  }

  BwdCoef c;
  c.k = inv_T * kLog2e;
  c.nl = -lse[row] * kLog2e;
  c.c0 = inv_T * ((HAS_ENT ? g2 * ex[row] : 0.f) - g1);
  c.c1 = -g2 * inv_T * inv_T;
  const float hot = g1 * inv_T;
  int y = -1;
  if (g_lp) {
    const int64_t yl = labels[row];
    if (yl >= 0 && yl < (int64_t)V) y = (int)yl;
  }
  // position of the label inside the vector body, or -1
  const int yb = (y >= sp.head && y < sp.tail0) ? (y - sp.head) : -1;
  const int yvec = yb >= 0 ? yb / E::VEC : -1;
  const int yj = yb >= 0 ? yb % E::VEC : 0;

  for (int i = tid; i < sp.head; i += kBwdThreads) {
    float g = grad1<HAS_ENT>(E::load1(x + i), c);
    if (i == y) g += hot;
    E::store1(d + i, g);
  }
  for (int i = sp.tail0 + tid; i < V; i += kBwdThreads) {
    float g = grad1<HAS_ENT>(E::load1(x + i), c);
    if (i == y) g += hot;
    E::store1(d + i, g);
  }

  auto do_vec = [&](const u32x4& in, int idx) {
    float v[E::VEC], g[E::VEC];
    E::unpack(in, v);
#pragma unroll
    for (int j = 0; j < E::VEC; ++j) g[j] = grad1<HAS_ENT>(v[j], c);
    if (idx == yvec) {
#pragma unroll
      for (int j = 0; j < E::VEC; ++j) g[j] += (j == yj) ? hot : 0.f;
    }
    st16<SIIRL_LPE_BWD_NT_STORE>(E::pack(g), dv + idx);
  };

  constexpr int kTile = kBwdThreads * kBwdUnroll;
  const int nfull = sp.nvec / kTile * kTile;
  for (int base = 0; base < nfull; base += kTile) {
    u32x4 buf[kBwdUnroll];
#pragma unroll
    for (int u = 0; u < kBwdUnroll; ++u) buf[u] = ld16<SIIRL_LPE_BWD_NT_LOAD>(xv + base + u * kBwdThreads + tid);
#pragma unroll
    for (int u = 0; u < kBwdUnroll; ++u) do_vec(buf[u], base + u * kBwdThreads + tid);
  }
  for (int i = nfull + tid; i < sp.nvec; i += kBwdThreads) {
    const u32x4 b = ld16<SIIRL_LPE_BWD_NT_LOAD>(xv + i);
    do_vec(b, i);
  }
}

// Flat variant of the backward for contiguous rows (row_stride == V, 16-byte aligned, V a multiple of the
// vector width): the [T, V] tensor is walked as one dense stream, workgroup b taking vectors
// [b * kFlatChunk, (b + 1) * kFlatChunk).  Workgroups in flight then cover one contiguous window of memory
// instead of one 16 KB piece in each of ~2000 different rows, which keeps DRAM pages open while they are used.
// A chunk is shorter than a row, so it touches at most two rows; their coefficients are wave-uniform.
// Measured at T=32768, V=152064 bf16: 3.2 ms (6.2 TB/s) against 3.85 ms for the row-per-workgroup kernel;
// 8 KB per workgroup (256 threads x 2 vectors) beats 4, 16, 32 and 64 KB, ordinary loads beat non-temporal ones.
#ifndef SIIRL_LPE_BWD_FLAT_ITER
#define SIIRL_LPE_BWD_FLAT_ITER 1
#endif
#ifndef SIIRL_LPE_BWD_FLAT_UNROLL
#define SIIRL_LPE_BWD_FLAT_UNROLL 2
#endif
#ifndef SIIRL_LPE_BWD_FLAT_NT_LOAD
#define SIIRL_LPE_BWD_FLAT_NT_LOAD 0
#endif
constexpr int kFlatIter = SIIRL_LPE_BWD_FLAT_ITER;
constexpr int kFlatUnroll = SIIRL_LPE_BWD_FLAT_UNROLL;
constexpr int kFlatChunk = kBwdThreads * kFlatUnroll * kFlatIter;  // vectors per workgroup

struct RowCoef {
  float nl, c0, c1, hot;
  int yvec, yj;
  bool zero;
};

template <class E, bool HAS_ENT>
__global__ __launch_bounds__(kBwdThreads) void lpe_bwd_flat_kernel(const typename E::elem_t* logits, int64_t T,
                                                                int vpr, int64_t total_vec,
                                                                const int64_t* __restrict__ labels, float inv_T,
                                                                const float* __restrict__ lse,
                                                                const float* __restrict__ ex,
                                                                const float* __restrict__ g_lp,
                                                                const float* __restrict__ g_ent,
                                                                typename E::elem_t* dlogits, uint32_t flags) {
  const int tid = threadIdx.x;
  const int64_t first = (int64_t)blockIdx.x * kFlatChunk;
  const int64_t row0 = first / vpr;
  const int rem0 = (int)(first - row0 * vpr);
  const float k = inv_T * kLog2e;
  RowCoef rc[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int64_t row = row0 + q;
    rc[q] = RowCoef{0.f, 0.f, 0.f, 0.f, -1, 0, true};
    if (row < T) {
      // A skipped row (label kSkipRow) takes no gradient: both upstream gradients count as zero, so with
      // SIIRL_BWD_SKIP_ZERO_ROWS it is written as zeros unread; without the flag its probabilities are forced to
      // zero (nl = -inf) and the arithmetic yields zeros for every logit that is not +inf or NaN.  (Making the row's
      // zero flag itself depend on the label, flag or no flag, cost this kernel 4 % at [32768, 152064]: 3.35 against
      // 3.21 ms.)
      const int64_t yl = labels != nullptr ? labels[row] : 0;
      const bool skipped = yl == kSkipRow;
      const float g1 = (g_lp && yl != kIgnoreIndex && !skipped) ? g_lp[row] : 0.f;
      const float g2 = (HAS_ENT && !skipped) ? g_ent[row] : 0.f;
      rc[q].zero = (flags & SIIRL_BWD_SKIP_ZERO_ROWS) && g1 == 0.f && g2 == 0.f;
      rc[q].nl = skipped ? -__builtin_inff() : -lse[row] * kLog2e;
      rc[q].c0 = inv_T * ((HAS_ENT ? g2 * ex[row] : 0.f) - g1);
      rc[q].c1 = -g2 * inv_T * inv_T;
      rc[q].hot = g1 * inv_T;
      if (g_lp) {
        const int64_t y = labels[row];
        if (y >= 0 && y < (int64_t)vpr * E::VEC) {
          rc[q].yvec = (int)(y / E::VEC);
          rc[q].yj = (int)(y % E::VEC);
        }
      }
    }
  }
  const u32x4* xv = reinterpret_cast<const u32x4*>(logits) + first;
  u32x4* dv = reinterpret_cast<u32x4*>(dlogits) + first;
  const int64_t left = total_vec - first;
  const int avail = left < kFlatChunk ? (int)left : kFlatChunk;
  constexpr int kTile = kBwdThreads * kFlatUnroll;
#pragma unroll 1
  for (int it = 0; it < kFlatIter; ++it) {
    u32x4 buf[kFlatUnroll];
#pragma unroll
    for (int u = 0; u < kFlatUnroll; ++u) {
      const int o = it * kTile + u * kBwdThreads + tid;
      const bool q = rem0 + o >= vpr;
      buf[u] = u32x4{0u, 0u, 0u, 0u};
      if (o < avail && !(q ? rc[1].zero : rc[0].zero)) buf[u] = ld16<SIIRL_LPE_BWD_FLAT_NT_LOAD>(xv + o);
    }
#pragma unroll
    for (int u = 0; u < kFlatUnroll; ++u) {
      const int o = it * kTile + u * kBwdThreads + tid;
      if (o >= avail) continue;
      const int r = rem0 + o;
      const bool q = r >= vpr;
      const RowCoef& c = q ? rc[1] : rc[0];
      const int rr = q ? r - vpr : r;
      float v[E::VEC], g[E::VEC];
      E::unpack(buf[u], v);
      const BwdCoef bc{k, c.nl, c.c0, c.c1};
#pragma unroll
      for (int j = 0; j < E::VEC; ++j) g[j] = c.zero ? 0.f : grad1<HAS_ENT>(v[j], bc);
      if (rr == c.yvec) {
#pragma unroll
        for (int j = 0; j < E::VEC; ++j) g[j] += (j == c.yj) ? c.hot : 0.f;
      }
      st16<SIIRL_LPE_BWD_NT_STORE>(E::pack(g), dv + o);
    }
  }
}

// ----------------------------------------------------------------------------------- fused forward + backward

// One workgroup (1024 threads, one per CU) per row does both passes: the online-softmax pass, then -- with the
// row's upstream gradients produced in-kernel from (logprob, entropy) by `Coef` -- the dlogits pass over the same
// row.  The first 152 KB of the row stay in LDS between the passes (half of a 152064-entry bf16 row), the rest is
// read a second time, last-read-first so that the L2 serves what it still holds.  HBM sees about 5 bytes per
// element instead of the 6 of separate forward and backward launches, and one launch less.
// Measured at T=32768, V=152064 bf16: 3.8 ms against 4.67 ms for forward + flat backward.  Keeping the second half
// of the row in registers as well (whole row on chip, 4 bytes per element) measured no faster: with one workgroup
// per CU the exponentials of the two passes no longer hide behind the memory stream (3.86 ms with the last two
// tiles and the ragged end in registers, 4.14 ms when those loads are all issued up front: more requests in flight
// per CU scatter over more DRAM pages).  Counter-measured traffic of this kernel at that size: 13.1 GB fetched (the
// L2 and the memory-side cache serve a third of the second read) + 10.0 GB written in 3.65 ms = 6.3 TB/s, the
// streaming-copy rate of the part.  A persistent variant that
// holds the whole row in registers and interleaves the dlogits pass of one row with the load and softmax pass of
// the workgroup's next row (4 bytes per element, nothing re-read) measured 4.3 ms (1024 threads) to 5.9 ms (512):
// the workgroup-wide merge between rows drains that CU's loads once per row.
#ifndef SIIRL_LPE_FUSED_THREADS
#define SIIRL_LPE_FUSED_THREADS 1024
#endif
#ifndef SIIRL_LPE_FUSED_UNROLL
#define SIIRL_LPE_FUSED_UNROLL 4
#endif
constexpr int kFusedThreads = SIIRL_LPE_FUSED_THREADS;
constexpr int kFusedUnroll = SIIRL_LPE_FUSED_UNROLL;

// upstream gradients given per row (the plain "backward with known grads" case)
struct GivenGrads {
  const float* g_lp;
  const float* g_ent;
  __device__ __forceinline__ void operator()(int64_t row, float lp, float ent, float& g1, float& g2) const {
    g1 = g_lp ? g_lp[row] : 0.f;
    g2 = g_ent ? g_ent[row] : 0.f;
  }
};

// Upstream gradients of the actor's loss for one token, from its log-prob and entropy: the policy loss `kind`
// (vanilla / cpgd / gpg: the token-separable ones), the KL loss, the entropy bonus and the CPGD drift term, each
// times its aggregation weight.  The aggregation weights depend on the mask alone and are given per token.
struct ActorCoef {
  tok::LossArgs a;         // clip bounds, coefficients, kind; its tensor fields are the per-token arrays below
  const float* w_pg;       // d agg / d loss_mat for the policy term
  const float* w_aux;      // the same for the entropy / KL / drift terms
  __device__ __forceinline__ void operator()(int64_t row, float lp, float ent, float& g1, float& g2) const {
    const float wp = w_pg[row], wa = w_aux[row];
    const float old = a.old_lp ? a.old_lp[row] : lp;  // on-policy: old = log_prob.detach()
    const float isw = a.isw ? a.isw[row] : 1.f;
    const tok::PgOut o = tok::pg_token(a.kind, lp, old, a.adv[row], isw, 0.f, a);
    float d = wp * o.dtok;
    if (a.drift_coef != 0.f) d += a.drift_coef * wa * tok::clamp_max(o.r_raw - 1.f, 2.f);
    if (a.ref) d += a.kl_coef * wa * tok::kl_token(lp, a.ref[row], a.kl_mode, a.kl_st).g;
    // a token outside the mask has weight 0; its log-prob may be anything (NaN for a padding label)
    g1 = (wp == 0.f && wa == 0.f) ? 0.f : a.scale * d;
    g2 = -a.scale * a.ent_coef * wa;
  }
};

template <class E, bool ENT, class Coef>
__global__ __launch_bounds__(kFusedThreads) void lpe_fused_kernel(const typename E::elem_t* logits, int64_t row_stride,
                                                                  int V, const int64_t* __restrict__ labels,
                                                                  float inv_T, Coef coef, float* __restrict__ logprob,
                                                                  float* __restrict__ entropy,
                                                                  typename E::elem_t* dlogits, int64_t d_stride,
                                                                  int lds_vecs) {
  using elem_t = typename E::elem_t;
  const int64_t row = blockIdx.x;
  const elem_t* x = logits + row * row_stride;
  elem_t* d = dlogits + row * d_stride;
  const int tid = threadIdx.x;
  const float k = inv_T * kLog2e;
  const RowSplit<E> sp(x, d, V);
  const u32x4* xv = reinterpret_cast<const u32x4*>(x + sp.head);
  u32x4* dv = reinterpret_cast<u32x4*>(d + sp.head);
  constexpr int kTile = kFusedThreads * kFusedUnroll;

  // A row labelled "skip" (a packed token outside the response window) is not read at all, as in the two-launch
  // kernels: log-prob and entropy 0, a gradient of zeros whatever the upstream coefficients would be.  The label is
  // the same for the whole workgroup, so every thread leaves here, before the first barrier.
  if (labels && labels[row] == kSkipRow) {
    if (tid == 0) {
      if (logprob) logprob[row] = 0.f;
      if (ENT && entropy) entropy[row] = 0.f;
    }
    for (int i = tid; i < sp.head; i += kFusedThreads) E::store1(d + i, 0.f);
    for (int i = sp.tail0 + tid; i < V; i += kFusedThreads) E::store1(d + i, 0.f);
    const u32x4 z = u32x4{0u, 0u, 0u, 0u};
    for (int i = tid; i < sp.nvec; i += kFusedThreads) st16<true>(z, dv + i);
    return;
  }

  // the first `cap` 16-byte vectors of the row are kept in LDS between the passes
  extern __shared__ __align__(16) char row_lds[];
  u32x4* keep = reinterpret_cast<u32x4*>(row_lds);
  const int cap = lds_vecs < sp.nvec ? lds_vecs : sp.nvec;
  // ---- pass 1: online softmax state (ordinary loads: the row should stay cached for pass 2)
  SoftState st{-1e30f, 0.f, 0.f};
  for (int i = tid; i < sp.head; i += kFusedThreads) absorb1<ENT>(st, E::load1(x + i), k);
  for (int i = sp.tail0 + tid; i < V; i += kFusedThreads) absorb1<ENT>(st, E::load1(x + i), k);
  // region A = vectors [0, capA): kept in LDS (whole tiles only, so that it has no ragged end); region C = the
  // rest of the row: read again in pass 2
  const int capA = cap / kTile * kTile;
  const int nfull = sp.nvec / kTile * kTile;
  for (int base = 0; base < nfull; base += kTile) {
    u32x4 buf[kFusedUnroll];
#pragma unroll
    for (int u = 0; u < kFusedUnroll; ++u) buf[u] = ld16<false>(xv + base + u * kFusedThreads + tid);
    if (base < capA) {
#pragma unroll
      for (int u = 0; u < kFusedUnroll; ++u) keep[base + u * kFusedThreads + tid] = buf[u];
    }
    absorb_vecs<E, ENT, kFusedUnroll>(st, buf, k);
  }
  for (int i = nfull + tid; i < sp.nvec; i += kFusedThreads) {
    u32x4 b = ld16<false>(xv + i);
    absorb_vecs<E, ENT, 1>(st, &b, k);
  }
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const float omx = __shfl_xor(st.mx, o, kWave);
    const float os = __shfl_xor(st.s, o, kWave);
    const float ot = __shfl_xor(st.t, o, kWave);
    merge(st, omx, os, ot, k);
  }
  __shared__ float sm[3 * (kFusedThreads / kWave)];
  __shared__ float bc[4];

  const int lane = tid & (kWave - 1), wid = tid / kWave;
  if (lane == 0) {
    sm[wid * 3 + 0] = st.mx;
    sm[wid * 3 + 1] = st.s;
    sm[wid * 3 + 2] = st.t;
  }
  __syncthreads();
  int y = -1;
  bool ignored = false;
  {
    const int64_t yl = labels ? labels[row] : -1;
    if (yl >= 0 && yl < (int64_t)V) y = (int)yl;
    ignored = labels && yl == kIgnoreIndex;
  }
  if (tid == 0) {
    for (int w = 1; w < kFusedThreads / kWave; ++w) merge(st, sm[w * 3], sm[w * 3 + 1], sm[w * 3 + 2], k);
    const float lse = st.mx * inv_T + logf(st.s);
    const float exv = ENT ? inv_T * (st.t / st.s) : 0.f;
    const float lp = y >= 0 ? E::load1(x + y) * inv_T - lse : (ignored ? 0.f : __builtin_nanf(""));
    bc[0] = lse;
    bc[1] = exv;
    bc[2] = lp;
    if (logprob) logprob[row] = lp;
    if (ENT && entropy) entropy[row] = lse - exv;
  }
  __syncthreads();
  const float lse = bc[0], exv = bc[1], lp = bc[2];

  // ---- the row's upstream gradients, then pass 2: dlogits
  float g1, g2;
  coef(row, lp, lse - exv, g1, g2);
  if (!ENT) g2 = 0.f;
  if (ignored) g1 = 0.f;
  BwdCoef c;
  c.k = k;
  c.nl = -lse * kLog2e;
  c.c0 = inv_T * (g2 * exv - g1);
  c.c1 = -g2 * inv_T * inv_T;
  const float hot = g1 * inv_T;
  const bool zero = g1 == 0.f && g2 == 0.f;
  const int yb = (y >= sp.head && y < sp.tail0) ? (y - sp.head) : -1;
  const int yvec = yb >= 0 ? yb / E::VEC : -1;
  const int yj = yb >= 0 ? yb % E::VEC : 0;

  if (zero) {  // nothing flows into this row (padding, prompt tokens): zeros, without the second read
    for (int i = tid; i < sp.head; i += kFusedThreads) E::store1(d + i, 0.f);
    for (int i = sp.tail0 + tid; i < V; i += kFusedThreads) E::store1(d + i, 0.f);
    const u32x4 z = u32x4{0u, 0u, 0u, 0u};
    for (int i = tid; i < sp.nvec; i += kFusedThreads) st16<true>(z, dv + i);
    return;
  }
  for (int i = tid; i < sp.head; i += kFusedThreads) {
    float g = grad1<ENT>(E::load1(x + i), c);
    if (i == y) g += hot;
    E::store1(d + i, g);
  }
  for (int i = sp.tail0 + tid; i < V; i += kFusedThreads) {
    float g = grad1<ENT>(E::load1(x + i), c);
    if (i == y) g += hot;
    E::store1(d + i, g);
  }
  auto do_vec = [&](const u32x4& in, int idx) {
    float v[E::VEC], g[E::VEC];
    E::unpack(in, v);
#pragma unroll
    for (int j = 0; j < E::VEC; ++j) g[j] = grad1<ENT>(v[j], c);
    if (idx == yvec) {
#pragma unroll
      for (int j = 0; j < E::VEC; ++j) g[j] += (j == yj) ? hot : 0.f;
    }
    st16<true>(E::pack(g), dv + idx);
  };
  for (int i = nfull + tid; i < sp.nvec; i += kFusedThreads) do_vec(ld16<false>(xv + i), i);
  // last read first: the end of the row is what the L2 still holds.  Each thread re-reads the LDS slots it wrote
  // itself, so no barrier is needed for them.
  for (int base = nfull - kTile; base >= 0; base -= kTile) {
    if (base < capA) {
#pragma unroll
      for (int u = 0; u < kFusedUnroll; ++u) {
        const int idx = base + u * kFusedThreads + tid;
        do_vec(keep[idx], idx);
      }
    } else {
      u32x4 buf[kFusedUnroll];
#pragma unroll
      for (int u = 0; u < kFusedUnroll; ++u) buf[u] = ld16<false>(xv + base + u * kFusedThreads + tid);
#pragma unroll
      for (int u = 0; u < kFusedUnroll; ++u) do_vec(buf[u], base + u * kFusedThreads + tid);
    }
  }
}

template <class E, class Coef>
int launch_fused(const void* logits, int64_t T, int V, int64_t row_stride, const int64_t* labels, float inv_T,
                 const Coef& coef, bool with_entropy, float* logprob, float* entropy, void* dlogits, int64_t d_stride,
                 hipStream_t st) {
  using elem_t = typename E::elem_t;
  dim3 grid((unsigned)T), block(kFusedThreads);
#ifndef SIIRL_LPE_FUSED_LDS_BYTES
#define SIIRL_LPE_FUSED_LDS_BYTES 155648
#endif
  constexpr int kLds = SIIRL_LPE_FUSED_LDS_BYTES;
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&lpe_fused_kernel<E, true, Coef>), kLds)) return rc;
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&lpe_fused_kernel<E, false, Coef>), kLds)) return rc;
  if (with_entropy)
    lpe_fused_kernel<E, true, Coef><<<grid, block, kLds, st>>>((const elem_t*)logits, row_stride, V, labels, inv_T, coef,
                                                            logprob, entropy, (elem_t*)dlogits, d_stride, kLds / 16);
  else
    lpe_fused_kernel<E, false, Coef><<<grid, block, kLds, st>>>((const elem_t*)logits, row_stride, V, labels, inv_T, coef,
                                                             logprob, entropy, (elem_t*)dlogits, d_stride, kLds / 16);
  SIIRL_LAUNCH_CHECK("lpe_fused_kernel");
  return SIIRL_OK;
}

template <class E>
int launch_fwd(const void* logits, int64_t T, int V, int64_t row_stride, const int64_t* labels, float inv_T,
               float* logprob, float* entropy, float* lse, float* ex, hipStream_t st) {
  using elem_t = typename E::elem_t;
  dim3 grid((unsigned)T), block(kFwdThreads);
  // Logits of up to kCacheResidentBytes (the part's 256 MB memory-side cache and a little more) are read with
  // ordinary loads, so that the backward pass that follows finds them cached: measured on [2048, 32000] fp32
  // (250 MiB) forward + backward 128 -> 117 us, [768, 152064] bf16 (223 MiB) 114 -> 103 us, the forward alone
  // unchanged; from 375 MiB upwards the non-temporal loads win (forward alone 60 against 70 us at that size).
  const bool nt = SIIRL_LPE_FWD_NT_LOAD && streams_past_cache((double)T * (double)V * (double)sizeof(elem_t));
  auto go = [&](auto ent_tag, auto nt_tag) {
    lpe_fwd_kernel<E, decltype(ent_tag)::value, decltype(nt_tag)::value><<<grid, block, 0, st>>>(
        (const elem_t*)logits, row_stride, V, labels, inv_T, logprob, decltype(ent_tag)::value ? entropy : nullptr, lse,
        decltype(ent_tag)::value ? ex : nullptr);
  };
  using Yes = std::true_type;
  using No = std::false_type;
  if (entropy) {
    if (nt) go(Yes{}, Yes{}); else go(Yes{}, No{});
  } else {
    if (nt) go(No{}, Yes{}); else go(No{}, No{});
  }
  SIIRL_LAUNCH_CHECK("lpe_fwd_kernel");
  return SIIRL_OK;
}

template <class E>
int launch_bwd(const void* logits, int64_t T, int V, int64_t row_stride, const int64_t* labels, float inv_T,
               const float* lse, const float* ex, const float* g_lp, const float* g_ent, void* dlogits,
               int64_t d_stride, uint32_t flags, hipStream_t st) {
  using elem_t = typename E::elem_t;
#if SIIRL_LPE_BWD_FLAT
  const bool aligned = (((uintptr_t)logits | (uintptr_t)dlogits) & 15u) == 0;
  if (aligned && row_stride == V && d_stride == V && V % E::VEC == 0 && V / E::VEC >= kFlatChunk) {
    const int vpr = V / E::VEC;
    const int64_t total_vec = T * (int64_t)vpr;
    const int64_t blocks = (total_vec + kFlatChunk - 1) / kFlatChunk;
    if (blocks <= 0x7fffffffLL) {
      dim3 grid((unsigned)blocks), block(kBwdThreads);
      if (g_ent)
        lpe_bwd_flat_kernel<E, true><<<grid, block, 0, st>>>((const elem_t*)logits, T, vpr, total_vec, labels, inv_T,
                                                             lse, ex, g_lp, g_ent, (elem_t*)dlogits, flags);
      else
        lpe_bwd_flat_kernel<E, false><<<grid, block, 0, st>>>((const elem_t*)logits, T, vpr, total_vec, labels, inv_T,
                                                              lse, nullptr, g_lp, nullptr, (elem_t*)dlogits, flags);
      SIIRL_LAUNCH_CHECK("lpe_bwd_flat_kernel");
      return SIIRL_OK;
    }
  }
#endif
  using elem_t = typename E::elem_t;
  dim3 grid((unsigned)T), block(kBwdThreads);
  if (g_ent)
    lpe_bwd_kernel<E, true><<<grid, block, 0, st>>>((const elem_t*)logits, row_stride, V, labels, inv_T, lse, ex,
                                                    g_lp, g_ent, (elem_t*)dlogits, d_stride, flags);
  else
    lpe_bwd_kernel<E, false><<<grid, block, 0, st>>>((const elem_t*)logits, row_stride, V, labels, inv_T, lse,
                                                     nullptr, g_lp, nullptr, (elem_t*)dlogits, d_stride, flags);
  SIIRL_LAUNCH_CHECK("lpe_bwd_kernel");
  return SIIRL_OK;
}

int check_common(const void* logits, int dt, int64_t T, int64_t V, int64_t row_stride, float inv_T) {
  SIIRL_REQUIRE(dt == SIIRL_F32 || dt == SIIRL_BF16 || dt == SIIRL_F16,
                "logits dtype %d not supported (f32, bf16, f16)", dt);
  SIIRL_REQUIRE(T >= 0 && T <= 0x7fffffffLL, "T=%lld out of range", (long long)T);
  SIIRL_REQUIRE(V >= 1 && V <= 0x3fffffffLL, "V=%lld out of range", (long long)V);
  SIIRL_REQUIRE(row_stride >= V, "row_stride %lld < V %lld", (long long)row_stride, (long long)V);
  SIIRL_REQUIRE(inv_T > 0.f && inv_T < 1e30f, "inv_temperature must be positive and finite");
  SIIRL_REQUIRE(T == 0 || logits != nullptr, "logits is NULL");
  SIIRL_REQUIRE(((uintptr_t)logits % dtype_size(dt)) == 0, "logits not aligned to its element size");
  return SIIRL_OK;
}

}  // namespace
}  // namespace siirl

using namespace siirl;

extern "C" int siirl_logprob_entropy_fwd(const void* logits, int logits_dtype, int64_t T, int64_t V,
                                         int64_t row_stride, const int64_t* labels, float inv_temperature,
                                         float* logprob, float* entropy, float* lse, float* ex,
                                         siirl_stream_t stream) {
  if (int rc = check_common(logits, logits_dtype, T, V, row_stride, inv_temperature)) return rc;
  if (T == 0) return SIIRL_OK;
  SIIRL_REQUIRE(lse != nullptr, "lse is NULL");
  SIIRL_REQUIRE((logprob == nullptr) == (labels == nullptr), "labels and logprob must be given together");
  SIIRL_REQUIRE(entropy == nullptr || ex != nullptr, "ex is required when entropy is requested");
  SIIRL_REQUIRE(logprob != nullptr || entropy != nullptr, "nothing requested: logprob and entropy are both NULL");
  hipStream_t st = (hipStream_t)stream;
  switch (logits_dtype) {
    case SIIRL_BF16:
      return launch_fwd<ElemBF16>(logits, T, (int)V, row_stride, labels, inv_temperature, logprob, entropy, lse, ex, st);
    case SIIRL_F16:
      return launch_fwd<ElemF16>(logits, T, (int)V, row_stride, labels, inv_temperature, logprob, entropy, lse, ex, st);
    default:
      return launch_fwd<ElemF32>(logits, T, (int)V, row_stride, labels, inv_temperature, logprob, entropy, lse, ex, st);
  }
}

extern "C" int siirl_logprob_entropy_bwd(const void* logits, int logits_dtype, int64_t T, int64_t V,
                                         int64_t row_stride, const int64_t* labels, float inv_temperature,
                                         const float* lse, const float* ex, const float* g_logprob,
                                         const float* g_entropy, void* dlogits, int64_t dlogits_row_stride,
                                         uint32_t flags, siirl_stream_t stream) {
  if (int rc = check_common(logits, logits_dtype, T, V, row_stride, inv_temperature)) return rc;
  if (T == 0) return SIIRL_OK;
  SIIRL_REQUIRE(dlogits != nullptr && lse != nullptr, "dlogits / lse is NULL");
  SIIRL_REQUIRE(dlogits_row_stride >= V, "dlogits_row_stride %lld < V", (long long)dlogits_row_stride);
  SIIRL_REQUIRE(g_logprob != nullptr || g_entropy != nullptr, "no upstream gradient given");
  SIIRL_REQUIRE(g_logprob == nullptr || labels != nullptr, "labels is required with g_logprob");
  SIIRL_REQUIRE(g_entropy == nullptr || ex != nullptr, "ex is required with g_entropy");
  SIIRL_REQUIRE((flags & ~SIIRL_BWD_SKIP_ZERO_ROWS) == 0, "unknown flags 0x%x", flags);
  SIIRL_REQUIRE(((uintptr_t)dlogits % dtype_size(logits_dtype)) == 0, "dlogits not aligned to its element size");
  if (dlogits == logits) {
    SIIRL_REQUIRE(dlogits_row_stride == row_stride, "in-place backward needs equal row strides");
  } else {
    const size_t es = dtype_size(logits_dtype);
    const uintptr_t a0 = (uintptr_t)logits, a1 = a0 + (size_t)((T - 1) * row_stride + V) * es;
    const uintptr_t b0 = (uintptr_t)dlogits, b1 = b0 + (size_t)((T - 1) * dlogits_row_stride + V) * es;
    SIIRL_REQUIRE(a1 <= b0 || b1 <= a0, "dlogits overlaps logits without being the same buffer");
  }
  hipStream_t st = (hipStream_t)stream;
  switch (logits_dtype) {
    case SIIRL_BF16:
      return launch_bwd<ElemBF16>(logits, T, (int)V, row_stride, labels, inv_temperature, lse, ex, g_logprob,
                                  g_entropy, dlogits, dlogits_row_stride, flags, st);
    case SIIRL_F16:
      return launch_bwd<ElemF16>(logits, T, (int)V, row_stride, labels, inv_temperature, lse, ex, g_logprob,
                                 g_entropy, dlogits, dlogits_row_stride, flags, st);
    default:
      return launch_bwd<ElemF32>(logits, T, (int)V, row_stride, labels, inv_temperature, lse, ex, g_logprob,
                                 g_entropy, dlogits, dlogits_row_stride, flags, st);
  }
}

extern "C" int siirl_logprob_entropy_fwd_bwd(const void* logits, int logits_dtype, int64_t T, int64_t V,
                                             int64_t row_stride, const int64_t* labels, float inv_temperature,
                                             const float* g_logprob, const float* g_entropy, float* logprob,
                                             float* entropy, void* dlogits, int64_t dlogits_row_stride,
                                             siirl_stream_t stream) {
  if (int rc = check_common(logits, logits_dtype, T, V, row_stride, inv_temperature)) return rc;
  if (T == 0) return SIIRL_OK;
  SIIRL_REQUIRE(dlogits != nullptr && dlogits != logits, "dlogits is NULL or the logits buffer (no in-place mode here)");
  SIIRL_REQUIRE(dlogits_row_stride >= V, "dlogits_row_stride %lld < V", (long long)dlogits_row_stride);
  SIIRL_REQUIRE(g_logprob != nullptr || g_entropy != nullptr, "no upstream gradient given");
  SIIRL_REQUIRE((g_logprob == nullptr && logprob == nullptr) || labels != nullptr, "labels is required with g_logprob / logprob");
  SIIRL_REQUIRE(((uintptr_t)dlogits % dtype_size(logits_dtype)) == 0, "dlogits not aligned to its element size");
  {
    const size_t es = dtype_size(logits_dtype);
    const uintptr_t a0 = (uintptr_t)logits, a1 = a0 + (size_t)((T - 1) * row_stride + V) * es;
    const uintptr_t b0 = (uintptr_t)dlogits, b1 = b0 + (size_t)((T - 1) * dlogits_row_stride + V) * es;
    SIIRL_REQUIRE(a1 <= b0 || b1 <= a0, "dlogits overlaps logits");
  }
  hipStream_t st = (hipStream_t)stream;
  const GivenGrads coef{g_logprob, g_entropy};
  const bool ent = g_entropy != nullptr || entropy != nullptr;
  switch (logits_dtype) {
    case SIIRL_BF16:
      return launch_fused<ElemBF16>(logits, T, (int)V, row_stride, labels, inv_temperature, coef, ent, logprob, entropy,
                                    dlogits, dlogits_row_stride, st);
    case SIIRL_F16:
      return launch_fused<ElemF16>(logits, T, (int)V, row_stride, labels, inv_temperature, coef, ent, logprob, entropy,
                                   dlogits, dlogits_row_stride, st);
    default:
      return launch_fused<ElemF32>(logits, T, (int)V, row_stride, labels, inv_temperature, coef, ent, logprob, entropy,
                                   dlogits, dlogits_row_stride, st);
  }
}

extern "C" int siirl_actor_step_fused(const void* logits, int logits_dtype, int64_t T, int64_t V, int64_t row_stride,
                                      const int64_t* labels, float inv_temperature, const float* old_log_prob,
                                      const float* advantages, const float* ref_log_prob, const float* is_weights,
                                      const float* w_policy, const float* w_aux, int loss_mode, float clip_low,
                                      float clip_high, float clip_c, float log_ratio_clamp, float entropy_coeff,
                                      int kl_mode, int kl_straight_through, float kl_coef, float policy_drift_coeff,
                                      float loss_scale, float* logprob, float* entropy, void* dlogits,
                                      int64_t dlogits_row_stride, siirl_stream_t stream) {
  if (int rc = check_common(logits, logits_dtype, T, V, row_stride, inv_temperature)) return rc;
  if (T == 0) return SIIRL_OK;
  SIIRL_REQUIRE(dlogits != nullptr && dlogits != logits, "dlogits is NULL or the logits buffer (no in-place mode here)");
  SIIRL_REQUIRE(dlogits_row_stride >= V, "dlogits_row_stride %lld < V", (long long)dlogits_row_stride);
  SIIRL_REQUIRE(labels && advantages && w_policy && w_aux && logprob, "NULL operand");
  SIIRL_REQUIRE(loss_mode == SIIRL_LOSS_VANILLA || loss_mode == SIIRL_LOSS_CPGD || loss_mode == SIIRL_LOSS_GPG,
                "loss mode %d is not token-separable (gspo and geo_mean need the two-pass path)", loss_mode);
  if (loss_mode != SIIRL_LOSS_GPG) SIIRL_REQUIRE(clip_c > 1.0f, "clip_ratio_c must be greater than 1.0, got %f", (double)clip_c);
  SIIRL_REQUIRE(log_ratio_clamp > 0.f, "log_ratio_clamp must be positive (20 in the reference, +inf for none)");
  if (ref_log_prob) SIIRL_REQUIRE(kl_mode >= 0 && kl_mode <= 3, "unknown kl mode %d", kl_mode);
  SIIRL_REQUIRE(entropy_coeff == 0.f || entropy != nullptr, "entropy output is required with a non-zero entropy_coeff");
  SIIRL_REQUIRE(((uintptr_t)dlogits % dtype_size(logits_dtype)) == 0, "dlogits not aligned to its element size");
  {
    const size_t es = dtype_size(logits_dtype);
    const uintptr_t a0 = (uintptr_t)logits, a1 = a0 + (size_t)((T - 1) * row_stride + V) * es;
    const uintptr_t b0 = (uintptr_t)dlogits, b1 = b0 + (size_t)((T - 1) * dlogits_row_stride + V) * es;
    SIIRL_REQUIRE(a1 <= b0 || b1 <= a0, "dlogits overlaps logits");
  }
  ActorCoef coef{};
  tok::LossArgs& a = coef.a;
  a.old_lp = old_log_prob; a.adv = advantages; a.ref = ref_log_prob; a.isw = loss_mode == SIIRL_LOSS_CPGD ? nullptr : is_weights;
  a.kind = loss_mode == SIIRL_LOSS_VANILLA ? tok::KIND_VANILLA : (loss_mode == SIIRL_LOSS_CPGD ? tok::KIND_CPGD : tok::KIND_GPG);
  a.kl_mode = kl_mode; a.kl_st = kl_straight_through;
  a.eps_lo = clip_low; a.eps_hi = clip_high; a.clip_c = clip_c; a.dclamp = log_ratio_clamp;
  if (loss_mode == SIIRL_LOSS_CPGD) {
    SIIRL_REQUIRE(clip_low < 1.0f && clip_high > -1.0f, "CPGD takes log(1 - clip_low) and log(1 + clip_high)");
    a.log_lo = (float)log(1.0 - (double)clip_low);
    a.log_hi = (float)log(1.0 + (double)clip_high);
  }
  a.ent_coef = entropy_coeff; a.kl_coef = ref_log_prob ? kl_coef : 0.f; a.drift_coef = policy_drift_coeff; a.scale = loss_scale;
  coef.w_pg = w_policy; coef.w_aux = w_aux;
  hipStream_t st = (hipStream_t)stream;
  const bool ent = entropy != nullptr;
  switch (logits_dtype) {
    case SIIRL_BF16:
      return launch_fused<ElemBF16>(logits, T, (int)V, row_stride, labels, inv_temperature, coef, ent, logprob, entropy,
                                    dlogits, dlogits_row_stride, st);
    case SIIRL_F16:
      return launch_fused<ElemF16>(logits, T, (int)V, row_stride, labels, inv_temperature, coef, ent, logprob, entropy,
                                   dlogits, dlogits_row_stride, st);
    default:
      return launch_fused<ElemF32>(logits, T, (int)V, row_stride, labels, inv_temperature, coef, ent, logprob, entropy,
                                   dlogits, dlogits_row_stride, st);
  }
}
