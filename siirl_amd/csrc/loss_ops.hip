// [B, L] loss arithmetic of the actor and critic updates: the registered policy-gradient losses (PPO / GRPO /
// DAPO "vanilla", GSPO, CPGD, GPG, GMPO "geo_mean"), the CPGD drift term, the clipped value loss, KL penalty,
// masked aggregation, and their hand-written backward.
//
// Replaces, of siirl/dag_worker/core_algos.py:  agg_loss :536-569, compute_policy_loss_cpgd :572-629,
// compute_policy_loss_vanilla :710-792, compute_policy_loss_gspo :795-862, compute_policy_loss_gpg :865-895,
// compute_policy_loss_geo_mean :1074-1153, compute_value_loss :1173-1212, kl_penalty :1215-1276; of
// siirl/utils/model_utils/torch_functional.py: masked_sum / masked_mean :146-168; and the composition of
// siirl/engine/actor/dp_actor.py:455-513 (drift term :488-494).
//
// Shape of the computation: one workgroup reduces a segment of kSeg tokens of one row into kNP partial
// sums (LDS tree per partial), a single-workgroup finish kernel folds segments into rows and rows into
// the scalars in double precision.  No atomics: results are reproducible run to run.  The backward is a
// plain elementwise kernel that re-evaluates the token and applies autograd's tie rules by hand.
#include "common.hpp"
#include "loss_token.hpp"

#include <mutex>

// Scratch of siirl_actor_loss_fwd_static, the entry point that allocates nothing: the segment partials, the row
// pre-pass sums and the finish records that the other forward entry points take from the caller's workspace.  One
// copy per GPU, held until the process ends, cut into slices ("slots") so that calls on different streams can each
// have their own.  In host code this name is only a handle for hipGetSymbolAddress; kernels receive the device
// address that call returns.
constexpr size_t kStaticScratchBytes = SIIRL_ACTOR_LOSS_STATIC_SCRATCH_BYTES;  // per slot
constexpr int kStaticSlots = SIIRL_ACTOR_LOSS_STATIC_SLOTS;
static __device__ __align__(256) unsigned char scratch[kStaticSlots * kStaticScratchBytes];

namespace siirl {
namespace {

// Threads of the two streaming kernels (partials, backward).  Measured at [5488, 8192] fp32 with an int64 mask,
// actor loss forward + backward: 128 threads x 16 tokens per thread 0.46 ms, 256 x 8 tokens 0.48-0.52 ms; longer
// segments change nothing further.
#ifndef SIIRL_LOSS_THREADS
#define SIIRL_LOSS_THREADS 128
#endif
#ifndef SIIRL_LOSS_SEG
#define SIIRL_LOSS_SEG 2048
#endif
constexpr int kThreads = 256;                  // every other kernel of this file
constexpr int kStream = SIIRL_LOSS_THREADS;
constexpr int kSeg = SIIRL_LOSS_SEG;  // tokens per workgroup
constexpr int kNP = 12;     // partials per segment (see enum P)

enum P { P_PG = 0, P_M, P_CLIP, P_NEGD, P_LOWER, P_ENT, P_KL, P_RSUM, P_RMIN, P_RMAX, P_AUX0, P_AUX1 };
// out[] of the finish kernel
enum O { O_LOSS = 0, O_PG, O_CLIPFRAC, O_PPOKL, O_CLIPLOWER, O_ENTLOSS, O_KLLOSS, O_RMEAN, O_RMIN, O_RMAX,
         O_MTOTAL, O_POLICY, O_DRIFT, O_COUNT = 16 };

using namespace tok;

// ---------------------------------------------------------------------------- row pre-pass (GSPO)

// per segment: GSPO { sum_t (lp - old) * m, sum_t m };  GEO { sum_t x * m, sum_t m, sum_t A * m,
// sum_t log(isw + 1e-10) * m }, x the token's clipped log-ratio
constexpr int kNPre = 4;
__global__ __launch_bounds__(kThreads) void row_prepass_kernel(LossArgs a, float* __restrict__ pre) {
  const int64_t b = blockIdx.x / a.nseg;
  const int seg = blockIdx.x % a.nseg;
  const int64_t t0 = (int64_t)seg * kSeg;
  float sd = 0.f, sm = 0.f, sa = 0.f, sw = 0.f;
  for (int i = threadIdx.x; i < kSeg; i += kThreads) {
    const int64_t t = t0 + i;
    if (t < a.L) {
      const int64_t idx = b * a.L + t;
      const float m = load_mask(a.mask, a.mask_dtype, idx);
      sm += m;
      if (a.kind == KIND_GSPO) {
        sd += (a.lp[idx] - a.old_lp[idx]) * m;
      } else {
        const float A = a.adv[idx];
        sd += pg_token(KIND_GEO, a.lp[idx], a.old_lp[idx], A, 1.f, 0.f, a).tok * m;
        sa += A * m;
        if (a.isw) sw += logf(a.isw[idx] + 1e-10f) * m;
      }
    }
  }
  __shared__ float sh[kThreads / kWave + 1];
  sd = block_sum(sd, sh);
  sm = block_sum(sm, sh);
  sa = block_sum(sa, sh);
  sw = block_sum(sw, sh);
  if (threadIdx.x == 0) {
    float* p = pre + (b * a.nseg + seg) * kNPre;
    p[0] = sd; p[1] = sm; p[2] = sa; p[3] = sw;
  }
}

// folds the pre-pass segments of each row.  GSPO: row_s[b] = sum d*m / max(sum m, 1).  GEO: row_s[b] is the
// sequence's loss -adv_b * exp(sum x*m / (n + 1e-8)) [* exp(sum log(w + 1e-10)*m / (n + 1e-8))], adv_b =
// sum A*m / (n + 1e-8), in the reference's float32 arithmetic.
__global__ __launch_bounds__(kThreads) void row_finish_kernel(const float* __restrict__ pre, int nseg, int64_t B,
                                                              int kind, int has_isw, float* __restrict__ row_s) {
  const int64_t b = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (b >= B) return;
  double sd = 0.0, sm = 0.0, sa = 0.0, sw = 0.0;
  for (int s = 0; s < nseg; ++s) {
    const float* p = pre + (b * nseg + s) * kNPre;
    sd += p[0]; sm += p[1]; sa += p[2]; sw += p[3];
  }
  if (kind == KIND_GSPO) {
    const float n = fmaxf((float)sm, 1.f);  // .clamp(min=1)
    row_s[b] = (float)sd / n;
  } else {
    const float n = (float)sm + 1e-8f;
    float v = -((float)sa / n) * expf((float)sd / n);
    if (has_isw) v *= expf((float)sw / n);
    row_s[b] = v;
  }
}

// ---------------------------------------------------------------------------- segment partials

// KIND >= 0 compiles the token formula of that loss alone (the common ones); KIND < 0 reads a.kind at run time.
template <int KIND>
__global__ __launch_bounds__(kStream) void loss_partials_kernel(LossArgs a, const float* __restrict__ row_s,
                                                                 float* __restrict__ partials) {
  const int kind = KIND >= 0 ? KIND : a.kind;
  const int64_t b = blockIdx.x / a.nseg;
  const int seg = blockIdx.x % a.nseg;
  const int64_t t0 = (int64_t)seg * kSeg;
  float acc[kNP];
#pragma unroll
  for (int k = 0; k < kNP; ++k) acc[k] = 0.f;
  acc[P_RMIN] = __builtin_inff();
  acc[P_RMAX] = -__builtin_inff();
  const float seq_s = (kind == KIND_GSPO) ? row_s[b] : 0.f;

  const bool vec = a.vec != 0, nt = a.nt != 0;
  for (int gq = threadIdx.x; gq < kSeg / 4; gq += kStream) {
    const int64_t t = t0 + 4 * gq;
    if (t >= a.L) break;
    const int nv = (int)((a.L - t) < 4 ? (a.L - t) : 4);
    const int64_t idx0 = b * a.L + t;
    const Quad m4 = load_mask_quad(a.mask, a.mask_dtype, idx0, vec, nv, nt);
    const Quad lp4 = load_quad(a.lp, idx0, vec, nv, 0.f, nt);
    const bool agg_only = kind == KIND_AGG;
    const Quad old4 = agg_only ? const_quad(0.f) : load_quad(a.old_lp, idx0, vec, nv, 0.f, nt);
    const Quad adv4 = agg_only ? const_quad(0.f) : load_quad(a.adv, idx0, vec, nv, 0.f, nt);
    const Quad isw4 = a.isw ? load_quad(a.isw, idx0, vec, nv, 1.f, nt) : const_quad(1.f);
    const Quad ent4 = a.ent ? load_quad(a.ent, idx0, vec, nv, 0.f, nt) : const_quad(0.f);
    const Quad ref4 = a.ref ? load_quad(a.ref, idx0, vec, nv, 0.f, nt) : const_quad(0.f);
    const Quad aux4 = ((KIND < 0 || KIND >= KIND_KL_COV) && a.aux) ? load_quad(a.aux, idx0, vec, nv, 0.f, nt) : const_quad(0.f);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (e >= nv) break;
      const float m = m4.v[e];
      acc[P_M] += m;
      if (agg_only) {
        acc[P_PG] += contrib(lp4.v[e], m, a.agg_mode);
        continue;
      }
      const float lp = lp4.v[e];
      const PgOut o = pg_token(kind, lp, old4.v[e], adv4.v[e], isw4.v[e], seq_s, a, aux4.v[e]);
      if (kind != KIND_GEO) acc[P_PG] += contrib(o.tok, m, a.agg_mode);  // GEO: the loss is per sequence (row_s)
      acc[P_CLIP] += contrib_where(o.clip, m);
      acc[P_NEGD] += contrib_where(o.negd, m);
      acc[P_LOWER] += contrib_where(o.lower, m);
      acc[P_RSUM] += o.r_raw;
      acc[P_RMIN] = fminf(acc[P_RMIN], o.r_raw);
      acc[P_RMAX] = fmaxf(acc[P_RMAX], o.r_raw);
      if (a.ent) acc[P_ENT] += contrib(ent4.v[e], m, a.aux_agg_mode);
      if (a.ref) acc[P_KL] += contrib(kl_token(lp, ref4.v[e], a.kl_mode, 0).v, m, a.aux_agg_mode);
      if (a.drift_coef != 0.f) acc[P_AUX0] += contrib(clamp_max(o.r_raw - 1.f, 2.f) * lp, m, a.aux_agg_mode);
    }
  }

  // one wave-level reduction per partial, one LDS exchange for all of them
  __shared__ float sh[kStream / kWave][kNP];
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x / kWave;
#pragma unroll
  for (int k = 0; k < kNP; ++k) {
    float v = acc[k];
    if (k == P_RMIN) {
#pragma unroll
      for (int o = kWave / 2; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, kWave));
    } else if (k == P_RMAX) {
#pragma unroll
      for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    } else {
      v = wave_sum(v);
    }
    if (lane == 0) sh[wid][k] = v;
  }
  __syncthreads();
  if (threadIdx.x < kNP) {
    const int k = threadIdx.x;
    float v = sh[0][k];
    for (int w = 1; w < kStream / kWave; ++w)
      v = k == P_RMIN ? fminf(v, sh[w][k]) : (k == P_RMAX ? fmaxf(v, sh[w][k]) : v + sh[w][k]);
    partials[(b * a.nseg + seg) * kNP + k] = v;
  }
}

// ---------------------------------------------------------------------------- very long rows

// The finish kernels give a row to one thread, which walks the row's segments.  A row of more than kFoldAbove
// segments (half a million tokens) first has its segment partials folded 64 to 1, one wave per group of 64, sums in
// double, as often as it takes; rows of ordinary length never come here, so their results do not depend on it.
constexpr int kFoldAbove = 256, kFoldBy = 64;
__global__ __launch_bounds__(kThreads) void fold_segments_kernel(const float* __restrict__ in, int64_t B, int nseg,
                                                                 int nseg2, float* __restrict__ out) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t g = (int64_t)blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;  // (row, group of segments)
  if (g >= B * nseg2) return;
  const int64_t b = g / nseg2;
  const int s2 = (int)(g - b * nseg2), s = s2 * kFoldBy + lane;
  const bool have = s < nseg;
  const float* p = in + (b * nseg + (have ? s : 0)) * kNP;
  float res = 0.f;
#pragma unroll
  for (int k = 0; k < kNP; ++k) {
    float r;
    if (k == P_RMIN) {
      float v = have ? p[k] : __builtin_inff();
#pragma unroll
      for (int o = kWave / 2; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, kWave));
      r = v;
    } else if (k == P_RMAX) {
      float v = have ? p[k] : -__builtin_inff();
#pragma unroll
      for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
      r = v;
    } else {
      r = (float)wave_sum(have ? (double)p[k] : 0.0);
    }
    if (lane == k) res = r;
  }
  if (lane < kNP) out[g * kNP + lane] = res;
}

// Folds `partials` ([B][nseg][kNP]) until a row has at most kFoldAbove segments, alternating between `spare` and
// `partials`; returns where the result lies and updates nseg.
int fold_long_rows(const float*& cur, float* partials, float* spare, int64_t B, int& nseg, hipStream_t st) {
  float* dst = spare;
  while (nseg > kFoldAbove) {
    const int nseg2 = (nseg + kFoldBy - 1) / kFoldBy;
    const int64_t groups = B * nseg2;
    fold_segments_kernel<<<dim3((unsigned)((groups + kThreads / kWave - 1) / (kThreads / kWave))), dim3(kThreads), 0, st>>>(
        cur, B, nseg, nseg2, dst);
    SIIRL_LAUNCH_CHECK("fold_segments_kernel");
    cur = dst;
    dst = dst == spare ? partials : spare;
    nseg = nseg2;
  }
  return SIIRL_OK;
}

// ---------------------------------------------------------------------------- finish

__device__ __forceinline__ double block_sum_d(double v, double* sh) { return block_sum(v, sh); }

// Aggregates a per-row numerator given the mode.  num/msum are row sums; returns this row's term of
// the batch sum whose final normaliser is applied by the caller.
__device__ __forceinline__ double row_term(double num, double msum, int agg) {
  return agg == SIIRL_AGG_SEQ_MEAN_TOKEN_MEAN ? num / msum : num;  // 0/0 -> NaN, as the reference
}
__device__ __forceinline__ double finish_term(double total, double mtotal, int agg, int64_t B, int64_t L) {
  switch (agg) {
    case SIIRL_AGG_TOKEN_MEAN: return total / (mtotal + 1e-8);
    case SIIRL_AGG_SEQ_MEAN_TOKEN_SUM: return total / (double)B;
    case SIIRL_AGG_SEQ_MEAN_TOKEN_MEAN: return total / (double)B;
    default: return total / (double)L;
  }
}

// running totals of the finish: nine sums (fp64) and the extremes of the raw ratio
enum T { T_PG = 0, T_M, T_CLIP, T_NEGD, T_LOWER, T_ENT, T_KL, T_RSUM, T_DRIFT, T_COUNT };
struct Totals {
  double v[T_COUNT];
  float rmin, rmax;
  __device__ void init() {
    for (int k = 0; k < T_COUNT; ++k) v[k] = 0.0;
    rmin = __builtin_inff();
    rmax = -__builtin_inff();
  }
};

// folds the segments of row b into the totals and writes the row's mask sum
__device__ __forceinline__ void fold_row(const LossArgs& a, const float* __restrict__ partials,
                                         const float* __restrict__ row_s, float* __restrict__ row_msum, int64_t b,
                                         Totals& t) {
  double r[kNP];
  for (int k = 0; k < kNP; ++k) r[k] = 0.0;
  for (int s = 0; s < a.nseg; ++s) {
    const float* p = partials + (b * a.nseg + s) * kNP;
    for (int k = 0; k < kNP; ++k) {
      if (k == P_RMIN) t.rmin = fminf(t.rmin, p[k]);
      else if (k == P_RMAX) t.rmax = fmaxf(t.rmax, p[k]);
      else r[k] += p[k];
    }
  }
  row_msum[b] = (float)r[P_M];
  t.v[T_M] += r[P_M];
  t.v[T_PG] += a.kind == KIND_GEO ? (double)row_s[b] : row_term(r[P_PG], r[P_M], a.agg_mode);
  t.v[T_DRIFT] += row_term(r[P_AUX0], r[P_M], a.aux_agg_mode);
  t.v[T_ENT] += row_term(r[P_ENT], r[P_M], a.aux_agg_mode);
  t.v[T_KL] += row_term(r[P_KL], r[P_M], a.aux_agg_mode);
  t.v[T_CLIP] += r[P_CLIP];
  t.v[T_NEGD] += r[P_NEGD];
  t.v[T_LOWER] += r[P_LOWER];
  t.v[T_RSUM] += r[P_RSUM];
}

// workgroup-wide reduction of the totals; the result is valid in thread 0
__device__ __forceinline__ void reduce_totals(Totals& t) {
  __shared__ double sh[kThreads / kWave + 1];
  for (int k = 0; k < T_COUNT; ++k) t.v[k] = block_sum_d(t.v[k], sh);
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    t.rmin = fminf(t.rmin, __shfl_xor(t.rmin, o, kWave));
    t.rmax = fmaxf(t.rmax, __shfl_xor(t.rmax, o, kWave));
  }
  __shared__ float shm[2 * (kThreads / kWave)];
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x / kWave;
  __syncthreads();
  if (lane == 0) {
    shm[wid] = t.rmin;
    shm[kThreads / kWave + wid] = t.rmax;
  }
  __syncthreads();
  if (threadIdx.x == 0)
    for (int w = 1; w < kThreads / kWave; ++w) {
      t.rmin = fminf(t.rmin, shm[w]);
      t.rmax = fmaxf(t.rmax, shm[kThreads / kWave + w]);
    }
}

__device__ __forceinline__ void write_result(const LossArgs& a, const Totals& t, float* __restrict__ out) {
  const double t_m = t.v[T_M];
  const double pg = a.kind == KIND_GEO ? t.v[T_PG] / (double)a.B : finish_term(t.v[T_PG], t_m, a.agg_mode, a.B, a.L);
  const double den = t_m + 1e-8;
  double policy = pg;
  double entl = 0.0, kll = 0.0, drl = 0.0;
  if (a.ent) {
    entl = finish_term(t.v[T_ENT], t_m, a.aux_agg_mode, a.B, a.L);
    policy = policy - entl * (double)a.ent_coef;
  }
  if (a.ref) {
    kll = finish_term(t.v[T_KL], t_m, a.aux_agg_mode, a.B, a.L);
    policy = policy + kll * (double)a.kl_coef;
  }
  if (a.drift_coef != 0.f) {
    drl = finish_term(t.v[T_DRIFT], t_m, a.aux_agg_mode, a.B, a.L);
    policy = policy + drl * (double)a.drift_coef;
  }
  for (int k = 0; k < O_COUNT; ++k) out[k] = 0.f;
  out[O_PG] = (float)pg;
  out[O_POLICY] = (float)policy;
  out[O_LOSS] = (float)(policy * (double)a.scale);
  out[O_MTOTAL] = (float)t_m;
  if (a.kind != KIND_AGG) {
    out[O_CLIPFRAC] = (float)(t.v[T_CLIP] / den);
    out[O_PPOKL] = (float)(t.v[T_NEGD] / den);
    out[O_CLIPLOWER] = (float)(t.v[T_LOWER] / den);
    out[O_ENTLOSS] = (float)entl;
    out[O_KLLOSS] = (float)kll;
    out[O_DRIFT] = (float)drl;
    out[O_RMEAN] = (float)(t.v[T_RSUM] / (double)(a.B * a.L));
    out[O_RMIN] = t.rmin;
    out[O_RMAX] = t.rmax;
  }
}

// small batches: one workgroup folds every row and writes the result block
__global__ __launch_bounds__(kThreads) void loss_finish_kernel(LossArgs a, const float* __restrict__ partials,
                                                               const float* __restrict__ row_s,
                                                               float* __restrict__ out,
                                                               float* __restrict__ row_msum) {
  Totals t;
  t.init();
  for (int64_t b = threadIdx.x; b < a.B; b += kThreads) fold_row(a, partials, row_s, row_msum, b, t);
  reduce_totals(t);
  if (threadIdx.x == 0) write_result(a, t, out);
}

// large batches, level 1: one thread per row, one record of totals per workgroup
constexpr int kFinRec = T_COUNT + 2;
__global__ __launch_bounds__(kThreads) void loss_rows_kernel(LossArgs a, const float* __restrict__ partials,
                                                             const float* __restrict__ row_s,
                                                             float* __restrict__ row_msum, double* __restrict__ rec) {
  Totals t;
  t.init();
  const int64_t b = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (b < a.B) fold_row(a, partials, row_s, row_msum, b, t);
  reduce_totals(t);
  if (threadIdx.x == 0) {
    double* r = rec + (int64_t)blockIdx.x * kFinRec;
    for (int k = 0; k < T_COUNT; ++k) r[k] = t.v[k];
    r[T_COUNT] = (double)t.rmin;
    r[T_COUNT + 1] = (double)t.rmax;
  }
}
// level 2: one workgroup folds the records in order
__global__ __launch_bounds__(kThreads) void loss_finish2_kernel(LossArgs a, const double* __restrict__ rec, int nrec,
                                                                float* __restrict__ out) {
  Totals t;
  t.init();
  for (int i = threadIdx.x; i < nrec; i += kThreads) {
    const double* r = rec + (int64_t)i * kFinRec;
    for (int k = 0; k < T_COUNT; ++k) t.v[k] += r[k];
    t.rmin = fminf(t.rmin, (float)r[T_COUNT]);
    t.rmax = fmaxf(t.rmax, (float)r[T_COUNT + 1]);
  }
  reduce_totals(t);
  if (threadIdx.x == 0) write_result(a, t, out);
}

// ---------------------------------------------------------------------------- backward

// aggregation weight of a token as m * c (see tok::agg_weight for the exact quotient form)
struct AggCoef {
  float c;
  bool where;  // token-mean goes through masked_mean: where(mask, v, 0) * mask
  __device__ __forceinline__ float operator()(float m) const { return (where && m == 0.f) ? 0.f : m * c; }
};
__device__ __forceinline__ AggCoef agg_coef(int agg, float mtotal, float mrow, int64_t B, int64_t L) {
  switch (agg) {
    case SIIRL_AGG_TOKEN_MEAN: return AggCoef{1.f / (mtotal + 1e-8f), true};
    case SIIRL_AGG_SEQ_MEAN_TOKEN_SUM: return AggCoef{1.f / (float)B, false};
    case SIIRL_AGG_SEQ_MEAN_TOKEN_MEAN: return AggCoef{1.f / mrow / (float)B, false};
    default: return AggCoef{1.f / (float)L, false};
  }
}

template <int KIND>
__global__ __launch_bounds__(kStream) void loss_bwd_kernel(LossArgs a, const float* __restrict__ g_out,
                                                            const float* __restrict__ saved_out,
                                                            const float* __restrict__ row_msum,
                                                            const float* __restrict__ row_s,
                                                            float* __restrict__ d_lp, float* __restrict__ d_ent) {
  const int kind = KIND >= 0 ? KIND : a.kind;
  const int64_t b = blockIdx.x / a.nseg;
  const int64_t t0 = (int64_t)(blockIdx.x % a.nseg) * kSeg;
  const float g = g_out[0] * a.scale;
  const float mtotal = saved_out[O_MTOTAL];
  const float mrow = row_msum[b];
  const float seq_s = (kind == KIND_GSPO || kind == KIND_GEO) ? row_s[b] : 0.f;
  const bool vec = a.vec != 0, nt = a.nt != 0;
  const bool agg_only = kind == KIND_AGG;
  // aggregation weights are m * c with c fixed for the row: one division per thread instead of up to three per token
  const AggCoef w_pg = agg_coef(a.agg_mode, mtotal, mrow, a.B, a.L);
  const AggCoef w_aux = agg_coef(a.aux_agg_mode, mtotal, mrow, a.B, a.L);
  const float geo_c = seq_s / (mrow + 1e-8f) / (float)a.B;
  for (int gq = threadIdx.x; gq < kSeg / 4; gq += kStream) {
    const int64_t t = t0 + 4 * gq;
    if (t >= a.L) break;
    const int nv = (int)((a.L - t) < 4 ? (a.L - t) : 4);
    const int64_t idx0 = b * a.L + t;
    const Quad m4 = load_mask_quad(a.mask, a.mask_dtype, idx0, vec, nv, nt);
    Quad dlp, dent;
    if (agg_only) {
#pragma unroll
      for (int e = 0; e < 4; ++e) dlp.v[e] = g * w_pg(m4.v[e]);
      store_quad(d_lp, idx0, vec, nv, dlp);
      continue;
    }
    const Quad lp4 = load_quad(a.lp, idx0, vec, nv, 0.f, nt);
    const Quad old4 = load_quad(a.old_lp, idx0, vec, nv, 0.f, nt);
    const Quad adv4 = load_quad(a.adv, idx0, vec, nv, 0.f, nt);
    const Quad isw4 = a.isw ? load_quad(a.isw, idx0, vec, nv, 1.f, nt) : const_quad(1.f);
    const Quad ref4 = a.ref ? load_quad(a.ref, idx0, vec, nv, 0.f, nt) : const_quad(0.f);
    const Quad aux4 = ((KIND < 0 || KIND >= KIND_KL_COV) && a.aux) ? load_quad(a.aux, idx0, vec, nv, 0.f, nt) : const_quad(0.f);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float m = m4.v[e], lp = lp4.v[e];
      const PgOut o = pg_token(kind, lp, old4.v[e], adv4.v[e], isw4.v[e], seq_s, a, aux4.v[e]);
      float d;
      if (kind == KIND_GEO)  // d mean_b(row loss) / d x = row loss * m / (n + 1e-8) / B
        d = geo_c * m * o.dtok;
      else
        d = w_pg(m) * o.dtok;
      const float wa = w_aux(m);
      if (a.drift_coef != 0.f)  // the weight clamp(exp(lp - old) - 1, max = 2) is detached
        d += a.drift_coef * wa * clamp_max(o.r_raw - 1.f, 2.f);
      dent.v[e] = 0.f;
      if (a.ent || a.ref) {
        if (a.ref) d += a.kl_coef * wa * kl_token(lp, ref4.v[e], a.kl_mode, a.kl_st).g;
        dent.v[e] = -g * a.ent_coef * wa;
      }
      dlp.v[e] = g * d;
    }
    store_quad(d_lp, idx0, vec, nv, dlp);
    if (a.ent && d_ent) store_quad(d_ent, idx0, vec, nv, dent);
  }
}

int launch_loss_bwd(const LossArgs& a, const float* g_out, const float* saved_out, const float* row_msum,
                    const float* row_s, float* d_lp, float* d_ent, hipStream_t st) {
  const dim3 grid((unsigned)(a.B * a.nseg)), block(kStream);
  switch (a.kind) {
    case KIND_VANILLA: loss_bwd_kernel<KIND_VANILLA><<<grid, block, 0, st>>>(a, g_out, saved_out, row_msum, row_s, d_lp, d_ent); break;
    case KIND_GSPO: loss_bwd_kernel<KIND_GSPO><<<grid, block, 0, st>>>(a, g_out, saved_out, row_msum, row_s, d_lp, d_ent); break;
    case KIND_AGG: loss_bwd_kernel<KIND_AGG><<<grid, block, 0, st>>>(a, g_out, saved_out, row_msum, row_s, d_lp, d_ent); break;
    case KIND_VALUE: loss_bwd_kernel<KIND_VALUE><<<grid, block, 0, st>>>(a, g_out, saved_out, row_msum, row_s, d_lp, d_ent); break;
    case KIND_KL_COV: loss_bwd_kernel<KIND_KL_COV><<<grid, block, 0, st>>>(a, g_out, saved_out, row_msum, row_s, d_lp, d_ent); break;
    case KIND_CLIP_COV: loss_bwd_kernel<KIND_CLIP_COV><<<grid, block, 0, st>>>(a, g_out, saved_out, row_msum, row_s, d_lp, d_ent); break;
    default: loss_bwd_kernel<-1><<<grid, block, 0, st>>>(a, g_out, saved_out, row_msum, row_s, d_lp, d_ent);
  }
  SIIRL_LAUNCH_CHECK("loss_bwd_kernel");
  return SIIRL_OK;
}

__global__ __launch_bounds__(kThreads) void fill_kernel(float* __restrict__ p, int64_t n, float v) {
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads) p[i] = v;
}

// ---------------------------------------------------------------------------- aggregation weights

// w[b, t] = d agg_loss / d loss_mat[b, t]: depends on the mask only (row sums and total from the partials pass)
__global__ __launch_bounds__(kThreads) void agg_weights_kernel(LossArgs a, const float* __restrict__ saved_out,
                                                               const float* __restrict__ row_msum,
                                                               float* __restrict__ w) {
  const int64_t b = blockIdx.x / a.nseg;
  const int64_t t0 = (int64_t)(blockIdx.x % a.nseg) * kSeg;
  const float mtotal = saved_out[O_MTOTAL], mrow = row_msum[b];
  for (int i = threadIdx.x; i < kSeg; i += kThreads) {
    const int64_t t = t0 + i;
    if (t >= a.L) break;
    const int64_t idx = b * a.L + t;
    w[idx] = agg_weight(a.agg_mode, load_mask(a.mask, a.mask_dtype, idx), mtotal, mrow, a.B, a.L);
  }
}

// ---------------------------------------------------------------------------- KL penalty (elementwise)

// four consecutive elements per thread and pass; `vec`: every operand is 16-byte aligned (one 16-byte access each)
__global__ __launch_bounds__(kThreads) void kl_fwd_kernel(const float* __restrict__ lp, const float* __restrict__ ref,
                                                          int64_t n, int mode, bool vec, float* __restrict__ out) {
  const int64_t nq = (n + 3) / 4;
  for (int64_t q = (int64_t)blockIdx.x * kThreads + threadIdx.x; q < nq; q += (int64_t)gridDim.x * kThreads) {
    const int64_t i = q * 4;
    const int nv = (int)(n - i < 4 ? n - i : 4);
    const bool v4 = vec && nv == 4;
    const Quad a = load_quad(lp, i, v4, nv, 0.f), b = load_quad(ref, i, v4, nv, 0.f);
    Quad o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o.v[e] = kl_token(a.v[e], b.v[e], mode, 0).v;
    store_quad(out, i, v4, nv, o);
  }
}
__global__ __launch_bounds__(kThreads) void kl_bwd_kernel(const float* __restrict__ g, const float* __restrict__ lp,
                                                          const float* __restrict__ ref, int64_t n, int mode, int st,
                                                          bool vec, float* __restrict__ d_lp, float* __restrict__ d_ref) {
  const int64_t nq = (n + 3) / 4;
  for (int64_t q = (int64_t)blockIdx.x * kThreads + threadIdx.x; q < nq; q += (int64_t)gridDim.x * kThreads) {
    const int64_t i = q * 4;
    const int nv = (int)(n - i < 4 ? n - i : 4);
    const bool v4 = vec && nv == 4;
    const Quad gg = load_quad(g, i, v4, nv, 0.f), a = load_quad(lp, i, v4, nv, 0.f), b = load_quad(ref, i, v4, nv, 0.f);
    Quad d, nd;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      d.v[e] = gg.v[e] * kl_token(a.v[e], b.v[e], mode, st).g;
      nd.v[e] = -d.v[e];  // every estimator depends on lp - ref only
    }
    if (d_lp) store_quad(d_lp, i, v4, nv, d);
    if (d_ref) store_quad(d_ref, i, v4, nv, nd);
  }
}

// ---------------------------------------------------------------------------- masked_sum / masked_mean

// row_sum[b] = sum_t where(m, v, 0) * m ; row_mean[b] = row_sum / (sum_t m + 1e-8); total2 = {sum, mean} over all
__global__ __launch_bounds__(kThreads) void masked_finish_kernel(const float* __restrict__ partials, int nseg,
                                                                 int64_t B, float* __restrict__ row_sum,
                                                                 float* __restrict__ row_mean,
                                                                 float* __restrict__ total2,
                                                                 float* __restrict__ row_msum,
                                                                 float* __restrict__ mask_total) {
  double tv = 0, tm = 0;
  for (int64_t b = threadIdx.x; b < B; b += kThreads) {
    double v = 0, m = 0;
    for (int s = 0; s < nseg; ++s) {
      v += partials[(b * nseg + s) * kNP + P_PG];
      m += partials[(b * nseg + s) * kNP + P_M];
    }
    if (row_sum) row_sum[b] = (float)v;
    if (row_mean) row_mean[b] = (float)(v / (m + 1e-8));
    if (row_msum) row_msum[b] = (float)m;
    tv += v;
    tm += m;
  }
  __shared__ double sh[kThreads / kWave + 1];
  tv = block_sum_d(tv, sh);
  tm = block_sum_d(tm, sh);
  if (threadIdx.x == 0 && total2) {
    total2[0] = (float)tv;
    total2[1] = (float)(tv / (tm + 1e-8));
  }
  if (threadIdx.x == 0 && mask_total) mask_total[0] = (float)tm;
}

// many rows: one thread per row writes the row's results, one {sum, mask sum} record per workgroup; then one
// workgroup folds the records (fp64 as above; the order of the additions differs from the one-level finish)
__global__ __launch_bounds__(kThreads) void masked_rows_kernel(const float* __restrict__ partials, int nseg, int64_t B,
                                                               float* __restrict__ row_sum,
                                                               float* __restrict__ row_mean,
                                                               float* __restrict__ row_msum, double* __restrict__ rec) {
  const int64_t b = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  double v = 0, m = 0;
  if (b < B) {
    for (int s = 0; s < nseg; ++s) {
      v += partials[(b * nseg + s) * kNP + P_PG];
      m += partials[(b * nseg + s) * kNP + P_M];
    }
    if (row_sum) row_sum[b] = (float)v;
    if (row_mean) row_mean[b] = (float)(v / (m + 1e-8));
    if (row_msum) row_msum[b] = (float)m;
  }
  __shared__ double sh[kThreads / kWave + 1];
  v = block_sum_d(v, sh);
  m = block_sum_d(m, sh);
  if (threadIdx.x == 0) {
    rec[2 * (int64_t)blockIdx.x] = v;
    rec[2 * (int64_t)blockIdx.x + 1] = m;
  }
}
__global__ __launch_bounds__(kThreads) void masked_finish2_kernel(const double* __restrict__ rec, int nrec,
                                                                  float* __restrict__ total2,
                                                                  float* __restrict__ mask_total) {
  double tv = 0, tm = 0;
  for (int i = threadIdx.x; i < nrec; i += kThreads) {
    tv += rec[2 * i];
    tm += rec[2 * i + 1];
  }
  __shared__ double sh[kThreads / kWave + 1];
  tv = block_sum_d(tv, sh);
  tm = block_sum_d(tm, sh);
  if (threadIdx.x == 0 && total2) {
    total2[0] = (float)tv;
    total2[1] = (float)(tv / (tm + 1e-8));
  }
  if (threadIdx.x == 0 && mask_total) mask_total[0] = (float)tm;
}

// backward of masked_sum / masked_mean: d[b, t] = g[b or 0] * m[b, t] (/ (mask sum of the reduced extent + 1e-8))
// Four tokens per thread and access when rows allow it (`vec`: L % 4 == 0, 16-byte aligned operands): a quad then
// lies inside one row.
__global__ __launch_bounds__(kThreads) void masked_bwd_kernel(const float* __restrict__ g, const void* mask,
                                                              int mask_dtype, int64_t B, int64_t L, int per_row,
                                                              const float* __restrict__ den, int vec, int nt,
                                                              float* __restrict__ d) {
  const int64_t n = B * L;
  const float all = per_row ? 0.f : (den ? g[0] / (den[0] + 1e-8f) : g[0]);
  if (vec) {
    for (int64_t q = (int64_t)blockIdx.x * kThreads + threadIdx.x; q < n / 4; q += (int64_t)gridDim.x * kThreads) {
      const int64_t i = 4 * q;
      float w = all;
      if (per_row) {
        const int64_t b = i / L;
        w = den ? g[b] / (den[b] + 1e-8f) : g[b];
      }
      Quad m4 = load_mask_quad(mask, mask_dtype, i, true, 4, nt != 0);
#pragma unroll
      for (int e = 0; e < 4; ++e) m4.v[e] = w * m4.v[e];
      store_quad(d, i, true, 4, m4);
    }
    return;
  }
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads) {
    float w = all;
    if (per_row) {
      const int64_t b = i / L;
      w = den ? g[b] / (den[b] + 1e-8f) : g[b];
    }
    d[i] = w * load_mask(mask, mask_dtype, i);
  }
}

// ---------------------------------------------------------------------------- KL penalty in the reward

// rewards = scores - beta * kld,  kld = kl(old, ref) * m ; row_kl[b] = masked_mean(kld, m) of the row
__global__ __launch_bounds__(kThreads) void kl_reward_kernel(const float* __restrict__ scores,
                                                             const float* __restrict__ old_lp,
                                                             const float* __restrict__ ref, const void* mask,
                                                             int mask_dtype, int64_t L, int kl_mode, float beta, bool vec,
                                                             float* __restrict__ rewards, float* __restrict__ row_kl) {
  const int64_t b = blockIdx.x;
  float sv = 0.f, sm = 0.f;
  for (int64_t t = (int64_t)threadIdx.x * 4; t < L; t += kThreads * 4) {  // four tokens per thread and pass
    const int64_t idx = b * L + t;
    const int nv = (int)(L - t < 4 ? L - t : 4);
    const Quad m = load_mask_quad(mask, mask_dtype, idx, vec, nv);
    const Quad o = load_quad(old_lp, idx, vec, nv, 0.f), r = load_quad(ref, idx, vec, nv, 0.f);
    const Quad s = load_quad(scores, idx, vec, nv, 0.f);
    Quad out;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float kld = kl_token(o.v[e], r.v[e], kl_mode, 0).v * m.v[e];
      out.v[e] = s.v[e] - beta * kld;
      if (e < nv) {
        sv += contrib_where(kld, m.v[e]);
        sm += m.v[e];
      }
    }
    store_quad(rewards, idx, vec, nv, out);
  }
  __shared__ float sh[kThreads / kWave + 1];
  sv = block_sum(sv, sh);
  sm = block_sum(sm, sh);
  if (threadIdx.x == 0) row_kl[b] = sv / (sm + 1e-8f);
}
__global__ __launch_bounds__(kThreads) void mean_rows_kernel(const float* __restrict__ row, int64_t B,
                                                             float* __restrict__ out) {
  double s = 0;
  for (int64_t b = threadIdx.x; b < B; b += kThreads) s += row[b];
  __shared__ double sh[kThreads / kWave + 1];
  s = block_sum_d(s, sh);
  if (threadIdx.x == 0) out[0] = (float)(s / (double)B);
}

// ---------------------------------------------------------------------------- covariance scores (clip_cov, kl_cov)

// Sums over the whole [B, L] batch that the two covariance losses centre their operands with, in a fixed grid so
// that the result does not depend on the launch: per workgroup {count of m > 0, sum A and sum lp over m > 0,
// sum m, sum A*m, sum lp*m} (floats per thread, doubles from the wave up), folded by one workgroup.
constexpr int kCovGrid = 1024;
constexpr int kCovSums = 6;
__global__ __launch_bounds__(kThreads) void cov_sums_kernel(const float* __restrict__ lp, const float* __restrict__ adv,
                                                            const void* mask, int mask_dtype, int64_t n, int vec,
                                                            int nt_in, double* __restrict__ part) {
  float s[kCovSums] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const int64_t nq = (n + 3) / 4;  // four tokens per thread and access
  for (int64_t q = (int64_t)blockIdx.x * kThreads + threadIdx.x; q < nq; q += (int64_t)gridDim.x * kThreads) {
    const int64_t i = 4 * q;
    const int nv = (int)((n - i) < 4 ? (n - i) : 4);
    const bool v = vec != 0 && nv == 4;
    const Quad m4 = load_mask_quad(mask, mask_dtype, i, v, nv, nt_in != 0);
    const Quad a4 = load_quad(adv, i, v, nv, 0.f, nt_in != 0), l4 = load_quad(lp, i, v, nv, 0.f, nt_in != 0);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (e >= nv) break;
      const float m = m4.v[e], a = a4.v[e], l = l4.v[e];
      if (m > 0.f) { s[0] += 1.f; s[1] += a; s[2] += l; }
      s[3] += m;
      s[4] += contrib_where(a, m);  // masked_mean: where(mask, v, 0) * mask
      s[5] += contrib_where(l, m);
    }
  }
  __shared__ double sh[kThreads / kWave + 1];
  for (int k = 0; k < kCovSums; ++k) {
    const double t = block_sum((double)s[k], sh);
    if (threadIdx.x == 0) part[(int64_t)blockIdx.x * kCovSums + k] = t;
  }
}
// stats[0..5] = {count of m > 0, sum of the mask, mean A, mean lp, and what the first two lost to float32 rounding
// (count = stats[0] + stats[4], mask sum = stats[1] + stats[5], exact in double)}; plain means over m > 0 (kl_cov,
// core_algos.py:1055) or masked means sum(v * m) / (sum(m) + 1e-8) in fp32 (clip_cov, :967-969)
__global__ __launch_bounds__(kThreads) void cov_stats_kernel(const double* __restrict__ part, int nparts, int masked_means,
                                                             float* __restrict__ stats) {
  __shared__ double sh[kThreads / kWave + 1];
  double t[kCovSums];
  for (int k = 0; k < kCovSums; ++k) {
    double v = 0.0;
    for (int i = threadIdx.x; i < nparts; i += kThreads) v += part[(int64_t)i * kCovSums + k];
    t[k] = block_sum(v, sh);
  }
  if (threadIdx.x == 0) {
    stats[0] = (float)t[0];
    stats[1] = (float)t[3];
    stats[4] = (float)(t[0] - (double)stats[0]);
    stats[5] = (float)(t[3] - (double)stats[1]);
    if (masked_means) {
      const float den = (float)t[3] + 1e-8f;
      stats[2] = (float)t[4] / den;
      stats[3] = (float)t[5] / den;
    } else {
      stats[2] = (float)(t[1] / t[0]);  // no token with m > 0: 0 / 0, and no score is finite anyway
      stats[3] = (float)(t[2] / t[0]);
    }
  }
}
// cov[b, t] = (A - mean A) * (lp - mean lp), minus infinity where the mask is not positive (neither loss ever picks
// such a token) and, for clip_cov, where the PPO clip already bites (l2 > l1)
__global__ __launch_bounds__(kThreads) void cov_scores_kernel(const float* __restrict__ old_lp, const float* __restrict__ lp,
                                                              const float* __restrict__ adv, const void* mask,
                                                              int mask_dtype, int64_t n, int vec, int nt_in,
                                                              int clip_mode, float lo, float hi,
                                                              const float* __restrict__ stats,
                                                              float* __restrict__ cov) {
  const float ma = stats[2], ml = stats[3];
  const int64_t nq = (n + 3) / 4;
  for (int64_t q = (int64_t)blockIdx.x * kThreads + threadIdx.x; q < nq; q += (int64_t)gridDim.x * kThreads) {
    const int64_t i = 4 * q;
    const int nv = (int)((n - i) < 4 ? (n - i) : 4);
    const bool v = vec != 0 && nv == 4;
    const Quad m4 = load_mask_quad(mask, mask_dtype, i, v, nv, nt_in != 0);
    const Quad a4 = load_quad(adv, i, v, nv, 0.f, nt_in != 0), l4 = load_quad(lp, i, v, nv, 0.f, nt_in != 0);
    const Quad o4 = clip_mode ? load_quad(old_lp, i, v, nv, 0.f, nt_in != 0) : const_quad(0.f);
    Quad c4;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float m = m4.v[e], a = a4.v[e], l = l4.v[e];
      float c = (a - ma) * (l - ml);
      if (clip_mode) {
        const float r = expf(l - o4.v[e]);
        const float l1 = -a * r, l2 = -a * clampf(r, lo, hi);
        if (!(m > 0.f) || l2 > l1) c = -__builtin_inff();
      } else if (!(m > 0.f)) {
        c = -__builtin_inff();
      }
      c4.v[e] = c;
    }
    store_quad(cov, i, v, nv, c4);
  }
}

// ---------------------------------------------------------------------------- host

int nseg_of(int64_t L) { return (int)((L + kSeg - 1) / kSeg); }

// tokens move four at a time when rows start 16-byte aligned for every operand (and outputs `o1`, `o2`)
void set_vec(LossArgs& a, const void* o1 = nullptr, const void* o2 = nullptr) {
  auto ok16 = [](const void* p) { return p == nullptr || ((uintptr_t)p & 15) == 0; };
  const size_t msz = a.mask_dtype == SIIRL_I64 ? 8 : (a.mask_dtype == SIIRL_U8 ? 1 : (a.mask_dtype == SIIRL_F32 || a.mask_dtype == SIIRL_I32 ? 4 : 2));
  const bool mask_ok = ((uintptr_t)a.mask & (msz * 4 > 16 ? 15 : msz * 4 - 1)) == 0;
  a.vec = (a.L % 4 == 0) && mask_ok && ok16(a.old_lp) && ok16(a.lp) && ok16(a.adv) && ok16(a.isw) && ok16(a.ent) &&
          ok16(a.ref) && ok16(a.aux) && ok16(o1) && ok16(o2);
  // bytes one pass reads: ordinary loads while they fit the memory-side cache, non-temporal ones beyond
  const int n_f32 = (a.old_lp != nullptr) + (a.lp != nullptr) + (a.adv != nullptr) + (a.isw != nullptr) + (a.ent != nullptr) +
                    (a.ref != nullptr) + (a.aux != nullptr);
  a.nt = streams_past_cache((double)a.B * (double)a.L * (double)(4 * n_f32 + (a.mask ? msz : 0)));
}

size_t ws_bytes_of(int64_t B, int64_t L) {
  const size_t ns = (size_t)nseg_of(L);
  return (size_t)B * ns * kNP * sizeof(float) + (size_t)B * ns * kNPre * sizeof(float) + 256 +
         (size_t)((B + kThreads - 1) / kThreads) * kFinRec * sizeof(double);
}
constexpr int64_t kTwoLevelRows = 2048;  // above this many rows the finish runs in two levels

int check_dims(int64_t B, int64_t L) {
  // an empty batch (B == 0) is served: the forward writes the aggregates of nothing, the backward does nothing
  SIIRL_REQUIRE(B >= 0 && L >= 1, "B=%lld must not be negative and L=%lld must be positive", (long long)B, (long long)L);
  SIIRL_REQUIRE(L <= (1LL << 40) && B * (int64_t)nseg_of(L) <= 0x7fffffffLL, "B=%lld x L=%lld exceeds the launch grid",
                (long long)B, (long long)L);
  return SIIRL_OK;
}
int check_mask_dtype(int dt) {
  SIIRL_REQUIRE(dt == SIIRL_U8 || dt == SIIRL_I64 || dt == SIIRL_I32 || dt == SIIRL_F32 || dt == SIIRL_BF16 ||
                    dt == SIIRL_F16, "mask dtype %d not supported", dt);
  return SIIRL_OK;
}
int check_agg(int agg) {
  SIIRL_REQUIRE(agg >= 0 && agg <= 3, "Invalid loss_agg_mode: %d", agg);
  return SIIRL_OK;
}


int launch_loss_partials(const LossArgs& a, const float* row_s, float* partials, hipStream_t st) {
  const dim3 grid((unsigned)(a.B * a.nseg)), block(kStream);
  switch (a.kind) {
    case KIND_VANILLA: loss_partials_kernel<KIND_VANILLA><<<grid, block, 0, st>>>(a, row_s, partials); break;
    case KIND_GSPO: loss_partials_kernel<KIND_GSPO><<<grid, block, 0, st>>>(a, row_s, partials); break;
    case KIND_AGG: loss_partials_kernel<KIND_AGG><<<grid, block, 0, st>>>(a, row_s, partials); break;
    case KIND_VALUE: loss_partials_kernel<KIND_VALUE><<<grid, block, 0, st>>>(a, row_s, partials); break;
    case KIND_KL_COV: loss_partials_kernel<KIND_KL_COV><<<grid, block, 0, st>>>(a, row_s, partials); break;
    case KIND_CLIP_COV: loss_partials_kernel<KIND_CLIP_COV><<<grid, block, 0, st>>>(a, row_s, partials); break;
    default: loss_partials_kernel<-1><<<grid, block, 0, st>>>(a, row_s, partials);
  }
  SIIRL_LAUNCH_CHECK("loss_partials_kernel");
  return SIIRL_OK;
}

int run_forward(LossArgs& a, float* out16, float* row_msum, float* row_s, void* ws, size_t ws_bytes,
                hipStream_t st) {
  if (a.B == 0) {  // the finish alone: zero sums give the reference's 0 (token-mean, -sum-norm) or NaN (seq-mean-*)
    a.nseg = nseg_of(a.L);
    loss_finish_kernel<<<1, dim3(kThreads), 0, st>>>(a, nullptr, row_s, out16, row_msum);
    SIIRL_LAUNCH_CHECK("loss_finish_kernel");
    return SIIRL_OK;
  }
  a.nseg = nseg_of(a.L);
  if (ws_bytes < ws_bytes_of(a.B, a.L) || ws == nullptr)
    return fail(SIIRL_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed for B=%lld L=%lld",
                ws_bytes, ws_bytes_of(a.B, a.L), (long long)a.B, (long long)a.L);
  SIIRL_REQUIRE(((uintptr_t)ws & 7) == 0, "workspace must be 8-byte aligned");
  set_vec(a);
  float* partials = (float*)ws;
  float* pre = partials + (size_t)a.B * a.nseg * kNP;
  dim3 grid((unsigned)(a.B * a.nseg)), block(kThreads);
  if (a.kind == KIND_GSPO || a.kind == KIND_GEO) {
    row_prepass_kernel<<<grid, block, 0, st>>>(a, pre);
    SIIRL_LAUNCH_CHECK("row_prepass_kernel");
    row_finish_kernel<<<dim3((unsigned)((a.B + kThreads - 1) / kThreads)), block, 0, st>>>(pre, a.nseg, a.B, a.kind,
                                                                                       a.isw != nullptr, row_s);
    SIIRL_LAUNCH_CHECK("row_finish_kernel");
  }
  if (int rc = launch_loss_partials(a, row_s, partials, st)) return rc;
  const size_t used = ((size_t)a.B * a.nseg * (kNP + kNPre) * sizeof(float) + 255) / 256 * 256;
  const float* folded = partials;  // the pre-pass sums are spent by now: their room serves the folding of long rows
  if (int rc = fold_long_rows(folded, partials, pre, a.B, a.nseg, st)) return rc;
  if (a.B <= kTwoLevelRows) {
    loss_finish_kernel<<<1, block, 0, st>>>(a, folded, row_s, out16, row_msum);
    SIIRL_LAUNCH_CHECK("loss_finish_kernel");
  } else {
    double* rec = reinterpret_cast<double*>((char*)ws + used);
    const int nrec = (int)((a.B + kThreads - 1) / kThreads);
    loss_rows_kernel<<<dim3((unsigned)nrec), block, 0, st>>>(a, folded, row_s, row_msum, rec);
    SIIRL_LAUNCH_CHECK("loss_rows_kernel");
    loss_finish2_kernel<<<1, block, 0, st>>>(a, rec, nrec, out16);
    SIIRL_LAUNCH_CHECK("loss_finish2_kernel");
  }
  return SIIRL_OK;
}

}  // namespace
}  // namespace siirl

using namespace siirl;

extern "C" size_t siirl_loss_workspace_bytes(int64_t B, int64_t L) {
  if (B < 1 || L < 1) return 0;
  return ws_bytes_of(B, L);
}

extern "C" int siirl_agg_loss_fwd(const float* loss_mat, const void* mask, int mask_dtype, int64_t B, int64_t L,
                                  int agg_mode, float* out16, float* row_msum, void* workspace,
                                  size_t workspace_bytes, siirl_stream_t stream) {
  if (int rc = check_dims(B, L)) return rc;
  if (int rc = check_mask_dtype(mask_dtype)) return rc;
  if (int rc = check_agg(agg_mode)) return rc;
  SIIRL_REQUIRE(out16 && (B == 0 || (loss_mat && mask && row_msum)), "NULL operand");
  LossArgs a{};
  a.lp = loss_mat; a.mask = mask; a.mask_dtype = mask_dtype; a.kind = KIND_AGG; a.agg_mode = agg_mode;
  a.aux_agg_mode = agg_mode; a.scale = 1.f; a.B = B; a.L = L;
  return run_forward(a, out16, row_msum, nullptr, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int siirl_agg_weights(const void* mask, int mask_dtype, int64_t B, int64_t L, int agg_mode, float* weights,
                                 float* out16, float* row_msum, void* workspace, size_t workspace_bytes,
                                 siirl_stream_t stream) {
  if (int rc = check_dims(B, L)) return rc;
  if (int rc = check_mask_dtype(mask_dtype)) return rc;
  if (int rc = check_agg(agg_mode)) return rc;
  SIIRL_REQUIRE(out16 && (B == 0 || (mask && weights && row_msum)), "NULL operand");
  LossArgs a{};
  // the partials pass over the weights buffer itself (its values are not used, only the mask sums are)
  a.lp = weights; a.mask = mask; a.mask_dtype = mask_dtype; a.kind = KIND_AGG; a.agg_mode = agg_mode;
  a.aux_agg_mode = agg_mode; a.scale = 1.f; a.B = B; a.L = L;
  hipStream_t st = (hipStream_t)stream;
  fill_kernel<<<dim3(1024), dim3(kThreads), 0, st>>>(weights, B * L, 0.f);
  SIIRL_LAUNCH_CHECK("fill_kernel");
  if (int rc = run_forward(a, out16, row_msum, nullptr, workspace, workspace_bytes, st)) return rc;
  if (B == 0) return SIIRL_OK;
  agg_weights_kernel<<<dim3((unsigned)(B * a.nseg)), dim3(kThreads), 0, st>>>(a, out16, row_msum, weights);
  SIIRL_LAUNCH_CHECK("agg_weights_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_agg_loss_bwd(const float* g_out, const void* mask, int mask_dtype, const float* out16,
                                  const float* row_msum, int64_t B, int64_t L, int agg_mode, float* d_loss_mat,
                                  siirl_stream_t stream) {
  if (int rc = check_dims(B, L)) return rc;
  if (int rc = check_mask_dtype(mask_dtype)) return rc;
  if (int rc = check_agg(agg_mode)) return rc;
  if (B == 0) return SIIRL_OK;
  SIIRL_REQUIRE(g_out && mask && out16 && row_msum && d_loss_mat, "NULL operand");
  LossArgs a{};
  a.mask = mask; a.mask_dtype = mask_dtype; a.kind = KIND_AGG; a.agg_mode = agg_mode; a.aux_agg_mode = agg_mode;
  a.scale = 1.f; a.B = B; a.L = L; a.nseg = nseg_of(L);
  set_vec(a, d_loss_mat);
  return launch_loss_bwd(a, g_out, out16, row_msum, nullptr, d_loss_mat, nullptr, (hipStream_t)stream);
}

static int fill_actor_args(LossArgs& a, const float* old_log_prob, const float* log_prob, const float* advantages,
                           const void* mask, int mask_dtype, const float* is_weights, const float* entropy,
                           const float* ref_log_prob, int64_t B, int64_t L, int loss_mode, float clip_low,
                           float clip_high, float clip_c, float log_ratio_clamp, int agg_mode, float entropy_coeff, int kl_mode,
                           int kl_straight_through, float kl_coef, float policy_drift_coeff, float loss_scale,
                           const float* token_aux = nullptr, bool cov = false) {
  if (int rc = check_dims(B, L)) return rc;
  if (int rc = check_mask_dtype(mask_dtype)) return rc;
  if (int rc = check_agg(agg_mode)) return rc;
  if (!cov)
    SIIRL_REQUIRE(loss_mode >= SIIRL_LOSS_VANILLA && loss_mode <= SIIRL_LOSS_GEO_MEAN, "Unsupported loss mode: %d",
                  loss_mode);
  else
    SIIRL_REQUIRE(loss_mode == SIIRL_LOSS_KL_COV || loss_mode == SIIRL_LOSS_CLIP_COV,
                  "loss mode %d takes no per-token selection (kl_cov and clip_cov do)", loss_mode);
  SIIRL_REQUIRE(B == 0 || (old_log_prob && log_prob && advantages && mask), "NULL operand");
  if (loss_mode == SIIRL_LOSS_VANILLA || loss_mode == SIIRL_LOSS_CPGD)
    SIIRL_REQUIRE(clip_c > 1.0f, "clip_ratio_c must be greater than 1.0, got %f", (double)clip_c);
  if (loss_mode == SIIRL_LOSS_CPGD) {
    SIIRL_REQUIRE(clip_low < 1.0f && clip_high > -1.0f, "CPGD takes log(1 - clip_low) and log(1 + clip_high)");
    a.log_lo = (float)log(1.0 - (double)clip_low);
    a.log_hi = (float)log(1.0 + (double)clip_high);
  }
  SIIRL_REQUIRE(log_ratio_clamp > 0.f, "log_ratio_clamp must be positive (20 in the reference, +inf for none)");
  if (ref_log_prob) SIIRL_REQUIRE(kl_mode >= 0 && kl_mode <= 3, "unknown kl mode %d", kl_mode);
  a.old_lp = old_log_prob; a.lp = log_prob; a.adv = advantages; a.mask = mask; a.mask_dtype = mask_dtype;
  a.isw = is_weights; a.ent = entropy; a.ref = ref_log_prob; a.aux = token_aux;
  static const int kind_of[] = {KIND_VANILLA, KIND_GSPO, KIND_CPGD, KIND_GPG, KIND_GEO, KIND_KL_COV, KIND_CLIP_COV};
  a.kind = kind_of[loss_mode];
  a.agg_mode = loss_mode == SIIRL_LOSS_GSPO ? SIIRL_AGG_SEQ_MEAN_TOKEN_MEAN : agg_mode;
  a.aux_agg_mode = agg_mode;
  a.kl_mode = kl_mode; a.kl_st = kl_straight_through;
  a.eps_lo = clip_low; a.eps_hi = clip_high; a.clip_c = clip_c; a.dclamp = log_ratio_clamp;
  a.ent_coef = entropy_coeff; a.kl_coef = kl_coef; a.drift_coef = policy_drift_coeff; a.scale = loss_scale;
  a.B = B; a.L = L; a.nseg = nseg_of(L);
  return SIIRL_OK;
}

extern "C" int siirl_actor_loss_fwd(const float* old_log_prob, const float* log_prob, const float* advantages,
                                    const void* mask, int mask_dtype, const float* is_weights, const float* entropy,
                                    const float* ref_log_prob, int64_t B, int64_t L, int loss_mode, float clip_low,
                                    float clip_high, float clip_c, float log_ratio_clamp, int agg_mode, float entropy_coeff, int kl_mode,
                                    int kl_straight_through, float kl_coef, float policy_drift_coeff, float loss_scale, float* out16,
                                    float* row_msum, float* row_s, void* workspace, size_t workspace_bytes,
                                    siirl_stream_t stream) {
  LossArgs a{};
  if (int rc = fill_actor_args(a, old_log_prob, log_prob, advantages, mask, mask_dtype, is_weights, entropy,
                               ref_log_prob, B, L, loss_mode, clip_low, clip_high, clip_c, log_ratio_clamp, agg_mode, entropy_coeff,
                               kl_mode, kl_straight_through, kl_coef, policy_drift_coeff, loss_scale))
    return rc;
  SIIRL_REQUIRE(out16 && (B == 0 || row_msum), "NULL output");
  SIIRL_REQUIRE(B == 0 || (loss_mode != SIIRL_LOSS_GSPO && loss_mode != SIIRL_LOSS_GEO_MEAN) || row_s,
                "row_s is required for the gspo and geo_mean losses");
  return run_forward(a, out16, row_msum, row_s, workspace, workspace_bytes, (hipStream_t)stream);
}

// Device address of `scratch` on each GPU, looked up on the first call made with that GPU current.
constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mu;

static int static_scratch_address(void** out) {
  int dev = -1;
  SIIRL_HIP_CHECK(hipGetDevice(&dev));
  SIIRL_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal %d is outside [0, %d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    SIIRL_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    SIIRL_REQUIRE(p != nullptr && ((uintptr_t)p & 255) == 0, "static scratch resolved to %p", p);
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return SIIRL_OK;
}

extern "C" int siirl_actor_loss_fwd_static(const float* old_log_prob, const float* log_prob, const float* advantages,
                                           const void* mask, int mask_dtype, const float* is_weights,
                                           const float* entropy, const float* ref_log_prob, int64_t B, int64_t L,
                                           int loss_mode, float clip_low, float clip_high, float clip_c,
                                           float log_ratio_clamp, int agg_mode, float entropy_coeff, int kl_mode,
                                           int kl_straight_through, float kl_coef, float policy_drift_coeff,
                                           float loss_scale, float* out16, float* row_msum, float* row_s,
                                           int slot, siirl_stream_t stream) {
  LossArgs a{};
  if (int rc = fill_actor_args(a, old_log_prob, log_prob, advantages, mask, mask_dtype, is_weights, entropy,
                               ref_log_prob, B, L, loss_mode, clip_low, clip_high, clip_c, log_ratio_clamp, agg_mode,
                               entropy_coeff, kl_mode, kl_straight_through, kl_coef, policy_drift_coeff, loss_scale))
    return rc;
  SIIRL_REQUIRE(slot >= 0 && slot < kStaticSlots, "slot %d is outside [0, %d)", slot, kStaticSlots);
  SIIRL_REQUIRE(out16 && (B == 0 || row_msum), "NULL output");
  SIIRL_REQUIRE(B == 0 || (loss_mode != SIIRL_LOSS_GSPO && loss_mode != SIIRL_LOSS_GEO_MEAN) || row_s,
                "row_s is required for the gspo and geo_mean losses");
  const size_t need = B == 0 ? 0 : ws_bytes_of(B, L);
  if (need > kStaticScratchBytes)
    return fail(SIIRL_ERR_WORKSPACE,
                "B=%lld x L=%lld needs %zu bytes of scratch, a slot of the static buffer holds %zu: use siirl_actor_loss_fwd "
                "with a workspace of the caller's", (long long)B, (long long)L, need, kStaticScratchBytes);
  void* ws = nullptr;
  if (int rc = static_scratch_address(&ws)) return rc;
  // every scratch word that the finish kernels read is written by this call's earlier kernels: nothing to clear
  return run_forward(a, out16, row_msum, row_s, (unsigned char*)ws + (size_t)slot * kStaticScratchBytes,
                     kStaticScratchBytes, (hipStream_t)stream);
}

extern "C" int siirl_actor_loss_bwd(const float* g_loss, const float* old_log_prob, const float* log_prob,
                                    const float* advantages, const void* mask, int mask_dtype,
                                    const float* is_weights, const float* entropy, const float* ref_log_prob,
                                    int64_t B, int64_t L, int loss_mode, float clip_low, float clip_high, float clip_c,
                                    float log_ratio_clamp, int agg_mode, float entropy_coeff, int kl_mode, int kl_straight_through,
                                    float kl_coef, float policy_drift_coeff, float loss_scale, const float* out16, const float* row_msum,
                                    const float* row_s, float* d_log_prob, float* d_entropy, siirl_stream_t stream) {
  LossArgs a{};
  if (int rc = fill_actor_args(a, old_log_prob, log_prob, advantages, mask, mask_dtype, is_weights, entropy,
                               ref_log_prob, B, L, loss_mode, clip_low, clip_high, clip_c, log_ratio_clamp, agg_mode, entropy_coeff,
                               kl_mode, kl_straight_through, kl_coef, policy_drift_coeff, loss_scale))
    return rc;
  if (B == 0) return SIIRL_OK;
  SIIRL_REQUIRE(g_loss && out16 && row_msum && d_log_prob, "NULL operand");
  SIIRL_REQUIRE((loss_mode != SIIRL_LOSS_GSPO && loss_mode != SIIRL_LOSS_GEO_MEAN) || row_s,
                "row_s is required for the gspo and geo_mean losses");
  SIIRL_REQUIRE(entropy == nullptr || d_entropy != nullptr, "d_entropy is required when entropy is given");
  set_vec(a, d_log_prob, d_entropy);
  return launch_loss_bwd(a, g_loss, out16, row_msum, row_s, d_log_prob, d_entropy, (hipStream_t)stream);
}

extern "C" size_t siirl_cov_workspace_bytes(void) { return (size_t)kCovGrid * kCovSums * sizeof(double); }

extern "C" int siirl_cov_scores(const float* old_log_prob, const float* log_prob, const float* advantages,
                                const void* mask, int mask_dtype, int64_t B, int64_t L, int loss_mode, float clip_low,
                                float clip_high, float* cov, float* stats, void* workspace, size_t workspace_bytes,
                                siirl_stream_t stream) {
  if (int rc = check_dims(B, L)) return rc;
  if (int rc = check_mask_dtype(mask_dtype)) return rc;
  SIIRL_REQUIRE(loss_mode == SIIRL_LOSS_KL_COV || loss_mode == SIIRL_LOSS_CLIP_COV,
                "covariance scores belong to the kl_cov and clip_cov losses (loss mode %d given)", loss_mode);
  SIIRL_REQUIRE(stats != nullptr, "NULL stats");
  SIIRL_REQUIRE(B == 0 || (log_prob && advantages && mask && cov), "NULL operand");
  SIIRL_REQUIRE(B == 0 || loss_mode != SIIRL_LOSS_CLIP_COV || old_log_prob, "clip_cov needs old_log_prob");
  if (workspace == nullptr || workspace_bytes < siirl_cov_workspace_bytes())
    return fail(SIIRL_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes,
                siirl_cov_workspace_bytes());
  SIIRL_REQUIRE(((uintptr_t)workspace & 7) == 0, "workspace must be 8-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const int64_t n = B * L;
  const int clip_mode = loss_mode == SIIRL_LOSS_CLIP_COV;
  const int64_t wgs = ((n + 3) / 4 + kThreads - 1) / kThreads;
  const int grid = (int)(wgs < 1 ? 1 : (wgs < kCovGrid ? wgs : kCovGrid));
  double* part = (double*)workspace;
  // four tokens per access when every operand starts on a 16-byte boundary (the mask: four of its elements)
  auto ok16 = [](const void* p) { return p == nullptr || ((uintptr_t)p & 15) == 0; };
  const size_t msz = dtype_size(mask_dtype);
  const int vec = ok16(old_log_prob) && ok16(log_prob) && ok16(advantages) && ok16(cov) &&
                  ((uintptr_t)mask & (msz * 4 > 16 ? 15 : msz * 4 - 1)) == 0;
  // the operands are read twice here and again by the loss
  const int nt_in = streams_past_cache((double)n * (double)(8 + msz + (clip_mode ? 4 : 0)));
  cov_sums_kernel<<<dim3((unsigned)grid), dim3(kThreads), 0, st>>>(log_prob, advantages, mask, mask_dtype, n, vec, nt_in,
                                                                  part);
  SIIRL_LAUNCH_CHECK("cov_sums_kernel");
  cov_stats_kernel<<<1, dim3(kThreads), 0, st>>>(part, grid, clip_mode, stats);
  SIIRL_LAUNCH_CHECK("cov_stats_kernel");
  if (n == 0) return SIIRL_OK;
  cov_scores_kernel<<<dim3((unsigned)grid), dim3(kThreads), 0, st>>>(old_log_prob, log_prob, advantages, mask, mask_dtype,
                                                                    n, vec, nt_in, clip_mode, 1.f - clip_low,
                                                                    1.f + clip_high, stats, cov);
  SIIRL_LAUNCH_CHECK("cov_scores_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_actor_loss_cov_fwd(const float* old_log_prob, const float* log_prob, const float* advantages,
                                        const void* mask, int mask_dtype, const float* is_weights, const float* entropy,
                                        const float* ref_log_prob, const float* token_aux, int64_t B, int64_t L,
                                        int loss_mode, float clip_low, float clip_high, int agg_mode, float entropy_coeff,
                                        int kl_mode, int kl_straight_through, float kl_coef, float policy_drift_coeff,
                                        float loss_scale, float* out16, float* row_msum, void* workspace,
                                        size_t workspace_bytes, siirl_stream_t stream) {
  LossArgs a{};
  SIIRL_REQUIRE(token_aux != nullptr || B == 0, "token_aux is NULL");
  if (int rc = fill_actor_args(a, old_log_prob, log_prob, advantages, mask, mask_dtype, is_weights, entropy,
                               ref_log_prob, B, L, loss_mode, clip_low, clip_high, 3.0f, 20.0f, agg_mode, entropy_coeff,
                               kl_mode, kl_straight_through, kl_coef, policy_drift_coeff, loss_scale,
                               token_aux, true))
    return rc;
  SIIRL_REQUIRE(out16 && (B == 0 || row_msum), "NULL output");
  return run_forward(a, out16, row_msum, nullptr, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int siirl_actor_loss_cov_bwd(const float* g_loss, const float* old_log_prob, const float* log_prob,
                                        const float* advantages, const void* mask, int mask_dtype,
                                        const float* is_weights, const float* entropy, const float* ref_log_prob,
                                        const float* token_aux, int64_t B, int64_t L, int loss_mode, float clip_low,
                                        float clip_high, int agg_mode, float entropy_coeff, int kl_mode,
                                        int kl_straight_through, float kl_coef, float policy_drift_coeff,
                                        float loss_scale, const float* out16, const float* row_msum, float* d_log_prob,
                                        float* d_entropy, siirl_stream_t stream) {
  LossArgs a{};
  SIIRL_REQUIRE(token_aux != nullptr || B == 0, "token_aux is NULL");
  if (int rc = fill_actor_args(a, old_log_prob, log_prob, advantages, mask, mask_dtype, is_weights, entropy,
                               ref_log_prob, B, L, loss_mode, clip_low, clip_high, 3.0f, 20.0f, agg_mode, entropy_coeff,
                               kl_mode, kl_straight_through, kl_coef, policy_drift_coeff, loss_scale,
                               token_aux, true))
    return rc;
  if (B == 0) return SIIRL_OK;
  SIIRL_REQUIRE(g_loss && out16 && row_msum && d_log_prob, "NULL operand");
  SIIRL_REQUIRE(entropy == nullptr || d_entropy != nullptr, "d_entropy is required when entropy is given");
  set_vec(a, d_log_prob, d_entropy);
  return launch_loss_bwd(a, g_loss, out16, row_msum, nullptr, d_log_prob, d_entropy, (hipStream_t)stream);
}

static int fill_value_args(LossArgs& a, const float* vpreds, const float* returns, const float* values,
                           const void* mask, int mask_dtype, int64_t B, int64_t L, float cliprange_value,
                           int agg_mode) {
  if (int rc = check_dims(B, L)) return rc;
  if (int rc = check_mask_dtype(mask_dtype)) return rc;
  if (int rc = check_agg(agg_mode)) return rc;
  SIIRL_REQUIRE(B == 0 || (vpreds && returns && values && mask), "NULL operand");
  a.old_lp = values; a.lp = vpreds; a.adv = returns; a.mask = mask; a.mask_dtype = mask_dtype;
  a.kind = KIND_VALUE; a.agg_mode = agg_mode; a.aux_agg_mode = agg_mode;
  a.eps_lo = cliprange_value; a.scale = 0.5f;
  a.B = B; a.L = L; a.nseg = nseg_of(L);
  return SIIRL_OK;
}

extern "C" int siirl_value_loss_fwd(const float* vpreds, const float* returns, const float* values, const void* mask,
                                    int mask_dtype, int64_t B, int64_t L, float cliprange_value, int agg_mode,
                                    float* out16, float* row_msum, void* workspace, size_t workspace_bytes,
                                    siirl_stream_t stream) {
  LossArgs a{};
  if (int rc = fill_value_args(a, vpreds, returns, values, mask, mask_dtype, B, L, cliprange_value, agg_mode)) return rc;
  SIIRL_REQUIRE(out16 && (B == 0 || row_msum), "NULL output");
  return run_forward(a, out16, row_msum, nullptr, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int siirl_value_loss_bwd(const float* g_loss, const float* vpreds, const float* returns,
                                    const float* values, const void* mask, int mask_dtype, int64_t B, int64_t L,
                                    float cliprange_value, int agg_mode, const float* out16, const float* row_msum,
                                    float* d_vpreds, siirl_stream_t stream) {
  LossArgs a{};
  if (int rc = fill_value_args(a, vpreds, returns, values, mask, mask_dtype, B, L, cliprange_value, agg_mode)) return rc;
  if (B == 0) return SIIRL_OK;
  SIIRL_REQUIRE(g_loss && out16 && row_msum && d_vpreds, "NULL operand");
  set_vec(a, d_vpreds);
  return launch_loss_bwd(a, g_loss, out16, row_msum, nullptr, d_vpreds, nullptr, (hipStream_t)stream);
}

extern "C" int siirl_kl_penalty_fwd(const float* logprob, const float* ref_logprob, int64_t n, int kl_mode, float* out,
                                    siirl_stream_t stream) {
  SIIRL_REQUIRE(n >= 0, "n < 0");
  SIIRL_REQUIRE(kl_mode >= 0 && kl_mode <= 3, "unknown kl mode %d", kl_mode);
  if (n == 0) return SIIRL_OK;
  SIIRL_REQUIRE(logprob && ref_logprob && out, "NULL operand");
  const int64_t want = ((n + 3) / 4 + kThreads - 1) / kThreads;
  const unsigned blocks = (unsigned)(want < 16384 ? want : 16384);
  const bool vec = (((uintptr_t)logprob | (uintptr_t)ref_logprob | (uintptr_t)out) & 15) == 0;
  kl_fwd_kernel<<<dim3(blocks), dim3(kThreads), 0, (hipStream_t)stream>>>(logprob, ref_logprob, n, kl_mode, vec, out);
  SIIRL_LAUNCH_CHECK("kl_fwd_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_kl_penalty_bwd(const float* g, const float* logprob, const float* ref_logprob, int64_t n,
                                    int kl_mode, int straight_through, float* d_logprob, float* d_ref_logprob,
                                    siirl_stream_t stream) {
  SIIRL_REQUIRE(n >= 0, "n < 0");
  SIIRL_REQUIRE(kl_mode >= 0 && kl_mode <= 3, "unknown kl mode %d", kl_mode);
  if (n == 0) return SIIRL_OK;
  SIIRL_REQUIRE(g && logprob && ref_logprob && (d_logprob || d_ref_logprob), "NULL operand");
  const int64_t want = ((n + 3) / 4 + kThreads - 1) / kThreads;
  const unsigned blocks = (unsigned)(want < 16384 ? want : 16384);
  const bool vec = (((uintptr_t)g | (uintptr_t)logprob | (uintptr_t)ref_logprob | (uintptr_t)d_logprob |
                     (uintptr_t)d_ref_logprob) & 15) == 0;
  kl_bwd_kernel<<<dim3(blocks), dim3(kThreads), 0, (hipStream_t)stream>>>(g, logprob, ref_logprob, n, kl_mode,
                                                                        straight_through, vec, d_logprob, d_ref_logprob);
  SIIRL_LAUNCH_CHECK("kl_bwd_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_masked_reduce(const float* values, const void* mask, int mask_dtype, int64_t B, int64_t L,
                                   float* row_sum, float* row_mean, float* total2, float* row_msum,
                                   float* mask_total, void* workspace, size_t workspace_bytes,
                                   siirl_stream_t stream) {
  if (int rc = check_dims(B, L)) return rc;
  if (int rc = check_mask_dtype(mask_dtype)) return rc;
  SIIRL_REQUIRE(B == 0 || (values && mask), "NULL operand");
  SIIRL_REQUIRE(row_sum || row_mean || total2 || row_msum || mask_total, "no output requested");
  LossArgs a{};
  a.lp = values; a.mask = mask; a.mask_dtype = mask_dtype; a.kind = KIND_AGG; a.agg_mode = SIIRL_AGG_TOKEN_MEAN;
  a.aux_agg_mode = a.agg_mode; a.scale = 1.f; a.B = B; a.L = L; a.nseg = nseg_of(L);
  if (B == 0) {  // sums of nothing
    masked_finish_kernel<<<1, dim3(kThreads), 0, (hipStream_t)stream>>>(nullptr, a.nseg, 0, row_sum, row_mean, total2,
                                                                        row_msum, mask_total);
    SIIRL_LAUNCH_CHECK("masked_finish_kernel");
    return SIIRL_OK;
  }
  if (workspace_bytes < ws_bytes_of(B, L) || workspace == nullptr)
    return fail(SIIRL_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes,
                ws_bytes_of(B, L));
  SIIRL_REQUIRE(((uintptr_t)workspace & 7) == 0, "workspace must be 8-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  float* partials = (float*)workspace;
  set_vec(a);
  if (int rc = launch_loss_partials(a, nullptr, partials, st)) return rc;
  const size_t used = ((size_t)B * a.nseg * (kNP + kNPre) * sizeof(float) + 255) / 256 * 256;
  const float* folded = partials;
  if (int rc = fold_long_rows(folded, partials, partials + (size_t)B * a.nseg * kNP, B, a.nseg, st)) return rc;
  if (B <= kTwoLevelRows) {
    masked_finish_kernel<<<1, dim3(kThreads), 0, st>>>(folded, a.nseg, B, row_sum, row_mean, total2, row_msum,
                                                       mask_total);
    SIIRL_LAUNCH_CHECK("masked_finish_kernel");
    return SIIRL_OK;
  }
  double* rec = reinterpret_cast<double*>((char*)workspace + used);  // room for kFinRec >= 2 doubles per workgroup
  const int nrec = (int)((B + kThreads - 1) / kThreads);
  masked_rows_kernel<<<dim3((unsigned)nrec), dim3(kThreads), 0, st>>>(folded, a.nseg, B, row_sum, row_mean, row_msum,
                                                                      rec);
  SIIRL_LAUNCH_CHECK("masked_rows_kernel");
  if (total2 || mask_total) {
    masked_finish2_kernel<<<1, dim3(kThreads), 0, st>>>(rec, nrec, total2, mask_total);
    SIIRL_LAUNCH_CHECK("masked_finish2_kernel");
  }
  return SIIRL_OK;
}

extern "C" int siirl_masked_reduce_bwd(const float* g, const void* mask, int mask_dtype, int64_t B, int64_t L,
                                       int per_row, const float* mask_sums, float* d_values, siirl_stream_t stream) {
  if (int rc = check_dims(B, L)) return rc;
  if (int rc = check_mask_dtype(mask_dtype)) return rc;
  if (B == 0) return SIIRL_OK;
  SIIRL_REQUIRE(g && mask && d_values, "NULL operand");
  LossArgs a{};  // only to decide whether rows can move as 16-byte quads
  a.mask = mask;
  a.mask_dtype = mask_dtype;
  a.B = B;
  a.L = L;
  set_vec(a, d_values);
  const int64_t want = (B * L / (a.vec ? 4 : 1) + kThreads - 1) / kThreads;
  const unsigned blocks = (unsigned)(want < 16384 ? (want < 1 ? 1 : want) : 16384);
  masked_bwd_kernel<<<dim3(blocks), dim3(kThreads), 0, (hipStream_t)stream>>>(g, mask, mask_dtype, B, L, per_row,
                                                                            mask_sums, a.vec, a.nt, d_values);
  SIIRL_LAUNCH_CHECK("masked_bwd_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_kl_in_reward(const float* token_level_scores, const float* old_log_prob,
                                  const float* ref_log_prob, const void* mask, int mask_dtype, int64_t B, int64_t L,
                                  int kl_mode, float beta, float* token_level_rewards, float* row_kl,
                                  float* current_kl, siirl_stream_t stream) {
  if (int rc = check_dims(B, L)) return rc;
  if (int rc = check_mask_dtype(mask_dtype)) return rc;
  SIIRL_REQUIRE(kl_mode >= 0 && kl_mode <= 3, "unknown kl mode %d", kl_mode);
  SIIRL_REQUIRE(current_kl && (B == 0 || (token_level_scores && old_log_prob && ref_log_prob && mask &&
                                          token_level_rewards && row_kl)), "NULL operand");
  hipStream_t st = (hipStream_t)stream;
  if (B > 0) {  // an empty batch has no rewards to write; its mean KL is the mean of nothing (NaN)
    LossArgs a{};  // only to decide whether rows can move as 16-byte quads
    a.old_lp = old_log_prob; a.ref = ref_log_prob; a.adv = token_level_scores; a.mask = mask; a.mask_dtype = mask_dtype;
    a.L = L;
    set_vec(a, token_level_rewards);
    kl_reward_kernel<<<dim3((unsigned)B), dim3(kThreads), 0, st>>>(token_level_scores, old_log_prob, ref_log_prob, mask,
                                                                  mask_dtype, L, kl_mode, beta, a.vec != 0,
                                                                  token_level_rewards, row_kl);
    SIIRL_LAUNCH_CHECK("kl_reward_kernel");
  }
  mean_rows_kernel<<<1, dim3(kThreads), 0, st>>>(row_kl, B, current_kl);
  SIIRL_LAUNCH_CHECK("mean_rows_kernel");
  return SIIRL_OK;
}
