// Per-token formulas of the [B, L] loss arithmetic, shared by the loss kernels and by the fused logits ->
// dlogits actor step: the registered policy losses (value and hand-derived gradient per token), the KL
// estimators, aggregation weights, and small load helpers.
//
// Follows siirl/dag_worker/core_algos.py: agg_loss :536-569, cpgd :572-629, vanilla :710-792, gspo :795-862,
// gpg :865-895, clip_cov :898-995, kl_cov :998-1071, geo_mean :1074-1153, value loss :1173-1212, kl_penalty
// :1215-1276; drift term
// siirl/engine/actor/dp_actor.py:488-494.
#pragma once
#include "common.hpp"

// Cache hints of the [B, L] streaming kernels.  Measured at [5488, 8192] fp32 with an int64 mask (actor loss forward +
// backward): non-temporal loads 0.467 -> 0.428 ms, non-temporal stores of the gradient a further 0.428 -> 0.420 ms.
// That is for operands several times the part's 256 MB memory-side cache.  A pass that reads less than
// kCacheResidentBytes (common.hpp) uses ordinary loads instead (`nt` of the load helpers below, decided on the host
// per launch): what the forward has read is then still cached when the backward reads it again -- forward + backward
// at [1024, 8192] (192 MiB per pass) 99.8 -> 94 us, at [512, 8192] 55.3 -> 51 us; at [2048, 8192] (384 MiB) the
// non-temporal loads are the faster ones again (166 against 183 us).  Stores are non-temporal at every size: ordinary
// ones gain nothing there (51.8 against 51.1 us, 94.9 against 94.4 us) and their write-back delays the next kernel.
#ifndef SIIRL_LOSS_NT_STORE
#define SIIRL_LOSS_NT_STORE 1
#endif
#ifndef SIIRL_LOSS_NT_LOAD
#define SIIRL_LOSS_NT_LOAD 1
#endif

namespace siirl {
namespace tok {

struct LossArgs {
  const float* old_lp;   // [B,L] or null (kind == KIND_AGG)
  const float* lp;       // [B,L]  (kind == KIND_AGG: the loss matrix to aggregate)
  const float* adv;      // [B,L]
  const void* mask;      // [B,L]
  const float* isw;      // [B,L] or null
  const float* ent;      // [B,L] or null
  const float* ref;      // [B,L] or null
  const float* aux;      // [B,L], the covariance losses only: kl_cov the coefficient of |lp - old| per token
                         // (ppo_kl_coef where selected, else 0), clip_cov non-zero where the token's loss is dropped
  int mask_dtype;
  int kind;              // KIND_*
  int agg_mode;          // aggregation of the policy term (GSPO: forced to seq-mean-token-mean)
  int aux_agg_mode;      // aggregation of the entropy and KL terms
  int kl_mode, kl_st;
  float eps_lo, eps_hi, clip_c, dclamp;
  float log_lo, log_hi;  // CPGD: float(log(1 - eps_lo)), float(log(1 + eps_hi)), logarithms taken in double
  float ent_coef, kl_coef, drift_coef, scale;
  int64_t B, L;
  int nseg;
  int vec;  // L % 4 == 0 and every operand 16-byte aligned: tokens are moved four at a time
  int nt;   // the operands of a pass exceed the memory-side cache: non-temporal loads
};
enum { KIND_AGG = 0, KIND_VANILLA = 1, KIND_GSPO = 2, KIND_CPGD = 3, KIND_GPG = 4, KIND_GEO = 5, KIND_VALUE = 6,
       KIND_KL_COV = 7, KIND_CLIP_COV = 8 };

// torch.clamp / torch.maximum / torch.minimum semantics (NaN propagates)
__device__ __forceinline__ float clampf(float x, float lo, float hi) { return x < lo ? lo : (x > hi ? hi : x); }
__device__ __forceinline__ float clamp_max(float x, float hi) { return x > hi ? hi : x; }
__device__ __forceinline__ float tmax(float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : fmaxf(a, b); }
__device__ __forceinline__ float tmin(float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : fminf(a, b); }

// masked contribution.  token-mean goes through masked_mean: where(mask, v, 0) * mask; the other modes
// multiply directly (a NaN under a zero mask poisons them, as in the reference).
__device__ __forceinline__ float contrib_where(float v, float m) { return m != 0.f ? v * m : 0.f; }
__device__ __forceinline__ float contrib(float v, float m, int agg) {
  return agg == SIIRL_AGG_TOKEN_MEAN ? contrib_where(v, m) : v * m;
}

// four consecutive tokens of one operand; `vec` selects one 16-byte access
struct Quad {
  float v[4];
};
__device__ __forceinline__ Quad load_quad(const float* __restrict__ p, int64_t idx, bool vec, int nv, float fill,
                                          bool nt = SIIRL_LOSS_NT_LOAD != 0) {
  Quad q;
  if (vec) {
    if (SIIRL_LOSS_NT_LOAD && nt) {
      const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p + idx));
      q.v[0] = u2f(t.x); q.v[1] = u2f(t.y); q.v[2] = u2f(t.z); q.v[3] = u2f(t.w);
    } else {
      const float4 t = *reinterpret_cast<const float4*>(p + idx);
      q.v[0] = t.x; q.v[1] = t.y; q.v[2] = t.z; q.v[3] = t.w;
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) q.v[e] = e < nv ? p[idx + e] : fill;
  }
  return q;
}
__device__ __forceinline__ Quad const_quad(float c) { return Quad{{c, c, c, c}}; }
__device__ __forceinline__ Quad load_mask_quad(const void* p, int dt, int64_t idx, bool vec, int nv,
                                               bool nt = SIIRL_LOSS_NT_LOAD != 0) {
  Quad q;
  if (vec && dt == SIIRL_I64) {
    longlong2 a, b;
    if (SIIRL_LOSS_NT_LOAD && nt) {
      const u32x4 ra = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>((const int64_t*)p + idx));
      const u32x4 rb = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>((const int64_t*)p + idx) + 1);
      a.x = (int64_t)(((uint64_t)ra.y << 32) | ra.x); a.y = (int64_t)(((uint64_t)ra.w << 32) | ra.z);
      b.x = (int64_t)(((uint64_t)rb.y << 32) | rb.x); b.y = (int64_t)(((uint64_t)rb.w << 32) | rb.z);
    } else {
      a = reinterpret_cast<const longlong2*>((const int64_t*)p + idx)[0];
      b = reinterpret_cast<const longlong2*>((const int64_t*)p + idx)[1];
    }
    // masks hold small integers: when every value in the wave fits 32 bits, one v_cvt_f32_i32 each replaces the
    // 64-bit conversion sequence (the wave-uniform test keeps the general path out of the way, not out of the code)
    const int32_t l0 = (int32_t)a.x, l1 = (int32_t)a.y, l2 = (int32_t)b.x, l3 = (int32_t)b.y;
    const bool wide = ((int64_t)l0 != a.x) | ((int64_t)l1 != a.y) | ((int64_t)l2 != b.x) | ((int64_t)l3 != b.y);
    if (__builtin_amdgcn_ballot_w64(wide) == 0) {
      q.v[0] = (float)l0; q.v[1] = (float)l1; q.v[2] = (float)l2; q.v[3] = (float)l3;
    } else {
      q.v[0] = (float)a.x; q.v[1] = (float)a.y; q.v[2] = (float)b.x; q.v[3] = (float)b.y;
    }
  } else if (vec && dt == SIIRL_U8) {
    const uint32_t u = *reinterpret_cast<const uint32_t*>((const uint8_t*)p + idx);
    q.v[0] = (float)(u & 0xffu); q.v[1] = (float)((u >> 8) & 0xffu); q.v[2] = (float)((u >> 16) & 0xffu);
    q.v[3] = (float)(u >> 24);
  } else if (vec && dt == SIIRL_F32) {
    q = load_quad((const float*)p, idx, true, 4, 0.f, nt);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) q.v[e] = e < nv ? load_mask(p, dt, idx + e) : 0.f;
  }
  return q;
}
__device__ __forceinline__ void store_quad(float* __restrict__ p, int64_t idx, bool vec, int nv, const Quad& q) {
  if (vec) {
#if SIIRL_LOSS_NT_STORE
    __builtin_nontemporal_store(u32x4{f2u(q.v[0]), f2u(q.v[1]), f2u(q.v[2]), f2u(q.v[3])}, reinterpret_cast<u32x4*>(p + idx));
#else
    *reinterpret_cast<float4*>(p + idx) = make_float4(q.v[0], q.v[1], q.v[2], q.v[3]);
#endif
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (e < nv) p[idx + e] = q.v[e];
  }
}

struct KlOut {
  float v, g;  // value and d value / d logprob
};
__device__ __forceinline__ KlOut kl_token(float lp, float ref, int mode, int straight_through) {
  const float x = lp - ref;
  KlOut o;
  switch (mode) {
    case SIIRL_KL_K1: o.v = x; o.g = 1.f; break;
    case SIIRL_KL_ABS: o.v = fabsf(x); o.g = x > 0.f ? 1.f : (x < 0.f ? -1.f : 0.f); break;
    case SIIRL_KL_K2: o.v = 0.5f * x * x; o.g = x; break;
    default: {  // K3
      const float kr = ref - lp;
      const float k = clampf(kr, -20.f, 20.f);
      const float e = expf(k);
      const float raw = e - k - 1.f;
      o.v = clampf(raw, -10.f, 10.f);
      const bool pass = (kr >= -20.f && kr <= 20.f) && (raw >= -10.f && raw <= 10.f);
      o.g = pass ? -(e - 1.f) : 0.f;
    }
  }
  if (straight_through) o.g = x;  // value of the estimator, gradient of k2
  return o;
}

struct PgOut {
  float tok, dtok;  // per-token loss and d tok / d logprob (before the aggregation weight)
  float clip, lower, negd, r_raw;
};

// seq_s: GSPO's sequence-level mean log-ratio (unused otherwise).  For KIND_GEO tok is the token's clipped
// log-ratio x (the loss itself is per sequence); for KIND_VALUE lp = vpreds, old = values, A = returns and
// eps_lo = cliprange_value.  aux: the token's entry of LossArgs::aux (0 for the losses that have none).
__device__ __forceinline__ PgOut pg_token(int kind, float lp, float old, float A, float isw, float seq_s,
                                          const LossArgs& a, float aux = 0.f) {
  const float eps_lo = a.eps_lo, eps_hi = a.eps_hi, clip_c = a.clip_c, dclamp = a.dclamp;
  PgOut o;
  const float raw = lp - old;
  o.r_raw = expf(raw);
  const float lo = 1.f - eps_lo, hi = 1.f + eps_hi;
  if (kind == KIND_CPGD) {
    // the log-probability is clipped, not the ratio; importance weights are not used by this loss
    o.negd = -raw;
    float clipped;
    bool pass;
    if (A > 0.f) {
      const float b = a.log_hi + old;
      clipped = lp > b ? b : lp;
      pass = lp <= b;
      o.clip = o.r_raw > hi ? 1.f : 0.f;
    } else {
      const float b = a.log_lo + old;
      clipped = lp < b ? b : lp;
      pass = lp >= b;
      o.clip = o.r_raw < lo ? 1.f : 0.f;
    }
    o.tok = -clipped * A;
    o.dtok = pass ? -A : 0.f;
    o.lower = (o.r_raw > clip_c && A < 0.f) ? 1.f : 0.f;
    return o;
  }
  if (kind == KIND_GPG) {
    o.negd = 0.f; o.clip = 0.f; o.lower = 0.f;
    o.tok = -lp * A * isw;
    o.dtok = -A * isw;
    return o;
  }
  if (kind == KIND_GEO) {
    o.negd = -raw;
    const float sgn = A > 0.f ? 1.f : (A < 0.f ? -1.f : (A == 0.f ? 0.f : A));  // torch.sign; NaN stays NaN
    const float dc = clampf(raw, -eps_lo, eps_hi);
    const float p = sgn * raw, q = sgn * dc;
    o.tok = sgn * tmin(p, q);
    const bool inside = raw >= -eps_lo && raw <= eps_hi;  // then p == q and both sides of the min pass 1/2
    o.dtok = (inside || p < q) ? sgn * sgn : 0.f;
    const bool clipped = raw != dc;
    o.clip = (clipped && A > 0.f) ? 1.f : 0.f;
    o.lower = (clipped && A < 0.f) ? 1.f : 0.f;
    return o;
  }
  if (kind == KIND_KL_COV) {
    // -A * ratio, unclipped; a selected token also pays aux * |lp - old|.  The ppo_kl slot reports mean |lp - old|.
    const float ad = fabsf(raw);
    o.negd = ad; o.clip = 0.f; o.lower = 0.f;
    const float base = -A * o.r_raw;
    const float sg = raw > 0.f ? 1.f : (raw < 0.f ? -1.f : raw);  // torch.sign: 0 at 0, NaN stays NaN
    o.tok = (aux != 0.f ? base + aux * ad : base) * isw;
    o.dtok = (aux != 0.f ? base + aux * sg : base) * isw;
    return o;
  }
  if (kind == KIND_CLIP_COV) {
    // the PPO clip surrogate without dual clip and without the clamp of the log-ratio; a dropped token (aux != 0)
    // contributes nothing and is what the clip-fraction slot counts
    o.negd = -raw; o.lower = 0.f;
    const float r = o.r_raw;
    const float l1 = -A * r;
    const float l2 = -A * clampf(r, lo, hi);
    const float corr = aux != 0.f ? 0.f : 1.f;
    o.clip = 1.f - corr;
    o.tok = tmax(l1, l2) * corr * isw;
    const float dl2 = (r >= lo && r <= hi) ? l1 : 0.f;  // d l1 / d lp = l1
    const float w1 = l1 > l2 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
    const float w2 = l2 > l1 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
    o.dtok = (w1 * l1 + w2 * dl2) * corr * isw;
    return o;
  }
  if (kind == KIND_VALUE) {
    o.negd = 0.f; o.lower = 0.f; o.r_raw = 1.f;
    const float vmax = old + eps_lo, vmin = old - eps_lo;
    const float inner = tmin(lp, vmax), vc = tmax(inner, vmin);
    const float e1 = lp - A, e2 = vc - A;
    const float l1 = e1 * e1, l2 = e2 * e2;
    o.tok = tmax(l1, l2);
    o.clip = l2 > l1 ? 1.f : 0.f;
    const float dinner = lp < vmax ? 1.f : (lp == vmax ? 0.5f : 0.f);
    const float dvc = inner > vmin ? dinner : (inner == vmin ? 0.5f * dinner : 0.f);
    const float w1 = l1 > l2 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
    const float w2 = l2 > l1 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
    o.dtok = w1 * 2.f * e1 + w2 * 2.f * e2 * dvc;
    return o;
  }
  if (kind == KIND_VANILLA) {
    const float d = clampf(raw, -dclamp, dclamp);
    const float r = d == raw ? o.r_raw : expf(d);  // the clamp rarely bites: one exponential serves both
    const float dr = (raw >= -dclamp && raw <= dclamp) ? r : 0.f;  // d r / d lp
    o.negd = -d;
    const float l1 = -A * r;
    const float rc = clampf(r, lo, hi);
    const float l2 = -A * rc;
    const float c1 = tmax(l1, l2);
    o.clip = l2 > l1 ? 1.f : 0.f;
    const float l3 = -A * clip_c;
    const float c2 = tmin(l3, c1);
    o.lower = (c1 > l3 && A < 0.f) ? 1.f : 0.f;
    o.tok = A < 0.f ? c2 : c1;
    // autograd: maximum / minimum give each side 1, 1/2 (tie) or 0; clamp passes inside [lo, hi] inclusive
    const float dl1 = -A * dr;
    const float dl2 = (r >= lo && r <= hi) ? -A * dr : 0.f;
    const float w1 = l1 > l2 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
    const float w2 = l2 > l1 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
    const float dc1 = w1 * dl1 + w2 * dl2;
    const float wc = c1 < l3 ? 1.f : (c1 == l3 ? 0.5f : 0.f);
    o.dtok = A < 0.f ? wc * dc1 : dc1;
  } else {  // GSPO
    o.negd = -raw;
    const float l = clamp_max(seq_s, 10.f);  // lp - lp.detach() == 0
    const float r = expf(l);
    const float dr = (seq_s <= 10.f) ? r : 0.f;
    const float l1 = -A * r;
    const float rc = clampf(r, lo, hi);
    const float l2 = -A * rc;
    o.tok = tmax(l1, l2);
    o.clip = l2 > l1 ? 1.f : 0.f;
    o.lower = 0.f;
    const float dl1 = -A * dr;
    const float dl2 = (r >= lo && r <= hi) ? -A * dr : 0.f;
    const float w1 = l1 > l2 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
    const float w2 = l2 > l1 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
    o.dtok = w1 * dl1 + w2 * dl2;
  }
  o.tok *= isw;  // importance weights multiply value and gradient alike
  o.dtok *= isw;
  return o;
}


// aggregation weight of token (b, t): d (aggregate) / d (loss_mat[b, t])
__device__ __forceinline__ float agg_weight(int agg, float m, float mtotal, float mrow, int64_t B, int64_t L) {
  switch (agg) {
    case SIIRL_AGG_TOKEN_MEAN: return m != 0.f ? m / (mtotal + 1e-8f) : 0.f;
    case SIIRL_AGG_SEQ_MEAN_TOKEN_SUM: return m / (float)B;
    case SIIRL_AGG_SEQ_MEAN_TOKEN_MEAN: return m / mrow / (float)B;
    default: return m / (float)L;
  }
}

}  // namespace tok
}  // namespace siirl
