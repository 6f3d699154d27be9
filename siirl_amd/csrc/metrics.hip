// Batch statistics the trainer logs from the tensors of the loss path, in one pass and one result block.
//
// Replaces compute_data_metric / _compute_response_info (siirl/utils/metrics/metric_utils.py:36-183): sequence
// score / reward sums, masked mean / max / min of advantages, returns and values, the value function's explained
// variance, response and prompt length statistics.  The reference issues ~40 reductions and as many .item() syncs;
// here a partials kernel over [B, L] segments and a one-workgroup finish write SIIRL_METRIC_COUNT floats.
#include "common.hpp"

namespace siirl {
namespace {

constexpr int kThreads = 256;
constexpr int kSeg = 4096;
constexpr int kNP = 16;
enum P { P_SCORE = 0, P_REWARD, P_CNT, P_ADV, P_RET, P_VAL, P_DIFF, P_DIFF2, P_RET2, P_ADVMAX, P_ADVMIN, P_RETMAX,
         P_RETMIN, P_VALMAX, P_VALMIN, P_PROMPT };

struct MetricArgs {
  const float* scores;   // token_level_scores  [B, L]
  const float* rewards;  // token_level_rewards [B, L]
  const float* adv;      // [B, L]
  const float* ret;      // [B, L]
  const float* val;      // [B, L] or null
  const void* rmask;     // response_mask [B, L]
  int rmask_dtype;
  const void* amask;     // attention_mask [B, S], S = P + L; the prompt part is its first P columns
  int amask_dtype;
  int64_t B, L, Pw;
  int nseg;
};

__device__ __forceinline__ double wave_max_d(double v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmax(v, __shfl_xor(v, o, kWave));
  return v;
}
__device__ __forceinline__ double block_max_d(double v, double* sh) {
  v = wave_max_d(v);
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x / kWave;
  __syncthreads();
  if (lane == 0) sh[wid] = v;
  __syncthreads();
  double r = sh[0];
  for (int w = 1; w < kThreads / kWave; ++w) r = fmax(r, sh[w]);
  return r;
}

__global__ __launch_bounds__(kThreads) void metric_partials_kernel(MetricArgs a, double* __restrict__ part) {
  const int64_t b = blockIdx.x / a.nseg;
  const int seg = blockIdx.x % a.nseg;
  const int64_t t0 = (int64_t)seg * kSeg;
  const double inf = (double)__builtin_inff();
  double s[9];
  for (int k = 0; k < 9; ++k) s[k] = 0.0;
  double mx[3] = {-inf, -inf, -inf}, mn[3] = {inf, inf, inf};
  for (int i = threadIdx.x; i < kSeg; i += kThreads) {
    const int64_t t = t0 + i;
    if (t >= a.L) break;
    const int64_t idx = b * a.L + t;
    s[P_SCORE] += (double)a.scores[idx];
    s[P_REWARD] += (double)a.rewards[idx];
    if (load_mask(a.rmask, a.rmask_dtype, idx) != 0.f) {  // response_mask.bool()
      const float ad = a.adv[idx], re = a.ret[idx];
      s[P_CNT] += 1.0;
      s[P_ADV] += (double)ad;
      s[P_RET] += (double)re;
      s[P_RET2] += (double)re * (double)re;
      mx[0] = fmax(mx[0], (double)ad); mn[0] = fmin(mn[0], (double)ad);
      mx[1] = fmax(mx[1], (double)re); mn[1] = fmin(mn[1], (double)re);
      if (a.val) {
        const float va = a.val[idx];
        const double d = (double)(re - va);  // the reference subtracts in float32
        s[P_VAL] += (double)va;
        s[P_DIFF] += d;
        s[P_DIFF2] += d * d;
        mx[2] = fmax(mx[2], (double)va); mn[2] = fmin(mn[2], (double)va);
      }
    }
  }
  double prompt = 0.0;
  if (seg == 0)
    for (int64_t c = threadIdx.x; c < a.Pw; c += kThreads)
      prompt += load_mask(a.amask, a.amask_dtype, b * (a.Pw + a.L) + c) != 0.f ? 1.0 : 0.0;
  __shared__ double sh[kThreads / kWave + 1];
  double* out = part + (b * a.nseg + seg) * kNP;
  for (int k = 0; k < 9; ++k) {
    const double v = block_sum(s[k], sh);
    if (threadIdx.x == 0) out[k] = v;
  }
  for (int k = 0; k < 3; ++k) {
    const double hi = block_max_d(mx[k], sh);
    const double lo = -block_max_d(-mn[k], sh);
    if (threadIdx.x == 0) {
      out[P_ADVMAX + 2 * k] = hi;
      out[P_ADVMAX + 2 * k + 1] = lo;
    }
  }
  prompt = block_sum(prompt, sh);
  if (threadIdx.x == 0) out[P_PROMPT] = prompt;
}

// running sum / max / min of a per-row quantity
struct Stat {
  double s, hi, lo, n;
  __device__ void init() { s = 0.0; hi = -(double)__builtin_inff(); lo = (double)__builtin_inff(); n = 0.0; }
  __device__ void add(double v) { s += v; hi = fmax(hi, v); lo = fmin(lo, v); n += 1.0; }
  __device__ void reduce(double* sh) {
    s = block_sum(s, sh);
    n = block_sum(n, sh);
    hi = block_max_d(hi, sh);
    lo = -block_max_d(-lo, sh);
  }
};

__global__ __launch_bounds__(kThreads) void metric_finish_kernel(MetricArgs a, const double* __restrict__ part,
                                                                 float* __restrict__ out) {
  const double inf = (double)__builtin_inff();
  Stat score, reward, rlen, plen, clen, wlen;
  score.init(); reward.init(); rlen.init(); plen.init(); clen.init(); wlen.init();
  double tot[9];
  for (int k = 0; k < 9; ++k) tot[k] = 0.0;
  double mx[3] = {-inf, -inf, -inf}, mn[3] = {inf, inf, inf};
  double rclip = 0.0, pclip = 0.0;
  for (int64_t b = threadIdx.x; b < a.B; b += kThreads) {
    double r[9];
    for (int k = 0; k < 9; ++k) r[k] = 0.0;
    for (int sgm = 0; sgm < a.nseg; ++sgm) {
      const double* p = part + (b * a.nseg + sgm) * kNP;
      for (int k = 0; k < 9; ++k) r[k] += p[k];
      for (int k = 0; k < 3; ++k) {
        mx[k] = fmax(mx[k], p[P_ADVMAX + 2 * k]);
        mn[k] = fmin(mn[k], p[P_ADVMAX + 2 * k + 1]);
      }
    }
    const double prompt = part[(b * a.nseg) * kNP + P_PROMPT];
    for (int k = 2; k < 9; ++k) tot[k] += r[k];
    const double sc = (double)(float)r[P_SCORE], rw = (double)(float)r[P_REWARD];  // float32 row sums, as .sum(-1)
    score.add(sc);
    reward.add(rw);
    rlen.add(r[P_CNT]);
    plen.add(prompt);
    if (r[P_CNT] == (double)a.L) rclip += 1.0;
    if (prompt == (double)a.Pw) pclip += 1.0;
    if (rw > 0.5) clen.add(r[P_CNT]); else wlen.add(r[P_CNT]);
  }
  __shared__ double sh[kThreads / kWave + 1];
  score.reduce(sh); reward.reduce(sh); rlen.reduce(sh); plen.reduce(sh); clen.reduce(sh); wlen.reduce(sh);
  for (int k = 2; k < 9; ++k) tot[k] = block_sum(tot[k], sh);
  for (int k = 0; k < 3; ++k) {
    mx[k] = block_max_d(mx[k], sh);
    mn[k] = -block_max_d(-mn[k], sh);
  }
  rclip = block_sum(rclip, sh);
  pclip = block_sum(pclip, sh);
  if (threadIdx.x != 0) return;
  const double B = (double)a.B, n = tot[P_CNT];
  int o = 0;
  auto put = [&](double v) { out[o++] = (float)v; };
  put(score.s / B); put(score.hi); put(score.lo);
  put(reward.s / B); put(reward.hi); put(reward.lo);
  put(tot[P_ADV] / n); put(mx[0]); put(mn[0]);
  put(tot[P_RET] / n); put(mx[1]); put(mn[1]);
  if (a.val) {
    put(tot[P_VAL] / n); put(mx[2]); put(mn[2]);
    const double var_diff = (tot[P_DIFF2] - tot[P_DIFF] * tot[P_DIFF] / n) / (n - 1.0);  // torch.var: unbiased
    const double var_ret = (tot[P_RET2] - tot[P_RET] * tot[P_RET] / n) / (n - 1.0);
    put(1.0 - var_diff / (var_ret + 1e-5));
  } else {
    put(0.0); put(0.0); put(0.0); put(0.0);
  }
  put(rlen.s / B); put(rlen.hi); put(rlen.lo); put(rclip / B);
  put(clen.n > 0 ? clen.hi : 0.0); put(clen.n > 0 ? clen.lo : 0.0); put(clen.n > 0 ? clen.s / clen.n : 0.0);
  put(wlen.n > 0 ? wlen.hi : 0.0); put(wlen.n > 0 ? wlen.lo : 0.0); put(wlen.n > 0 ? wlen.s / wlen.n : 0.0);
  put(plen.s / B); put(plen.hi); put(plen.lo); put(pclip / B);
  put(n);
  while (o < 32) put(0.0);
}

int check_mask(int dt) {
  SIIRL_REQUIRE(dt == SIIRL_U8 || dt == SIIRL_I64 || dt == SIIRL_I32 || dt == SIIRL_F32 || dt == SIIRL_BF16 ||
                    dt == SIIRL_F16, "mask dtype %d not supported", dt);
  return SIIRL_OK;
}
int nseg_of(int64_t L) { return (int)((L + kSeg - 1) / kSeg); }

}  // namespace
}  // namespace siirl

using namespace siirl;

extern "C" size_t siirl_data_metrics_workspace_bytes(int64_t B, int64_t L) {
  if (B < 1 || L < 1) return 0;
  return (size_t)B * nseg_of(L) * kNP * sizeof(double);
}

extern "C" int siirl_data_metrics(const float* token_level_scores, const float* token_level_rewards,
                                  const float* advantages, const float* returns, const float* values,
                                  const void* response_mask, int response_mask_dtype, const void* attention_mask,
                                  int attention_mask_dtype, int64_t B, int64_t L, int64_t prompt_width, float* out32,
                                  void* workspace, size_t workspace_bytes, siirl_stream_t stream) {
  SIIRL_REQUIRE(B >= 1 && L >= 1 && prompt_width >= 0 && B * (int64_t)nseg_of(L) <= 0x7fffffffLL,
                "B=%lld L=%lld prompt_width=%lld out of range", (long long)B, (long long)L, (long long)prompt_width);
  if (int rc = check_mask(response_mask_dtype)) return rc;
  if (prompt_width > 0)
    if (int rc = check_mask(attention_mask_dtype)) return rc;
  SIIRL_REQUIRE(token_level_scores && token_level_rewards && advantages && returns && response_mask && out32 &&
                    (prompt_width == 0 || attention_mask), "NULL operand");
  const size_t need = siirl_data_metrics_workspace_bytes(B, L);
  if (workspace == nullptr || workspace_bytes < need)
    return fail(SIIRL_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes, need);
  SIIRL_REQUIRE(((uintptr_t)workspace & 7) == 0, "workspace must be 8-byte aligned");
  MetricArgs a{token_level_scores, token_level_rewards, advantages, returns, values, response_mask,
               response_mask_dtype, attention_mask, attention_mask_dtype, B, L, prompt_width, nseg_of(L)};
  hipStream_t st = (hipStream_t)stream;
  metric_partials_kernel<<<dim3((unsigned)(B * a.nseg)), dim3(kThreads), 0, st>>>(a, (double*)workspace);
  SIIRL_LAUNCH_CHECK("metric_partials_kernel");
  metric_finish_kernel<<<1, dim3(kThreads), 0, st>>>(a, (const double*)workspace, out32);
  SIIRL_LAUNCH_CHECK("metric_finish_kernel");
  return SIIRL_OK;
}
