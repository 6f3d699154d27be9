// Outcome-reward placement with DAPO's overlong penalty.
//
// Replaces the tensor arithmetic of DAPORewardManager.__call__ (siirl/engine/reward_manager/dapo.py:57-126): per
// trajectory, valid_response_length = sum of the attention mask over the response columns; the scalar score, plus
// min(-(valid - (max_resp_len - buffer_len)) / buffer_len * penalty_factor, 0) when the overlong buffer is
// enabled, is written at the last valid response token of an otherwise zero float32 [B, L] tensor.  The penalty
// is float32 arithmetic, as in the reference where the valid length is a 0-d tensor; a row without valid tokens
// lands on index -1, i.e. the last column, as Python indexing does.  Scoring itself (tokenizer, rule functions) is the caller's.
#include "common.hpp"

namespace siirl {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ double mask_value(const void* p, int dt, int64_t i) { return (double)load_mask(p, dt, i); }

__global__ __launch_bounds__(kThreads) void place_reward_kernel(const double* __restrict__ scores, const void* amask,
                                                                int amask_dtype, int64_t Pw, int64_t L, int enable,
                                                                double max_resp_len, double buffer_len,
                                                                double penalty_factor, float* __restrict__ reward,
                                                                double* __restrict__ overlong,
                                                                int64_t* __restrict__ valid_len) {
  const int64_t b = blockIdx.x;
  double n = 0.0;
  for (int64_t t = threadIdx.x; t < L; t += kThreads) {
    n += mask_value(amask, amask_dtype, b * (Pw + L) + Pw + t);
    reward[b * L + t] = 0.f;
  }
  __shared__ double sh[kThreads / kWave + 1];
  n = block_sum(n, sh);
  __syncthreads();  // the zero fill above is complete before the one non-zero store
  if (threadIdx.x != 0) return;
  const int64_t valid = (int64_t)n;
  // valid is a 0-d integer tensor in the reference, so the penalty is float32 tensor arithmetic:
  // (-exceed / buffer_len) * penalty_factor, min with 0, and score + penalty, each rounded to float32
  float r = (float)scores[b], pen = 0.f;
  if (enable) {
    const float exceed = (float)((double)valid - (max_resp_len - buffer_len));
    pen = fminf((-exceed / (float)buffer_len) * (float)penalty_factor, 0.f);
    r = r + pen;
  }
  int64_t pos = valid - 1;
  if (pos < 0) pos += L;
  if (pos >= 0 && pos < L) reward[b * L + pos] = r;
  if (overlong) overlong[b] = (double)pen;
  if (valid_len) valid_len[b] = valid;
}

}  // namespace
}  // namespace siirl

using namespace siirl;

extern "C" int siirl_place_outcome_reward(const double* scores, const void* attention_mask, int mask_dtype, int64_t B,
                                          int64_t prompt_width, int64_t L, int overlong_enable, double max_resp_len,
                                          double overlong_buffer_len, double overlong_penalty_factor,
                                          float* reward_tensor, double* overlong_reward, int64_t* valid_response_length,
                                          siirl_stream_t stream) {
  SIIRL_REQUIRE(B >= 1 && L >= 1 && prompt_width >= 0 && B <= 0x7fffffffLL, "B=%lld L=%lld prompt_width=%lld out of range",
                (long long)B, (long long)L, (long long)prompt_width);
  SIIRL_REQUIRE(mask_dtype == SIIRL_U8 || mask_dtype == SIIRL_I64 || mask_dtype == SIIRL_I32 || mask_dtype == SIIRL_F32 ||
                    mask_dtype == SIIRL_BF16 || mask_dtype == SIIRL_F16, "mask dtype %d not supported", mask_dtype);
  SIIRL_REQUIRE(scores && attention_mask && reward_tensor, "NULL operand");
  SIIRL_REQUIRE(!overlong_enable || overlong_buffer_len != 0.0, "overlong buffer length must not be zero");
  place_reward_kernel<<<dim3((unsigned)B), dim3(kThreads), 0, (hipStream_t)stream>>>(
      scores, attention_mask, mask_dtype, prompt_width, L, overlong_enable, max_resp_len, overlong_buffer_len,
      overlong_penalty_factor, reward_tensor, overlong_reward, valid_response_length);
  SIIRL_LAUNCH_CHECK("place_reward_kernel");
  return SIIRL_OK;
}
