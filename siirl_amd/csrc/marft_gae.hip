// Multi-agent GAE over reversed trajectories (MARFT): compute_marft_gae_advantage_return,
// siirl/dag_worker/core_algos.py:351-458, before its whitening.
//
// The batch holds, per request, `len` consecutive rows (the request's trajectory steps, last step first); every row
// has one response per agent (n_agents tensors [B, L_a] of rewards, values and an integer mask whose row sum is the
// number of generated tokens, which sit at the front of the row).  One accumulator walks the whole request: rows in
// batch order, inside a row the agents from the last to the first, inside an agent the tokens from the last
// generated one to the first:
//   last token of an agent:  delta = rew + gamma * V_next - V,  V_next = the next agent's first value in the same row;
//                            for the last agent the first agent's first value in the row before (0 in the first row)
//   any other token:         delta = gamma * V[t + 1] - V[t]          (rewards count at an agent's last token only)
//   gae = delta + (gamma * lam) * gae ;  advantage[t] = gae ;  return[t] = gae + V[t]
// in the reference's float32 operation order (this file is compiled with -ffp-contract=off: no multiply-add is
// fused), so the results are the reference's bit for bit.  The reference does this with a Python loop over every
// token; here one wave owns a request: 64 tokens at a time are loaded and their deltas formed in parallel, then the
// recurrence runs along the 64 lanes in order (a neighbour-to-neighbour shift per step) and the results leave
// coalesced.  Requests are independent, so waves never wait for each other.
#include "common.hpp"

namespace siirl {
namespace {

constexpr int kMaxAgents = SIIRL_MARFT_MAX_AGENTS;
constexpr int kDppWaveShr1 = 0x138;  // DPP control: lane i reads lane i - 1 across the whole wave

struct MarftArgs {
  const float* rew[kMaxAgents];
  const float* val[kMaxAgents];
  const void* mask[kMaxAgents];
  float* adv[kMaxAgents];
  float* ret[kMaxAgents];
  int64_t width[kMaxAgents];
  int64_t B;
  int n_agents, mask_dtype, store_mode;
  float gamma, gamma_lam;
};

// what an assignment into a tensor of the mask's dtype keeps of a float32: itself (float outputs), its integer part
// (integer masks) or whether it is non-zero (bool masks)
__device__ __forceinline__ float stored(float x, int mode) {
  if (mode == SIIRL_MARFT_STORE_TRUNCATED) return truncf(x);
  if (mode == SIIRL_MARFT_STORE_NONZERO) return x != 0.f ? 1.f : 0.f;
  return x;
}

__device__ __forceinline__ int64_t wave_uniform(int64_t x) {  // tells the compiler: the same in every lane
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)x);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)x >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

// What a lane loads for its token: the value, and the value after it or (at the agent's last token) the reward.
struct Fetched {
  float v, other;
};

template <typename M>
__global__ __launch_bounds__(kWave) void marft_gae_kernel(MarftArgs a, const int64_t* __restrict__ chain_start,
                                                          const int64_t* __restrict__ chain_len,
                                                          int32_t* __restrict__ status) {
  const int lane = threadIdx.x;
  const int64_t row0 = wave_uniform(chain_start[blockIdx.x]), len = wave_uniform(chain_len[blockIdx.x]);
  if (row0 < 0 || len <= 0 || row0 + len > a.B) {
    if (lane == 0 && len > 0) atomicMax(status, 2);  // rows outside the batch: nothing of this request is written
    return;
  }
  float gae = 0.f;
  for (int64_t tr = 0; tr < len; ++tr) {
    const int64_t row = row0 + tr;
    for (int ag = a.n_agents - 1; ag >= 0; --ag) {
      const int64_t L = a.width[ag];
      // the row's token count: four loads in flight per lane
      const M* __restrict__ mrow = (const M*)a.mask[ag] + row * L;
      int64_t gen = 0;
      int64_t c = lane;
      for (; c + 3 * kWave < L; c += 4 * kWave) {
        const M m0 = mrow[c], m1 = mrow[c + kWave], m2 = mrow[c + 2 * kWave], m3 = mrow[c + 3 * kWave];
        gen += ((int64_t)m0 + (int64_t)m1) + ((int64_t)m2 + (int64_t)m3);
      }
      for (; c < L; c += kWave) gen += (int64_t)mrow[c];
#pragma unroll
      for (int o = kWave / 2; o > 0; o >>= 1) {
        const int lo = __shfl_xor((int)(uint32_t)gen, o, kWave), hi = __shfl_xor((int)(uint32_t)((uint64_t)gen >> 32), o, kWave);
        gen += (int64_t)(((uint64_t)(uint32_t)hi << 32) | (uint32_t)lo);
      }
      gen = wave_uniform(gen);
      if (gen > L) {  // a mask that is not 0/1: the reference would index past the row
        if (lane == 0) atomicMax(status, 1);
        gen = L;
      }
      if (gen <= 0) continue;
      const float* __restrict__ v = a.val[ag] + row * L;
      const float* __restrict__ r = a.rew[ag] + row * L;
      bool has_next = true;
      float v_after = 0.f;  // the value that follows this agent's last token
      if (ag == a.n_agents - 1) {
        has_next = tr > 0;
        if (has_next) v_after = a.val[0][(row - 1) * a.width[0]];
      } else {
        v_after = a.val[ag + 1][row * a.width[ag + 1]];
      }
      // lane 0 holds the latest token of the block that ends at `top`
      auto fetch = [&](int64_t top) {
        const int64_t t = top - lane;
        Fetched f{0.f, 0.f};
        if (t >= 0) {
          f.v = v[t];
          f.other = t == gen - 1 ? r[t] : v[t + 1];
        }
        return f;
      };
      // Per block of 64 tokens: what the block needs was loaded while the block before it was walked; its results
      // are stored, and the next block's operands loaded, just before the walk, so that every memory operation has a
      // whole walk to complete in before anything waits for it.
      float* __restrict__ adv_row = a.adv[ag] + row * L;
      float* __restrict__ ret_row = a.ret[ag] + row * L;
      const int nblocks = __builtin_amdgcn_readfirstlane((int)((gen + kWave - 1) / kWave));
      Fetched cur = fetch(gen - 1);
      float held_adv = 0.f, held_ret = 0.f;
      int64_t held_t = -1;
      for (int blk = 0; blk < nblocks; ++blk) {
        const int64_t top = gen - 1 - (int64_t)blk * kWave;
        const int64_t t = top - lane;
        float d = 0.f;
        if (t == gen - 1)
          d = has_next ? (cur.other + a.gamma * v_after) - cur.v : cur.other - cur.v;
        else if (t >= 0)
          d = a.gamma * cur.other - cur.v;
        const float v_here = cur.v;
        if (held_t >= 0) {
          adv_row[held_t] = held_adv;
          ret_row[held_t] = held_ret;
        }
        if (blk + 1 < nblocks) cur = fetch(top - kWave);
        const int n = __builtin_amdgcn_readfirstlane((int)(top + 1 < kWave ? top + 1 : kWave));
        // The recurrence along the lanes: every step each lane takes its neighbour's value (lane - 1, a whole-wave
        // shift; lane 0 takes the accumulator carried into the block) and forms d + gamma_lam * that.  After step k
        // the lanes 0 .. k hold their final values, which later steps recompute unchanged; the other lanes hold
        // garbage until their turn.  Two dependent float32 instructions per token, no cross-lane reads of the result.
        // A short last block runs all 64 steps as well (lanes beyond its n tokens are never looked at): no loop control.
        float mine = 0.f;
#pragma unroll
        for (int k = 0; k < kWave; ++k) {
          const float before = u2f((uint32_t)__builtin_amdgcn_update_dpp((int)f2u(gae), (int)f2u(mine), kDppWaveShr1,
                                                                         0xf, 0xf, false));
          mine = d + a.gamma_lam * before;
        }
        gae = u2f((uint32_t)__builtin_amdgcn_readlane((int)f2u(mine), n - 1));
        held_t = t;
        held_adv = stored(mine, a.store_mode);
        held_ret = stored(mine + v_here, a.store_mode);
      }
      if (held_t >= 0) {
        adv_row[held_t] = held_adv;
        ret_row[held_t] = held_ret;
      }
    }
  }
}

__global__ __launch_bounds__(256) void marft_clear_kernel(float* __restrict__ p, float* __restrict__ q, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    p[i] = 0.f;
    q[i] = 0.f;
  }
}
__global__ void marft_clear_status_kernel(int32_t* status) { status[threadIdx.x] = 0; }

}  // namespace
}  // namespace siirl

using namespace siirl;

extern "C" int siirl_marft_gae(const float* const* token_level_rewards, const float* const* values,
                               const void* const* masks, int mask_dtype, const int64_t* widths, int n_agents, int64_t B,
                               const int64_t* chain_start, const int64_t* chain_len, int64_t n_chains, float gamma,
                               float gamma_lam, int store_mode, float* const* advantages, float* const* returns,
                               int32_t* status, siirl_stream_t stream) {
  SIIRL_REQUIRE(n_agents >= 1 && n_agents <= kMaxAgents, "n_agents=%d must lie in [1, %d]", n_agents, kMaxAgents);
  SIIRL_REQUIRE(B >= 0 && n_chains >= 0 && n_chains < (1LL << 31), "B=%lld n_chains=%lld out of range", (long long)B,
                (long long)n_chains);
  SIIRL_REQUIRE(mask_dtype == SIIRL_U8 || mask_dtype == SIIRL_I32 || mask_dtype == SIIRL_I64,
                "the token counts come from an integer mask (uint8 / bool, int32 or int64; dtype %d given)", mask_dtype);
  SIIRL_REQUIRE(store_mode >= SIIRL_MARFT_STORE_FLOAT && store_mode <= SIIRL_MARFT_STORE_NONZERO, "unknown store mode %d",
                store_mode);
  SIIRL_REQUIRE(token_level_rewards && values && masks && widths && advantages && returns && status, "NULL operand");
  SIIRL_REQUIRE(n_chains == 0 || (chain_start && chain_len), "NULL chain list");
  MarftArgs a{};
  a.B = B;
  a.n_agents = n_agents;
  a.mask_dtype = mask_dtype;
  a.store_mode = store_mode;
  a.gamma = gamma;
  a.gamma_lam = gamma_lam;
  for (int g = 0; g < n_agents; ++g) {
    SIIRL_REQUIRE(widths[g] >= 1 && widths[g] < (1LL << 31), "agent %d: row length %lld out of range", g, (long long)widths[g]);
    SIIRL_REQUIRE(B == 0 || (token_level_rewards[g] && values[g] && masks[g] && advantages[g] && returns[g]),
                  "agent %d: NULL operand", g);
    SIIRL_REQUIRE(B * widths[g] < (1LL << 40), "agent %d: %lld x %lld tokens are too many", g, (long long)B, (long long)widths[g]);
    a.rew[g] = token_level_rewards[g];
    a.val[g] = values[g];
    a.mask[g] = masks[g];
    a.adv[g] = advantages[g];
    a.ret[g] = returns[g];
    a.width[g] = widths[g];
  }
  hipStream_t st = (hipStream_t)stream;
  marft_clear_status_kernel<<<1, 1, 0, st>>>(status);
  SIIRL_LAUNCH_CHECK("marft_clear_status_kernel");
  if (B == 0) return SIIRL_OK;
  for (int g = 0; g < n_agents; ++g) {
    const int64_t n = B * widths[g];
    const int64_t want = (n + 255) / 256;
    marft_clear_kernel<<<dim3((unsigned)(want < 4096 ? want : 4096)), dim3(256), 0, st>>>(advantages[g], returns[g], n);
    SIIRL_LAUNCH_CHECK("marft_clear_kernel");
  }
  if (n_chains == 0) return SIIRL_OK;
  const dim3 grid((unsigned)n_chains), block(kWave);
  if (mask_dtype == SIIRL_U8)
    marft_gae_kernel<uint8_t><<<grid, block, 0, st>>>(a, chain_start, chain_len, status);
  else if (mask_dtype == SIIRL_I32)
    marft_gae_kernel<int32_t><<<grid, block, 0, st>>>(a, chain_start, chain_len, status);
  else
    marft_gae_kernel<int64_t><<<grid, block, 0, st>>>(a, chain_start, chain_len, status);
  SIIRL_LAUNCH_CHECK("marft_gae_kernel");
  return SIIRL_OK;
}
