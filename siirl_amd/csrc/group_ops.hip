// Per-prompt group statistics: GRPO outcome advantage and the DAPO dynamic-sampling keep mask.
//
// Replaces compute_grpo_outcome_advantage (siirl/dag_worker/core_algos.py:279-348) and the group test of
// dynamic_sampling (siirl/user_interface/filter_interface/dapo.py:66-93).
//
// Groups are defined by equal uid; uids are arbitrary int64 and need not be contiguous.  Each thread owns
// one trajectory i and visits the members of its group in batch order, so that every group statistic is
// accumulated in the order the reference uses; exact integer bookkeeping, no atomics.  When the uid array is
// non-decreasing (the layout the reference's data loader produces, and what an ascending filter keeps) a
// group is one contiguous run and a thread per trajectory walks just that run: O(B * n); every workgroup checks
// the ordering for itself (O(B) coalesced compares).  Otherwise that kernel only marks its outputs as pending and
// a second kernel gives every trajectory a whole wave: the uids pass through LDS in tiles shared by the 16 waves of
// a workgroup, each lane compares one entry per step, and the few hits of a step are taken in order from the
// ballot -- O(B^2) compares spread over all lanes, same member order, same arithmetic, bit-identical results.
// B is a rollout batch (10^3..10^5).
//
// The keep mask reproduces np.std(values) > 0 bit for bit: numpy sums with an 8-accumulator pairwise
// scheme in the dtype of the values, so e.g. three equal fp64 values 0.1 have std 1.4e-17 > 0.  This
// file is compiled with -ffp-contract=off so that (v - mean)^2 is rounded as numpy rounds it.
#include "common.hpp"
#include "loss_token.hpp"

namespace siirl {
namespace {

constexpr int kThreads = 256;   // streaming kernels (row sums, broadcast)
constexpr int kGroupThreads = 64;  // all-pairs kernels: one wave per workgroup, so B = 8192 already fills 128 CUs

// ---------------------------------------------------------------------------- row sums

// scores[b] = sum_t x[b, t]  (double accumulation, one workgroup per row)
__global__ __launch_bounds__(kThreads) void row_sum_kernel(const float* __restrict__ x, int64_t L,
                                                           float* __restrict__ out) {
  const int64_t b = blockIdx.x;
  const float* r = x + b * L;
  double s = 0.0;
  if (L % 4 == 0 && ((uintptr_t)x & 15) == 0) {  // rows start 16-byte aligned
    const u32x4* r4 = reinterpret_cast<const u32x4*>(r);
    for (int64_t t = threadIdx.x; t < L / 4; t += kThreads) {
      const u32x4 v = __builtin_nontemporal_load(r4 + t);  // read once
      s += ((double)u2f(v.x) + (double)u2f(v.y)) + ((double)u2f(v.z) + (double)u2f(v.w));
    }
  } else {
    for (int64_t t = threadIdx.x; t < L; t += kThreads) s += (double)r[t];
  }
  __shared__ double sh[kThreads / kWave + 1];
  s = block_sum(s, sh);
  if (threadIdx.x == 0) out[b] = (float)s;
}

// true iff uid[0] <= uid[1] <= ... ; evaluated by the whole workgroup (one wave), result uniform
__device__ __forceinline__ bool uid_non_decreasing(const int64_t* __restrict__ uid, int64_t B) {
  int bad = 0;  // no short circuit: the loads of successive iterations stay independent
#pragma unroll 8
  for (int64_t j = threadIdx.x; j + 1 < B; j += kGroupThreads) bad |= (uid[j] > uid[j + 1]) ? 1 : 0;
  return __all(bad == 0);
}
// the run [lo, hi) of positions around i that share uid[i] (uid non-decreasing)
__device__ __forceinline__ void run_of(const int64_t* __restrict__ uid, int64_t B, int64_t i, int64_t& lo, int64_t& hi) {
  const int64_t my = uid[i];
  lo = i;
  while (lo > 0 && uid[lo - 1] == my) --lo;
  hi = i + 1;
  while (hi < B && uid[hi] == my) ++hi;
}


// ---------------------------------------------------------------------------- GRPO advantage

constexpr uint32_t kPendingBits = 0x7fc0deadu;  // a NaN no arithmetic here produces: "left to the wave kernel"
constexpr uint8_t kPendingKeep = 2;
constexpr int kWaveThreads = 1024;                // wave-per-trajectory kernels: 16 trajectories per workgroup
constexpr int kWaveTile = 4096;                   // uids staged per step (32 KB of LDS)

__device__ __forceinline__ float grpo_value(double s, double mean, double sd, float eps, int norm_by_std) {
  // the reference evaluates (s - mean) / (std + eps) on fp32 0-d tensors; round the pieces likewise
  const float num = (float)s - (float)mean;
  return norm_by_std ? num / ((float)sd + eps) : num;
}

// a[i] = (s_i - mean_g) / (std_g + eps), unbiased std; a group of one uses mean 0, std 1.  Thread per trajectory
// over contiguous runs; when the uids are not non-decreasing every output is marked pending instead.
__global__ __launch_bounds__(kGroupThreads) void grpo_group_kernel(const float* __restrict__ scores,
                                                              const int64_t* __restrict__ uid, int64_t B, float eps,
                                                              int norm_by_std, float* __restrict__ a_out) {
  const int64_t i = (int64_t)blockIdx.x * kGroupThreads + threadIdx.x;
  const bool runs = uid_non_decreasing(uid, B);
  if (i >= B) return;
  if (!runs) {
    a_out[i] = u2f(kPendingBits);
    return;
  }
  int64_t lo, hi;
  run_of(uid, B, i, lo, hi);
  const int n = (int)(hi - lo);
  double sum = 0.0;
  for (int64_t j = lo; j < hi; ++j) sum += (double)scores[j];
  const double mean = n > 1 ? sum / (double)n : 0.0;
  double ss = 0.0;
  if (n > 1)
    for (int64_t j = lo; j < hi; ++j) {
      const double d = (double)scores[j] - mean;
      ss += d * d;
    }
  const double sd = n > 1 ? sqrt(ss / (double)(n - 1)) : 1.0;
  a_out[i] = grpo_value((double)scores[i], mean, sd, eps, norm_by_std);
}

// Stages uid[base, base + kWaveTile) into LDS (all threads of the workgroup), then calls f(j) on the calling wave for
// every j in the tile with uid[j] == my, in ascending order.  Every lane of the wave sees the same sequence of j.
template <typename F>
__device__ __forceinline__ void wave_members(const int64_t* __restrict__ uid, int64_t B, int64_t my, bool active,
                                             int64_t* s_uid, F&& f) {
  const int lane = threadIdx.x & (kWave - 1);
  for (int64_t base = 0; base < B; base += kWaveTile) {
    __syncthreads();
    for (int k = threadIdx.x; k < kWaveTile; k += kWaveThreads) s_uid[k] = base + k < B ? uid[base + k] : 0;
    __syncthreads();
    const int lim = (int)((B - base) < kWaveTile ? (B - base) : kWaveTile);
    if (active)
      for (int k0 = 0; k0 < lim; k0 += kWave) {
        const int k = k0 + lane;
        unsigned long long bal = __ballot(k < lim && s_uid[k] == my);
        while (bal) {
          const int l = __builtin_ctzll(bal);
          bal &= bal - 1;
          f(base + k0 + l);
        }
      }
  }
}

// The pending outputs of grpo_group_kernel: one wave per trajectory.
__global__ __launch_bounds__(kWaveThreads) void grpo_group_wave_kernel(const float* __restrict__ scores,
                                                                        const int64_t* __restrict__ uid, int64_t B,
                                                                        float eps, int norm_by_std,
                                                                        float* __restrict__ a_out) {
  __shared__ int64_t s_uid[kWaveTile];
  const int64_t i = (int64_t)blockIdx.x * (kWaveThreads / kWave) + threadIdx.x / kWave;
  const bool active = i < B && f2u(a_out[i]) == kPendingBits;
  if (!__syncthreads_or(active ? 1 : 0)) return;  // ordered uids: the first kernel has done everything
  const int64_t my = active ? uid[i] : 0;
  int n = 0;
  double sum = 0.0;
  wave_members(uid, B, my, active, s_uid, [&](int64_t j) {
    ++n;
    sum += (double)scores[j];
  });
  const double mean = n > 1 ? sum / (double)n : 0.0;
  double ss = 0.0;
  if (__syncthreads_or((active && n > 1) ? 1 : 0))
    wave_members(uid, B, my, active && n > 1, s_uid, [&](int64_t j) {
      const double d = (double)scores[j] - mean;
      ss += d * d;
    });
  if (!active) return;
  const double sd = n > 1 ? sqrt(ss / (double)(n - 1)) : 1.0;
  if ((threadIdx.x & (kWave - 1)) == 0) a_out[i] = grpo_value((double)scores[i], mean, sd, eps, norm_by_std);
}

// out[b, t] = a[b] * mask[b, t]; one workgroup per 4096-token segment of a row, four tokens per access
constexpr int kBcastSeg = 4096;
__global__ __launch_bounds__(kThreads) void broadcast_mask_kernel(const float* __restrict__ a, const void* mask,
                                                                  int mask_dtype, int64_t L, int nseg, int vec,
                                                                  float* __restrict__ out) {
  const int64_t b = blockIdx.x / nseg;
  const int64_t t0 = (int64_t)(blockIdx.x % nseg) * kBcastSeg;
  const float ab = a[b];
  for (int q = threadIdx.x; q < kBcastSeg / 4; q += kThreads) {
    const int64_t t = t0 + 4 * q;
    if (t >= L) break;
    const int nv = (int)((L - t) < 4 ? (L - t) : 4);
    const int64_t idx = b * L + t;
    tok::Quad m4 = tok::load_mask_quad(mask, mask_dtype, idx, vec != 0, nv);
#pragma unroll
    for (int e = 0; e < 4; ++e) m4.v[e] = ab * m4.v[e];
    tok::store_quad(out, idx, vec != 0, nv, m4);
  }
}

// ---------------------------------------------------------------------------- numpy pairwise sum

// Streaming restatement of numpy's pairwise_sum for one block of n <= 128 values fed in order.
template <typename T>
struct NpBlock {
  T r0, r1, r2, r3, r4, r5, r6, r7, res;
  int n, nb, k;
  __device__ void begin(int n_) {
    n = n_;
    nb = n < 8 ? 0 : n - (n % 8);
    k = 0;
    r0 = r1 = r2 = r3 = r4 = r5 = r6 = r7 = T(0);
    res = T(0);
  }
  __device__ T fold() const { return ((r0 + r1) + (r2 + r3)) + ((r4 + r5) + (r6 + r7)); }
  __device__ void push(T v) {
    if (k < nb) {
      switch (k & 7) {
        case 0: r0 += v; break;
        case 1: r1 += v; break;
        case 2: r2 += v; break;
        case 3: r3 += v; break;
        case 4: r4 += v; break;
        case 5: r5 += v; break;
        case 6: r6 += v; break;
        default: r7 += v;
      }
    } else {
      if (k == nb && nb > 0) res = fold();
      res += v;
    }
    ++k;
  }
  __device__ T finish() const { return (nb > 0 && n == nb) ? fold() : res; }
};

// Pull-style iterator over the members of uid `my`, in batch order, from global memory.
template <typename T>
struct MemberCursor {
  const int64_t* uid;
  const T* val;
  int64_t B, j;
  int64_t my;
  __device__ T next() {
    while (j < B && uid[j] != my) ++j;
    return val[j++];
  }
};

// numpy's pairwise_sum over n members with an optional transform (v - mean)^2; explicit stack instead of
// recursion.  Leaves hold at most 128 values; n2 = n/2 rounded down to a multiple of 8.
template <typename T, bool SQDEV>
__device__ T np_pairwise(MemberCursor<T>& cur, int n, T mean) {
  struct Frame {
    int n, stage;
    T left;
  };
  Frame st[40];
  int sp = 0;
  st[0] = {n, 0, T(0)};
  T ret = T(0);
  while (sp >= 0) {
    Frame& f = st[sp];
    if (f.n <= 128) {
      NpBlock<T> blk;
      blk.begin(f.n);
      for (int q = 0; q < f.n; ++q) {
        T v = cur.next();
        if (SQDEV) {
          const T d = v - mean;
          v = d * d;
        }
        blk.push(v);
      }
      ret = blk.finish();
      --sp;
      while (sp >= 0) {
        Frame& p = st[sp];
        if (p.stage == 1) {  // left child done: run the right child
          p.left = ret;
          p.stage = 2;
          int n2 = p.n / 2;
          n2 -= n2 % 8;
          st[++sp] = {p.n - n2, 0, T(0)};
          break;
        }
        ret = p.left + ret;  // right child done
        --sp;
      }
    } else {
      f.stage = 1;
      int n2 = f.n / 2;
      n2 -= n2 % 8;
      st[++sp] = {n2, 0, T(0)};
    }
  }
  return ret;
}

// keep[i] = group of i has one member, or np.std(group values) > 0.  Thread per trajectory over contiguous runs;
// when the uids are not non-decreasing every output is marked pending instead.
template <typename T>
__global__ __launch_bounds__(kGroupThreads) void keep_mask_kernel(const T* __restrict__ val, const int64_t* __restrict__ uid,
                                                             int64_t B, uint8_t* __restrict__ keep,
                                                             int32_t* __restrict__ group_size) {
  const int64_t i = (int64_t)blockIdx.x * kGroupThreads + threadIdx.x;
  const bool runs = uid_non_decreasing(uid, B);
  if (i >= B) return;
  if (!runs) {
    keep[i] = kPendingKeep;
    return;
  }
  const int64_t my = uid[i];
  int64_t lo, hi;
  run_of(uid, B, i, lo, hi);
  const int n = (int)(hi - lo);
  T mean, ssq;
  if (n <= 128) {
    NpBlock<T> blk;
    blk.begin(n);
    if (n > 1)
      for (int64_t j = lo; j < hi; ++j) blk.push(val[j]);
    mean = blk.finish() / (T)n;
    blk.begin(n);
    if (n > 1)
      for (int64_t j = lo; j < hi; ++j) {
        const T d = val[j] - mean;
        blk.push(d * d);
      }
    ssq = blk.finish();
  } else {
    MemberCursor<T> c1{uid, val, B, lo, my};
    mean = np_pairwise<T, false>(c1, n, T(0)) / (T)n;
    MemberCursor<T> c2{uid, val, B, lo, my};
    ssq = np_pairwise<T, true>(c2, n, mean);
  }
  const T sd = sqrt(ssq / (T)n);
  keep[i] = (n == 1 || sd > T(0)) ? 1 : 0;
  if (group_size) group_size[i] = n;
}

// The pending outputs of keep_mask_kernel: one wave per trajectory, members visited in batch order.
template <typename T>
__global__ __launch_bounds__(kWaveThreads) void keep_mask_wave_kernel(const T* __restrict__ val,
                                                                       const int64_t* __restrict__ uid, int64_t B,
                                                                       uint8_t* __restrict__ keep,
                                                                       int32_t* __restrict__ group_size) {
  __shared__ int64_t s_uid[kWaveTile];
  const int64_t i = (int64_t)blockIdx.x * (kWaveThreads / kWave) + threadIdx.x / kWave;
  const bool active = i < B && keep[i] == kPendingKeep;
  if (!__syncthreads_or(active ? 1 : 0)) return;  // ordered uids: the first kernel has done everything
  const int64_t my = active ? uid[i] : 0;
  int n = 0;
  wave_members(uid, B, my, active, s_uid, [&](int64_t) { ++n; });
  const bool small = n <= 128;
  T mean = T(0), ssq = T(0);
  NpBlock<T> blk;
  blk.begin(small ? n : 0);
  if (__syncthreads_or((active && small && n > 1) ? 1 : 0)) {
    wave_members(uid, B, my, active && small && n > 1, s_uid, [&](int64_t j) { blk.push(val[j]); });
    mean = blk.finish() / (T)n;
    blk.begin(small ? n : 0);
    wave_members(uid, B, my, active && small && n > 1, s_uid, [&](int64_t j) {
      const T d = val[j] - mean;
      blk.push(d * d);
    });
    ssq = blk.finish();
  }
  if (!active) return;
  if (!small) {  // rare: groups of more than 128, numpy recurses; every lane walks the same members
    MemberCursor<T> c1{uid, val, B, 0, my};
    mean = np_pairwise<T, false>(c1, n, T(0)) / (T)n;
    MemberCursor<T> c2{uid, val, B, 0, my};
    ssq = np_pairwise<T, true>(c2, n, mean);
  }
  const T sd = sqrt(ssq / (T)n);
  if ((threadIdx.x & (kWave - 1)) == 0) {
    keep[i] = (n == 1 || sd > T(0)) ? 1 : 0;
    if (group_size) group_size[i] = n;
  }
}

}  // namespace
}  // namespace siirl

using namespace siirl;

extern "C" int siirl_grpo_outcome_advantage(const float* token_level_rewards, const void* mask, int mask_dtype,
                                            const int64_t* uid, int64_t B, int64_t L, float epsilon,
                                            int norm_adv_by_std, float* advantages, float* scratch_2B,
                                            siirl_stream_t stream) {
  SIIRL_REQUIRE(B >= 0 && L >= 1, "B=%lld L=%lld out of range", (long long)B, (long long)L);
  if (B == 0) return SIIRL_OK;
  SIIRL_REQUIRE(B <= 0x7fffffffLL, "B too large");
  SIIRL_REQUIRE(token_level_rewards && mask && uid && advantages && scratch_2B, "NULL operand");
  SIIRL_REQUIRE(mask_dtype == SIIRL_U8 || mask_dtype == SIIRL_I64 || mask_dtype == SIIRL_I32 ||
                    mask_dtype == SIIRL_F32 || mask_dtype == SIIRL_BF16 || mask_dtype == SIIRL_F16,
                "mask dtype %d not supported", mask_dtype);
  hipStream_t st = (hipStream_t)stream;
  float* scores = scratch_2B;
  float* a = scratch_2B + B;
  row_sum_kernel<<<dim3((unsigned)B), dim3(kThreads), 0, st>>>(token_level_rewards, L, scores);
  SIIRL_LAUNCH_CHECK("row_sum_kernel");
  grpo_group_kernel<<<dim3((unsigned)((B + kGroupThreads - 1) / kGroupThreads)), dim3(kGroupThreads), 0, st>>>(
      scores, uid, B, epsilon, norm_adv_by_std, a);
  SIIRL_LAUNCH_CHECK("grpo_group_kernel");
  constexpr int kPerWg = kWaveThreads / kWave;
  grpo_group_wave_kernel<<<dim3((unsigned)((B + kPerWg - 1) / kPerWg)), dim3(kWaveThreads), 0, st>>>(
      scores, uid, B, epsilon, norm_adv_by_std, a);
  SIIRL_LAUNCH_CHECK("grpo_group_wave_kernel");
  const int64_t nseg = (L + kBcastSeg - 1) / kBcastSeg;
  SIIRL_REQUIRE(B * nseg <= 0x7fffffffLL, "B=%lld x L=%lld exceeds the launch grid", (long long)B, (long long)L);
  const size_t mask_es = dtype_size(mask_dtype);
  const bool vec = L % 4 == 0 && ((uintptr_t)advantages & 15) == 0 &&
                   ((uintptr_t)mask % (mask_es * 4 < 16 ? mask_es * 4 : 16)) == 0;
  broadcast_mask_kernel<<<dim3((unsigned)(B * nseg)), dim3(kThreads), 0, st>>>(a, mask, mask_dtype, L, (int)nseg,
                                                                              vec ? 1 : 0, advantages);
  SIIRL_LAUNCH_CHECK("broadcast_mask_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_group_keep_mask(const void* metric, int metric_dtype, const int64_t* uid, int64_t B,
                                     uint8_t* keep, int32_t* group_size, siirl_stream_t stream) {
  SIIRL_REQUIRE(B >= 0 && B <= 0x7fffffffLL, "B=%lld out of range", (long long)B);
  if (B == 0) return SIIRL_OK;
  SIIRL_REQUIRE(metric && uid && keep, "NULL operand");
  SIIRL_REQUIRE(metric_dtype == SIIRL_F32 || metric_dtype == SIIRL_F64, "metric dtype %d not supported (f32, f64)",
                metric_dtype);
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)((B + kGroupThreads - 1) / kGroupThreads)), block(kGroupThreads);
  constexpr int kPerWg = kWaveThreads / kWave;
  const dim3 wgrid((unsigned)((B + kPerWg - 1) / kPerWg)), wblock(kWaveThreads);
  if (metric_dtype == SIIRL_F32) {
    keep_mask_kernel<float><<<grid, block, 0, st>>>((const float*)metric, uid, B, keep, group_size);
    SIIRL_LAUNCH_CHECK("keep_mask_kernel");
    keep_mask_wave_kernel<float><<<wgrid, wblock, 0, st>>>((const float*)metric, uid, B, keep, group_size);
  } else {
    keep_mask_kernel<double><<<grid, block, 0, st>>>((const double*)metric, uid, B, keep, group_size);
    SIIRL_LAUNCH_CHECK("keep_mask_kernel");
    keep_mask_wave_kernel<double><<<wgrid, wblock, 0, st>>>((const double*)metric, uid, B, keep, group_size);
  }
  SIIRL_LAUNCH_CHECK("keep_mask_wave_kernel");
  return SIIRL_OK;
}
