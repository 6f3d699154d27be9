// The k largest entries of a [n] fp32 score vector, marked in place of torch.topk + scatter: KL-Cov gives the
// max(1, int(n_valid * kl_cov_ratio)) tokens of largest covariance an extra KL term
// (siirl/dag_worker/core_algos.py:1055-1063: torch.topk(cov, k).indices, then an indexed assignment).
//
// Radix select on an order-preserving 32-bit key, three histogram passes (11 + 11 + 10 bits from the top), each a
// streaming read of the scores; a workgroup keeps eight copies of the 2048-bin histogram in LDS (lanes spread over
// them) and adds its non-empty bins to the pass's histogram in memory (integer atomics: the sums are exact whatever
// the order), one workgroup walks down from the top bin to the one that holds the k-th largest.  After the third
// pass the cut is a single key value: entries above it are taken; of the entries equal to it as many as are still
// missing, lowest index first (counted per chunk, then ranked inside each chunk with a scan).  The same input marks
// the same tokens on every run.
// NaN sorts above everything, as for torch.topk; -0 and +0 are one value.
#include "common.hpp"

namespace siirl {
namespace {

constexpr int kSelThreads = 1024;
constexpr int kSelGrid = 256;  // one workgroup per compute unit
constexpr int kBins = 2048;
constexpr int kCopies = 8;     // LDS copies of the histogram: 64 KB
constexpr int kTile = kSelThreads * 4;

struct SelState {
  uint32_t prefix;      // key bits fixed so far (from the top)
  uint32_t need;        // how many of the entries that match the prefix are still to be taken
  uint32_t ties_total;  // after the last pass: entries equal to the cut
  uint32_t pad;
};

__device__ __forceinline__ uint32_t key_of(float v) {
  uint32_t u = f2u(v);
  if (v != v) return 0xffffffffu;
  if (u == 0x80000000u) u = 0u;
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// chunk of workgroup w: [w * per, min(n, (w + 1) * per)), per a multiple of the tile
__device__ __forceinline__ void chunk_of(int64_t n, int64_t per, int64_t& lo, int64_t& hi) {
  lo = (int64_t)blockIdx.x * per;
  hi = lo + per < n ? lo + per : n;
  if (lo > n) lo = n;
}

// Access mode of a launch: bit 0 = 16-byte accesses (aligned operands), bit 1 = non-temporal loads.  The passes of
// one call read the same vector up to five times: one that fits the memory-side cache is read with ordinary loads
// so that the later passes find it there (three histogram passes over 180 MB: 94.5 -> 89.6 us), a larger one
// streams past the caches.  The marks are always stored non-temporally: ordinary stores made this kernel 9 us
// faster and the loss kernel that runs next 33 us slower (it then shares the memory with their write-back).
constexpr int kVec = 1, kNt = 2;
__device__ __forceinline__ u32x4 load16(const float* __restrict__ p, bool nt) {
  return nt ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)) : *reinterpret_cast<const u32x4*>(p);
}

// four consecutive scores from index i (a multiple of 4 when vec); entries at or beyond hi are reported as absent
__device__ __forceinline__ int load4(const float* __restrict__ x, int64_t i, int64_t hi, int mode, float (&v)[4]) {
  if (i + 4 <= hi && (mode & kVec)) {
    const u32x4 t = load16(x + i, (mode & kNt) != 0);
    v[0] = u2f(t.x); v[1] = u2f(t.y); v[2] = u2f(t.z); v[3] = u2f(t.w);
    return 4;
  }
  int c = 0;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if (i + e < hi) {
      v[e] = x[i + e];
      c = e + 1;
    }
  return c;
}

// PASS 0: bins are key bits 31..21; PASS 1: bits 20..10 of the keys whose top 11 bits equal the prefix; PASS 2: bits
// 9..0 of the keys whose top 22 bits do.
template <int PASS>
__global__ __launch_bounds__(kSelThreads) void select_hist_kernel(const float* __restrict__ x, int64_t n, int64_t per,
                                                                  int mode, const SelState* __restrict__ st,
                                                                  uint32_t* __restrict__ ghist) {
  __shared__ uint32_t hist[kCopies][kBins];
  for (int i = threadIdx.x; i < kCopies * kBins; i += kSelThreads) (&hist[0][0])[i] = 0u;
  __syncthreads();
  const uint32_t prefix = PASS == 0 ? 0u : st->prefix;
  uint32_t* mine = hist[threadIdx.x & (kCopies - 1)];
  int64_t lo, hi;
  chunk_of(n, per, lo, hi);
  auto count = [&](float val) {
    const uint32_t k = key_of(val);
    uint32_t bin;
    bool counted = true;
    if (PASS == 0) {
      bin = k >> 21;
    } else if (PASS == 1) {
      bin = (k >> 10) & 2047u;
      counted = (k >> 21) == (prefix >> 21);
    } else {
      bin = k & 1023u;
      counted = (k >> 10) == (prefix >> 10);
    }
    if (counted) {
      // a wave whose entries all fall into one bin (a masked stretch: all -inf) adds once
      const uint32_t b0 = __builtin_amdgcn_readfirstlane(bin);
      const uint64_t all = __ballot(1), same = __ballot(bin == b0);
      if (same == all) {
        if ((int)(threadIdx.x & (kWave - 1)) == __ffsll((unsigned long long)all) - 1)
          atomicAdd(&mine[b0], (uint32_t)__popcll(all));
      } else {
        atomicAdd(&mine[bin], 1u);
      }
    }
  };
  // whole tiles, four 16-byte loads in flight per thread; then what is left, one (possibly partial) vector at a time
  constexpr int kInFlight = 4;
  int64_t i = lo + 4 * (int64_t)threadIdx.x;
  if (mode & kVec) {
    const bool nt = (mode & kNt) != 0;
    for (; i + (int64_t)(kInFlight - 1) * kTile + 4 <= hi; i += (int64_t)kInFlight * kTile) {
      u32x4 t[kInFlight];
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) t[u] = load16(x + i + (int64_t)u * kTile, nt);
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        count(u2f(t[u].x));
        count(u2f(t[u].y));
        count(u2f(t[u].z));
        count(u2f(t[u].w));
      }
    }
  }
  for (; i < hi; i += kTile) {
    float v[4];
    const int c = load4(x, i, hi, mode, v);
    if (c > 0) count(v[0]);
    if (c > 1) count(v[1]);
    if (c > 2) count(v[2]);
    if (c > 3) count(v[3]);
  }
  __syncthreads();
  for (int b = threadIdx.x; b < kBins; b += kSelThreads) {
    uint32_t s = 0;
#pragma unroll
    for (int c = 0; c < kCopies; ++c) s += hist[c][b];
    if (s) atomicAdd(&ghist[PASS * kBins + b], s);
  }
}

// Finds, from the top bin of the pass's histogram down, the bin in which the running count reaches `need`.
template <int PASS>
__global__ __launch_bounds__(kSelThreads) void select_scan_kernel(const uint32_t* __restrict__ ghist, uint32_t k_first,
                                                                  SelState* __restrict__ st) {
  __shared__ uint32_t cnt[kBins];
  __shared__ uint32_t wsum[kSelThreads / kWave];
  for (int b = threadIdx.x; b < kBins; b += kSelThreads) cnt[b] = ghist[PASS * kBins + b];
  __syncthreads();
  // thread t owns bins 2t (lower) and 2t + 1; above(t) = entries in bins beyond 2t + 1
  const int t = threadIdx.x;
  const uint32_t c0 = cnt[2 * t], c1 = cnt[2 * t + 1];
  const uint32_t own = c0 + c1;
  const int lane = t & (kWave - 1), w = t / kWave;
  uint32_t incl = own;  // suffix sum inside the wave: this lane and the lanes above it
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const uint32_t up = __shfl_down(incl, o, kWave);
    if (lane + o < kWave) incl += up;
  }
  if (lane == 0) wsum[w] = incl;
  __syncthreads();
  uint32_t above = incl - own;
  for (int q = w + 1; q < kSelThreads / kWave; ++q) above += wsum[q];
  const uint32_t need = PASS == 0 ? k_first : st->need;
  const uint32_t prefix = PASS == 0 ? 0u : st->prefix;
  __syncthreads();  // every thread has read the state before one of them rewrites it
  int bin = -1;
  uint32_t before = 0;
  if (above < need && need <= above + c1) {
    bin = 2 * t + 1;
    before = above;
  } else if (above + c1 < need && need <= above + own) {
    bin = 2 * t;
    before = above + c1;
  }
  if (bin >= 0) {
    const int shift = PASS == 0 ? 21 : (PASS == 1 ? 10 : 0);
    st->prefix = prefix | ((uint32_t)bin << shift);
    st->need = need - before;
    st->ties_total = cnt[bin];
  }
}

// per chunk: entries equal to the cut.  Skipped (zeros) when every such entry is taken anyway.
__global__ __launch_bounds__(kSelThreads) void select_count_ties_kernel(const float* __restrict__ x, int64_t n, int64_t per,
                                                                        int mode, const SelState* __restrict__ st,
                                                                        uint32_t* __restrict__ ties) {
  __shared__ double sh[kSelThreads / kWave + 1];
  uint32_t c = 0;
  if (st->need != st->ties_total) {
    const uint32_t cut = st->prefix;
    int64_t lo, hi;
    chunk_of(n, per, lo, hi);
    for (int64_t i = lo + 4 * (int64_t)threadIdx.x; i < hi; i += kTile) {
      float v[4];
      const int m = load4(x, i, hi, mode, v);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (e < m) c += key_of(v[e]) == cut ? 1u : 0u;
    }
  }
  const double total = block_sum((double)c, sh);  // exact: a chunk holds fewer than 2^32 entries
  if (threadIdx.x == 0) ties[blockIdx.x] = (uint32_t)total;
}

__global__ __launch_bounds__(kSelThreads) void select_clear_kernel(float* __restrict__ aux, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * kSelThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kSelThreads) aux[i] = 0.f;
}
__global__ __launch_bounds__(kSelThreads) void select_init_kernel(uint32_t* __restrict__ ghist) {
  ghist[blockIdx.x * kSelThreads + threadIdx.x] = 0u;  // grid: 3 * kBins / kSelThreads workgroups
}

// aux[i] = coef where the entry is taken, 0 elsewhere
__global__ __launch_bounds__(kSelThreads) void select_mark_kernel(const float* __restrict__ x, int64_t n, int64_t per, int mode,
                                                                  const SelState* __restrict__ st,
                                                                  const uint32_t* __restrict__ ties, float coef,
                                                                  float* __restrict__ aux) {
  __shared__ uint32_t wsum[kSelThreads / kWave];
  __shared__ uint32_t run;
  const uint32_t cut = st->prefix, quota = st->need;
  const bool all_ties = st->need == st->ties_total;
  uint32_t base = 0;  // entries equal to the cut in the chunks before this one
  if (!all_ties)
    for (int b = 0; b < (int)blockIdx.x; ++b) base += ties[b];
  if (threadIdx.x == 0) run = base;
  __syncthreads();
  int64_t lo, hi;
  chunk_of(n, per, lo, hi);
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  for (int64_t t0 = lo; t0 < hi; t0 += kTile) {  // every thread runs every tile: the barriers below are uniform
    const int64_t i = t0 + 4 * (int64_t)threadIdx.x;
    float v[4];
    const int m = i < hi ? load4(x, i, hi, mode, v) : 0;
    uint32_t key[4] = {0u, 0u, 0u, 0u};
    uint32_t mine = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (e < m) {
        key[e] = key_of(v[e]);
        mine += key[e] == cut ? 1u : 0u;
      }
    uint32_t first = 0;  // rank, among all entries equal to the cut, of this thread's first one
    if (!all_ties) {
      uint32_t incl = mine;
#pragma unroll
      for (int o = 1; o < kWave; o <<= 1) {
        const uint32_t dn = __shfl_up(incl, o, kWave);
        if (lane >= o) incl += dn;
      }
      if (lane == kWave - 1) wsum[w] = incl;
      __syncthreads();
      uint32_t before = run;
      for (int q = 0; q < w; ++q) before += wsum[q];
      first = before + incl - mine;
      uint32_t tile_total = 0;
      for (int q = 0; q < kSelThreads / kWave; ++q) tile_total += wsum[q];
      __syncthreads();
      if (threadIdx.x == 0) run += tile_total;
      __syncthreads();
    }
    float out[4];
    uint32_t r = first;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      bool take = key[e] > cut;
      if (e < m && key[e] == cut) {
        take = all_ties || r < quota;
        ++r;
      }
      out[e] = take ? coef : 0.f;
    }
    if (m == 4 && (mode & kVec)) {
      const u32x4 o{f2u(out[0]), f2u(out[1]), f2u(out[2]), f2u(out[3])};
      __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(aux + i));  // (see kNt: stores always)
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (e < m) aux[i + e] = out[e];
    }
  }
}

// ------------------------------------------------------------------------------ entries inside an open interval

// Clip-Cov's candidate list (siirl/dag_worker/core_algos.py:974-975: nonzero of lb < cov < ub): first the number of
// such entries per chunk, then their flat indices in ascending order, each chunk writing behind the chunks before it
// and ranking its own entries tile by tile with a scan.
__global__ __launch_bounds__(kSelThreads) void range_count_kernel(const float* __restrict__ x, int64_t n, int64_t per, int mode,
                                                                  float lo_open, float hi_open,
                                                                  uint32_t* __restrict__ counts) {
  __shared__ double sh[kSelThreads / kWave + 1];
  int64_t lo, hi;
  chunk_of(n, per, lo, hi);
  uint32_t c = 0;
  for (int64_t i = lo + 4 * (int64_t)threadIdx.x; i < hi; i += kTile) {
    float v[4];
    const int m = load4(x, i, hi, mode, v);
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (e < m) c += (v[e] > lo_open && v[e] < hi_open) ? 1u : 0u;
  }
  const double total = block_sum((double)c, sh);
  if (threadIdx.x == 0) counts[blockIdx.x] = (uint32_t)total;
}
// counts[grid] = the sum of the chunk counts (one workgroup)
__global__ __launch_bounds__(kSelGrid) void range_total_kernel(uint32_t* __restrict__ counts, int grid,
                                                               uint32_t* __restrict__ total) {
  __shared__ double sh[kSelGrid / kWave + 1];
  const double t = block_sum(threadIdx.x < (unsigned)grid ? (double)counts[threadIdx.x] : 0.0, sh);
  if (threadIdx.x == 0) {
    counts[grid] = (uint32_t)t;
    *total = (uint32_t)t;
  }
}
__global__ __launch_bounds__(kSelThreads) void range_write_kernel(const float* __restrict__ x, int64_t n, int64_t per, int mode,
                                                                  float lo_open, float hi_open,
                                                                  const uint32_t* __restrict__ counts,
                                                                  int64_t* __restrict__ indices, int64_t capacity) {
  __shared__ uint32_t wsum[kSelThreads / kWave];
  __shared__ uint32_t run;
  uint32_t base = 0;
  for (int b = 0; b < (int)blockIdx.x; ++b) base += counts[b];
  if (threadIdx.x == 0) run = base;
  __syncthreads();
  int64_t lo, hi;
  chunk_of(n, per, lo, hi);
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  for (int64_t t0 = lo; t0 < hi; t0 += kTile) {  // every thread runs every tile: the barriers are uniform
    const int64_t i = t0 + 4 * (int64_t)threadIdx.x;
    float v[4];
    const int m = i < hi ? load4(x, i, hi, mode, v) : 0;
    bool in[4];
    uint32_t mine = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      in[e] = e < m && v[e] > lo_open && v[e] < hi_open;
      mine += in[e] ? 1u : 0u;
    }
    uint32_t incl = mine;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const uint32_t dn = __shfl_up(incl, o, kWave);
      if (lane >= o) incl += dn;
    }
    if (lane == kWave - 1) wsum[w] = incl;
    __syncthreads();
    uint32_t r = run + incl - mine;
    for (int q = 0; q < w; ++q) r += wsum[q];
    uint32_t tile_total = 0;
    for (int q = 0; q < kSelThreads / kWave; ++q) tile_total += wsum[q];
    __syncthreads();
    if (threadIdx.x == 0) run += tile_total;
    __syncthreads();
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (in[e]) {
        if ((int64_t)r < capacity) indices[r] = i + e;  // (the scores changed since they were counted: no write past the end)
        ++r;
      }
  }
}

int access_mode(bool aligned, int64_t n) {
  return (aligned ? kVec : 0) | (streams_past_cache(4.0 * (double)n) ? kNt : 0);
}

struct SelWs {
  size_t part, state, ties, total;
};
SelWs sel_ws() {
  SelWs w;
  w.part = 0;  // three histograms, one per pass
  w.state = (size_t)3 * kBins * sizeof(uint32_t);
  w.ties = w.state + 256;
  w.total = w.ties + (size_t)kSelGrid * sizeof(uint32_t);
  return w;
}

}  // namespace
}  // namespace siirl

using namespace siirl;

// chunk layout shared by the interval pair: `per` entries per workgroup, `grid` workgroups
static void range_chunks(int64_t n, int64_t& per, int& grid) {
  per = ((n + kSelGrid - 1) / kSelGrid + kTile - 1) / kTile * kTile;
  grid = (int)((n + per - 1) / per);
}

extern "C" size_t siirl_range_select_workspace_bytes(void) { return (size_t)(kSelGrid + 1) * sizeof(uint32_t); }

extern "C" int siirl_range_select_count(const float* scores, int64_t n, float lower_open, float upper_open,
                                        uint32_t* count, void* workspace, size_t workspace_bytes, siirl_stream_t stream) {
  SIIRL_REQUIRE(n >= 0 && n < (1LL << 32), "n=%lld out of range (below 2^32)", (long long)n);
  SIIRL_REQUIRE(count != nullptr && (n == 0 || scores != nullptr), "NULL operand");
  if (workspace == nullptr || workspace_bytes < siirl_range_select_workspace_bytes())
    return fail(SIIRL_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes,
                siirl_range_select_workspace_bytes());
  SIIRL_REQUIRE(((uintptr_t)workspace & 3) == 0 && ((uintptr_t)count & 3) == 0, "workspace and count must be 4-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  uint32_t* counts = (uint32_t*)workspace;
  int64_t per = kTile;
  int grid = 0;
  if (n > 0) {
    range_chunks(n, per, grid);
    const int mode = access_mode(((uintptr_t)scores & 15) == 0, n);
    range_count_kernel<<<dim3((unsigned)grid), dim3(kSelThreads), 0, st>>>(scores, n, per, mode, lower_open, upper_open, counts);
    SIIRL_LAUNCH_CHECK("range_count_kernel");
  }
  range_total_kernel<<<1, dim3(kSelGrid), 0, st>>>(counts, grid, count);
  SIIRL_LAUNCH_CHECK("range_total_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_range_select_write(const float* scores, int64_t n, float lower_open, float upper_open,
                                        const void* workspace, int64_t* indices, int64_t capacity,
                                        siirl_stream_t stream) {
  SIIRL_REQUIRE(n >= 0 && n < (1LL << 32) && capacity >= 0, "n=%lld (below 2^32) or capacity=%lld out of range",
                (long long)n, (long long)capacity);
  if (n == 0 || capacity == 0) return SIIRL_OK;
  SIIRL_REQUIRE(scores && workspace && indices, "NULL operand");
  int64_t per;
  int grid;
  range_chunks(n, per, grid);
  const int mode = access_mode(((uintptr_t)scores & 15) == 0, n);
  range_write_kernel<<<dim3((unsigned)grid), dim3(kSelThreads), 0, (hipStream_t)stream>>>(
      scores, n, per, mode, lower_open, upper_open, (const uint32_t*)workspace, indices, capacity);
  SIIRL_LAUNCH_CHECK("range_write_kernel");
  return SIIRL_OK;
}

extern "C" size_t siirl_topk_mark_workspace_bytes(void) { return sel_ws().total; }

extern "C" int siirl_topk_mark(const float* scores, int64_t n, int64_t k, float value, float* marks, void* workspace,
                               size_t workspace_bytes, siirl_stream_t stream) {
  SIIRL_REQUIRE(n >= 0 && n < (1LL << 32), "n=%lld out of range (below 2^32)", (long long)n);
  SIIRL_REQUIRE(k >= 0 && k <= n, "k=%lld must lie in [0, n=%lld]", (long long)k, (long long)n);
  if (n == 0) return SIIRL_OK;
  SIIRL_REQUIRE(scores && marks, "NULL operand");
  SIIRL_REQUIRE(scores != marks, "marks must not alias scores");
  const SelWs ws = sel_ws();
  if (workspace == nullptr || workspace_bytes < ws.total)
    return fail(SIIRL_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes, ws.total);
  SIIRL_REQUIRE(((uintptr_t)workspace & 15) == 0, "workspace must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  char* base = (char*)workspace;
  uint32_t* part = (uint32_t*)(base + ws.part);
  SelState* state = (SelState*)(base + ws.state);
  uint32_t* ties = (uint32_t*)(base + ws.ties);
  const int mode = access_mode((((uintptr_t)scores | (uintptr_t)marks) & 15) == 0, n);
  const int64_t per = ((n + kSelGrid - 1) / kSelGrid + kTile - 1) / kTile * kTile;
  const int grid = (int)((n + per - 1) / per);  // <= kSelGrid; chunks beyond n do not exist
  const dim3 g((unsigned)grid), b(kSelThreads);
  if (k == 0) {
    select_clear_kernel<<<g, b, 0, st>>>(marks, n);
    SIIRL_LAUNCH_CHECK("select_clear_kernel");
    return SIIRL_OK;
  }
  static_assert(3 * kBins % kSelThreads == 0, "the histograms are cleared by whole workgroups");
  select_init_kernel<<<dim3(3 * kBins / kSelThreads), b, 0, st>>>(part);
  SIIRL_LAUNCH_CHECK("select_init_kernel");
  select_hist_kernel<0><<<g, b, 0, st>>>(scores, n, per, mode, state, part);
  SIIRL_LAUNCH_CHECK("select_hist_kernel<0>");
  select_scan_kernel<0><<<1, b, 0, st>>>(part, (uint32_t)k, state);
  SIIRL_LAUNCH_CHECK("select_scan_kernel<0>");
  select_hist_kernel<1><<<g, b, 0, st>>>(scores, n, per, mode, state, part);
  SIIRL_LAUNCH_CHECK("select_hist_kernel<1>");
  select_scan_kernel<1><<<1, b, 0, st>>>(part, 0u, state);
  SIIRL_LAUNCH_CHECK("select_scan_kernel<1>");
  select_hist_kernel<2><<<g, b, 0, st>>>(scores, n, per, mode, state, part);
  SIIRL_LAUNCH_CHECK("select_hist_kernel<2>");
  select_scan_kernel<2><<<1, b, 0, st>>>(part, 0u, state);
  SIIRL_LAUNCH_CHECK("select_scan_kernel<2>");
  select_count_ties_kernel<<<g, b, 0, st>>>(scores, n, per, mode, state, ties);
  SIIRL_LAUNCH_CHECK("select_count_ties_kernel");
  select_mark_kernel<<<g, b, 0, st>>>(scores, n, per, mode, state, ties, value, marks);
  SIIRL_LAUNCH_CHECK("select_mark_kernel");
  return SIIRL_OK;
}
