// lm_head projection fused with log-prob / entropy: logits = hidden[T,H] . W[V,H]^T are produced tile by tile on
// the matrix cores and consumed in the epilogue; no [T, V] tensor is needed (the forward may park its tiles for the
// backward, see below).
//
// Replaces FusedLinearForPPO (siirl/utils/experimental/torch_functional.py:20-211) and linear_cross_entropy
// (siirl/utils/kernel/linear_cross_entropy.py:40-117 -> siirl/utils/kernel/kernels.py:507-696,1378-1586); the
// per-tile online-softmax state (max, sum exp, sum x*exp) is the one of kernels.py:254-266,343-350.
//
// One GEMM core, C[M,N] = A[M,K] . B[N,K]^T, 16-bit operands, fp32 accumulation, 256 x 256 x 64 workgroup tile,
// 8 waves (2 x 4) of 128 x 64 (8 x 4 MFMA 16x16x32 tiles, 128 accumulator registers each).  The 16x16x32 shape moves
// half the accumulator data per flop of the 32x32x16 one; with random operand bits the matrix cores then sustain
// 1.79 instead of 1.62 PFLOP/s in an LDS-fed loop at this part's power limit, which is what sets these kernels' time.
//   * A (K-major rows) goes global -> LDS by DMA (global_load_lds_dwordx4, no staging registers, no ds_write)
//     into a ring of four 32 KB stages.  Rows are unpadded; 16-byte chunks are XOR-swizzled by (row / 2) % 8 so
//     that the ds_read_b128 fragment reads are conflict-free.  A stage is issued three K-steps before it is read
//     and published (barrier) one step before, so the first fragments of the next step are read ahead of the
//     barrier and the matrix cores do not drain at it.
//   * B never touches the LDS: it is prepared once per call in the MFMA operand's lane order ("fragment-packed")
//     and each lane loads its 16-byte operands straight into registers, one K-step ahead.
//   * all loads of the main loop are inline asm with hand-placed s_waitcnt vmcnt: the compiler's own tracking
//     would wait for every outstanding DMA before each LDS read.
// Four epilogues: softmax partials (forward), dlogits in both layouts (backward), fp32 accumulate (d hidden),
// bf16 store (d weight).  The backward walks the vocabulary in slabs: recompute the slab's logits, write
// dlogits[T, slab] and its transpose, then dH += dlogits . W_slab and dW_slab = dlogits^T . hidden as two more
// runs of the same core against packed transposed copies of W and hidden.
// Optionally the forward also parks the fp32 accumulator tiles in memory (4 bytes per logit, in the accumulator's
// own lane order, so stores and loads are whole 1 KB wave accesses); the backward then replays the tiles through
// the same dlogits epilogue instead of recomputing the GEMM: a third of the backward's matrix work is traded for
// one streaming pass.
#include "common.hpp"

namespace siirl {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Workgroup tile 256 x 256 x 64, 8 waves as 2 (M) x 4 (N), two per SIMD, one workgroup per CU (the LDS ring).
// (Measured alternatives at T=16384, H=3584, V=152064, with the 32x32x16 MFMA: 128-row tiles with two workgroups per
// CU 1.5-4 % slower; 4 waves of 128 x 128, one per SIMD, 5-14 % slower.)
constexpr int BM = 256, BN = 256, BK = 64;
constexpr int WM = 2, WN = 4;  // wave grid over the workgroup tile
constexpr int kThreads = WM * WN * 64;
constexpr int kWavesPerSimd = kThreads / 256;
constexpr int MI = BM / (WM * 16), NJ = BN / (WN * 16);  // 16x16 MFMA tiles per wave: 8 x 4
constexpr int KS = BK / 32;                              // K = 32 slices per K-step
static_assert(MI == 8 && NJ == 4 && KS == 2, "the K-step schedule is written for 8 x 4 tiles and two K slices");
constexpr int kRowBytes = BK * 2;             // unpadded rows, 16-byte chunks XOR-swizzled by (row / 2) % 8
constexpr int kTileBytes = BM * kRowBytes;    // 32768
constexpr int kStageBytes = kTileBytes;       // A tile only: B goes global -> registers
constexpr int kStages = 4;
constexpr int kSmemBytes = kStages * kStageBytes;  // 131072
constexpr int kDmaPerWave = kTileBytes / 1024 / (kThreads / 64);  // 1 KB per wave instruction
#ifndef SIIRL_SLAB
#define SIIRL_SLAB 8192
#endif
constexpr int kSlab = SIIRL_SLAB;                   // vocabulary columns per backward slab
static_assert(kSlab % 256 == 0, "a slab is a whole number of workgroup tiles");
#ifndef SIIRL_DH_GROUP
#define SIIRL_DH_GROUP 8
#endif
constexpr int kDhGroup = SIIRL_DH_GROUP;      // slabs of dlogits kept before d hidden and d weight are updated: fewer
                                              // fp32 read-modify-write passes over [T, H] (about 6 % of a d-hidden
                                              // launch at 4 slabs), and 8 x 448 d-weight tiles fill 14 rounds of
                                              // the 256 CUs exactly; measured 4 / 8 / all 19 slabs of V = 152064:
                                              // 34.4 / 33.7 / 33.2 ms per backward
constexpr int kLdPad = 64;                    // extra elements per row of D: keeps a tile's rows off a
                                              // power-of-two stride, which would put them all in one memory channel

struct GemmArgs {
  const uint16_t* A;
  int64_t lda;
  const u32x4* Bp;  // fragment-packed B (see pack layout), already offset to the first K block of this GEMM
  int64_t kb_total; // 32-wide K blocks per 16-row block of the packed buffer
  int M, N, K;  // K is a multiple of BK; rows beyond M are clamped on load and masked by the epilogue
  int tiles_m, tiles_n;
  int splits;  // K is cut into `splits` runs of K-steps; run s is tile column tn + s * tiles_n of the raster
  int blk_m;   // tiles along M of an XCD's block of 32 tiles
};

struct TileCoord {
  int tm, tn;
  bool valid;
};
// XCD-aware rasterisation.  Workgroups are dispatched round-robin over the 8 XCDs, each with its own L2, so
// workgroup id runs on XCD id % 8 as that XCD's (id / 8)-th workgroup.  The tile grid is cut into blocks of
// blk_m x blk_n tiles (32 tiles: one XCD's resident set; blk_m is the launch's choice among 2, 4, 8, 16); block b
// goes to XCD b % 8 and its tiles to 32 consecutive workgroups of that XCD, so the workgroups sharing an L2 at any
// time share blk_m A-tiles and blk_n B-tiles instead of streaming 32 different A-tiles.  Blocks sweep M fastest
// inside a strip of blk_n N-tiles, which keeps a strip's B-tiles hot across the 8 XCDs.  (Sweeping N fastest instead, which would stream the big
// operand from memory once rather than once per strip, measured 4 % slower forward and 8-17 % slower backward GEMMs
// at T=16384, H=3584, V=152064: the L2 reuse inside a strip matters more than the bytes from memory.)
constexpr int kXcd = 8, kBlkTiles = 32;
__host__ __device__ inline int64_t raster_grid(int tiles_m, int tiles_n, int blk_m) {
  const int blk_n = kBlkTiles / blk_m;
  const int64_t blocks = (int64_t)((tiles_m + blk_m - 1) / blk_m) * ((tiles_n + blk_n - 1) / blk_n);
  return (blocks + kXcd - 1) / kXcd * kXcd * kBlkTiles;
}
__device__ __forceinline__ TileCoord tile_of(const GemmArgs& g, int id) {
  const int blk_m = g.blk_m, blk_n = kBlkTiles / blk_m;
  const int xcd = id % kXcd, l = id / kXcd;
  const int blk = (l / kBlkTiles) * kXcd + xcd, j = l % kBlkTiles;
  const int mb = (g.tiles_m + blk_m - 1) / blk_m;
  const int tm = (blk % mb) * blk_m + j % blk_m;
  const int tn = (blk / mb) * blk_n + j / blk_m;
  return {tm, tn, tm < g.tiles_m && tn < g.tiles_n * g.splits};
}

// Accumulator coordinates of lane `lane` in wave (wm, wn): element r (0..3) of acc[i][j] is
//   row = wm*128 + i*16 + (lane/16)*4 + r ,  col = wn*64 + j*16 + lane%16   (tile-relative)
__device__ __forceinline__ int acc_row(int wm, int i, int r, int lane) {
  return wm * (MI * 16) + i * 16 + (lane >> 4) * 4 + r;
}
__device__ __forceinline__ int acc_col(int wn, int j, int lane) { return wn * (NJ * 16) + j * 16 + (lane & 15); }

// m0 (the DMA's LDS base) is a reserved register: naming it in a clobber list is right but draws a warning
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
// F16: the 16-bit operands are IEEE half instead of bf16 (the same data movement, the other MFMA)
template <class Epi, bool AT = false, bool F16 = false>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(kWavesPerSimd, kWavesPerSimd))) void gemm_nt_kernel(GemmArgs g, Epi epi) {
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int wm = w / WN, wn = w % WN;
  const TileCoord tc = tile_of(g, blockIdx.x);
  if (!tc.valid) return;
  const int split = tc.tn / g.tiles_n;
  const int m0 = tc.tm * BM, n0 = (tc.tn - split * g.tiles_n) * BN;
  // this workgroup's run of K-steps (the host keeps every run non-empty)
  const int kt_per = (g.K / BK + g.splits - 1) / g.splits;
  const int kt_first = split * kt_per;
  const int KT = (g.K / BK - kt_first < kt_per) ? g.K / BK - kt_first : kt_per;

  // A: global -> LDS by DMA (global_load_lds_dwordx4): wave instruction I = w * kDmaPerWave + i fills the 1 KB
  // [I * 1024, I * 1024 + 1024) of the stage.
  //   A[M][K] (AT = false): 16-byte slot sl = I * 64 + lane holds row sl / 8, chunk (sl % 8) ^ ((row / 2) % 8).  Rows
  //     past the matrix edge are clamped to the last row.
  //   A given as [K][M], M contiguous (AT = true): the stage is 64 K-rows of 512 bytes; slot sl holds K-row sl / 32,
  //     chunk (sl % 32) ^ 2 * (row % 4), i.e. the 32-byte segments of a row are XOR-swizzled by the row so that the
  //     four K-rows a transposing fragment read touches lie in different banks.  Columns past M are read as they are
  //     (the row pitch covers whole tiles) and only reach output rows that the epilogue masks.
  const int wu = __builtin_amdgcn_readfirstlane(w);
  const char* gA = AT ? reinterpret_cast<const char*>(g.A + (int64_t)kt_first * BK * g.lda + m0)
                      : reinterpret_cast<const char*>(g.A + (int64_t)m0 * g.lda + (int64_t)kt_first * BK);
  const int64_t a_step = AT ? (int64_t)BK * g.lda * 2 : (int64_t)BK * 2;  // bytes from one K-step to the next
  uint32_t offA[kDmaPerWave];
#pragma unroll
  for (int i = 0; i < kDmaPerWave; ++i) {
    const int sl = (wu * kDmaPerWave + i) * 64 + lane;
    if constexpr (AT) {
      const int row = sl >> 5;
      const int ch = (sl & 31) ^ ((row & 3) << 1);
      offA[i] = (uint32_t)row * (uint32_t)g.lda * 2u + ch * 16;
    } else {
      int row = sl >> 3;
      const int ch = (sl & 7) ^ ((row >> 1) & 7);
      row = (m0 + row < g.M) ? row : g.M - 1 - m0;
      offA[i] = (uint32_t)row * (uint32_t)g.lda * 2u + ch * 16;
    }
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
  // B: fragment-packed, one 16-byte load per lane per MFMA operand, no LDS.  N-tile j of the wave, K slice s of the
  // K-step: chunk ((n0 / 16 + wn * NJ + j) * kb_total + kt * KS + s) * 64 + lane.
  const char* gB =
      reinterpret_cast<const char*>(g.Bp + ((int64_t)(n0 >> 4) * g.kb_total + (int64_t)kt_first * KS) * 64);
  uint32_t offB[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) offB[j] = (uint32_t)(((wn * NJ + j) * g.kb_total * 64 + lane) * 16);

  floatx4 acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

  u32x4 b0[NJ][KS], b1[NJ][KS];
  auto dma = [&](int stage, int kt, int i0 = 0, int i1 = kDmaPerWave) {
    const char* base = gA + (int64_t)kt * a_step;
#pragma unroll
    for (int i = i0; i < i1; ++i) {
      const uint32_t dst = lds0 + stage * kStageBytes + (wu * kDmaPerWave + i) * 1024;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(offA[i]), "s"(base) : "m0", "memory");
    }
  };
  auto bload = [&](u32x4 (&b)[NJ][KS], int kt, int j) {
    const char* base = gB + (int64_t)kt * (KS * 1024);
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(b[j][0]) : "v"(offB[j]), "s"(base));
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:1024" : "=v"(b[j][1]) : "v"(offB[j]), "s"(base));
  };
  // waits until only this wave's last kDmaPerWave loads (one stage of DMA) are in flight and ties the B registers
  // to the wait
  static_assert(NJ * KS == 8 && kDmaPerWave % 2 == 0, "see the load schedule of a K-step");
  auto bwait = [&](u32x4 (&b)[NJ][KS]) {
    asm volatile("s_waitcnt vmcnt(%[n])"
                 : "+v"(b[0][0]), "+v"(b[0][1]), "+v"(b[1][0]), "+v"(b[1][1]), "+v"(b[2][0]), "+v"(b[2][1]),
                   "+v"(b[3][0]), "+v"(b[3][1])
                 : [n] "n"(kDmaPerWave)
                 : "memory");
  };

#pragma unroll
  for (int j = 0; j < NJ; ++j) bload(b0, 0, j);
  dma(0, 0);
  dma(1, KT > 1 ? 1 : 0);
  dma(2, KT > 2 ? 2 : 0);
  bwait(b0);
  __syncthreads();

  // A fragments of MFMA group gq = 2 * s + hf: K slice s (32 columns), row blocks hf * 4 .. hf * 4 + 3 of the wave's
  // eight 16-row blocks.  AT = false: lane (m = lane % 16, 8-column chunk lane / 16 of the slice) reads its 8
  // consecutive K entries as one 16-byte chunk of row m.  AT = true: the stage holds K-rows, so the 8 entries come
  // from two transposing reads (ds_read_b64_tr_b16): in each block of 16 lanes, lane 4 e + c addresses the 8 bytes of
  // K-row e, M-chunk c, and receives the entries of K-rows 0..3 at M = its own index in the block; block lane / 16
  // takes the 8 K-rows lane / 16 * 8 .. + 7 of the slice.
  const int m15 = lane & 15, kq = lane >> 4, sw = m15 >> 1;
  const int frag_row = (wm * (MI * 16) + m15) * kRowBytes;
  int xk[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) xk[s] = frag_row + (((s * 4 + kq) ^ sw) << 4);
  const int tq = m15 >> 2;
  const int xt0 = (kq * 8 + tq) * 512 + wm * 256 + (lane & 3) * 8 + (tq << 5);  // row block ii: xt0 ^ (ii << 5)

  // step kt: stage kt % 4 is read; B(kt + 1) and DMA(kt + 3) are issued (K-steps past the end are clamped to the
  // last one: they land in stages that are not read again); the barrier at the end publishes stage
  // (kt + 2) % 4, whose DMA was issued one step earlier, and frees stage kt % 4 for DMA(kt + 4).
  // A fragments are read one MFMA group ahead; the group after the last one of a step is the first of the next
  // step, whose stage was published by the previous barrier, so the reads cross the barrier.
  bf16x8 afa[4], afb[4];
  auto fread = [&](bf16x8 (&af)[4], int stage, int gq) {
    const char* cur = smem + stage * kStageBytes;
    const int s = gq >> 1, hf = gq & 1;
    if constexpr (AT) {
      typedef short s16x4 __attribute__((ext_vector_type(4)));
      typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
#pragma unroll
      for (int ii = 0; ii < 4; ++ii) {
        const char* at = cur + (xt0 ^ (ii << 5)) + s * (32 * 512) + hf * 128;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(at));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(at + 4 * 512));
        af[ii] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    } else {
#pragma unroll
      for (int ii = 0; ii < 4; ++ii)
        af[ii] = *reinterpret_cast<const bf16x8*>(cur + xk[s] + (hf * 4 + ii) * 16 * kRowBytes);
    }
  };
  auto mma = [&](bf16x8 (&af)[4], u32x4 (&bc)[NJ][KS], int gq) {
    const int s = gq >> 1, hf = gq & 1;
#pragma unroll
    for (int ii = 0; ii < 4; ++ii)
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj) {
        // boustrophedon over the N-tiles: consecutive MFMAs always share one operand (0.5-0.8 % faster at T=16384,
        // H=3584, V=152064 than restarting at N-tile 0 for every row block: fewer operand wires toggle)
        const int j = (ii & 1) ? NJ - 1 - jj : jj;
        floatx4& c = acc[hf * 4 + ii][j];
        if constexpr (F16)
          c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, af[ii]), __builtin_bit_cast(f16x8, bc[j][s]), c, 0, 0, 0);
        else
          c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[ii], __builtin_bit_cast(bf16x8, bc[j][s]), c, 0, 0, 0);
      }
  };
  fread(afa, 0, 0);
  // One K-step: four groups of 16 MFMAs.  The 12 vector-memory instructions are spread over the step (B for two
  // N-tiles before each of the first two groups, half of the DMA before each of the last two) instead of being issued
  // in one burst, and the wave raises its priority while it issues MFMAs so that its SIMD partner's loads do not
  // delay them.
  auto mma_prio = [&](bf16x8 (&af)[4], u32x4 (&bc)[NJ][KS], int gq) {
    __builtin_amdgcn_s_setprio(1);
    mma(af, bc, gq);
    __builtin_amdgcn_s_setprio(0);
  };
  auto step = [&](int kt, u32x4 (&bc)[NJ][KS], u32x4 (&bn)[NJ][KS]) {
    const int stage = kt & 3;
    const int ktb = kt + 1 < KT ? kt + 1 : KT - 1, kta = kt + 3 < KT ? kt + 3 : KT - 1;
#pragma unroll
    for (int j = 0; j < NJ / 2; ++j) bload(bn, ktb, j);
    fread(afb, stage, 1);
    mma_prio(afa, bc, 0);
#pragma unroll
    for (int j = NJ / 2; j < NJ; ++j) bload(bn, ktb, j);
    fread(afa, stage, 2);
    mma_prio(afb, bc, 1);
    dma((stage + 3) & 3, kta, 0, kDmaPerWave / 2);
    fread(afb, stage, 3);
    mma_prio(afa, bc, 2);
    dma((stage + 3) & 3, kta, kDmaPerWave / 2, kDmaPerWave);
    fread(afa, (stage + 1) & 3, 0);
    mma_prio(afb, bc, 3);
    bwait(bn);
    __syncthreads();
  };
  int kt = 0;
  for (; kt + 2 <= KT; kt += 2) {
    step(kt, b0, b1);
    step(kt + 1, b1, b0);
  }
  if (kt < KT) step(kt, b0, b1);
  // the clamped DMA of the last steps may still be in flight and the epilogue reuses the LDS
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  epi(acc, m0, n0, tc.tm, split, wm, wn, lane, tid, smem);
}
#pragma clang diagnostic pop

// ------------------------------------------------------------------------------ parked accumulator tiles

// Tile (tm, tn) of the forward GEMM occupies kQuads * kThreads 16-byte slots; slot c * kThreads + tid holds thread
// tid's acc[i][j] (four registers), c = i * NJ + j.  A wave instruction therefore moves one contiguous KB, and the
// tile can be handed to any epilogue exactly as the main loop would have left it.
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int kQuads = MI * NJ;
constexpr int64_t kSavedTileBytes = (int64_t)kQuads * kThreads * 16;  // BM * BN * 4
__device__ __forceinline__ f32x4* saved_tile(float* base, int tm, int tn, int tiles_n) {
  return reinterpret_cast<f32x4*>(base) + ((int64_t)tm * tiles_n + tn) * (kQuads * kThreads);
}

// Runs an epilogue over parked tiles: workgroup b takes tile (tm_first + b / tiles_n, b % tiles_n) and calls the
// epilogue with vocabulary row m0 counted from the first tile row of the launch.
template <class Epi>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(kWavesPerSimd, kWavesPerSimd))) void replay_tiles_kernel(
    const float* __restrict__ saved, int tiles_n, int tm_first, Epi epi) {
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int wm = w / WN, wn = w % WN;
  const int tml = blockIdx.x / tiles_n, tn = blockIdx.x - tml * tiles_n;
  const f32x4* src = saved_tile(const_cast<float*>(saved), tm_first + tml, tn, tiles_n) + tid;
  floatx4 acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = __builtin_nontemporal_load(src + (i * NJ + j) * kThreads);
  epi(acc, tml * BM, tn * BN, tml, 0, wm, wn, lane, tid, smem);
}

// ------------------------------------------------------------------------------ epilogue: softmax partials

// The two fused GEMMs run "transposed": M is the vocabulary (A = W), N the tokens (B = hidden).  In the MFMA
// accumulator layout a lane then owns one token (column) and its registers run over vocabulary rows, so the
// softmax reductions over the vocabulary are in-register, followed by two exchanges between the four lanes that
// share a token and a merge of the WM waves through LDS -- no 16-lane butterfly per row.
//
// Per token of the tile: mx = max_v z, s = sum exp(z - mx), t = sum z * exp(z - mx) over the tile's 256
// vocabulary rows, z = acc * inv_T; one (mx, s, t) per token is written to part[tm][.][token].
struct SoftmaxPartialsEpi {
  float inv_T;
  int T, V;
  float* part;  // [tiles_m][3][T]
  float* save;  // null, or the parked accumulator tiles (see saved_tile)
  int tiles_n;
  __device__ __forceinline__ void operator()(floatx4 (&acc)[MI][NJ], int m0, int n0, int tm, int split, int wm, int wn,
                                             int lane, int tid, char* smem) const {
    // Parking costs about 11 us per tile (256 KB per workgroup): the workgroup's own drain, not a burst of the round.
    if (save) {
      f32x4* dst = saved_tile(save, tm, n0 / BN, tiles_n) + tid;
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) dst[(i * NJ + j) * kThreads] = acc[i][j];
    }
    float* sh = reinterpret_cast<float*>(smem);  // [WM][BN][3]; the main loop's last barrier freed the LDS
    const float k = kLog2e;
    const float ninf = -__builtin_inff();
    const bool full = m0 + BM <= V;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      float mx = ninf;
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const bool ok = full || (m0 + acc_row(wm, i, r, lane) < V);
          mx = fmaxf(mx, ok ? acc[i][j][r] * inv_T : ninf);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
      mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
      float s = 0.f, t = 0.f;
      if (mx > ninf) {
        const float nmk = -mx * k;
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const bool ok = full || (m0 + acc_row(wm, i, r, lane) < V);
            const float x = acc[i][j][r] * inv_T;
            const float e = ok ? fast_exp2(fmaf(x, k, nmk)) : 0.f;
            s += e;
            t = fmaf(ok ? x : 0.f, e, t);
          }
      }
      s += __shfl_xor(s, 16, kWave);
      t += __shfl_xor(t, 16, kWave);
      s += __shfl_xor(s, 32, kWave);
      t += __shfl_xor(t, 32, kWave);
      if (lane < 16) {
        float* d = sh + (wm * BN + acc_col(wn, j, lane)) * 3;
        d[0] = mx;
        d[1] = s;
        d[2] = t;
      }
    }
    __syncthreads();
    const int tok = n0 + tid;
    if (tid < BN && tok < T) {
      float M = ninf;
#pragma unroll
      for (int q = 0; q < WM; ++q) M = fmaxf(M, sh[(q * BN + tid) * 3]);
      float ss = 0.f, tt = 0.f;
#pragma unroll
      for (int q = 0; q < WM; ++q) {
        const float* a = sh + (q * BN + tid) * 3;
        const float f = a[0] > ninf ? fast_exp2((a[0] - M) * k) : 0.f;
        ss += a[1] * f;
        tt += a[2] * f;
      }
      float* o = part + (int64_t)tm * 3 * T;
      o[tok] = M;
      o[(int64_t)T + tok] = ss;
      o[2 * (int64_t)T + tok] = tt;
    }
  }
};

// ------------------------------------------------------------------------------ epilogue: dlogits

// d raw_logit = inv_T * ( g_lp * (1[v == y] - p) - g_h * p * (z - ex) ),  p = exp(z - lse), z = acc * inv_T,
// written as bf16 to D[token][v] (ld = ldd); v is slab-relative and is the M dimension of this GEMM.  Rows v in
// [Vs, Vpad) are written as zeros: they are K-padding of the d-hidden GEMM that consumes D.  A lane owns one token,
// so the per-token coefficients are loaded once per lane and D gets 8-byte stores.  This one token-major layout
// serves both consumers: d hidden reads it as its A[M = token][K = vocabulary], d weight as A given by K-rows.
struct DlogitsEpi {
  float inv_T;
  int T, Vs, Vpad;
  int64_t v0;  // first vocabulary column of the slab
  const float* lse;
  const float* ex;
  const float* g_lp;  // may be null
  const float* g_h;   // may be null
  const int64_t* labels;
  uint16_t* D;
  int64_t ldd;
  // One lane's part of the tile.  With a = raw accumulator (z = a * inv_T) the gradient is
  //   d = p * (c0 + c1 * a) + [v == y] * cy,   p = exp2(a * ek + nl),
  // ek = inv_T * log2(e), nl = -lse * log2(e), c1 = -g_h * inv_T^2, c0 = inv_T * (g_h * ex - g_lp), cy = g_lp * inv_T:
  // two fused multiply-adds, one exp2 and one multiply per logit.  FULL: every vocabulary row of the tile is inside
  // the slab.
  template <bool FULL>
  __device__ __forceinline__ void tile(floatx4 (&acc)[MI][NJ], int m0, int n0, int wm, int wn, int lane) const {
    const float ek = inv_T * kLog2e;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int tok = n0 + acc_col(wn, j, lane);
      if (tok >= T) continue;
      const float g1 = g_lp ? g_lp[tok] : 0.f;
      const float g2 = g_h ? g_h[tok] : 0.f;
      const float nl = -lse[tok] * kLog2e;
      const float exv = g_h ? ex[tok] : 0.f;
      const float c1 = -g2 * inv_T * inv_T, c0 = inv_T * (g2 * exv - g1), cy = g1 * inv_T;
      int y = -1;
      if (g_lp) {
        const int64_t yl = labels[tok] - v0;
        if (yl >= 0 && yl < Vs) y = (int)yl;
      }
      uint16_t* drow = D + (int64_t)tok * ldd;
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        const int v = m0 + acc_row(wm, i, 0, lane);  // 4 consecutive vocabulary rows of the slab
        float d[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float a = acc[i][j][e];
          const float p = fast_exp2(fmaf(a, ek, nl));
          float g = p * fmaf(a, c1, c0);
          if (v + e == y) g += cy;
          d[e] = (FULL || v + e < Vs) ? g : 0.f;
        }
        // the four lanes that share the token hold 16 consecutive rows: 32 contiguous bytes per token and store
        if (FULL || v < Vpad) *reinterpret_cast<uint2*>(drow + v) = make_uint2(pack_bf16(d[0], d[1]), pack_bf16(d[2], d[3]));
      }
    }
  }
  __device__ __forceinline__ void operator()(floatx4 (&acc)[MI][NJ], int m0, int n0, int tm, int split, int wm, int wn,
                                             int lane, int tid, char* smem) const {
    if (m0 + BM <= Vs)
      tile<true>(acc, m0, n0, wm, wn, lane);
    else
      tile<false>(acc, m0, n0, wm, wn, lane);
  }
};

// ------------------------------------------------------------------------------ epilogues: plain stores

struct AccumF32Epi {  // C_s[row][col] = (beta ? C_s : 0) + acc, one fp32 buffer C_s = C + s * split_stride per K run
  float* C;
  int64_t ldc, split_stride;
  int M, N, beta;
  __device__ __forceinline__ void operator()(floatx4 (&acc)[MI][NJ], int m0, int n0, int tm, int split, int wm, int wn, int lane, int tid,
                             char* smem) const {
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = m0 + acc_row(wm, i, r, lane);
        if (row >= M) continue;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          const int col = n0 + acc_col(wn, j, lane);
          if (col >= N) continue;
          float* p = C + split * split_stride + (int64_t)row * ldc + col;
          *p = beta ? *p + acc[i][j][r] : acc[i][j][r];
        }
      }
  }
};

struct StoreEpi {  // C[row][col] = acc, rounded to the output type (out_dtype: SIIRL_BF16, SIIRL_F16 or SIIRL_F32)
  void* C;
  int64_t ldc;
  int M, N, out_dtype;
  __device__ __forceinline__ void operator()(floatx4 (&acc)[MI][NJ], int m0, int n0, int tm, int split, int wm, int wn, int lane, int tid,
                             char* smem) const {
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = m0 + acc_row(wm, i, r, lane);
        if (row >= M) continue;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          const int col = n0 + acc_col(wn, j, lane);
          if (col >= N) continue;
          const int64_t at = (int64_t)row * ldc + col;
          if (out_dtype == SIIRL_BF16)
            reinterpret_cast<uint16_t*>(C)[at] = (uint16_t)(pack_bf16(acc[i][j][r], 0.f) & 0xffffu);
          else if (out_dtype == SIIRL_F16)
            reinterpret_cast<uint16_t*>(C)[at] = (uint16_t)(pack_f16(acc[i][j][r], 0.f) & 0xffffu);
          else
            reinterpret_cast<float*>(C)[at] = acc[i][j][r];
        }
      }
  }
};

// ------------------------------------------------------------------------------ small kernels

// Fragment-packed B operand.  For a K-major matrix B[n][k] the packed buffer holds, for each block of 16 rows nb
// and each block of 32 columns kb, the 64 x 16 bytes that one 16x16x32 MFMA takes as its B operand, in lane order:
//   chunk index ((nb * KB + kb) * 64 + l),  l = (n % 16) + 16 * ((k % 32) / 8),  8 consecutive k per chunk.
// Rows n >= N and columns k >= K are zero.  One thread per chunk.
__global__ __launch_bounds__(256) void pack_b_kernel(const uint16_t* __restrict__ in, int64_t ld_in, int N, int K,
                                                     u32x4* __restrict__ out, int64_t KB, int64_t chunks) {
  const int64_t ch = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (ch >= chunks) return;
  const int l = (int)(ch & 63);
  const int64_t blk = ch >> 6, kb = blk % KB, nb = blk / KB;
  const int64_t n = nb * 16 + (l & 15), k = kb * 32 + (l >> 4) * 8;
  u32x4 v = {0u, 0u, 0u, 0u};
  if (n < N && k < K) v = *reinterpret_cast<const u32x4*>(in + n * ld_in + k);  // K % 8 == 0
  out[ch] = v;
}

// The same packing of the transpose: B[n][k] = in[k][n] with in of shape [R = K][C = N].  A workgroup stages a
// 64 x 64 tile through LDS and emits its 512 chunks.
// from_f16: the input holds IEEE halves, the packed output bf16 (round to nearest even).
__device__ __forceinline__ uint32_t half2_to_bf16x2(uint32_t w) { return pack_bf16(f16_lo(w), f16_hi(w)); }
__global__ __launch_bounds__(256) void transpose_pack_b_kernel(const uint16_t* __restrict__ in, int64_t ld_in, int R,
                                                               int C, u32x4* __restrict__ out, int64_t KB, int from_f16) {
  __shared__ __align__(16) uint16_t tile[64][72];  // 144-byte rows: 16-byte aligned, 36 dwords (column reads spread)
  const int r0 = blockIdx.x * 64, c0 = blockIdx.y * 64;  // r = k, c = n
  // 16 bytes (8 columns) per thread and pass, 8 threads per row, 32 rows per pass; ld_in and c0 are multiples of 8
  for (int q = threadIdx.x; q < 512; q += 256) {
    const int rr = q >> 3, cc = (q & 7) * 8;
    const int r = r0 + rr, c = c0 + cc;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (r < R) {
      if (c + 8 <= C) {
        v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(in + (int64_t)r * ld_in + c));
      } else if (c < C) {
        uint16_t t[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) t[e] = c + e < C ? in[(int64_t)r * ld_in + c + e] : (uint16_t)0;
        v = u32x4{(uint32_t)t[0] | ((uint32_t)t[1] << 16), (uint32_t)t[2] | ((uint32_t)t[3] << 16),
                  (uint32_t)t[4] | ((uint32_t)t[5] << 16), (uint32_t)t[6] | ((uint32_t)t[7] << 16)};
      }
    }
    if (from_f16) v = u32x4{half2_to_bf16x2(v.x), half2_to_bf16x2(v.y), half2_to_bf16x2(v.z), half2_to_bf16x2(v.w)};
    *reinterpret_cast<u32x4*>(&tile[rr][cc]) = v;
  }
  __syncthreads();
  for (int q = threadIdx.x; q < 512; q += 256) {
    const int nl = q & 63, kc = q >> 6;  // local n, local chunk of 8 k
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = (uint32_t)tile[kc * 8 + 2 * e][nl] | ((uint32_t)tile[kc * 8 + 2 * e + 1][nl] << 16);
    const int64_t n = c0 + nl, k = r0 + kc * 8;
    const int64_t ch = ((n >> 4) * KB + (k >> 5)) * 64 + (n & 15) + 16 * ((k >> 3) & 3);
    out[ch] = u32x4{w[0], w[1], w[2], w[3]};
  }
}

// label_logit[row] = inv_T * <hidden[row], W[labels[row]]>, one wave per row (NaN for a label outside [0, V))
__global__ __launch_bounds__(256) void label_logit_kernel(const uint16_t* __restrict__ hidden,
                                                          const uint16_t* __restrict__ W,
                                                          const int64_t* __restrict__ labels, int T, int H, int64_t V,
                                                          float inv_T, float* __restrict__ out, int f16) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= T) return;
  const int64_t y = labels[row];
  if (y < 0 || y >= V) {
    if (lane == 0) out[row] = __builtin_nanf("");
    return;
  }
  const u32x4* a = reinterpret_cast<const u32x4*>(hidden + (int64_t)row * H);
  const u32x4* b = reinterpret_cast<const u32x4*>(W + y * (int64_t)H);
  float s = 0.f;
  for (int i = lane; i < H / 8; i += kWave) {
    const u32x4 u = a[i], v = b[i];
    if (f16)
      s += f16_lo(u.x) * f16_lo(v.x) + f16_hi(u.x) * f16_hi(v.x) + f16_lo(u.y) * f16_lo(v.y) + f16_hi(u.y) * f16_hi(v.y) +
           f16_lo(u.z) * f16_lo(v.z) + f16_hi(u.z) * f16_hi(v.z) + f16_lo(u.w) * f16_lo(v.w) + f16_hi(u.w) * f16_hi(v.w);
    else
      s += bf16_lo(u.x) * bf16_lo(v.x) + bf16_hi(u.x) * bf16_hi(v.x) + bf16_lo(u.y) * bf16_lo(v.y) +
           bf16_hi(u.y) * bf16_hi(v.y) + bf16_lo(u.z) * bf16_lo(v.z) + bf16_hi(u.z) * bf16_hi(v.z) +
           bf16_lo(u.w) * bf16_lo(v.w) + bf16_hi(u.w) * bf16_hi(v.w);
  }
  s = wave_sum(s);
  if (lane == 0) out[row] = s * inv_T;
}

// folds the per-tile partials of each token: lse, ex, entropy, logprob.  A workgroup handles kMergeTok tokens;
// kMergeGrp thread groups each merge every kMergeGrp-th tile online, then the states are merged through LDS.
constexpr int kMergeTok = 16, kMergeGrp = 16;
static_assert(kMergeTok * kMergeGrp == 256, "one thread per (token, group)");
__global__ __launch_bounds__(256) void merge_partials_kernel(const float* __restrict__ part, int nparts, int T,
                                                             const float* __restrict__ label_logit,
                                                             float* __restrict__ logprob, float* __restrict__ entropy,
                                                             float* __restrict__ lse_out, float* __restrict__ ex_out) {
  __shared__ float sh[kMergeGrp][kMergeTok][3];
  const int tl = threadIdx.x % kMergeTok, grp = threadIdx.x / kMergeTok;
  const int row = blockIdx.x * kMergeTok + tl;
  float M = -__builtin_inff(), s = 0.f, t = 0.f;
  if (row < T) {
    for (int p = grp; p < nparts; p += kMergeGrp) {
      const float* q = part + (int64_t)p * 3 * T;
      const float m = q[row];
      if (m > -__builtin_inff()) {
        const float Mn = fmaxf(M, m);
        const float fo = fast_exp2((M - Mn) * kLog2e), fn = fast_exp2((m - Mn) * kLog2e);
        s = s * fo + q[(int64_t)T + row] * fn;
        t = t * fo + q[2 * (int64_t)T + row] * fn;
        M = Mn;
      }
    }
  }
  sh[grp][tl][0] = M;
  sh[grp][tl][1] = s;
  sh[grp][tl][2] = t;
  __syncthreads();
  if (grp != 0 || row >= T) return;
  float Mx = M;
#pragma unroll
  for (int g = 1; g < kMergeGrp; ++g) Mx = fmaxf(Mx, sh[g][tl][0]);
  double ss = 0.0, tt = 0.0;
#pragma unroll
  for (int g = 0; g < kMergeGrp; ++g) {
    const float m = sh[g][tl][0];
    if (m > -__builtin_inff()) {
      const float f = fast_exp2((m - Mx) * kLog2e);
      ss += (double)(sh[g][tl][1] * f);
      tt += (double)(sh[g][tl][2] * f);
    }
  }
  const float lse = Mx + logf((float)ss);
  const float exv = (float)(tt / ss);
  lse_out[row] = lse;
  if (ex_out) ex_out[row] = exv;
  if (entropy) entropy[row] = lse - exv;
  if (logprob) logprob[row] = label_logit[row] - lse;
}

// out = in (+ in2), rounded to out_dtype (SIIRL_BF16, SIIRL_F16 or SIIRL_F32)
__global__ __launch_bounds__(256) void sum_convert_kernel(const float* __restrict__ in, const float* __restrict__ in2,
                                                          void* __restrict__ out, int64_t n, int out_dtype) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const float v = in2 ? in[i] + in2[i] : in[i];
    if (out_dtype == SIIRL_BF16)
      reinterpret_cast<uint16_t*>(out)[i] = (uint16_t)(pack_bf16(v, 0.f) & 0xffffu);
    else if (out_dtype == SIIRL_F16)
      reinterpret_cast<uint16_t*>(out)[i] = (uint16_t)(pack_f16(v, 0.f) & 0xffffu);
    else
      reinterpret_cast<float*>(out)[i] = v;
  }
}

// fp32 operands are staged as three bf16 terms per element so that the bf16 matrix cores reproduce the product to
// 2^-16: x = hi + lo + O(2^-16 x) with hi = bf16(x), lo = bf16(x - hi), and
//   a . b ~ a_hi . b_hi + a_hi . b_lo + a_lo . b_hi .
// A row of K floats becomes a row of 3 K bf16: [hi | hi | lo] for the A operand (role 0), [hi | lo | hi] for the B
// operand (role 1); the GEMM then simply runs over K' = 3 K.  The first K columns are bf16(x): what the two gradient
// GEMMs use.  Four elements per thread.
__global__ __launch_bounds__(256) void split3_kernel(const float* __restrict__ in, int64_t rows, int64_t K,
                                                     uint16_t* __restrict__ out, int role) {
  const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;  // quad index
  const int64_t kq = K / 4;
  if (q >= rows * kq) return;
  const int64_t r = q / kq, k = (q - r * kq) * 4;
  const float4 x = *reinterpret_cast<const float4*>(in + r * K + k);
  const uint32_t h01 = pack_bf16(x.x, x.y), h23 = pack_bf16(x.z, x.w);
  const uint32_t l01 = pack_bf16(x.x - bf16_lo(h01), x.y - bf16_hi(h01));
  const uint32_t l23 = pack_bf16(x.z - bf16_lo(h23), x.w - bf16_hi(h23));
  uint16_t* o = out + r * 3 * K + k;
  *reinterpret_cast<uint2*>(o) = make_uint2(h01, h23);
  *reinterpret_cast<uint2*>(o + K) = role == 0 ? make_uint2(h01, h23) : make_uint2(l01, l23);
  *reinterpret_cast<uint2*>(o + 2 * K) = role == 0 ? make_uint2(l01, l23) : make_uint2(h01, h23);
}

// ------------------------------------------------------------------------------ host

inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

// AT: A is given by its K-rows (A[K][M], M contiguous, row pitch lda >= tiles_m * BM, K readable rows)
template <class Epi, bool AT = false, bool F16 = false>
int launch_gemm(const uint16_t* A, int64_t lda, const u32x4* Bp, int64_t kb_total, int M, int N, int K, const Epi& epi,
                hipStream_t st, const char* what, int splits = 1, int blk_m = 8) {
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_nt_kernel<Epi, AT, F16>), kSmemBytes)) return rc;
  GemmArgs g{A, lda, Bp, kb_total, M, N, K, (M + BM - 1) / BM, (N + BN - 1) / BN, splits, blk_m};
  if (AT && lda < (int64_t)g.tiles_m * BM) return fail(SIIRL_ERR_INVALID_ARGUMENT, "%s: row pitch %lld is shorter than %d tiles", what, (long long)lda, g.tiles_m);
  const int64_t tiles = raster_grid(g.tiles_m, g.tiles_n * splits, blk_m);
  gemm_nt_kernel<Epi, AT, F16><<<dim3((unsigned)tiles), dim3(kThreads), kSmemBytes, st>>>(g, epi);
  SIIRL_LAUNCH_CHECK(what);
  return SIIRL_OK;
}

// Tiles along M of an XCD's block, per GEMM of the fused path.  Measured at T=16384, H=3584, V=152064 (ms per step
// for blocks of 2 x 16 / 4 x 8 / 8 x 4 / 16 x 2 tiles): forward 13.34 / 13.32 / 13.67 / 15.16; recompute + dlogits
// 13.97 / 14.17 / 14.30 / 14.90 (1 x 32: slower again); d hidden 13.49 / 13.31 / 13.50 / 13.74; d weight 13.77 /
// 13.50 / 13.40 / 14.24.  The A operand of the first two is W, streamed from memory once per strip of blk_n token
// tiles: wider strips read it less often.
constexpr int kBlkFwd = 4, kBlkRecompute = 2, kBlkDHidden = 4, kBlkDWeight = 8;

// Two K runs when that fills the 256 compute units' last round noticeably better (896 tiles = 3.5 rounds become
// 1792 = 7) and the GEMM is deep enough for the second fp32 buffer's extra pass not to matter.
inline int pick_splits(int M, int N, int K) {
  const int64_t tiles = (int64_t)((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  auto eff = [](int64_t t) { return (double)t / (double)((t + 255) / 256 * 256); };
  if (K / BK < 128) return 1;
  return eff(2 * tiles) > eff(tiles) * 1.05 ? 2 : 1;
}

// K of the logits GEMM for operands of `dtype`: the hidden size, or three bf16 terms per fp32 element (split3_kernel)
inline int64_t logits_k(int dtype, int64_t H) { return dtype == SIIRL_F32 ? 3 * H : H; }

int check_fused(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V, float inv_T, int dtype) {
  SIIRL_REQUIRE(dtype == SIIRL_BF16 || dtype == SIIRL_F16 || dtype == SIIRL_F32,
                "fused lm_head path takes bf16, fp16 or fp32 operands (dtype %d given)", dtype);
  // 32-bit byte offsets inside a 256-row tile bound the row pitch of every A operand (W: K, D: group of slabs + pad)
  SIIRL_REQUIRE(T >= 1 && T < (1LL << 22) && V >= 1 && V < (1LL << 30), "T=%lld (< 4194304) V=%lld out of range",
                (long long)T, (long long)V);
  SIIRL_REQUIRE(H >= BK && H % BK == 0 && logits_k(dtype, H) < (1 << 22),
                "hidden size %lld must be a positive multiple of %d (below %d)", (long long)H, BK,
                (1 << 22) / (dtype == SIIRL_F32 ? 3 : 1));
  SIIRL_REQUIRE(hidden && weight, "NULL operand");
  SIIRL_REQUIRE(((uintptr_t)hidden & 15) == 0 && ((uintptr_t)weight & 15) == 0, "operands must be 16-byte aligned");
  SIIRL_REQUIRE(inv_T > 0.f && inv_T < 1e30f, "inv_temperature must be positive and finite");
  return SIIRL_OK;
}
int check_ws_align(const void* ws) {
  SIIRL_REQUIRE(((uintptr_t)ws & 255) == 0, "workspace must be 256-byte aligned");
  return SIIRL_OK;
}

// hs / wsp: the three-term bf16 copies of fp32 operands ([T][3 H], [V][3 H]); absent for 16-bit operands
struct FwdWs {
  size_t part, label, hp, hs, wsp, total;
};
FwdWs fwd_ws(int64_t T, int64_t H, int64_t V, int dtype) {
  FwdWs w;
  const int64_t tiles_v = (V + BM - 1) / BM, Kc = logits_k(dtype, H);
  size_t off = 0;
  w.part = off; off += round_up((size_t)tiles_v * 3 * T * 4, 256);
  w.label = off; off += round_up((size_t)T * 4, 256);
  w.hp = off; off += (size_t)round_up(T, BN) * Kc * 2;
  w.hs = off; off += dtype == SIIRL_F32 ? round_up((size_t)T * Kc * 2, 256) : 0;
  w.wsp = off; off += dtype == SIIRL_F32 ? round_up((size_t)V * Kc * 2, 256) : 0;
  w.total = off;
  return w;
}

struct BwdWs {
  size_t hp, wtp, htp, d, dh32, hs, wsp, total;
  int64_t ldwt, ldt, hpad, ldd_row;  // ldt: token count padded to BK (the K of the d-weight GEMM); ldd_row: pitch of D
};
BwdWs bwd_ws(int64_t T, int64_t H, int64_t V, bool want_dh, bool want_dw, int dtype) {
  BwdWs w;
  const int64_t Kc = logits_k(dtype, H);
  w.ldwt = round_up(V, BK);
  w.ldt = round_up(T, BK);
  w.ldd_row = (int64_t)kDhGroup * kSlab + kLdPad;
  w.hpad = round_up(H, BN);
  size_t off = 0;
  w.hp = off; off += (size_t)round_up(T, BN) * Kc * 2;
  w.wtp = off; off += want_dh ? (size_t)w.hpad * w.ldwt * 2 : 0;
  w.htp = off; off += want_dw ? (size_t)w.hpad * w.ldt * 2 : 0;
  w.d = off; off += round_up((size_t)w.ldt * w.ldd_row * 2, 256);  // rows [T, ldt) are K-padding of d weight: zeros
  w.dh32 = off; off += want_dh ? 2 * round_up((size_t)T * H * 4, 256) : 0;  // one buffer per K run
  w.hs = off; off += dtype == SIIRL_F32 ? round_up((size_t)T * Kc * 2, 256) : 0;
  w.wsp = off; off += dtype == SIIRL_F32 ? round_up((size_t)V * Kc * 2, 256) : 0;
  w.total = off;
  return w;
}

// fp32 operands -> their three-term bf16 copies (hidden in the B role, weight in the A role)
int stage_f32(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V, uint16_t* hs, uint16_t* wsp,
              hipStream_t st) {
  const int64_t qh = T * (H / 4), qw = V * (H / 4);
  split3_kernel<<<dim3((unsigned)((qh + 255) / 256)), dim3(256), 0, st>>>((const float*)hidden, T, H, hs, 1);
  SIIRL_LAUNCH_CHECK("split3_kernel(hidden)");
  split3_kernel<<<dim3((unsigned)((qw + 255) / 256)), dim3(256), 0, st>>>((const float*)weight, V, H, wsp, 0);
  SIIRL_LAUNCH_CHECK("split3_kernel(weight)");
  return SIIRL_OK;
}

__global__ __launch_bounds__(256) void zero_fill_kernel(u32x4* __restrict__ p, int64_t n16) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (int64_t)gridDim.x * 256) p[i] = u32x4{0u, 0u, 0u, 0u};
}

int pack_hidden(const uint16_t* h, int64_t T, int64_t H, u32x4* out, hipStream_t st) {
  const int64_t chunks = round_up(T, BN) * H / 8;
  pack_b_kernel<<<dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, st>>>(h, H, (int)T, (int)H, out, H / 32, chunks);
  SIIRL_LAUNCH_CHECK("pack_b_kernel");
  return SIIRL_OK;
}

// The per-token operands of the backward for the listed token rows only (a row index outside [0, T) yields zero
// gradients: the row then contributes nothing).
__global__ __launch_bounds__(256) void gather_token_operands_kernel(const int64_t* __restrict__ rows, int64_t n, int64_t T,
                                                                    const int64_t* __restrict__ labels,
                                                                    const float* __restrict__ lse,
                                                                    const float* __restrict__ ex,
                                                                    const float* __restrict__ g_lp,
                                                                    const float* __restrict__ g_ent,
                                                                    int64_t* __restrict__ labels_c, float* __restrict__ lse_c,
                                                                    float* __restrict__ ex_c, float* __restrict__ g_lp_c,
                                                                    float* __restrict__ g_ent_c) {
  const int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (j >= n) return;
  const int64_t r = rows[j];
  const bool ok = r >= 0 && r < T;
  labels_c[j] = ok && labels ? labels[r] : -1;
  lse_c[j] = ok ? lse[r] : 0.f;
  ex_c[j] = ok && ex ? ex[r] : 0.f;
  g_lp_c[j] = ok && g_lp ? g_lp[r] : 0.f;
  g_ent_c[j] = ok && g_ent ? g_ent[r] : 0.f;
}

struct RowsWs {
  size_t hidden, labels, lse, ex, g_lp, g_ent, dh, inner, inner_bytes, total;
};
RowsWs rows_ws(int64_t n, int64_t H, int64_t V, bool want_dh, bool want_dw, int dtype) {
  const size_t es = dtype_size(dtype);
  RowsWs w;
  size_t off = 0;
  auto take = [&off](size_t bytes) {
    const size_t at = off;
    off += round_up(bytes, 256);
    return at;
  };
  w.hidden = take((size_t)n * H * es);
  w.labels = take((size_t)n * 8);
  w.lse = take((size_t)n * 4);
  w.ex = take((size_t)n * 4);
  w.g_lp = take((size_t)n * 4);
  w.g_ent = take((size_t)n * 4);
  w.dh = take(want_dh ? (size_t)n * H * es : 0);
  w.inner = off;
  w.inner_bytes = n > 0 ? bwd_ws(n, H, V, want_dh, want_dw, dtype).total : 0;
  w.total = off + w.inner_bytes;
  return w;
}

}  // namespace
}  // namespace siirl

using namespace siirl;

extern "C" size_t siirl_fused_linear_fwd_workspace_bytes_dtype(int dtype, int64_t T, int64_t H, int64_t V) {
  if (T < 1 || V < 1 || H < 1 || dtype_size(dtype) == 0) return 0;
  return fwd_ws(T, H, V, dtype).total;
}
extern "C" size_t siirl_fused_linear_fwd_workspace_bytes(int64_t T, int64_t H, int64_t V) {
  return siirl_fused_linear_fwd_workspace_bytes_dtype(SIIRL_BF16, T, H, V);
}

extern "C" size_t siirl_fused_linear_bwd_workspace_bytes_dtype(int dtype, int64_t T, int64_t H, int64_t V,
                                                               int want_d_hidden, int want_d_weight) {
  if (T < 1 || V < 1 || H < 1 || dtype_size(dtype) == 0) return 0;
  return bwd_ws(T, H, V, want_d_hidden != 0, want_d_weight != 0, dtype).total;
}
extern "C" size_t siirl_fused_linear_bwd_workspace_bytes(int64_t T, int64_t H, int64_t V, int want_d_hidden,
                                                         int want_d_weight) {
  return siirl_fused_linear_bwd_workspace_bytes_dtype(SIIRL_BF16, T, H, V, want_d_hidden, want_d_weight);
}

extern "C" size_t siirl_fused_linear_saved_logits_bytes(int64_t T, int64_t V) {
  if (T < 1 || V < 1) return 0;
  return (size_t)(((V + BM - 1) / BM) * ((T + BN - 1) / BN) * kSavedTileBytes);
}

extern "C" int siirl_fused_linear_logprob_entropy_fwd(const void* hidden, const void* weight, int dtype,
                                                      const int64_t* labels, int64_t T, int64_t H, int64_t V,
                                                      float inv_temperature, float* logprob, float* entropy, float* lse,
                                                      float* ex, float* saved_logits, void* workspace,
                                                      size_t workspace_bytes, siirl_stream_t stream) {
  if (int rc = check_fused(hidden, weight, T, H, V, inv_temperature, dtype)) return rc;
  SIIRL_REQUIRE(lse != nullptr, "lse is NULL");
  SIIRL_REQUIRE(((uintptr_t)saved_logits & 15) == 0, "saved_logits must be 16-byte aligned");
  SIIRL_REQUIRE((logprob == nullptr) == (labels == nullptr), "labels and logprob must be given together");
  SIIRL_REQUIRE(entropy == nullptr || ex != nullptr, "ex is required when entropy is requested");
  const FwdWs ws = fwd_ws(T, H, V, dtype);
  if (workspace == nullptr || workspace_bytes < ws.total)
    return fail(SIIRL_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes, ws.total);
  if (int rc = check_ws_align(workspace)) return rc;
  hipStream_t st = (hipStream_t)stream;
  float* part = reinterpret_cast<float*>((char*)workspace + ws.part);
  float* label_logit = reinterpret_cast<float*>((char*)workspace + ws.label);
  const uint16_t* h = (const uint16_t*)hidden;
  const uint16_t* w = (const uint16_t*)weight;
  const int64_t Kc = logits_k(dtype, H);
  const bool f16 = dtype == SIIRL_F16;
  if (dtype == SIIRL_F32) {
    uint16_t* hs = (uint16_t*)((char*)workspace + ws.hs);
    uint16_t* wsp = (uint16_t*)((char*)workspace + ws.wsp);
    if (int rc = stage_f32(hidden, weight, T, H, V, hs, wsp, st)) return rc;
    h = hs;
    w = wsp;
  }
  if (labels) {
    label_logit_kernel<<<dim3((unsigned)((T + 3) / 4)), dim3(256), 0, st>>>(h, w, labels, (int)T, (int)Kc, V,
                                                                          inv_temperature, label_logit, (int)f16);
    SIIRL_LAUNCH_CHECK("label_logit_kernel");
  }
  u32x4* hp = reinterpret_cast<u32x4*>((char*)workspace + ws.hp);
  if (int rc = pack_hidden(h, T, Kc, hp, st)) return rc;
  SoftmaxPartialsEpi epi{inv_temperature, (int)T, (int)V, part, saved_logits, (int)((T + BN - 1) / BN)};
  if (int rc = f16 ? launch_gemm<SoftmaxPartialsEpi, false, true>(w, Kc, hp, Kc / 32, (int)V, (int)T, (int)Kc, epi, st,
                                                                  "gemm_nt_kernel<SoftmaxPartialsEpi, f16>", 1, kBlkFwd)
                   : launch_gemm(w, Kc, hp, Kc / 32, (int)V, (int)T, (int)Kc, epi, st, "gemm_nt_kernel<SoftmaxPartialsEpi>", 1,
                                 kBlkFwd))
    return rc;
  const int tiles_v = (int)((V + BM - 1) / BM);
  merge_partials_kernel<<<dim3((unsigned)((T + kMergeTok - 1) / kMergeTok)), dim3(256), 0, st>>>(part, tiles_v, (int)T, label_logit,
                                                                               logprob, entropy, lse, ex);
  SIIRL_LAUNCH_CHECK("merge_partials_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_fused_linear_logprob_entropy_bwd(const void* hidden, const void* weight, int dtype,
                                                      const int64_t* labels, int64_t T, int64_t H, int64_t V,
                                                      float inv_temperature, const float* lse, const float* ex,
                                                      const float* saved_logits, const float* g_logprob,
                                                      const float* g_entropy, void* d_hidden, void* d_weight,
                                                      void* workspace, size_t workspace_bytes, siirl_stream_t stream) {
  if (int rc = check_fused(hidden, weight, T, H, V, inv_temperature, dtype)) return rc;
  SIIRL_REQUIRE(lse != nullptr, "lse is NULL");
  SIIRL_REQUIRE(((uintptr_t)saved_logits & 15) == 0, "saved_logits must be 16-byte aligned");
  SIIRL_REQUIRE(g_logprob != nullptr || g_entropy != nullptr, "no upstream gradient given");
  SIIRL_REQUIRE(g_logprob == nullptr || labels != nullptr, "labels is required with g_logprob");
  SIIRL_REQUIRE(g_entropy == nullptr || ex != nullptr, "ex is required with g_entropy");
  SIIRL_REQUIRE(d_hidden != nullptr || d_weight != nullptr, "neither d_hidden nor d_weight requested");
  const bool want_dh = d_hidden != nullptr, want_dw = d_weight != nullptr;
  const BwdWs ws = bwd_ws(T, H, V, want_dh, want_dw, dtype);
  if (workspace == nullptr || workspace_bytes < ws.total)
    return fail(SIIRL_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes, ws.total);
  if (int rc = check_ws_align(workspace)) return rc;
  hipStream_t st = (hipStream_t)stream;
  char* base = (char*)workspace;
  u32x4* hp = (u32x4*)(base + ws.hp);          // packed hidden: B[n = token][k = K of the logits GEMM]
  u32x4* Wtp = (u32x4*)(base + ws.wtp);        // packed W^T:    B[n = H][k = vocabulary]
  u32x4* Htp = (u32x4*)(base + ws.htp);        // packed hidden^T: B[n = H][k = token]
  uint16_t* D = (uint16_t*)(base + ws.d);      // [ldt][ldd_row]: kDhGroup slabs side by side
  float* dH32 = (float*)(base + ws.dh32);      // [T][H]
  const uint16_t* h = (const uint16_t*)hidden;
  const uint16_t* w = (const uint16_t*)weight;
  // The logits are recomputed from the operands as given (fp16: the half MFMA; fp32: three bf16 terms per element,
  // K = 3 H).  The two gradient GEMMs multiply the bf16 dlogits with bf16 copies of hidden and W (for fp16 and fp32
  // operands: rounded to bf16 while they are transposed and packed) and write their fp32 sums in the operands' dtype.
  const int64_t Kc = logits_k(dtype, H);
  const bool f16 = dtype == SIIRL_F16;
  if (dtype == SIIRL_F32) {
    uint16_t* hs = (uint16_t*)(base + ws.hs);
    uint16_t* wsp = (uint16_t*)(base + ws.wsp);
    if (int rc = stage_f32(hidden, weight, T, H, V, hs, wsp, st)) return rc;
    h = hs;
    w = wsp;
  }

  if (!saved_logits)
    if (int rc = pack_hidden(h, T, Kc, hp, st)) return rc;
  if (want_dh) {
    transpose_pack_b_kernel<<<dim3((unsigned)(ws.ldwt / 64), (unsigned)(ws.hpad / 64)), dim3(256), 0, st>>>(
        w, Kc, (int)V, (int)H, Wtp, ws.ldwt / 32, (int)f16);
    SIIRL_LAUNCH_CHECK("transpose_pack_b_kernel(W)");
  }
  if (want_dw) {
    transpose_pack_b_kernel<<<dim3((unsigned)(ws.ldt / 64), (unsigned)(ws.hpad / 64)), dim3(256), 0, st>>>(
        h, Kc, (int)T, (int)H, Htp, ws.ldt / 32, (int)f16);
    SIIRL_LAUNCH_CHECK("transpose_pack_b_kernel(hidden)");
  }
  if (want_dw && ws.ldt > T) {  // the token rows that only pad the K of the d-weight GEMM (ldd_row * 2 % 16 == 0)
    const int64_t n16 = (ws.ldt - T) * ws.ldd_row * 2 / 16;
    zero_fill_kernel<<<dim3((unsigned)((n16 + 255) / 256 < 1024 ? (n16 + 255) / 256 : 1024)), dim3(256), 0, st>>>(
        reinterpret_cast<u32x4*>(D + T * ws.ldd_row), n16);
    SIIRL_LAUNCH_CHECK("zero_fill_kernel");
  }
  int dh_splits = 1;
  const int64_t dh32_stride = (int64_t)(round_up((size_t)T * H * 4, 256) / 4);
  int slab_idx = 0;
  const int tiles_t = (int)((T + BN - 1) / BN);
  for (int64_t v0 = 0; v0 < V; v0 += kSlab, ++slab_idx) {
    const int N = (int)((V - v0) < kSlab ? (V - v0) : kSlab);
    const int Npad = (int)round_up(N, BK);
    const int gs = slab_idx % kDhGroup;  // position of this slab in its group of D columns
    if (!saved_logits) {
      DlogitsEpi epi{inv_temperature, (int)T, N, Npad, v0, lse, ex, g_logprob, g_entropy, labels,
                     D + (int64_t)gs * kSlab, ws.ldd_row};
      if (int rc = f16 ? launch_gemm<DlogitsEpi, false, true>(w + v0 * Kc, Kc, hp, Kc / 32, N, (int)T, (int)Kc, epi, st,
                                                              "gemm_nt_kernel<DlogitsEpi, f16>", 1, kBlkRecompute)
                       : launch_gemm(w + v0 * Kc, Kc, hp, Kc / 32, N, (int)T, (int)Kc, epi, st, "gemm_nt_kernel<DlogitsEpi>", 1,
                                     kBlkRecompute))
        return rc;
    } else if (gs == 0) {
      // the whole group's dlogits in one pass over the tiles the forward parked
      const int64_t left = V - v0, cap = (int64_t)kDhGroup * kSlab;
      const int Ng = (int)(left < cap ? left : cap);
      DlogitsEpi epi{inv_temperature, (int)T, Ng, (int)round_up(Ng, BK), v0, lse, ex, g_logprob, g_entropy, labels,
                     D, ws.ldd_row};
      const void* fn = reinterpret_cast<const void*>(&replay_tiles_kernel<DlogitsEpi>);
      if (int rc = allow_dynamic_lds(fn, kSmemBytes)) return rc;
      const int64_t wgs = (int64_t)((Ng + BM - 1) / BM) * tiles_t;
      replay_tiles_kernel<DlogitsEpi><<<dim3((unsigned)wgs), dim3(kThreads), kSmemBytes, st>>>(
          saved_logits, tiles_t, (int)(v0 / BM), epi);
      SIIRL_LAUNCH_CHECK("replay_tiles_kernel<DlogitsEpi>");
    }
    if (want_dh && (gs == kDhGroup - 1 || v0 + kSlab >= V)) {
      // dH[T, H] += D[T, K] . Wt[H, g0 : g0 + K]^T over the group's columns (only the last slab can be partial)
      const int64_t g0 = v0 - (int64_t)gs * kSlab;
      const int K = gs * kSlab + Npad;
      // the first group decides whether d hidden is accumulated as two K runs; a shallower last group then still
      // writes both buffers (its second run may be short, never empty: K >= 2 K-steps)
      if (g0 == 0) dh_splits = pick_splits((int)T, (int)H, K);
      const int splits = (K / BK >= 2) ? dh_splits : 1;
      AccumF32Epi acc{dH32, H, dh32_stride, (int)T, (int)H, g0 > 0 ? 1 : 0};
      if (int rc = launch_gemm(D, ws.ldd_row, Wtp + (g0 / 32) * 64, ws.ldwt / 32, (int)T, (int)H, K, acc, st,
                               "gemm_nt_kernel<AccumF32Epi>", splits, kBlkDHidden))
        return rc;
    }
    if (want_dw && (gs == kDhGroup - 1 || v0 + kSlab >= V)) {
      // dW[g0 : g0 + M, H] = D[ldt, M]^T . Ht[H, ldt]^T over the group's vocabulary rows: D is the A operand given
      // by its K-rows (tokens)
      const int64_t g0 = v0 - (int64_t)gs * kSlab;
      const int M = gs * kSlab + N;
      StoreEpi sto{(char*)d_weight + g0 * H * (int64_t)dtype_size(dtype), H, M, (int)H, dtype};
      if (int rc = launch_gemm<StoreEpi, true>(D, ws.ldd_row, Htp, ws.ldt / 32, M, (int)H, (int)ws.ldt, sto, st,
                                               "gemm_nt_kernel<StoreEpi, A by K-rows>", 1, kBlkDWeight))
        return rc;
    }
  }
  if (want_dh) {
    const int64_t n = T * H;
    const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    sum_convert_kernel<<<dim3(blocks), dim3(256), 0, st>>>(dH32, dh_splits > 1 ? dH32 + dh32_stride : nullptr, d_hidden, n,
                                                           dtype);
    SIIRL_LAUNCH_CHECK("sum_convert_kernel");
  }
  return SIIRL_OK;
}

extern "C" size_t siirl_fused_linear_bwd_rows_workspace_bytes_dtype(int dtype, int64_t n_rows, int64_t H, int64_t V,
                                                                    int want_d_hidden, int want_d_weight) {
  if (n_rows < 0 || H <= 0 || V <= 0 || dtype_size(dtype) == 0) return 0;
  return rows_ws(n_rows, H, V, want_d_hidden != 0, want_d_weight != 0, dtype).total;
}
extern "C" size_t siirl_fused_linear_bwd_rows_workspace_bytes(int64_t n_rows, int64_t H, int64_t V, int want_d_hidden,
                                                              int want_d_weight) {
  return siirl_fused_linear_bwd_rows_workspace_bytes_dtype(SIIRL_BF16, n_rows, H, V, want_d_hidden, want_d_weight);
}

extern "C" int siirl_fused_linear_logprob_entropy_bwd_rows(const void* hidden, const void* weight, int dtype,
                                                           const int64_t* labels, int64_t T, int64_t H, int64_t V,
                                                           float inv_temperature, const float* lse, const float* ex,
                                                           const float* g_logprob, const float* g_entropy,
                                                           const int64_t* rows, int64_t n_rows, void* d_hidden,
                                                           void* d_weight, void* workspace, size_t workspace_bytes,
                                                           siirl_stream_t stream) {
  if (int rc = check_fused(hidden, weight, T, H, V, inv_temperature, dtype)) return rc;
  SIIRL_REQUIRE(n_rows >= 0 && n_rows <= T, "n_rows=%lld must lie in [0, T=%lld]", (long long)n_rows, (long long)T);
  SIIRL_REQUIRE(n_rows == 0 || rows != nullptr, "rows is NULL");
  SIIRL_REQUIRE(lse != nullptr, "lse is NULL");
  SIIRL_REQUIRE(g_logprob != nullptr || g_entropy != nullptr, "no upstream gradient given");
  SIIRL_REQUIRE(g_logprob == nullptr || labels != nullptr, "labels is required with g_logprob");
  SIIRL_REQUIRE(g_entropy == nullptr || ex != nullptr, "ex is required with g_entropy");
  SIIRL_REQUIRE(d_hidden != nullptr || d_weight != nullptr, "neither d_hidden nor d_weight requested");
  const bool want_dh = d_hidden != nullptr, want_dw = d_weight != nullptr;
  if (n_rows == 0) {  // no row carries a gradient: both results are zero
    if (want_dh)
      if (int rc = siirl_scatter_rows(nullptr, nullptr, 0, H * (int64_t)dtype_size(dtype), T, d_hidden, stream)) return rc;
    if (want_dw)
      if (int rc = siirl_scatter_rows(nullptr, nullptr, 0, H * (int64_t)dtype_size(dtype), V, d_weight, stream)) return rc;
    return SIIRL_OK;
  }
  const RowsWs ws = rows_ws(n_rows, H, V, want_dh, want_dw, dtype);
  const int64_t row_bytes = H * (int64_t)dtype_size(dtype);
  if (workspace == nullptr || workspace_bytes < ws.total)
    return fail(SIIRL_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes, ws.total);
  if (int rc = check_ws_align(workspace)) return rc;
  hipStream_t st = (hipStream_t)stream;
  char* base = (char*)workspace;
  void* hidden_c = base + ws.hidden;
  int64_t* labels_c = (int64_t*)(base + ws.labels);
  float* lse_c = (float*)(base + ws.lse);
  float* ex_c = (float*)(base + ws.ex);
  float* g_lp_c = (float*)(base + ws.g_lp);
  float* g_ent_c = (float*)(base + ws.g_ent);
  void* dh_c = base + ws.dh;
  if (int rc = siirl_gather_rows(hidden, rows, n_rows, row_bytes, T, hidden_c, stream)) return rc;
  gather_token_operands_kernel<<<dim3((unsigned)((n_rows + 255) / 256)), dim3(256), 0, st>>>(
      rows, n_rows, T, labels, lse, ex, g_logprob, g_entropy, labels_c, lse_c, ex_c, g_lp_c, g_ent_c);
  SIIRL_LAUNCH_CHECK("gather_token_operands_kernel");
  if (int rc = siirl_fused_linear_logprob_entropy_bwd(hidden_c, weight, dtype, labels_c, n_rows, H, V, inv_temperature,
                                                      lse_c, ex_c, nullptr, g_logprob ? g_lp_c : nullptr,
                                                      g_entropy ? g_ent_c : nullptr, want_dh ? dh_c : nullptr, d_weight,
                                                      base + ws.inner, ws.inner_bytes, stream))
    return rc;
  if (want_dh)
    if (int rc = siirl_scatter_rows(dh_c, rows, n_rows, row_bytes, T, d_hidden, stream)) return rc;
  return SIIRL_OK;
}
