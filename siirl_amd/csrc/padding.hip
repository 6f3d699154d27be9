// Remove-padding bookkeeping around the per-token loss path: token indices of the attended positions, gathers
// to and scatters from the packed ("rmpad") layout, and the response window of the padded result.
//
// Replaces the calls the actor makes around its log-prob computation (siirl/engine/actor/dp_actor.py:112-127,
// 214-231): flash-attn's bert_padding unpad_input / index_first_axis / pad_input (flash-attn 2.7.3 / 2.8.2, a
// third-party dependency: indices = nonzero(mask.flatten()), cu_seqlens = [0, cumsum(mask.sum(-1))]),
// torch.roll(input_ids_rmpad, -1) for the labels, and the [:, -response_length - 1 : -1] slice.
// All of it is integer / index work: results are exact.
#include "common.hpp"

namespace siirl {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ bool mask_on(const void* p, int dt, int64_t i) {
  switch (dt) {
    case SIIRL_U8: return ((const uint8_t*)p)[i] != 0;
    case SIIRL_I64: return ((const int64_t*)p)[i] != 0;
    case SIIRL_I32: return ((const int32_t*)p)[i] != 0;
    case SIIRL_F32: return ((const float*)p)[i] != 0.f;
    case SIIRL_BF16: return (((const uint16_t*)p)[i] & 0x7fffu) != 0;
    case SIIRL_F16: return (((const uint16_t*)p)[i] & 0x7fffu) != 0;
    default: return false;
  }
}

// seqlens[b] = number of attended positions of row b
__global__ __launch_bounds__(kThreads) void seqlens_kernel(const void* mask, int mask_dtype, int64_t S,
                                                           int32_t* __restrict__ seqlens) {
  const int64_t b = blockIdx.x;
  int n = 0;
  for (int64_t s = threadIdx.x; s < S; s += kThreads) n += mask_on(mask, mask_dtype, b * S + s) ? 1 : 0;
  __shared__ double sh[kThreads / kWave + 1];
  const double tot = block_sum((double)n, sh);  // exact for any count below 2^53
  if (threadIdx.x == 0) seqlens[b] = (int32_t)tot;
}

// cu_seqlens[0] = 0, cu_seqlens[b + 1] = sum_{i <= b} seqlens[i]; info = {total, max seqlen}.  One workgroup.
__global__ __launch_bounds__(kThreads) void cu_seqlens_kernel(const int32_t* __restrict__ seqlens, int64_t B,
                                                              int32_t* __restrict__ cu, int64_t* __restrict__ info) {
  __shared__ int32_t sh[kThreads];
  __shared__ int32_t carry_s, max_s;
  if (threadIdx.x == 0) {
    carry_s = 0;
    max_s = 0;
    cu[0] = 0;
  }
  __syncthreads();
  for (int64_t base = 0; base < B; base += kThreads) {
    const int64_t i = base + threadIdx.x;
    const int32_t v = i < B ? seqlens[i] : 0;
    sh[threadIdx.x] = v;
    __syncthreads();
    for (int off = 1; off < kThreads; off <<= 1) {  // Hillis-Steele inclusive scan
      const int32_t add = (int)threadIdx.x >= off ? sh[threadIdx.x - off] : 0;
      __syncthreads();
      sh[threadIdx.x] += add;
      __syncthreads();
    }
    const int32_t carry = carry_s;
    if (i < B) cu[i + 1] = carry + sh[threadIdx.x];
    atomicMax(&max_s, v);
    __syncthreads();
    if (threadIdx.x == 0) carry_s = carry + sh[kThreads - 1];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    info[0] = carry_s;
    info[1] = max_s;
  }
}

// indices[cu[b] + r] = b * S + s for the r-th attended position s of row b, in order.  One workgroup per row.
__global__ __launch_bounds__(kThreads) void indices_kernel(const void* mask, int mask_dtype, int64_t S,
                                                           const int32_t* __restrict__ cu,
                                                           int64_t* __restrict__ indices) {
  const int64_t b = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x / kWave;
  __shared__ int wave_cnt[kThreads / kWave];
  __shared__ int base_s;
  if (threadIdx.x == 0) base_s = cu[b];
  __syncthreads();
  for (int64_t s0 = 0; s0 < S; s0 += kThreads) {
    const int64_t s = s0 + threadIdx.x;
    const bool on = s < S && mask_on(mask, mask_dtype, b * S + s);
    const unsigned long long bal = __ballot(on);
    const int before = __popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) wave_cnt[wid] = __popcll(bal);
    __syncthreads();
    int off = base_s;
    for (int w = 0; w < wid; ++w) off += wave_cnt[w];
    if (on) indices[off + before] = b * S + s;
    __syncthreads();
    if (threadIdx.x == 0) {
      int t = 0;
      for (int w = 0; w < kThreads / kWave; ++w) t += wave_cnt[w];
      base_s += t;
    }
    __syncthreads();
  }
}

// dst[j] = src[indices[j]] (GATHER) or dst[indices[j]] = src[j] (scatter), rows of `units` elements of U (16 bytes
// when the rows allow it, else 4).  Workgroups are laid out as (piece of a row, row): a row's index is read once per
// workgroup and no address needs a division; every row is moved by 16-byte accesses that bypass the caches (each
// byte is touched once).
template <bool GATHER, typename U>
__global__ __launch_bounds__(kThreads) void move_rows_kernel(const U* __restrict__ src,
                                                             const int64_t* __restrict__ indices, int64_t n,
                                                             int64_t units, int64_t indexed_rows,
                                                             U* __restrict__ dst) {
  for (int64_t j = blockIdx.y; j < n; j += gridDim.y) {
    const int64_t r = indices[j];
    const bool ok = r >= 0 && r < indexed_rows;  // an index outside the indexed tensor never touches memory
    const U* __restrict__ from = GATHER ? src + r * units : src + j * units;
    U* __restrict__ to = GATHER ? dst + j * units : dst + r * units;
    if (!ok && !GATHER) continue;
    for (int64_t u = (int64_t)blockIdx.x * kThreads + threadIdx.x; u < units; u += (int64_t)gridDim.x * kThreads) {
      if (ok)
        __builtin_nontemporal_store(__builtin_nontemporal_load(from + u), to + u);
      else
        __builtin_nontemporal_store(U{}, to + u);
    }
  }
}

// The same for short rows (a workgroup would be mostly idle on one of them): elements of all rows in one flat range.
template <bool GATHER, typename U>
__global__ __launch_bounds__(kThreads) void move_short_rows_kernel(const U* __restrict__ src,
                                                                   const int64_t* __restrict__ indices, int64_t n,
                                                                   int units, int64_t indexed_rows, U* __restrict__ dst) {
  const int64_t total = n * units;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kThreads) {
    const int64_t j = i / units;
    const int u = (int)(i - j * units);
    const int64_t r = indices[j];
    const bool ok = r >= 0 && r < indexed_rows;
    if (GATHER) dst[i] = ok ? src[r * units + u] : U{};
    else if (ok) dst[r * units + u] = src[i];
  }
}

template <typename U>
__global__ __launch_bounds__(kThreads) void fill_zero_kernel(U* __restrict__ p, int64_t units) {
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < units; i += (int64_t)gridDim.x * kThreads)
    __builtin_nontemporal_store(U{}, p + i);
}

// ids_rmpad[j] = input_ids[indices[j]],  labels[j] = input_ids[indices[(j + 1) % nnz]]  (torch.roll(..., -1))
__global__ __launch_bounds__(kThreads) void unpad_ids_kernel(const int64_t* __restrict__ input_ids, int64_t n_ids,
                                                             const int64_t* __restrict__ indices, int64_t nnz,
                                                             int64_t* __restrict__ ids_rmpad,
                                                             int64_t* __restrict__ labels) {
  auto at = [&](int64_t r) { return (r >= 0 && r < n_ids) ? input_ids[r] : (int64_t)-1; };
  for (int64_t j = (int64_t)blockIdx.x * kThreads + threadIdx.x; j < nnz; j += (int64_t)gridDim.x * kThreads) {
    if (ids_rmpad) ids_rmpad[j] = at(indices[j]);
    if (labels) labels[j] = at(indices[j + 1 < nnz ? j + 1 : 0]);
  }
}

// labels[j] = SIIRL_LABEL_SKIP_ROW for the packed tokens whose log-prob the response window [S - L - 1, S - 2] of
// their sequence does not keep
__global__ __launch_bounds__(kThreads) void mark_outside_response_kernel(const int64_t* __restrict__ indices, int64_t nnz,
                                                                         int64_t S, int64_t L,
                                                                         int64_t* __restrict__ labels) {
  for (int64_t j = (int64_t)blockIdx.x * kThreads + threadIdx.x; j < nnz; j += (int64_t)gridDim.x * kThreads) {
    const int64_t r = indices[j];
    const int64_t s = r >= 0 ? r % S : -1;
    if (s < S - L - 1 || s > S - 2) labels[j] = SIIRL_LABEL_SKIP_ROW;
  }
}

// out[b, t] = values[j] for the j with indices[j] == b * S + (S - L - 1 + t); positions nobody writes stay 0
__global__ __launch_bounds__(kThreads) void response_scatter_kernel(const float* __restrict__ values,
                                                                    const int64_t* __restrict__ indices, int64_t nnz,
                                                                    int64_t B, int64_t S, int64_t L,
                                                                    float* __restrict__ out) {
  for (int64_t j = (int64_t)blockIdx.x * kThreads + threadIdx.x; j < nnz; j += (int64_t)gridDim.x * kThreads) {
    const int64_t pos = indices[j], b = pos / S, t = pos - b * S - (S - L - 1);
    if (pos >= 0 && b < B && t >= 0 && t < L) out[b * L + t] = values[j];
  }
}
__global__ __launch_bounds__(kThreads) void response_gather_kernel(const float* __restrict__ grad,
                                                                   const int64_t* __restrict__ indices, int64_t nnz,
                                                                   int64_t B, int64_t S, int64_t L,
                                                                   float* __restrict__ d_values) {
  for (int64_t j = (int64_t)blockIdx.x * kThreads + threadIdx.x; j < nnz; j += (int64_t)gridDim.x * kThreads) {
    const int64_t pos = indices[j], b = pos / S, t = pos - b * S - (S - L - 1);
    d_values[j] = (pos >= 0 && b < B && t >= 0 && t < L) ? grad[b * L + t] : 0.f;
  }
}

// Response mask from generated ids: 1 up to and including the first end-of-sequence token of the row, 0 after it
// (siirl/utils/model_utils/torch_functional.py:209-254).  One wave per row walks the row 64 ids at a time; a ballot
// finds the first hit of the chunk.  Every wave of the launch leaves its loop after ceil(L / 64) steps.
struct EosSet {
  int64_t tok[SIIRL_MAX_EOS_TOKENS];
  int n;
};

__device__ __forceinline__ void store_mask(void* p, int dt, int64_t i, bool on) {
  switch (dt) {
    case SIIRL_U8: ((uint8_t*)p)[i] = on ? 1 : 0; break;
    case SIIRL_I64: ((int64_t*)p)[i] = on ? 1 : 0; break;
    case SIIRL_I32: ((int32_t*)p)[i] = on ? 1 : 0; break;
    case SIIRL_F32: ((float*)p)[i] = on ? 1.f : 0.f; break;
    case SIIRL_BF16: ((uint16_t*)p)[i] = on ? 0x3f80u : 0u; break;
    case SIIRL_F16: ((uint16_t*)p)[i] = on ? 0x3c00u : 0u; break;
    default: break;
  }
}

__global__ __launch_bounds__(kThreads) void eos_mask_kernel(const void* __restrict__ ids, int id_dtype, int64_t B,
                                                            int64_t L, EosSet eos, void* __restrict__ mask,
                                                            int mask_dtype) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t b = (int64_t)blockIdx.x * (kThreads / kWave) + (threadIdx.x / kWave);
  if (b >= B) return;
  bool ended = false;  // wave-uniform: an end-of-sequence token lies in an earlier chunk
  for (int64_t t0 = 0; t0 < L; t0 += kWave) {
    const int64_t t = t0 + lane;
    bool hit = false;
    if (t < L && !ended) {
      const int64_t id = id_dtype == SIIRL_I64 ? ((const int64_t*)ids)[b * L + t] : (int64_t)((const int32_t*)ids)[b * L + t];
      for (int k = 0; k < eos.n; ++k) hit |= id == eos.tok[k];
    }
    const unsigned long long hits = __builtin_amdgcn_ballot_w64(hit);
    const int first = hits ? __builtin_ctzll(hits) : kWave;
    if (t < L) store_mask(mask, mask_dtype, b * L + t, !ended && lane <= first);
    ended |= hits != 0;
  }
}

unsigned blocks_for(int64_t n) {
  const int64_t b = (n + kThreads - 1) / kThreads;
  return (unsigned)(b < 1 ? 1 : (b > 16384 ? 16384 : b));
}

// rows of `row_bytes` move as 16-byte units when both tensors allow it, else as 4-byte words
bool rows_by_16(const void* a, const void* b, int64_t row_bytes) {
  return row_bytes % 16 == 0 && (((uintptr_t)a | (uintptr_t)b) & 15) == 0;
}
// (pieces of a row, rows): enough workgroups to fill the part, at most 65535 rows in flight
dim3 rows_grid(int64_t n, int64_t units) {
  const int64_t per_row = (units + kThreads - 1) / kThreads;
  const int64_t gx = per_row < 1 ? 1 : (per_row > 32 ? 32 : per_row);
  return dim3((unsigned)gx, (unsigned)(n > 65535 ? 65535 : n));
}
template <bool GATHER>
void launch_move_rows(const void* src, const int64_t* indices, int64_t n, int64_t row_bytes, int64_t indexed_rows, void* dst,
                      hipStream_t st) {
  const bool by16 = rows_by_16(src, dst, row_bytes);
  const int64_t units = by16 ? row_bytes / 16 : row_bytes / 4;
  if (units < kThreads / 2) {  // short rows: several per workgroup
    const dim3 grid(blocks_for(n * units));
    if (by16)
      move_short_rows_kernel<GATHER, u32x4><<<grid, dim3(kThreads), 0, st>>>((const u32x4*)src, indices, n, (int)units,
                                                                             indexed_rows, (u32x4*)dst);
    else
      move_short_rows_kernel<GATHER, uint32_t><<<grid, dim3(kThreads), 0, st>>>((const uint32_t*)src, indices, n, (int)units,
                                                                                indexed_rows, (uint32_t*)dst);
  } else if (by16) {
    move_rows_kernel<GATHER, u32x4><<<rows_grid(n, units), dim3(kThreads), 0, st>>>((const u32x4*)src, indices, n, units,
                                                                                    indexed_rows, (u32x4*)dst);
  } else {
    move_rows_kernel<GATHER, uint32_t><<<rows_grid(n, units), dim3(kThreads), 0, st>>>((const uint32_t*)src, indices, n, units,
                                                                                       indexed_rows, (uint32_t*)dst);
  }
}
void launch_fill_zero(void* p, int64_t bytes, hipStream_t st) {  // bytes: a multiple of 4
  if (bytes % 16 == 0 && ((uintptr_t)p & 15) == 0)
    fill_zero_kernel<u32x4><<<dim3(blocks_for(bytes / 16)), dim3(kThreads), 0, st>>>((u32x4*)p, bytes / 16);
  else
    fill_zero_kernel<uint32_t><<<dim3(blocks_for(bytes / 4)), dim3(kThreads), 0, st>>>((uint32_t*)p, bytes / 4);
}

int check_mask(int dt) {
  SIIRL_REQUIRE(dt == SIIRL_U8 || dt == SIIRL_I64 || dt == SIIRL_I32 || dt == SIIRL_F32 || dt == SIIRL_BF16 ||
                    dt == SIIRL_F16, "mask dtype %d not supported", dt);
  return SIIRL_OK;
}

}  // namespace
}  // namespace siirl

using namespace siirl;

extern "C" int siirl_unpad_indices(const void* attention_mask, int mask_dtype, int64_t B, int64_t S,
                                   int32_t* seqlens, int32_t* cu_seqlens, int64_t* indices, int64_t* info2,
                                   siirl_stream_t stream) {
  SIIRL_REQUIRE(B >= 1 && S >= 1 && B <= 0x7fffffffLL && B * S <= 0x7fffffffLL,
                "B=%lld S=%lld out of range (cu_seqlens is int32)", (long long)B, (long long)S);
  if (int rc = check_mask(mask_dtype)) return rc;
  SIIRL_REQUIRE(attention_mask && seqlens && cu_seqlens && indices && info2, "NULL operand");
  hipStream_t st = (hipStream_t)stream;
  seqlens_kernel<<<dim3((unsigned)B), dim3(kThreads), 0, st>>>(attention_mask, mask_dtype, S, seqlens);
  SIIRL_LAUNCH_CHECK("seqlens_kernel");
  cu_seqlens_kernel<<<1, dim3(kThreads), 0, st>>>(seqlens, B, cu_seqlens, info2);
  SIIRL_LAUNCH_CHECK("cu_seqlens_kernel");
  indices_kernel<<<dim3((unsigned)B), dim3(kThreads), 0, st>>>(attention_mask, mask_dtype, S, cu_seqlens, indices);
  SIIRL_LAUNCH_CHECK("indices_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_gather_rows(const void* src, const int64_t* indices, int64_t n, int64_t row_bytes,
                                 int64_t src_rows, void* dst, siirl_stream_t stream) {
  SIIRL_REQUIRE(n >= 0 && src_rows >= 0 && row_bytes >= 4 && row_bytes % 4 == 0,
                "n=%lld src_rows=%lld row_bytes=%lld: rows are whole 4-byte words", (long long)n, (long long)src_rows,
                (long long)row_bytes);
  if (n == 0) return SIIRL_OK;
  SIIRL_REQUIRE(src && indices && dst, "NULL operand");
  launch_move_rows<true>(src, indices, n, row_bytes, src_rows, dst, (hipStream_t)stream);
  SIIRL_LAUNCH_CHECK("move_rows_kernel<gather>");
  return SIIRL_OK;
}

extern "C" int siirl_scatter_rows(const void* src, const int64_t* indices, int64_t n, int64_t row_bytes,
                                  int64_t total_rows, void* dst, siirl_stream_t stream) {
  SIIRL_REQUIRE(n >= 0 && total_rows >= 0 && row_bytes >= 4 && row_bytes % 4 == 0,
                "n=%lld total_rows=%lld row_bytes=%lld: rows are whole 4-byte words", (long long)n,
                (long long)total_rows, (long long)row_bytes);
  if (total_rows == 0) return SIIRL_OK;
  SIIRL_REQUIRE(dst && (n == 0 || (src && indices)), "NULL operand");
  hipStream_t st = (hipStream_t)stream;
  launch_fill_zero(dst, total_rows * row_bytes, st);
  SIIRL_LAUNCH_CHECK("fill_zero_kernel");
  if (n == 0) return SIIRL_OK;
  launch_move_rows<false>(src, indices, n, row_bytes, total_rows, dst, st);
  SIIRL_LAUNCH_CHECK("move_rows_kernel<scatter>");
  return SIIRL_OK;
}

extern "C" int siirl_unpad_ids_labels(const int64_t* input_ids, int64_t n_ids, const int64_t* indices, int64_t nnz,
                                      int64_t* ids_rmpad, int64_t* labels_rolled, siirl_stream_t stream) {
  SIIRL_REQUIRE(nnz >= 0 && n_ids >= 0, "nnz=%lld n_ids=%lld must not be negative", (long long)nnz, (long long)n_ids);
  if (nnz == 0) return SIIRL_OK;
  SIIRL_REQUIRE(input_ids && indices && (ids_rmpad || labels_rolled), "NULL operand");
  unpad_ids_kernel<<<dim3(blocks_for(nnz)), dim3(kThreads), 0, (hipStream_t)stream>>>(input_ids, n_ids, indices, nnz,
                                                                                     ids_rmpad, labels_rolled);
  SIIRL_LAUNCH_CHECK("unpad_ids_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_response_scatter(const float* values, const int64_t* indices, int64_t nnz, int64_t B, int64_t S,
                                      int64_t L, float* out, siirl_stream_t stream) {
  SIIRL_REQUIRE(nnz >= 0 && B >= 1 && S >= 2 && L >= 1 && L <= S - 1, "nnz=%lld B=%lld S=%lld L=%lld: need 1 <= L <= S - 1",
                (long long)nnz, (long long)B, (long long)S, (long long)L);
  SIIRL_REQUIRE(out && (nnz == 0 || (values && indices)), "NULL operand");
  hipStream_t st = (hipStream_t)stream;
  launch_fill_zero(out, B * L * 4, st);
  SIIRL_LAUNCH_CHECK("fill_zero_kernel");
  if (nnz == 0) return SIIRL_OK;
  response_scatter_kernel<<<dim3(blocks_for(nnz)), dim3(kThreads), 0, st>>>(values, indices, nnz, B, S, L, out);
  SIIRL_LAUNCH_CHECK("response_scatter_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_response_gather(const float* grad, const int64_t* indices, int64_t nnz, int64_t B, int64_t S,
                                     int64_t L, float* d_values, siirl_stream_t stream) {
  SIIRL_REQUIRE(nnz >= 0 && B >= 1 && S >= 2 && L >= 1 && L <= S - 1, "nnz=%lld B=%lld S=%lld L=%lld: need 1 <= L <= S - 1",
                (long long)nnz, (long long)B, (long long)S, (long long)L);
  if (nnz == 0) return SIIRL_OK;
  SIIRL_REQUIRE(grad && indices && d_values, "NULL operand");
  response_gather_kernel<<<dim3(blocks_for(nnz)), dim3(kThreads), 0, (hipStream_t)stream>>>(grad, indices, nnz, B, S, L,
                                                                                           d_values);
  SIIRL_LAUNCH_CHECK("response_gather_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_eos_response_mask(const void* response_id, int id_dtype, int64_t B, int64_t L,
                                       const int64_t* eos_tokens, int n_eos, void* mask, int mask_dtype,
                                       siirl_stream_t stream) {
  SIIRL_REQUIRE(B >= 0 && L >= 0 && B <= 0x7fffffffLL, "B=%lld L=%lld out of range", (long long)B, (long long)L);
  SIIRL_REQUIRE(id_dtype == SIIRL_I64 || id_dtype == SIIRL_I32, "response_id dtype %d must be int64 or int32", id_dtype);
  SIIRL_REQUIRE(n_eos >= 0 && n_eos <= SIIRL_MAX_EOS_TOKENS, "n_eos=%d must be in [0, %d]", n_eos, SIIRL_MAX_EOS_TOKENS);
  if (int rc = check_mask(mask_dtype)) return rc;
  if (B == 0 || L == 0) return SIIRL_OK;
  SIIRL_REQUIRE(response_id && mask && (n_eos == 0 || eos_tokens), "NULL operand");
  EosSet eos;
  eos.n = n_eos;
  for (int k = 0; k < SIIRL_MAX_EOS_TOKENS; ++k) eos.tok[k] = k < n_eos ? eos_tokens[k] : 0;
  constexpr int rows_per_wg = kThreads / kWave;
  eos_mask_kernel<<<dim3((unsigned)((B + rows_per_wg - 1) / rows_per_wg)), dim3(kThreads), 0, (hipStream_t)stream>>>(
      response_id, id_dtype, B, L, eos, mask, mask_dtype);
  SIIRL_LAUNCH_CHECK("eos_mask_kernel");
  return SIIRL_OK;
}

extern "C" int siirl_mark_rows_outside_response(const int64_t* indices, int64_t nnz, int64_t S, int64_t L,
                                                int64_t* labels, siirl_stream_t stream) {
  SIIRL_REQUIRE(nnz >= 0 && S >= 1 && L >= 0 && L < S, "nnz=%lld S=%lld response_length=%lld out of range (0 <= L < S)",
                (long long)nnz, (long long)S, (long long)L);
  if (nnz == 0) return SIIRL_OK;
  SIIRL_REQUIRE(indices && labels, "NULL operand");
  mark_outside_response_kernel<<<dim3(blocks_for(nnz)), dim3(kThreads), 0, (hipStream_t)stream>>>(indices, nnz, S, L,
                                                                                                 labels);
  SIIRL_LAUNCH_CHECK("mark_outside_response_kernel");
  return SIIRL_OK;
}
