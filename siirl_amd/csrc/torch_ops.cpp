// torch.library layer of siirl_amd: TORCH_LIBRARY(siirl_hip, m).
//
// Host-only C++ (no device code): every operator checks its operands, allocates its outputs with ATen, and hands
// raw device pointers plus torch's current stream to the C ABI of libsiirl_hip.so (include/siirl_hip.h).  Two levels:
//
//   * plain operators, one per C entry point of the path (logprob_entropy_fwd / _bwd / _bwd_, grpo_advantage,
//     group_keep_mask, agg_loss_fwd / _bwd, policy_loss_fwd / _bwd, kl_penalty_fwd / _bwd, masked_reduce_fwd / _bwd,
//     fused_linear_logprob_entropy_fwd / _bwd): registered for the CUDA key only, functional unless their schema
//     says otherwise, with fake kernels registered from Python (siirl_amd/ops.py) for FakeTensor tracing;
//   * differentiable operators (logprob_entropy, actor_loss, agg_loss, kl_penalty, value_loss, masked_reduce,
//     fused_linear_logprob_entropy): torch::autograd::Function nodes over the plain ones, so that an eager forward
//     and its backward cost one dispatcher call each and no Python frame.  They are what the Python mirrors of the
//     reference's functions (siirl/utils/model_utils/torch_functional.py:56-168, siirl/dag_worker/core_algos.py:536-862,
//     1173-1276, siirl/utils/experimental/torch_functional.py:70-211) call.
//
// There is no CPU kernel: a CPU tensor has no kernel to dispatch to and raises.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/hip/HIPGraphsC10Utils.h>
#include <torch/csrc/autograd/custom_function.h>
#include <torch/library.h>

#include <tuple>
#include <vector>

#include "../../include/siirl_hip.h"

namespace {

using at::Tensor;
using c10::optional;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

// ----------------------------------------------------------------------------------------- plumbing

void check_rc(int rc, const char* what) {
  if (rc == SIIRL_OK) return;
  const char* msg = siirl_hip_last_error();
  if (rc == SIIRL_ERR_INVALID_ARGUMENT) TORCH_CHECK_VALUE(false, what, ": ", msg);
  if (rc == SIIRL_ERR_UNSUPPORTED) TORCH_CHECK_NOT_IMPLEMENTED(false, what, ": ", msg);
  TORCH_CHECK(false, what, " failed (status ", rc, "): ", msg);
}

int dtype_code(at::ScalarType t) {
  switch (t) {
    case at::kFloat: return SIIRL_F32;
    case at::kBFloat16: return SIIRL_BF16;
    case at::kHalf: return SIIRL_F16;
    case at::kDouble: return SIIRL_F64;
    case at::kLong: return SIIRL_I64;
    case at::kInt: return SIIRL_I32;
    case at::kByte: case at::kBool: return SIIRL_U8;
    default: TORCH_CHECK_TYPE(false, "dtype ", t, " is not supported by libsiirl_hip");
  }
}

void require_gpu(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), "siirl_amd: `", name, "` is on ", t.device(),
              "; these ops run on the GPU only (no CPU fallback)");
}

// torch on ROCm presents its HIP devices and streams under the CUDA device type
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;

siirl_stream_t stream_of(const Tensor& t) {
  return (siirl_stream_t)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

template <typename T = void>
T* ptr(const Tensor& t) {
  return t.defined() ? reinterpret_cast<T*>(t.data_ptr()) : nullptr;
}
template <typename T = void>
T* ptr(const optional<Tensor>& t) {
  return (t.has_value() && t->defined()) ? reinterpret_cast<T*>(t->data_ptr()) : nullptr;
}

bool has(const optional<Tensor>& t) { return t.has_value() && t->defined(); }

Tensor empty_f32(at::IntArrayRef shape, const Tensor& like) {
  return at::empty(shape, like.options().dtype(at::kFloat).memory_format(c10::nullopt));
}

// fp32, contiguous, on `dev`.  Called below the autograd keys (inside a node's forward / backward), where no
// conversion records a graph; a tensor that already qualifies is returned as it is.
Tensor f32c(const Tensor& t, const c10::Device& dev) {
  if (t.scalar_type() == at::kFloat && t.device() == dev && t.is_contiguous()) return t;
  Tensor r = t;
  if (r.device() != dev) r = r.to(dev);
  if (r.scalar_type() != at::kFloat) r = r.to(at::kFloat);
  return r.contiguous();
}
optional<Tensor> f32c(const optional<Tensor>& t, const c10::Device& dev) {
  if (!has(t)) return c10::nullopt;
  return f32c(*t, dev);
}

// a mask in a dtype the kernels read as is (anything else becomes fp32), contiguous, on `dev`
Tensor mask_arg(const Tensor& mask, const c10::Device& dev) {
  Tensor m = mask;
  if (m.device() != dev) m = m.to(dev);
  switch (m.scalar_type()) {
    case at::kBool: case at::kByte: case at::kInt: case at::kLong: case at::kFloat: case at::kBFloat16: case at::kHalf:
      break;
    default: m = m.to(at::kFloat);
  }
  return m.contiguous();
}

Tensor as_2d(const Tensor& t) {
  if (t.dim() == 2) return t;
  if (t.dim() == 1) return t.unsqueeze(0);
  if (t.dim() == 0) return t.reshape({1, 1});
  return t.reshape({-1, t.size(-1)});
}

void require_f32c(const Tensor& t, const char* name) {
  require_gpu(t, name);
  TORCH_CHECK_VALUE(t.scalar_type() == at::kFloat && t.is_contiguous(), "siirl_amd: `", name,
                    "` must be a contiguous float32 tensor");
}
void require_f32c(const optional<Tensor>& t, const char* name) {
  if (has(t)) require_f32c(*t, name);
}

int mask_code(const Tensor& mask) {
  TORCH_CHECK_VALUE(mask.is_contiguous(), "siirl_amd: the mask must be contiguous");
  return dtype_code(mask.scalar_type());
}

// The plain operators hand raw pointers to kernels whose grids are sized from ONE operand: every other operand must
// live on that operand's device and hold as many elements as the kernel will read or write.
void require_on(const Tensor& t, const Tensor& like, const char* name) {
  TORCH_CHECK(t.device() == like.device(), "siirl_amd: `", name, "` is on ", t.device(), ", expected ", like.device());
}
void require_mask(const Tensor& mask, const Tensor& like, const char* name = "mask") {
  require_on(mask, like, name);
  TORCH_CHECK_VALUE(mask.sizes() == like.sizes(), "siirl_amd: `", name, "` has shape ", mask.sizes(), ", expected ",
                    like.sizes());
}
void require_f32_like(const Tensor& t, const Tensor& like, const char* name) {
  require_on(t, like, name);
  TORCH_CHECK_VALUE(t.scalar_type() == at::kFloat && t.is_contiguous() && t.sizes() == like.sizes(), "siirl_amd: `", name,
                    "` must be a contiguous float32 tensor of shape ", like.sizes(), ", got ", t.scalar_type(), " ",
                    t.sizes());
}
void require_f32_like(const optional<Tensor>& t, const Tensor& like, const char* name) {
  if (has(t)) require_f32_like(*t, like, name);
}
void require_f32_n(const Tensor& t, int64_t n, const Tensor& like, const char* name) {
  require_on(t, like, name);
  TORCH_CHECK_VALUE(t.scalar_type() == at::kFloat && t.is_contiguous() && t.numel() == n, "siirl_amd: `", name,
                    "` must be a contiguous float32 tensor of ", n, " elements, got ", t.scalar_type(), " ", t.sizes());
}
void require_f32_n(const optional<Tensor>& t, int64_t n, const Tensor& like, const char* name) {
  if (has(t)) require_f32_n(*t, n, like, name);
}

Tensor loss_workspace(int64_t B, int64_t L, const Tensor& like, size_t* n) {
  *n = siirl_loss_workspace_bytes(B, L);
  return at::empty({(int64_t)*n}, like.options().dtype(at::kByte).memory_format(c10::nullopt));
}

// A (..., V) tensor with unit inner stride as blocks of uniformly strided rows: {element offset, rows, row stride}.
// A contiguous tensor or a row-sliced 2-D view is one block; a [B, S, V] slice along S gives B blocks.
struct RowBlock { int64_t off, rows, stride; };

void row_blocks(const Tensor& x, std::vector<RowBlock>& out) {
  const int64_t V = x.size(-1);
  TORCH_CHECK_VALUE(x.stride(-1) == 1 || V <= 1, "siirl_amd: the vocab axis of logits must have stride 1");
  if (x.numel() == 0) return;  // no rows: no blocks (an empty leading axis must not yield one)
  std::vector<std::pair<int64_t, int64_t>> dims;  // (size, stride) of the leading axes, size-1 axes dropped
  for (int64_t d = 0; d + 1 < x.dim(); ++d)
    if (x.size(d) != 1) dims.emplace_back(x.size(d), x.stride(d));
  if (dims.empty()) {
    out.push_back({0, x.numel() ? 1 : 0, std::max<int64_t>(V, 1)});
    return;
  }
  int64_t n_in = dims.back().first;
  const int64_t s_in = dims.back().second;
  size_t k = dims.size() - 1;
  while (k > 0 && dims[k - 1].second == n_in * s_in) {
    n_in *= dims[k - 1].first;
    --k;
  }
  TORCH_CHECK_VALUE(s_in >= V, "siirl_amd: overlapping logits rows are not supported");
  std::vector<int64_t> idx(k, 0);
  while (true) {
    int64_t off = 0;
    for (size_t d = 0; d < k; ++d) off += idx[d] * dims[d].second;
    out.push_back({off, n_in, s_in});
    size_t d = k;
    while (d > 0) {
      if (++idx[d - 1] < dims[d - 1].first) break;
      idx[d - 1] = 0;
      --d;
    }
    if (d == 0) break;
  }
}

// The blocks as a flat list {offset, rows, stride, ...}: host-side arithmetic on sizes and strides only, any device.
std::vector<int64_t> row_blocks_op(const Tensor& x) {
  TORCH_CHECK_VALUE(x.dim() >= 1, "row blocks need at least one axis");
  std::vector<RowBlock> blocks;
  row_blocks(x, blocks);
  std::vector<int64_t> flat;
  for (const auto& b : blocks) {
    flat.push_back(b.off);
    flat.push_back(b.rows);
    flat.push_back(b.stride);
  }
  return flat;
}

std::vector<int64_t> lead_shape(const Tensor& logits) {
  auto s = logits.sizes();
  return std::vector<int64_t>(s.begin(), s.end() - 1);
}

// ------------------------------------------------------------------ log-prob / entropy: plain operators

void check_logits(const Tensor& logits) {
  require_gpu(logits, "logits");
  TORCH_CHECK_TYPE(logits.dim() >= 1, "logits must be a tensor of shape (..., vocab_size)");
  TORCH_CHECK_VALUE(logits.size(-1) >= 1, "logits have an empty vocabulary axis (V=0)");
  const auto t = logits.scalar_type();
  TORCH_CHECK_TYPE(t == at::kFloat || t == at::kBFloat16 || t == at::kHalf, "logits dtype ", t,
                   " is not supported (float32, bfloat16, float16)");
}

std::tuple<Tensor, Tensor, Tensor, Tensor> lpe_fwd(const Tensor& logits, const optional<Tensor>& labels_in,
                                                   double inv_temperature, bool want_entropy) {
  check_logits(logits);
  const auto lead = lead_shape(logits);
  const int64_t V = logits.size(-1);
  const bool want_lp = has(labels_in);
  Tensor labels;
  if (want_lp) {
    TORCH_CHECK_VALUE(labels_in->sizes() == at::IntArrayRef(lead), "labels shape ", labels_in->sizes(),
                      " does not match logits ", logits.sizes());
    labels = *labels_in;
    if (labels.device() != logits.device()) labels = labels.to(logits.device());
    if (labels.scalar_type() != at::kLong) labels = labels.to(at::kLong);
    labels = labels.contiguous();
  }
  const std::vector<int64_t> none{0};
  Tensor lp = empty_f32(want_lp ? at::IntArrayRef(lead) : at::IntArrayRef(none), logits);
  Tensor ent = empty_f32(want_entropy ? at::IntArrayRef(lead) : at::IntArrayRef(none), logits);
  Tensor ex = empty_f32(want_entropy ? at::IntArrayRef(lead) : at::IntArrayRef(none), logits);
  Tensor lse = empty_f32(lead, logits);
  std::vector<RowBlock> blocks;
  row_blocks(logits, blocks);
  const int code = dtype_code(logits.scalar_type());
  const int64_t es = logits.element_size();
  DeviceGuard guard(logits.device());
  siirl_stream_t st = stream_of(logits);
  const char* base = ptr<char>(logits);
  int64_t done = 0;
  for (const auto& b : blocks) {
    if (b.rows == 0) continue;
    int rc = siirl_logprob_entropy_fwd(base + b.off * es, code, b.rows, V, b.stride,
                                       want_lp ? ptr<int64_t>(labels) + done : nullptr, (float)inv_temperature,
                                       want_lp ? ptr<float>(lp) + done : nullptr,
                                       want_entropy ? ptr<float>(ent) + done : nullptr, ptr<float>(lse) + done,
                                       want_entropy ? ptr<float>(ex) + done : nullptr, st);
    check_rc(rc, "siirl_logprob_entropy_fwd");
    done += b.rows;
  }
  return {lp, ent, lse, ex};
}

// writes the gradient of `logits` into `out` (which may be `logits` itself)
void lpe_bwd_launch(const Tensor& logits, const optional<Tensor>& labels_in, double inv_temperature, const Tensor& lse_in,
                    const optional<Tensor>& ex_in, const optional<Tensor>& g_lp_in, const optional<Tensor>& g_ent_in,
                    const Tensor& out, bool skip_zero_rows) {
  check_logits(logits);
  const auto dev = logits.device();
  const int64_t V = logits.size(-1);
  const int64_t es = logits.element_size();
  const int code = dtype_code(logits.scalar_type());
  const optional<Tensor> g_lp = f32c(g_lp_in, dev), g_ent = f32c(g_ent_in, dev), ex = f32c(ex_in, dev);
  const Tensor lse = f32c(lse_in, dev);
  Tensor labels;
  if (has(labels_in)) {
    labels = *labels_in;
    if (labels.device() != dev) labels = labels.to(dev);
    if (labels.scalar_type() != at::kLong) labels = labels.to(at::kLong);
    labels = labels.contiguous();
  }
  TORCH_CHECK_VALUE(!has(g_lp) || labels.defined(), "labels are required with g_logprob");
  TORCH_CHECK_VALUE(!has(g_ent) || has(ex), "ex is required with g_entropy");
  const int64_t rows = logits.numel() / V;
  auto per_row = [&](int64_t n, const char* name) {
    TORCH_CHECK_VALUE(n == rows, "siirl_amd: `", name, "` has ", n, " elements for ", rows, " rows of logits");
  };
  per_row(lse.numel(), "lse");
  if (has(ex)) per_row(ex->numel(), "ex");
  if (has(g_lp)) per_row(g_lp->numel(), "g_logprob");
  if (has(g_ent)) per_row(g_ent->numel(), "g_entropy");
  if (labels.defined()) per_row(labels.numel(), "labels");
  require_on(out, logits, "dlogits");
  TORCH_CHECK_TYPE(out.scalar_type() == logits.scalar_type(), "siirl_amd: dlogits must have the dtype of logits");
  std::vector<RowBlock> in_blocks, out_blocks;
  row_blocks(logits, in_blocks);
  const bool inplace = out.is_same(logits) || (out.data_ptr() == logits.data_ptr() && out.strides() == logits.strides());
  if (inplace) {
    out_blocks = in_blocks;
  } else {  // a fresh contiguous tensor: rows follow one another whatever the blocking of the input
    TORCH_CHECK_VALUE(out.is_contiguous() && out.sizes() == logits.sizes(),
                      "siirl_amd: dlogits must be contiguous and shaped like logits");
    int64_t r = 0;
    for (const auto& b : in_blocks) {
      out_blocks.push_back({r * V, b.rows, V});
      r += b.rows;
    }
  }
  DeviceGuard guard(dev);
  siirl_stream_t st = stream_of(logits);
  const uint32_t flags = skip_zero_rows ? SIIRL_BWD_SKIP_ZERO_ROWS : 0u;
  int64_t done = 0;
  for (size_t i = 0; i < in_blocks.size(); ++i) {
    const auto& b = in_blocks[i];
    if (b.rows == 0) continue;
    int rc = siirl_logprob_entropy_bwd(ptr<char>(logits) + b.off * es, code, b.rows, V, b.stride,
                                       labels.defined() ? ptr<int64_t>(labels) + done : nullptr, (float)inv_temperature,
                                       ptr<float>(lse) + done, has(g_ent) ? ptr<float>(ex) + done : nullptr,
                                       has(g_lp) ? ptr<float>(g_lp) + done : nullptr,
                                       has(g_ent) ? ptr<float>(g_ent) + done : nullptr,
                                       ptr<char>(out) + out_blocks[i].off * es, out_blocks[i].stride, flags, st);
    check_rc(rc, "siirl_logprob_entropy_bwd");
    done += b.rows;
  }
}

Tensor lpe_bwd(const Tensor& logits, const optional<Tensor>& labels, double inv_temperature, const Tensor& lse,
               const optional<Tensor>& ex, const optional<Tensor>& g_lp, const optional<Tensor>& g_ent,
               bool skip_zero_rows) {
  Tensor out = at::empty(logits.sizes(), logits.options().memory_format(c10::MemoryFormat::Contiguous));
  lpe_bwd_launch(logits, labels, inv_temperature, lse, ex, g_lp, g_ent, out, skip_zero_rows);
  return out;
}

void lpe_bwd_inplace(Tensor& logits, const optional<Tensor>& labels, double inv_temperature, const Tensor& lse,
                     const optional<Tensor>& ex, const optional<Tensor>& g_lp, const optional<Tensor>& g_ent,
                     bool skip_zero_rows) {
  lpe_bwd_launch(logits, labels, inv_temperature, lse, ex, g_lp, g_ent, logits, skip_zero_rows);
}

// ------------------------------------------------------------------ log-prob / entropy: differentiable operator

// (logits, labels) -> (logprob, entropy) with one forward pass and one backward pass over the rows.
// `defer`: a one-element int32 CPU tensor the caller keeps; a non-zero value at backward time turns an in-place
// backward into an out-of-place one (the caller found a second reader of the same logits after this node was built).
struct LogprobEntropyFn : public torch::autograd::Function<LogprobEntropyFn> {
  static variable_list forward(AutogradContext* ctx, const Tensor& logits, const optional<Tensor>& labels,
                               double inv_temperature, bool want_entropy, bool inplace_backward, bool skip_zero_rows,
                               const optional<Tensor>& defer) {
    at::AutoDispatchBelowADInplaceOrView below;
    auto [lp, ent, lse, ex] = lpe_fwd(logits, labels, inv_temperature, want_entropy);
    ctx->save_for_backward({logits, has(labels) ? *labels : Tensor(), lse, ex});
    ctx->saved_data["inv_t"] = inv_temperature;
    ctx->saved_data["want_entropy"] = want_entropy;
    ctx->saved_data["inplace"] = inplace_backward;
    ctx->saved_data["skip"] = skip_zero_rows;
    if (has(defer)) ctx->saved_data["defer"] = *defer;
    ctx->set_materialize_grads(false);
    if (!has(labels)) ctx->mark_non_differentiable({lp});
    if (!want_entropy) ctx->mark_non_differentiable({ent});
    return {lp, ent};
  }

  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    const auto saved = ctx->get_saved_variables();
    Tensor logits = saved[0];
    const Tensor& labels = saved[1];
    const Tensor& lse = saved[2];
    const Tensor& ex = saved[3];
    const bool want_entropy = ctx->saved_data["want_entropy"].toBool();
    optional<Tensor> g_lp, g_ent;
    if (labels.defined() && grads[0].defined()) g_lp = grads[0];
    if (want_entropy && grads[1].defined()) g_ent = grads[1];
    variable_list none(7);
    if (!has(g_lp) && !has(g_ent)) return none;
    const double inv_t = ctx->saved_data["inv_t"].toDouble();
    const bool skip = ctx->saved_data["skip"].toBool();
    bool inplace = ctx->saved_data["inplace"].toBool();
    auto it = ctx->saved_data.find("defer");
    if (inplace && it != ctx->saved_data.end() && it->second.toTensor().item<int>() != 0) inplace = false;
    at::AutoDispatchBelowADInplaceOrView below;
    // (the labels go along without a log-prob gradient too: they mark the rows the forward skipped)
    const optional<Tensor> lab = labels.defined() ? optional<Tensor>(labels) : c10::nullopt;
    const optional<Tensor> exo = has(g_ent) ? optional<Tensor>(ex) : c10::nullopt;
    if (inplace) {
      lpe_bwd_inplace(logits, lab, inv_t, lse, exo, g_lp, g_ent, skip);
      torch::autograd::impl::bump_version(logits);  // the saved activation now holds its own gradient
      none[0] = logits;
    } else {
      none[0] = lpe_bwd(logits, lab, inv_t, lse, exo, g_lp, g_ent, skip);
    }
    return none;
  }
};

std::tuple<Tensor, Tensor> logprob_entropy(const Tensor& logits, const optional<Tensor>& labels, double inv_temperature,
                                           bool want_entropy, bool inplace_backward, bool skip_zero_rows,
                                           const optional<Tensor>& defer) {
  auto out = LogprobEntropyFn::apply(logits, labels, inv_temperature, want_entropy, inplace_backward, skip_zero_rows,
                                     defer);
  return {out[0], out[1]};
}

// ------------------------------------------------------------------ group operators

Tensor grpo_advantage(const Tensor& rewards, const Tensor& mask, const Tensor& uid, double epsilon, bool norm_by_std) {
  require_f32c(rewards, "token_level_rewards");
  TORCH_CHECK_VALUE(rewards.dim() == 2, "token_level_rewards must be [B, L]");
  const int64_t B = rewards.size(0), L = rewards.size(1);
  TORCH_CHECK_VALUE(uid.scalar_type() == at::kLong && uid.numel() == B && mask.dim() == 2 && mask.size(0) == B &&
                        mask.size(1) == L, "siirl_amd: uid must be int64 [B] and mask [B, L]");
  require_on(mask, rewards, "mask");
  require_on(uid, rewards, "uid");
  Tensor adv = empty_f32({B, L}, rewards);
  Tensor scratch = empty_f32({2 * std::max<int64_t>(B, 1)}, rewards);
  Tensor u = uid.contiguous();
  DeviceGuard guard(rewards.device());
  check_rc(siirl_grpo_outcome_advantage(ptr<float>(rewards), ptr(mask), mask_code(mask), ptr<int64_t>(u), B, L,
                                        (float)epsilon, (int)norm_by_std, ptr<float>(adv), ptr<float>(scratch),
                                        stream_of(rewards)),
           "siirl_grpo_outcome_advantage");
  return adv;
}

std::tuple<Tensor, Tensor> group_keep_mask(const Tensor& metric, const Tensor& uid) {
  require_gpu(metric, "metric");
  const int64_t B = uid.numel();
  TORCH_CHECK_VALUE(metric.numel() == B && uid.scalar_type() == at::kLong,
                    "siirl_amd: metric and uid must have one entry per trajectory, uid int64");
  require_on(uid, metric, "uid");
  Tensor keep = at::empty({B}, metric.options().dtype(at::kByte));
  Tensor gsz = at::empty({B}, metric.options().dtype(at::kInt));
  Tensor met = metric.contiguous(), u = uid.contiguous();
  DeviceGuard guard(metric.device());
  check_rc(siirl_group_keep_mask(ptr(met), dtype_code(met.scalar_type()), ptr<int64_t>(u), B, ptr<uint8_t>(keep),
                                 ptr<int32_t>(gsz), stream_of(metric)),
           "siirl_group_keep_mask");
  return {keep, gsz};
}

// ------------------------------------------------------------------ aggregation

std::tuple<Tensor, Tensor> agg_loss_fwd(const Tensor& loss_mat, const Tensor& mask, int64_t agg_mode) {
  require_f32c(loss_mat, "loss_mat");
  TORCH_CHECK_VALUE(loss_mat.dim() == 2, "loss_mat must be [B, L]");
  require_mask(mask, loss_mat);
  const int64_t B = loss_mat.size(0), L = loss_mat.size(1);
  Tensor out16 = empty_f32({16}, loss_mat), row_msum = empty_f32({B}, loss_mat);
  size_t nws;
  Tensor ws = loss_workspace(B, L, loss_mat, &nws);
  DeviceGuard guard(loss_mat.device());
  check_rc(siirl_agg_loss_fwd(ptr<float>(loss_mat), ptr(mask), mask_code(mask), B, L, (int)agg_mode, ptr<float>(out16),
                              ptr<float>(row_msum), ptr(ws), nws, stream_of(loss_mat)),
           "siirl_agg_loss_fwd");
  return {out16, row_msum};
}

Tensor agg_loss_bwd(const Tensor& g, const Tensor& mask, const Tensor& out16, const Tensor& row_msum, int64_t agg_mode) {
  TORCH_CHECK_VALUE(mask.dim() == 2, "mask must be [B, L]");
  const int64_t B = mask.size(0), L = mask.size(1);
  require_f32c(g, "g");
  TORCH_CHECK_VALUE(g.numel() == 1, "siirl_amd: `g` is the gradient of the scalar loss (one element)");
  require_f32_n(out16, 16, g, "out16");
  require_f32_n(row_msum, B, g, "row_msum");
  require_on(mask, g, "mask");
  Tensor d = empty_f32({B, L}, out16);
  DeviceGuard guard(out16.device());
  check_rc(siirl_agg_loss_bwd(ptr<float>(g), ptr(mask), mask_code(mask), ptr<float>(out16), ptr<float>(row_msum), B, L,
                              (int)agg_mode, ptr<float>(d), stream_of(out16)),
           "siirl_agg_loss_bwd");
  return d;
}

Tensor scalar_grad(const Tensor& g) {  // upstream gradient of a 0-d output as a one-element fp32 device buffer
  Tensor r = g.detach();
  if (r.scalar_type() != at::kFloat) r = r.to(at::kFloat);
  return r.reshape({1}).contiguous();
}

struct AggLossFn : public torch::autograd::Function<AggLossFn> {
  static Tensor forward(AutogradContext* ctx, const Tensor& loss_mat, const Tensor& loss_mask, int64_t agg_mode) {
    at::AutoDispatchBelowADInplaceOrView below;
    require_gpu(loss_mat, "loss_mat");
    const auto dev = loss_mat.device();
    Tensor v = as_2d(f32c(loss_mat, dev));
    Tensor m = as_2d(mask_arg(loss_mask, dev));
    if (m.sizes() != v.sizes()) m = m.expand(v.sizes()).contiguous();
    auto [out16, row_msum] = agg_loss_fwd(v, m, agg_mode);
    ctx->save_for_backward({m, out16, row_msum});
    ctx->saved_data["agg"] = agg_mode;
    ctx->saved_data["shape"] = loss_mat.sizes().vec();
    ctx->saved_data["dtype"] = (int64_t)loss_mat.scalar_type();
    return out16.select(0, SIIRL_OUT_PG_LOSS);
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    const auto saved = ctx->get_saved_variables();
    at::AutoDispatchBelowADInplaceOrView below;
    Tensor d = agg_loss_bwd(scalar_grad(grads[0]), saved[0], saved[1], saved[2], ctx->saved_data["agg"].toInt());
    d = d.reshape(ctx->saved_data["shape"].toIntVector());
    const auto dt = (at::ScalarType)ctx->saved_data["dtype"].toInt();
    if (dt != at::kFloat) d = d.to(dt);
    return {d, Tensor(), Tensor()};
  }
};

Tensor agg_loss(const Tensor& loss_mat, const Tensor& loss_mask, int64_t agg_mode) {
  return AggLossFn::apply(loss_mat, loss_mask, agg_mode);
}

// ------------------------------------------------------------------ masked_sum / masked_mean

// values, mask: [B, L] -> (result, mask sums): per_row ? ([B], [B]) : ({sum, mean}, [1]).  The mean divides by
// (sum of the mask + 1e-8); the mask sums are what the backward divides by.
std::tuple<Tensor, Tensor> masked_reduce_fwd(const Tensor& values, const Tensor& mask, bool per_row, bool want_mean) {
  require_f32c(values, "values");
  TORCH_CHECK_VALUE(values.dim() == 2 && mask.sizes() == values.sizes(), "values and mask must be [B, L]");
  require_on(mask, values, "mask");
  const int64_t B = values.size(0), L = values.size(1);
  size_t nws;
  Tensor ws = loss_workspace(B, L, values, &nws);
  Tensor out = empty_f32({per_row ? B : 2}, values);
  Tensor msum = empty_f32({per_row ? B : 1}, values);
  if (per_row && B == 0) return {out, msum};  // no rows: nothing to reduce, nothing to launch
  DeviceGuard guard(values.device());
  check_rc(siirl_masked_reduce(ptr<float>(values), ptr(mask), mask_code(mask), B, L,
                               (per_row && !want_mean) ? ptr<float>(out) : nullptr,
                               (per_row && want_mean) ? ptr<float>(out) : nullptr, per_row ? nullptr : ptr<float>(out),
                               per_row ? ptr<float>(msum) : nullptr, per_row ? nullptr : ptr<float>(msum), ptr(ws), nws,
                               stream_of(values)),
           "siirl_masked_reduce");
  return {out, msum};
}

// d values[b, t] = g[b or 0] * mask[b, t] (/ (mask_sums[b or 0] + 1e-8) for the mean)
Tensor masked_reduce_bwd(const Tensor& g, const Tensor& mask, bool per_row, const optional<Tensor>& mask_sums) {
  TORCH_CHECK_VALUE(mask.dim() == 2, "mask must be [B, L]");
  const int64_t B = mask.size(0), L = mask.size(1);
  require_f32c(g, "g");
  require_f32c(mask_sums, "mask_sums");
  require_on(mask, g, "mask");
  if (has(mask_sums)) require_on(*mask_sums, g, "mask_sums");
  TORCH_CHECK_VALUE(g.numel() == (per_row ? B : 1) && (!has(mask_sums) || mask_sums->numel() == g.numel()),
                    "g and mask_sums must have one entry per reduced row");
  Tensor d = empty_f32({B, L}, g);
  DeviceGuard guard(g.device());
  check_rc(siirl_masked_reduce_bwd(ptr<float>(g), ptr(mask), mask_code(mask), B, L, (int)per_row, ptr<float>(mask_sums),
                                   ptr<float>(d), stream_of(g)),
           "siirl_masked_reduce_bwd");
  return d;
}

struct MaskedReduceFn : public torch::autograd::Function<MaskedReduceFn> {
  static Tensor forward(AutogradContext* ctx, const Tensor& values2d, const Tensor& mask2d, bool per_row,
                        bool want_mean) {
    at::AutoDispatchBelowADInplaceOrView below;
    auto [out, msum] = masked_reduce_fwd(values2d, mask2d, per_row, want_mean);
    ctx->save_for_backward({mask2d, want_mean ? msum : Tensor()});
    ctx->saved_data["per_row"] = per_row;
    return per_row ? out : out.select(0, want_mean ? 1 : 0);
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    const auto saved = ctx->get_saved_variables();
    at::AutoDispatchBelowADInplaceOrView below;
    Tensor g = grads[0].detach();
    if (g.scalar_type() != at::kFloat) g = g.to(at::kFloat);
    g = g.reshape({-1}).contiguous();
    optional<Tensor> msum;
    if (saved[1].defined()) msum = saved[1];
    return {masked_reduce_bwd(g, saved[0], ctx->saved_data["per_row"].toBool(), msum), Tensor(), Tensor(), Tensor()};
  }
};

// values / mask of any shape (mask broadcastable); `axes` empty = all elements.  fp32 result.
Tensor masked_reduce(const Tensor& values, const Tensor& mask, at::IntArrayRef axes, bool want_mean) {
  require_gpu(values, "values");
  const auto dev = values.device();
  const int64_t nd = values.dim();
  std::vector<bool> red(nd, axes.empty());
  for (int64_t a : axes) red[at::maybe_wrap_dim(a, nd)] = true;
  bool all = true;
  for (bool r : red) all = all && r;
  Tensor v = values;
  if (v.scalar_type() != at::kFloat) v = v.to(at::kFloat);
  Tensor m = mask_arg(mask, dev);
  if (m.sizes() != v.sizes()) m = m.expand(v.sizes());
  std::vector<int64_t> keep_shape;
  if (all || nd == 0) {
    if (v.numel() == 0) {  // the sum of nothing: B = 0 rows of one element
      v = v.reshape({0, 1});
      m = m.reshape({0, 1});
    } else {
      // rows for the kernels' two-level fold: the tensor's own last axis, or a power of two that divides the count
      // (one row of millions of tokens would leave the fold of its segments to a single thread)
      const int64_t n = v.numel();
      int64_t cols = nd >= 2 && v.size(-1) >= 256 ? v.size(-1) : n;
      if (cols == n && n > (1 << 16))
        for (int64_t c = 8192; c >= 256; c >>= 1)
          if (n % c == 0) { cols = c; break; }
      v = v.reshape({n / cols, cols});
      m = m.reshape({n / cols, cols});
    }
  } else {
    std::vector<int64_t> perm;
    int64_t n_red = 1;
    for (int64_t d = 0; d < nd; ++d)
      if (!red[d]) { perm.push_back(d); keep_shape.push_back(v.size(d)); }
    for (int64_t d = 0; d < nd; ++d)
      if (red[d]) { perm.push_back(d); n_red *= v.size(d); }
    if (n_red == 0) return at::zeros(keep_shape, v.options()) + v.sum() * 0;  // empty reduced extent: zeros
    v = v.permute(perm).reshape({-1, n_red});
    m = m.permute(perm).reshape({-1, n_red});
  }
  v = v.contiguous();
  m = m.contiguous();
  Tensor out = MaskedReduceFn::apply(v, m, !(all || nd == 0), want_mean);
  if (!(all || nd == 0)) out = out.reshape(keep_shape);
  return out;
}

// ------------------------------------------------------------------ the actor's loss

struct LossCfg {
  int64_t loss_mode, agg_mode, kl_mode;
  double clip_low, clip_high, clip_c, log_ratio_clamp, entropy_coeff, kl_coef, drift_coef, scale;
  bool kl_st;
};

bool is_cov_loss(int64_t loss_mode) { return loss_mode == SIIRL_LOSS_KL_COV || loss_mode == SIIRL_LOSS_CLIP_COV; }

void policy_loss_fwd_launch(const Tensor& old, const Tensor& lp, const Tensor& adv, const Tensor& mask,
                            const optional<Tensor>& isw, const optional<Tensor>& ent, const optional<Tensor>& ref,
                            const optional<Tensor>& aux, const LossCfg& c, float* out16, float* row_msum, float* row_s,
                            void* ws, size_t nws) {
  require_f32c(lp, "log_prob");
  require_f32c(old, "old_log_prob");
  require_f32c(adv, "advantages");
  require_f32c(isw, "is_weights");
  require_f32c(ent, "entropy");
  require_f32c(ref, "ref_log_prob");
  TORCH_CHECK_VALUE(lp.dim() == 2, "log_prob must be [B, L]");
  require_f32_like(old, lp, "old_log_prob");
  require_f32_like(adv, lp, "advantages");
  require_f32_like(isw, lp, "is_weights");
  require_f32_like(ent, lp, "entropy");
  require_f32_like(ref, lp, "ref_log_prob");
  require_mask(mask, lp);
  require_f32_like(aux, lp, "token_aux");
  TORCH_CHECK_VALUE(has(aux) == is_cov_loss(c.loss_mode), "siirl_amd: token_aux goes with the kl_cov and clip_cov losses");
  const int64_t B = lp.size(0), L = lp.size(1);
  DeviceGuard guard(lp.device());
  if (has(aux)) {
    check_rc(siirl_actor_loss_cov_fwd(ptr<float>(old), ptr<float>(lp), ptr<float>(adv), ptr(mask), mask_code(mask),
                                      ptr<float>(isw), ptr<float>(ent), ptr<float>(ref), ptr<float>(aux), B, L,
                                      (int)c.loss_mode, (float)c.clip_low, (float)c.clip_high, (int)c.agg_mode,
                                      (float)c.entropy_coeff, (int)c.kl_mode, (int)c.kl_st, (float)c.kl_coef,
                                      (float)c.drift_coef, (float)c.scale, out16, row_msum, ws, nws, stream_of(lp)),
             "siirl_actor_loss_cov_fwd");
    return;
  }
  check_rc(siirl_actor_loss_fwd(ptr<float>(old), ptr<float>(lp), ptr<float>(adv), ptr(mask), mask_code(mask),
                                ptr<float>(isw), ptr<float>(ent), ptr<float>(ref), B, L, (int)c.loss_mode,
                                (float)c.clip_low, (float)c.clip_high, (float)c.clip_c, (float)c.log_ratio_clamp,
                                (int)c.agg_mode, (float)c.entropy_coeff, (int)c.kl_mode, (int)c.kl_st, (float)c.kl_coef,
                                (float)c.drift_coef, (float)c.scale, out16, row_msum, row_s, ws, nws, stream_of(lp)),
           "siirl_actor_loss_fwd");
}

std::tuple<Tensor, Tensor, Tensor> policy_loss_fwd_impl(const Tensor& old, const Tensor& lp, const Tensor& adv,
                                                        const Tensor& mask, const optional<Tensor>& isw,
                                                        const optional<Tensor>& ent, const optional<Tensor>& ref,
                                                        const optional<Tensor>& aux, const LossCfg& c) {
  TORCH_CHECK_VALUE(lp.dim() == 2, "log_prob must be [B, L]");
  const int64_t B = lp.size(0), L = lp.size(1);
  Tensor out16 = empty_f32({16}, lp), row_msum = empty_f32({B}, lp), row_s = empty_f32({B}, lp);
  size_t nws;
  Tensor ws = loss_workspace(B, L, lp, &nws);
  policy_loss_fwd_launch(old, lp, adv, mask, isw, ent, ref, aux, c, ptr<float>(out16), ptr<float>(row_msum),
                         ptr<float>(row_s), ptr(ws), nws);
  return {out16, row_msum, row_s};
}

std::tuple<Tensor, Tensor> policy_loss_bwd_impl(const Tensor& g, const Tensor& old, const Tensor& lp, const Tensor& adv,
                                                const Tensor& mask, const optional<Tensor>& isw,
                                                const optional<Tensor>& ent, const optional<Tensor>& ref,
                                                const optional<Tensor>& aux, const LossCfg& c, const Tensor& out16,
                                                const Tensor& row_msum, const Tensor& row_s) {
  require_f32c(lp, "log_prob");
  require_f32c(g, "g_loss");
  require_f32c(old, "old_log_prob");
  require_f32c(adv, "advantages");
  require_f32c(isw, "is_weights");
  require_f32c(ent, "entropy");
  require_f32c(ref, "ref_log_prob");
  TORCH_CHECK_VALUE(lp.dim() == 2, "log_prob must be [B, L]");
  require_f32_like(old, lp, "old_log_prob");
  require_f32_like(adv, lp, "advantages");
  require_f32_like(isw, lp, "is_weights");
  require_f32_like(ent, lp, "entropy");
  require_f32_like(ref, lp, "ref_log_prob");
  require_mask(mask, lp);
  const int64_t B = lp.size(0), L = lp.size(1);
  require_f32_n(g, 1, lp, "g_loss");
  require_f32_n(out16, 16, lp, "out16");
  require_f32_n(row_msum, B, lp, "row_msum");
  require_f32_n(row_s, B, lp, "row_s");
  require_f32_like(aux, lp, "token_aux");
  TORCH_CHECK_VALUE(has(aux) == is_cov_loss(c.loss_mode), "siirl_amd: token_aux goes with the kl_cov and clip_cov losses");
  Tensor d_lp = empty_f32({B, L}, lp);
  const std::vector<int64_t> full{B, L}, none{0};
  Tensor d_ent = empty_f32(has(ent) ? at::IntArrayRef(full) : at::IntArrayRef(none), lp);
  DeviceGuard guard(lp.device());
  if (has(aux)) {
    check_rc(siirl_actor_loss_cov_bwd(ptr<float>(g), ptr<float>(old), ptr<float>(lp), ptr<float>(adv), ptr(mask),
                                      mask_code(mask), ptr<float>(isw), ptr<float>(ent), ptr<float>(ref),
                                      ptr<float>(aux), B, L, (int)c.loss_mode, (float)c.clip_low, (float)c.clip_high,
                                      (int)c.agg_mode, (float)c.entropy_coeff, (int)c.kl_mode, (int)c.kl_st,
                                      (float)c.kl_coef, (float)c.drift_coef, (float)c.scale, ptr<float>(out16),
                                      ptr<float>(row_msum), ptr<float>(d_lp), has(ent) ? ptr<float>(d_ent) : nullptr,
                                      stream_of(lp)),
             "siirl_actor_loss_cov_bwd");
    return {d_lp, d_ent};
  }
  check_rc(siirl_actor_loss_bwd(ptr<float>(g), ptr<float>(old), ptr<float>(lp), ptr<float>(adv), ptr(mask),
                                mask_code(mask), ptr<float>(isw), ptr<float>(ent), ptr<float>(ref), B, L,
                                (int)c.loss_mode, (float)c.clip_low, (float)c.clip_high, (float)c.clip_c,
                                (float)c.log_ratio_clamp, (int)c.agg_mode, (float)c.entropy_coeff, (int)c.kl_mode,
                                (int)c.kl_st, (float)c.kl_coef, (float)c.drift_coef, (float)c.scale, ptr<float>(out16),
                                ptr<float>(row_msum), ptr<float>(row_s), ptr<float>(d_lp),
                                has(ent) ? ptr<float>(d_ent) : nullptr, stream_of(lp)),
           "siirl_actor_loss_bwd");
  return {d_lp, d_ent};
}

std::tuple<Tensor, Tensor, Tensor> policy_loss_fwd(const Tensor& old, const Tensor& lp, const Tensor& adv,
                                                   const Tensor& mask, const optional<Tensor>& isw,
                                                   const optional<Tensor>& ent, const optional<Tensor>& ref,
                                                   int64_t loss_mode, double clip_low, double clip_high, double clip_c,
                                                   double log_ratio_clamp, int64_t agg_mode, double entropy_coeff,
                                                   int64_t kl_mode, bool kl_st, double kl_coef, double drift_coef,
                                                   double scale, const optional<Tensor>& aux) {
  return policy_loss_fwd_impl(old, lp, adv, mask, isw, ent, ref, aux,
                              LossCfg{loss_mode, agg_mode, kl_mode, clip_low, clip_high, clip_c, log_ratio_clamp,
                                      entropy_coeff, kl_coef, drift_coef, scale, kl_st});
}

std::tuple<Tensor, Tensor> policy_loss_bwd(const Tensor& g, const Tensor& old, const Tensor& lp, const Tensor& adv,
                                           const Tensor& mask, const optional<Tensor>& isw, const optional<Tensor>& ent,
                                           const optional<Tensor>& ref, int64_t loss_mode, double clip_low,
                                           double clip_high, double clip_c, double log_ratio_clamp, int64_t agg_mode,
                                           double entropy_coeff, int64_t kl_mode, bool kl_st, double kl_coef,
                                           double drift_coef, double scale, const Tensor& out16, const Tensor& row_msum,
                                           const Tensor& row_s, const optional<Tensor>& aux) {
  return policy_loss_bwd_impl(g, old, lp, adv, mask, isw, ent, ref, aux,
                              LossCfg{loss_mode, agg_mode, kl_mode, clip_low, clip_high, clip_c, log_ratio_clamp,
                                      entropy_coeff, kl_coef, drift_coef, scale, kl_st},
                              out16, row_msum, row_s);
}

// Scores that the covariance losses pick their tokens from: (cov [B, L], stats {count of mask > 0, sum of the mask,
// mean advantage, mean log-prob, float32 residues of the first two}).  No gradient: the pick is a set of indices.
std::tuple<Tensor, Tensor> cov_scores(const optional<Tensor>& old, const Tensor& lp, const Tensor& adv, const Tensor& mask,
                                      int64_t loss_mode, double clip_low, double clip_high) {
  require_f32c(lp, "log_prob");
  TORCH_CHECK_VALUE(lp.dim() == 2, "log_prob must be [B, L]");
  require_f32_like(adv, lp, "advantages");
  require_f32_like(old, lp, "old_log_prob");
  require_mask(mask, lp);
  TORCH_CHECK_VALUE(is_cov_loss(loss_mode), "siirl_amd: covariance scores belong to the kl_cov and clip_cov losses");
  TORCH_CHECK_VALUE(loss_mode != SIIRL_LOSS_CLIP_COV || has(old), "siirl_amd: clip_cov needs old_log_prob");
  const int64_t B = lp.size(0), L = lp.size(1);
  Tensor cov = at::empty_like(lp), stats = empty_f32({6}, lp);
  const size_t nws = siirl_cov_workspace_bytes();
  Tensor ws = at::empty({(int64_t)nws}, lp.options().dtype(at::kByte));
  DeviceGuard guard(lp.device());
  check_rc(siirl_cov_scores(ptr<float>(old), ptr<float>(lp), ptr<float>(adv), ptr(mask), mask_code(mask), B, L,
                            (int)loss_mode, (float)clip_low, (float)clip_high, ptr<float>(cov), ptr<float>(stats),
                            ptr(ws), nws, stream_of(lp)),
           "siirl_cov_scores");
  return {cov, stats};
}

// marks (shaped like scores): `value` at the k largest scores, 0 elsewhere
Tensor topk_mark(const Tensor& scores, int64_t k, double value) {
  require_f32c(scores, "scores");
  const int64_t n = scores.numel();
  TORCH_CHECK(k >= 0 && k <= n, "siirl_amd: k=", k, " is out of range for ", n, " scores");  // torch.topk: RuntimeError
  Tensor marks = at::empty_like(scores);
  const size_t nws = siirl_topk_mark_workspace_bytes();
  Tensor ws = at::empty({(int64_t)nws}, scores.options().dtype(at::kByte));
  DeviceGuard guard(scores.device());
  check_rc(siirl_topk_mark(ptr<float>(scores), n, k, (float)value, ptr<float>(marks), ptr(ws), nws, stream_of(scores)),
           "siirl_topk_mark");
  return marks;
}

// int64 flat indices, ascending, of the scores inside the open interval (lower, upper).  One host sync: the length
// of the list, as torch.nonzero has.
Tensor range_indices(const Tensor& scores, double lower, double upper) {
  require_f32c(scores, "scores");
  const int64_t n = scores.numel();
  const size_t nws = siirl_range_select_workspace_bytes();
  Tensor ws = at::empty({(int64_t)nws + 4}, scores.options().dtype(at::kByte));  // chunk counts, then the total
  uint32_t* count = reinterpret_cast<uint32_t*>(ptr<char>(ws) + nws);
  DeviceGuard guard(scores.device());
  siirl_stream_t st = stream_of(scores);
  check_rc(siirl_range_select_count(ptr<float>(scores), n, (float)lower, (float)upper, count, ptr(ws), nws, st),
           "siirl_range_select_count");
  const int64_t total = (int64_t)ws.narrow(0, (int64_t)nws, 4).view(at::kInt).item<int32_t>() & 0xffffffffLL;
  Tensor idx = at::empty({total}, scores.options().dtype(at::kLong));
  check_rc(siirl_range_select_write(ptr<float>(scores), n, (float)lower, (float)upper, ptr(ws), ptr<int64_t>(idx),
                                    total, st),
           "siirl_range_select_write");
  return idx;
}

constexpr int kActorOuts = 13;  // SIIRL_OUT_LOSS .. SIIRL_OUT_DRIFT_LOSS

// One fused forward (partials + finish) and one elementwise backward for the whole micro-batch loss.  The 13 scalars
// of the result block are the outputs; the gradient enters through pg_loss (`policy_only`) or through the scaled
// total; the other scalars are metrics.
struct ActorLossFn : public torch::autograd::Function<ActorLossFn> {
  static variable_list forward(AutogradContext* ctx, const Tensor& log_prob, const optional<Tensor>& entropy,
                               const Tensor& old_log_prob, const Tensor& advantages, const Tensor& response_mask,
                               const optional<Tensor>& is_weights, const optional<Tensor>& ref_log_prob,
                               int64_t loss_mode, double clip_low, double clip_high, double clip_c,
                               double log_ratio_clamp, int64_t agg_mode, double entropy_coeff, int64_t kl_mode,
                               bool kl_st, double kl_coef, double drift_coef, double scale, bool policy_only,
                               const optional<Tensor>& token_aux) {
    at::AutoDispatchBelowADInplaceOrView below;
    require_gpu(log_prob, "log_prob");
    const auto dev = log_prob.device();
    Tensor lp = as_2d(f32c(log_prob, dev));
    const auto shape = lp.sizes();
    Tensor old = as_2d(f32c(old_log_prob, dev)), adv = as_2d(f32c(advantages, dev));
    Tensor m = as_2d(mask_arg(response_mask, dev));
    optional<Tensor> isw, ent, ref, aux;
    if (has(is_weights)) isw = as_2d(f32c(*is_weights, dev));
    if (has(entropy)) ent = as_2d(f32c(*entropy, dev));
    if (has(ref_log_prob)) ref = as_2d(f32c(*ref_log_prob, dev));
    if (has(token_aux)) aux = as_2d(f32c(*token_aux, dev));
    auto same = [&](const Tensor& t, const char* name) {
      TORCH_CHECK_VALUE(t.sizes() == shape, name, " has shape ", t.sizes(), ", expected ", shape);
    };
    same(old, "old_log_prob");
    same(adv, "advantages");
    same(m, "response_mask");
    if (isw) same(*isw, "rollout_is_weights");
    if (ent) same(*ent, "entropy");
    if (ref) same(*ref, "ref_log_prob");
    if (aux) same(*aux, "token_aux");
    const LossCfg c{loss_mode, agg_mode, kl_mode, clip_low, clip_high, clip_c, log_ratio_clamp, entropy_coeff,
                    kl_coef, drift_coef, scale, kl_st};
    // one allocation for the result block, the two per-row vectors kept for the backward, and the scratch
    // (64 floats | B | B | workspace at a 256-byte boundary of a 512-byte aligned block)
    TORCH_CHECK_VALUE(lp.dim() == 2, "log_prob must be [B, L]");
    const int64_t B = lp.size(0), L = lp.size(1);
    const size_t nws = siirl_loss_workspace_bytes(B, L);
    const int64_t head = (64 + 2 * B + 63) / 64 * 64;  // floats before the workspace
    Tensor buf = empty_f32({head + (int64_t)((nws + 3) / 4)}, lp);
    Tensor out16 = buf.narrow(0, 0, 16), row_msum = buf.narrow(0, 64, B), row_s = buf.narrow(0, 64 + B, B);
    policy_loss_fwd_launch(old, lp, adv, m, isw, ent, ref, aux, c, ptr<float>(out16), ptr<float>(row_msum),
                           ptr<float>(row_s), ptr<float>(buf) + head, nws);
    ctx->save_for_backward({lp, old, adv, m, out16, row_msum, row_s, isw ? *isw : Tensor(), ent ? *ent : Tensor(),
                            ref ? *ref : Tensor(), aux ? *aux : Tensor()});
    ctx->saved_data["i"] = std::vector<int64_t>{loss_mode, agg_mode, kl_mode, (int64_t)kl_st, (int64_t)policy_only,
                                                (int64_t)log_prob.scalar_type(),
                                                has(entropy) ? (int64_t)entropy->scalar_type() : -1};
    ctx->saved_data["d"] = std::vector<double>{clip_low, clip_high, clip_c, log_ratio_clamp, entropy_coeff, kl_coef,
                                               drift_coef, scale};
    ctx->saved_data["lp_shape"] = log_prob.sizes().vec();
    if (has(entropy)) ctx->saved_data["ent_shape"] = entropy->sizes().vec();
    ctx->set_materialize_grads(false);
    variable_list outs = out16.unbind(0);
    outs.resize(kActorOuts);
    const int diff = policy_only ? SIIRL_OUT_PG_LOSS : SIIRL_OUT_LOSS;
    variable_list nondiff;
    for (int i = 0; i < kActorOuts; ++i)
      if (i != diff) nondiff.push_back(outs[i]);
    ctx->mark_non_differentiable(nondiff);
    return outs;
  }

  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    const auto iv = ctx->saved_data["i"].toIntVector();
    const auto dv = ctx->saved_data["d"].toDoubleVector();
    const bool policy_only = iv[4] != 0;
    const Tensor& g_in = grads[policy_only ? SIIRL_OUT_PG_LOSS : SIIRL_OUT_LOSS];
    variable_list none(21);
    if (!g_in.defined()) return none;
    const auto s = ctx->get_saved_variables();
    at::AutoDispatchBelowADInplaceOrView below;
    const LossCfg c{iv[0], iv[1], iv[2], dv[0], dv[1], dv[2], dv[3], dv[4], dv[5], dv[6], dv[7], iv[3] != 0};
    optional<Tensor> isw, ent, ref, aux;
    if (s[7].defined()) isw = s[7];
    if (s[8].defined()) ent = s[8];
    if (s[9].defined()) ref = s[9];
    if (s[10].defined()) aux = s[10];
    auto [d_lp, d_ent] = policy_loss_bwd_impl(scalar_grad(g_in), s[1], s[0], s[2], s[3], isw, ent, ref, aux, c, s[4],
                                              s[5], s[6]);
    d_lp = d_lp.reshape(ctx->saved_data["lp_shape"].toIntVector());
    if ((at::ScalarType)iv[5] != at::kFloat) d_lp = d_lp.to((at::ScalarType)iv[5]);
    none[0] = d_lp;
    if (ent) {
      d_ent = d_ent.reshape(ctx->saved_data["ent_shape"].toIntVector());
      if ((at::ScalarType)iv[6] != at::kFloat) d_ent = d_ent.to((at::ScalarType)iv[6]);
      none[1] = d_ent;
    }
    return none;
  }
};

std::vector<Tensor> actor_loss(const Tensor& log_prob, const optional<Tensor>& entropy, const Tensor& old_log_prob,
                               const Tensor& advantages, const Tensor& response_mask,
                               const optional<Tensor>& is_weights, const optional<Tensor>& ref_log_prob,
                               int64_t loss_mode, double clip_low, double clip_high, double clip_c,
                               double log_ratio_clamp, int64_t agg_mode, double entropy_coeff, int64_t kl_mode,
                               bool kl_st, double kl_coef, double drift_coef, double scale, bool policy_only,
                               const optional<Tensor>& token_aux) {
  return ActorLossFn::apply(log_prob, entropy, old_log_prob, advantages, response_mask, is_weights, ref_log_prob,
                            loss_mode, clip_low, clip_high, clip_c, log_ratio_clamp, agg_mode, entropy_coeff, kl_mode,
                            kl_st, kl_coef, drift_coef, scale, policy_only, token_aux);
}

// ------------------------------------------------------------------ value loss

struct ValueLossFn : public torch::autograd::Function<ValueLossFn> {
  static variable_list forward(AutogradContext* ctx, const Tensor& vpreds, const Tensor& returns, const Tensor& values,
                               const Tensor& response_mask, double cliprange_value, int64_t agg_mode) {
    at::AutoDispatchBelowADInplaceOrView below;
    require_gpu(vpreds, "vpreds");
    const auto dev = vpreds.device();
    Tensor vp = as_2d(f32c(vpreds, dev)), ret = as_2d(f32c(returns, dev)), val = as_2d(f32c(values, dev));
    Tensor m = as_2d(mask_arg(response_mask, dev));
    const int64_t B = vp.size(0), L = vp.size(1);
    TORCH_CHECK_VALUE(ret.sizes() == vp.sizes(), "returns has shape ", ret.sizes(), ", expected ", vp.sizes());
    TORCH_CHECK_VALUE(val.sizes() == vp.sizes(), "values has shape ", val.sizes(), ", expected ", vp.sizes());
    TORCH_CHECK_VALUE(m.sizes() == vp.sizes(), "response_mask has shape ", m.sizes(), ", expected ", vp.sizes());
    Tensor out16 = empty_f32({16}, vp), row_msum = empty_f32({B}, vp);
    size_t nws;
    Tensor ws = loss_workspace(B, L, vp, &nws);
    {
      DeviceGuard guard(dev);
      check_rc(siirl_value_loss_fwd(ptr<float>(vp), ptr<float>(ret), ptr<float>(val), ptr(m), mask_code(m), B, L,
                                    (float)cliprange_value, (int)agg_mode, ptr<float>(out16), ptr<float>(row_msum),
                                    ptr(ws), nws, stream_of(vp)),
               "siirl_value_loss_fwd");
    }
    ctx->save_for_backward({vp, ret, val, m, out16, row_msum});
    ctx->saved_data["clip"] = cliprange_value;
    ctx->saved_data["agg"] = agg_mode;
    ctx->saved_data["shape"] = vpreds.sizes().vec();
    ctx->saved_data["dtype"] = (int64_t)vpreds.scalar_type();
    Tensor loss = out16.select(0, SIIRL_OUT_LOSS), frac = out16.select(0, SIIRL_OUT_PG_CLIPFRAC);
    ctx->mark_non_differentiable({frac});
    return {loss, frac};
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    variable_list none(6);
    if (!grads[0].defined()) return none;
    const auto s = ctx->get_saved_variables();
    at::AutoDispatchBelowADInplaceOrView below;
    const Tensor& vp = s[0];
    const int64_t B = vp.size(0), L = vp.size(1);
    Tensor g = scalar_grad(grads[0]);
    Tensor d = empty_f32({B, L}, vp);
    {
      DeviceGuard guard(vp.device());
      check_rc(siirl_value_loss_bwd(ptr<float>(g), ptr<float>(vp), ptr<float>(s[1]), ptr<float>(s[2]), ptr(s[3]),
                                    mask_code(s[3]), B, L, (float)ctx->saved_data["clip"].toDouble(),
                                    (int)ctx->saved_data["agg"].toInt(), ptr<float>(s[4]), ptr<float>(s[5]),
                                    ptr<float>(d), stream_of(vp)),
               "siirl_value_loss_bwd");
    }
    d = d.reshape(ctx->saved_data["shape"].toIntVector());
    const auto dt = (at::ScalarType)ctx->saved_data["dtype"].toInt();
    if (dt != at::kFloat) d = d.to(dt);
    none[0] = d;
    return none;
  }
};

std::tuple<Tensor, Tensor> value_loss(const Tensor& vpreds, const Tensor& returns, const Tensor& values,
                                      const Tensor& response_mask, double cliprange_value, int64_t agg_mode) {
  auto out = ValueLossFn::apply(vpreds, returns, values, response_mask, cliprange_value, agg_mode);
  return {out[0], out[1]};
}

// ------------------------------------------------------------------ KL penalty

Tensor kl_penalty_fwd(const Tensor& lp, const Tensor& ref, int64_t kl_mode) {
  require_f32c(lp, "log_prob");
  require_f32c(ref, "ref_log_prob");
  TORCH_CHECK_VALUE(ref.sizes() == lp.sizes(), "siirl_amd: log_prob and ref_log_prob must have one shape");
  require_on(ref, lp, "ref_log_prob");
  Tensor out = at::empty_like(lp);
  DeviceGuard guard(lp.device());
  check_rc(siirl_kl_penalty_fwd(ptr<float>(lp), ptr<float>(ref), lp.numel(), (int)kl_mode, ptr<float>(out),
                                stream_of(lp)),
           "siirl_kl_penalty_fwd");
  return out;
}

std::tuple<Tensor, Tensor> kl_penalty_bwd(const Tensor& g, const Tensor& lp, const Tensor& ref, int64_t kl_mode,
                                          bool straight_through, bool need_lp, bool need_ref) {
  require_f32c(g, "g");
  require_f32c(lp, "log_prob");
  require_f32_like(ref, lp, "ref_log_prob");
  require_f32_like(g, lp, "g");
  const std::vector<int64_t> none{0};
  Tensor d_lp = empty_f32(need_lp ? lp.sizes() : at::IntArrayRef(none), lp);
  Tensor d_ref = empty_f32(need_ref ? lp.sizes() : at::IntArrayRef(none), lp);
  if (need_lp || need_ref) {
    DeviceGuard guard(lp.device());
    check_rc(siirl_kl_penalty_bwd(ptr<float>(g), ptr<float>(lp), ptr<float>(ref), lp.numel(), (int)kl_mode,
                                  (int)straight_through, need_lp ? ptr<float>(d_lp) : nullptr,
                                  need_ref ? ptr<float>(d_ref) : nullptr, stream_of(lp)),
             "siirl_kl_penalty_bwd");
  }
  return {d_lp, d_ref};
}

struct KlPenaltyFn : public torch::autograd::Function<KlPenaltyFn> {
  static Tensor forward(AutogradContext* ctx, const Tensor& logprob, const Tensor& ref_logprob, int64_t kl_mode,
                        bool straight_through) {
    at::AutoDispatchBelowADInplaceOrView below;
    require_gpu(logprob, "logprob");
    const auto dev = logprob.device();
    Tensor lp = f32c(logprob, dev), ref = f32c(ref_logprob, dev);
    if (ref.sizes() != lp.sizes()) ref = ref.expand(lp.sizes()).contiguous();
    Tensor out = kl_penalty_fwd(lp, ref, kl_mode);
    ctx->save_for_backward({lp, ref});
    ctx->saved_data["i"] = std::vector<int64_t>{kl_mode, (int64_t)straight_through, (int64_t)logprob.scalar_type(),
                                                (int64_t)ref_logprob.scalar_type()};
    ctx->saved_data["ref_shape"] = ref_logprob.sizes().vec();
    if (logprob.scalar_type() != at::kFloat) out = out.to(logprob.scalar_type());
    return out;
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    const auto s = ctx->get_saved_variables();
    const auto iv = ctx->saved_data["i"].toIntVector();
    const bool need_lp = ctx->needs_input_grad(0), need_ref = ctx->needs_input_grad(1);
    at::AutoDispatchBelowADInplaceOrView below;
    Tensor g = f32c(grads[0], s[0].device());
    auto [d_lp, d_ref] = kl_penalty_bwd(g, s[0], s[1], iv[0], iv[1] != 0, need_lp, need_ref);
    variable_list out(4);
    if (need_lp) out[0] = (at::ScalarType)iv[2] == at::kFloat ? d_lp : d_lp.to((at::ScalarType)iv[2]);
    if (need_ref) {
      const auto ref_shape = ctx->saved_data["ref_shape"].toIntVector();
      if (at::IntArrayRef(ref_shape) != s[0].sizes()) d_ref = d_ref.sum_to_size(ref_shape);
      out[1] = (at::ScalarType)iv[3] == at::kFloat ? d_ref : d_ref.to((at::ScalarType)iv[3]);
    }
    return out;
  }
};

Tensor kl_penalty(const Tensor& logprob, const Tensor& ref_logprob, int64_t kl_mode, bool straight_through) {
  return KlPenaltyFn::apply(logprob, ref_logprob, kl_mode, straight_through);
}

// ------------------------------------------------------------------ lm_head fused with log-prob / entropy

// hidden states and weights: bfloat16, float16 or float32, both of one dtype
int fused_operand_dtype(const Tensor& hidden, const Tensor& weight) {
  for (const Tensor* t : {&hidden, &weight}) {
    require_gpu(*t, t == &hidden ? "hidden" : "weight");
    TORCH_CHECK_TYPE(t->dim() == 2 && t->is_contiguous() &&
                         (t->scalar_type() == at::kBFloat16 || t->scalar_type() == at::kHalf || t->scalar_type() == at::kFloat),
                     "siirl_amd: `", t == &hidden ? "hidden" : "weight",
                     "` must be a contiguous 2-D bfloat16, float16 or float32 tensor");
  }
  TORCH_CHECK_TYPE(hidden.scalar_type() == weight.scalar_type(), "siirl_amd: hidden (", hidden.scalar_type(),
                   ") and weight (", weight.scalar_type(), ") must have one dtype");
  return hidden.scalar_type() == at::kBFloat16 ? SIIRL_BF16 : hidden.scalar_type() == at::kHalf ? SIIRL_F16 : SIIRL_F32;
}

std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor> fused_linear_fwd(const Tensor& hidden, const Tensor& weight,
                                                                    const Tensor& labels, double inv_temperature,
                                                                    bool save_logits) {
  const int dt = fused_operand_dtype(hidden, weight);
  const int64_t T = hidden.size(0), H = hidden.size(1), V = weight.size(0);
  TORCH_CHECK_VALUE(weight.size(1) == H && labels.dim() == 1 && labels.size(0) == T && labels.scalar_type() == at::kLong,
                    "shape mismatch: hidden ", hidden.sizes(), ", weight ", weight.sizes(), ", labels ", labels.sizes());
  require_on(weight, hidden, "weight");
  require_on(labels, hidden, "labels");
  Tensor lp = empty_f32({T}, hidden), ent = empty_f32({T}, hidden), lse = empty_f32({T}, hidden),
         ex = empty_f32({T}, hidden);
  Tensor saved = empty_f32({0}, hidden);
  if (save_logits) {
    try {
      saved = empty_f32({(int64_t)(siirl_fused_linear_saved_logits_bytes(T, V) / 4)}, hidden);
    } catch (const c10::OutOfMemoryError&) {
      save_logits = false;  // no room to keep the logits: the backward recomputes them
    }
  }
  const size_t nws = siirl_fused_linear_fwd_workspace_bytes_dtype(dt, T, H, V);
  Tensor ws = at::empty({(int64_t)std::max<size_t>(nws, 256)}, hidden.options().dtype(at::kByte));
  Tensor y = labels.contiguous();
  DeviceGuard guard(hidden.device());
  check_rc(siirl_fused_linear_logprob_entropy_fwd(ptr(hidden), ptr(weight), dt, ptr<int64_t>(y), T, H, V,
                                                  (float)inv_temperature, ptr<float>(lp), ptr<float>(ent),
                                                  ptr<float>(lse), ptr<float>(ex),
                                                  save_logits ? ptr<float>(saved) : nullptr, ptr(ws), nws,
                                                  stream_of(hidden)),
           "siirl_fused_linear_logprob_entropy_fwd");
  return {lp, ent, lse, ex, saved};
}

std::tuple<Tensor, Tensor> fused_linear_bwd(const Tensor& hidden, const Tensor& weight, const Tensor& labels,
                                            double inv_temperature, const Tensor& lse, const Tensor& ex,
                                            const optional<Tensor>& g_lp, const optional<Tensor>& g_ent,
                                            bool need_hidden, bool need_weight, const optional<Tensor>& saved_in,
                                            bool skip_zero_rows) {
  const int dt = fused_operand_dtype(hidden, weight);
  require_f32c(g_lp, "g_logprob");
  require_f32c(g_ent, "g_entropy");
  const int64_t T = hidden.size(0), H = hidden.size(1), V = weight.size(0);
  TORCH_CHECK_VALUE(weight.size(1) == H && labels.dim() == 1 && labels.size(0) == T && labels.scalar_type() == at::kLong,
                    "shape mismatch: hidden ", hidden.sizes(), ", weight ", weight.sizes(), ", labels ", labels.sizes());
  require_on(weight, hidden, "weight");
  require_on(labels, hidden, "labels");
  require_f32_n(lse, T, hidden, "lse");
  require_f32_n(ex, T, hidden, "ex");
  require_f32_n(g_lp, T, hidden, "g_logprob");
  require_f32_n(g_ent, T, hidden, "g_entropy");
  const std::vector<int64_t> none{0};
  Tensor d_h = at::empty(need_hidden ? hidden.sizes() : at::IntArrayRef(none), hidden.options());
  Tensor d_w = at::empty(need_weight ? weight.sizes() : at::IntArrayRef(none), weight.options());
  optional<Tensor> saved;
  if (has(saved_in) && saved_in->numel() != 0) {
    saved = saved_in;
    require_on(*saved, hidden, "saved");
    TORCH_CHECK_VALUE(saved->scalar_type() == at::kFloat && saved->is_contiguous() &&
                          (size_t)saved->numel() * 4 == siirl_fused_linear_saved_logits_bytes(T, V),
                      "saved is not the buffer the forward op returned for these shapes");
  }
  Tensor y = labels.contiguous();
  DeviceGuard guard(hidden.device());
  // Token rows whose upstream gradients are both zero (the prompt tokens of a packed batch: only the response slice
  // of the log-probs reaches the loss) drop out of all three GEMMs.  Finding them costs one host synchronisation,
  // so not under stream capture; parked logits are indexed by the forward's token tiles, so not with them either.
  if (skip_zero_rows && !has(saved) && T > 0 && (has(g_lp) || has(g_ent)) &&
      c10::hip::currentStreamCaptureStatusMayInitCtx() == c10::hip::CaptureStatus::None) {
    Tensor live = has(g_lp) ? g_lp->ne(0) : g_ent->ne(0);
    if (has(g_lp) && has(g_ent)) live = live.logical_or(g_ent->ne(0));
    Tensor rows = at::nonzero(live).reshape({-1});
    const int64_t n = rows.size(0);
    if (n < T) {
      const size_t nws = siirl_fused_linear_bwd_rows_workspace_bytes_dtype(dt, n, H, V, (int)need_hidden, (int)need_weight);
      Tensor ws = at::empty({(int64_t)std::max<size_t>(nws, 256)}, hidden.options().dtype(at::kByte));
      check_rc(siirl_fused_linear_logprob_entropy_bwd_rows(
                   ptr(hidden), ptr(weight), dt, ptr<int64_t>(y), T, H, V, (float)inv_temperature, ptr<float>(lse),
                   ptr<float>(ex), ptr<float>(g_lp), ptr<float>(g_ent), ptr<int64_t>(rows), n,
                   need_hidden ? ptr(d_h) : nullptr, need_weight ? ptr(d_w) : nullptr, ptr(ws), nws, stream_of(hidden)),
               "siirl_fused_linear_logprob_entropy_bwd_rows");
      return {d_h, d_w};
    }
  }
  const size_t nws = siirl_fused_linear_bwd_workspace_bytes_dtype(dt, T, H, V, (int)need_hidden, (int)need_weight);
  Tensor ws = at::empty({(int64_t)std::max<size_t>(nws, 256)}, hidden.options().dtype(at::kByte));
  check_rc(siirl_fused_linear_logprob_entropy_bwd(ptr(hidden), ptr(weight), dt, ptr<int64_t>(y), T, H, V,
                                                  (float)inv_temperature, ptr<float>(lse), ptr<float>(ex),
                                                  ptr<float>(saved), ptr<float>(g_lp), ptr<float>(g_ent),
                                                  need_hidden ? ptr(d_h) : nullptr, need_weight ? ptr(d_w) : nullptr,
                                                  ptr(ws), nws, stream_of(hidden)),
           "siirl_fused_linear_logprob_entropy_bwd");
  return {d_h, d_w};
}

struct FusedLinearFn : public torch::autograd::Function<FusedLinearFn> {
  static variable_list forward(AutogradContext* ctx, const Tensor& hidden, const Tensor& weight, const Tensor& labels,
                               double inv_temperature, bool save_logits, bool skip_zero_rows) {
    at::AutoDispatchBelowADInplaceOrView below;
    require_gpu(hidden, "hidden");
    require_gpu(weight, "weight");
    TORCH_CHECK_TYPE(hidden.scalar_type() == weight.scalar_type() &&
                         (hidden.scalar_type() == at::kBFloat16 || hidden.scalar_type() == at::kHalf ||
                          hidden.scalar_type() == at::kFloat),
                     "siirl_amd: the fused lm_head path takes hidden states and weights of one dtype, bfloat16, "
                     "float16 or float32 (got ", hidden.scalar_type(), " and ", weight.scalar_type(), ")");
    Tensor h = hidden.detach().contiguous(), w = weight.detach().contiguous();
    Tensor y = labels.detach();
    if (y.device() != h.device()) y = y.to(h.device());
    if (y.scalar_type() != at::kLong) y = y.to(at::kLong);
    y = y.contiguous();
    TORCH_CHECK_VALUE(h.dim() == 2 && w.dim() == 2 && w.size(1) == h.size(1) && y.dim() == 1 && y.size(0) == h.size(0),
                      "shape mismatch: hidden ", h.sizes(), ", weight ", w.sizes(), ", labels ", y.sizes());
    auto [lp, ent, lse, ex, saved] = fused_linear_fwd(h, w, y, inv_temperature, save_logits);
    ctx->save_for_backward({h, w, y, lse, ex, saved});
    ctx->saved_data["inv_t"] = inv_temperature;
    ctx->saved_data["skip_zero_rows"] = skip_zero_rows;
    ctx->set_materialize_grads(false);
    return {lp, ent};
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    const bool need_h = ctx->needs_input_grad(0), need_w = ctx->needs_input_grad(1);
    variable_list out(6);
    if ((!grads[0].defined() && !grads[1].defined()) || !(need_h || need_w)) return out;
    const auto s = ctx->get_saved_variables();
    at::AutoDispatchBelowADInplaceOrView below;
    optional<Tensor> g_lp, g_ent;
    if (grads[0].defined()) g_lp = f32c(grads[0], s[0].device());
    if (grads[1].defined()) g_ent = f32c(grads[1], s[0].device());
    auto [d_h, d_w] = fused_linear_bwd(s[0], s[1], s[2], ctx->saved_data["inv_t"].toDouble(), s[3], s[4], g_lp, g_ent,
                                       need_h, need_w, s[5], ctx->saved_data["skip_zero_rows"].toBool());
    if (need_h) out[0] = d_h;
    if (need_w) out[1] = d_w;
    return out;
  }
};

// `save_limit_bytes`: largest fp32 logit buffer the forward may park for the backward (0: never park).
std::tuple<Tensor, Tensor> fused_linear_logprob_entropy(const Tensor& hidden, const Tensor& weight, const Tensor& labels,
                                                        double inv_temperature, int64_t save_limit_bytes,
                                                        bool skip_zero_rows) {
  bool save = false;
  if (save_limit_bytes > 0 && at::GradMode::is_enabled() && (hidden.requires_grad() || weight.requires_grad()) &&
      hidden.dim() == 2 && weight.dim() == 2)
    save = (int64_t)siirl_fused_linear_saved_logits_bytes(hidden.size(0), weight.size(0)) <= save_limit_bytes;
  auto out = FusedLinearFn::apply(hidden, weight, labels, inv_temperature, save, skip_zero_rows);
  return {out[0], out[1]};
}

}  // namespace

TORCH_LIBRARY(siirl_hip, m) {
  // plain operators (CUDA kernels below; fake kernels in siirl_amd/ops.py)
  m.def("logprob_entropy_fwd(Tensor logits, Tensor? labels, float inv_temperature, bool want_entropy) -> "
        "(Tensor, Tensor, Tensor, Tensor)");
  m.def("logprob_entropy_bwd(Tensor logits, Tensor? labels, float inv_temperature, Tensor lse, Tensor? ex, "
        "Tensor? g_logprob, Tensor? g_entropy, bool skip_zero_rows) -> Tensor");
  m.def("logprob_entropy_bwd_(Tensor(a!) logits, Tensor? labels, float inv_temperature, Tensor lse, Tensor? ex, "
        "Tensor? g_logprob, Tensor? g_entropy, bool skip_zero_rows) -> ()");
  m.def("grpo_advantage(Tensor token_level_rewards, Tensor mask, Tensor uid, float epsilon, bool norm_by_std) -> Tensor");
  m.def("group_keep_mask(Tensor metric, Tensor uid) -> (Tensor, Tensor)");
  m.def("agg_loss_fwd(Tensor loss_mat, Tensor mask, int agg_mode) -> (Tensor, Tensor)");
  m.def("agg_loss_bwd(Tensor g, Tensor mask, Tensor out16, Tensor row_msum, int agg_mode) -> Tensor");
  m.def("masked_reduce_fwd(Tensor values, Tensor mask, bool per_row, bool want_mean) -> (Tensor, Tensor)");
  m.def("masked_reduce_bwd(Tensor g, Tensor mask, bool per_row, Tensor? mask_sums) -> Tensor");
  m.def("policy_loss_fwd(Tensor old_log_prob, Tensor log_prob, Tensor advantages, Tensor mask, Tensor? is_weights, "
        "Tensor? entropy, Tensor? ref_log_prob, int loss_mode, float clip_low, float clip_high, float clip_c, "
        "float log_ratio_clamp, int agg_mode, float entropy_coeff, int kl_mode, bool kl_straight_through, "
        "float kl_coef, float policy_drift_coeff, float loss_scale, Tensor? token_aux=None) -> (Tensor, Tensor, Tensor)");
  m.def("policy_loss_bwd(Tensor g_loss, Tensor old_log_prob, Tensor log_prob, Tensor advantages, Tensor mask, "
        "Tensor? is_weights, Tensor? entropy, Tensor? ref_log_prob, int loss_mode, float clip_low, float clip_high, "
        "float clip_c, float log_ratio_clamp, int agg_mode, float entropy_coeff, int kl_mode, "
        "bool kl_straight_through, float kl_coef, float policy_drift_coeff, float loss_scale, Tensor out16, "
        "Tensor row_msum, Tensor row_s, Tensor? token_aux=None) -> (Tensor, Tensor)");
  m.def("cov_scores(Tensor? old_log_prob, Tensor log_prob, Tensor advantages, Tensor mask, int loss_mode, "
        "float clip_low, float clip_high) -> (Tensor, Tensor)");
  m.def("topk_mark(Tensor scores, int k, float value) -> Tensor");
  m.def("range_indices(Tensor scores, float lower, float upper) -> Tensor");
  m.def("kl_penalty_fwd(Tensor log_prob, Tensor ref_log_prob, int kl_mode) -> Tensor");
  m.def("kl_penalty_bwd(Tensor g, Tensor log_prob, Tensor ref_log_prob, int kl_mode, bool straight_through, "
        "bool need_log_prob, bool need_ref) -> (Tensor, Tensor)");
  m.def("fused_linear_logprob_entropy_fwd(Tensor hidden, Tensor weight, Tensor labels, float inv_temperature, "
        "bool save_logits=False) -> (Tensor, Tensor, Tensor, Tensor, Tensor)");
  m.def("fused_linear_logprob_entropy_bwd(Tensor hidden, Tensor weight, Tensor labels, float inv_temperature, "
        "Tensor lse, Tensor ex, Tensor? g_logprob, Tensor? g_entropy, bool need_hidden, bool need_weight, "
        "Tensor? saved=None, bool skip_zero_rows=False) -> (Tensor, Tensor)");
  // how the log-prob operators cut a (..., V) view into launches; no device work (used by the host-side tests)
  m.def("row_blocks(Tensor x) -> int[]", &row_blocks_op);
  // differentiable operators (autograd nodes in C++; eager use only)
  m.def("logprob_entropy(Tensor logits, Tensor? labels, float inv_temperature, bool want_entropy, "
        "bool inplace_backward, bool skip_zero_rows, Tensor? defer=None) -> (Tensor, Tensor)", &logprob_entropy);
  m.def("actor_loss(Tensor log_prob, Tensor? entropy, Tensor old_log_prob, Tensor advantages, Tensor response_mask, "
        "Tensor? is_weights, Tensor? ref_log_prob, int loss_mode, float clip_low, float clip_high, float clip_c, "
        "float log_ratio_clamp, int agg_mode, float entropy_coeff, int kl_mode, bool kl_straight_through, "
        "float kl_coef, float policy_drift_coeff, float loss_scale, bool policy_only, Tensor? token_aux=None) -> Tensor[]",
        &actor_loss);
  m.def("agg_loss(Tensor loss_mat, Tensor loss_mask, int agg_mode) -> Tensor", &agg_loss);
  m.def("masked_reduce(Tensor values, Tensor mask, int[] axes, bool want_mean) -> Tensor", &masked_reduce);
  m.def("value_loss(Tensor vpreds, Tensor returns, Tensor values, Tensor response_mask, float cliprange_value, "
        "int agg_mode) -> (Tensor, Tensor)", &value_loss);
  m.def("kl_penalty(Tensor logprob, Tensor ref_logprob, int kl_mode, bool straight_through) -> Tensor", &kl_penalty);
  m.def("fused_linear_logprob_entropy(Tensor hidden, Tensor weight, Tensor labels, float inv_temperature, "
        "int save_limit_bytes, bool skip_zero_rows=False) -> (Tensor, Tensor)", &fused_linear_logprob_entropy);
}

TORCH_LIBRARY_IMPL(siirl_hip, CUDA, m) {
  m.impl("logprob_entropy_fwd", &lpe_fwd);
  m.impl("logprob_entropy_bwd", &lpe_bwd);
  m.impl("logprob_entropy_bwd_", &lpe_bwd_inplace);
  m.impl("grpo_advantage", &grpo_advantage);
  m.impl("group_keep_mask", &group_keep_mask);
  m.impl("agg_loss_fwd", &agg_loss_fwd);
  m.impl("agg_loss_bwd", &agg_loss_bwd);
  m.impl("masked_reduce_fwd", &masked_reduce_fwd);
  m.impl("masked_reduce_bwd", &masked_reduce_bwd);
  m.impl("policy_loss_fwd", &policy_loss_fwd);
  m.impl("policy_loss_bwd", &policy_loss_bwd);
  m.impl("cov_scores", &cov_scores);
  m.impl("topk_mark", &topk_mark);
  m.impl("range_indices", &range_indices);
  m.impl("kl_penalty_fwd", &kl_penalty_fwd);
  m.impl("kl_penalty_bwd", &kl_penalty_bwd);
  m.impl("fused_linear_logprob_entropy_fwd", &fused_linear_fwd);
  m.impl("fused_linear_logprob_entropy_bwd", &fused_linear_bwd);
}
