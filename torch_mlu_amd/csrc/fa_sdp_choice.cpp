// Backend selector for F.scaled_dot_product_attention on HIP tensors.
//
// Mirrors torch_mlu's selector: the stub registration of _fused_sdp_choice.cpp:37-77 (there for PrivateUse1, here for
// the CUDA slot that HIP tensors use), select_sdp_backend (sdp_utils.cpp:97-147) and the input constraints of
// sdp_utils.h:99-472 with their warning texts.  What is not mirrored are the MLU-specific heuristics
// (sdp_utils.h:475-524: device series, "split condition", "valid data ratio") and the xformers-derived priority order
// (sdp_utils.cpp:8-53): on MI355X the flash kernels of this build are preferred whenever they are eligible — they
// take GQA, head dims up to 256, and single-query decode (split-KV) —, then its mem-efficient entry points (additive
// attn_mask, top-left causal on non-square problems), and everything else is left to PyTorch's own
// choice among its remaining backends.
#include <ATen/ATen.h>
#include <ATen/Context.h>
#include <ATen/NestedTensorImpl.h>
#include <ATen/core/LegacyTypeDispatch.h>
#include <ATen/native/DispatchStub.h>
#include <ATen/native/transformers/attention.h>
#include <c10/util/Exception.h>
#include <torch/library.h>

#include <algorithm>
#include <array>
#include <sstream>

namespace torch_mlu_amd {
namespace sdp {

// Same values as torch_mlu/csrc/aten/operators/cnnl/transformers/sdp_utils.h (and PyTorch's sdp::SDPBackend).
enum class SDPBackend : int64_t { error = -1, math = 0, flash_attention = 1, efficient_attention = 2 };

struct sdp_params {
  const at::Tensor& query;
  const at::Tensor& key;
  const at::Tensor& value;
  const std::optional<at::Tensor>& attn_mask;
  double dropout;
  bool is_causal;
  bool enable_gqa;
};

bool input_requires_grad(const sdp_params& p) {
  return at::GradMode::is_enabled() &&
         (p.query.requires_grad() || p.key.requires_grad() || p.value.requires_grad());
}

bool check_runtime_disabled_flash(const sdp_params&, bool debug) {
  if (!at::globalContext().userEnabledFlashSDP()) {
    if (debug) TORCH_WARN("Flash attention has been runtime disabled.");
    return false;
  }
  return true;
}

bool has_nested_inputs(const sdp_params& p) { return p.query.is_nested() || p.key.is_nested() || p.value.is_nested(); }

// check_requires_grad_and_nested, sdp_utils.h (reference: sdp_utils.cpp:82-87): the mem-efficient kernels take nested
// inputs for inference only.
bool check_requires_grad_and_nested(const sdp_params& p, bool debug) {
  if (has_nested_inputs(p) && input_requires_grad(p)) {
    if (debug) TORCH_WARN("Memory efficient attention currently doesn't support training with NT inputs.");
    return false;
  }
  return true;
}

// Not in the reference: the nested wrapper of this build's mem-efficient op packs three nested tensors that hold the
// same number of sequences with one head count each (no broadcasting between them).
bool check_nested_same_structure(const sdp_params& p, bool debug) {
  const bool all = p.query.is_nested() && p.key.is_nested() && p.value.is_nested();
  if (!all || p.query.size(0) != p.key.size(0) || p.query.size(0) != p.value.size(0) ||
      p.key.size(1) != p.value.size(1) || p.key.size(1) <= 0 || p.query.size(1) % p.key.size(1) != 0 ||
      (!p.enable_gqa && p.query.size(1) != p.key.size(1))) {
    if (debug) TORCH_WARN("The mem-efficient kernels of this build need nested query, key and value with the same "
                          "number of sequences and matching head counts.");
    return false;
  }
  return true;
}

// Nested inputs (sdp_utils.h:168-200, 283-370): PyTorch's nested-tensor kernel of the flash op packs them and calls
// aten::_flash_attention_forward with cu_seqlens, i.e. this build's packed op.  What it cannot pack is refused here,
// with the reference's messages: a ragged head count, an empty sequence, batch sizes or head counts that are neither
// equal nor 1.
bool check_nested_sizes_one(const at::Tensor& t, const char* name, bool debug) {
  if (!t.is_nested()) return true;
  const auto* impl = at::native::get_nested_tensor_impl(t);
  if (!impl->opt_size(1).has_value()) {
    if (debug) TORCH_WARN("Fused kernels do not support ragged num_head_dims, ", name, "has a ragged num_heads.");
    return false;
  }
  const at::Tensor& sizes = impl->get_nested_sizes();
  const int64_t* ptr = sizes.data_ptr<int64_t>();
  const int64_t n = t.size(0), stride = sizes.stride(0);
  for (int64_t i = 0; i < n; ++i)
    if (ptr[i * stride + 1] == 0) {
      if (debug) TORCH_WARN("Fused kernels do not support seq_len == 0, ", name, "has a seq len of 0.");
      return false;
    }
  return true;
}

bool broadcastable(int64_t q, int64_t k, int64_t v, const char* what, bool debug) {
  const int64_t mx = std::max(q, std::max(k, v));
  if ((q != mx && q != 1) || (k != mx && k != 1) || (v != mx && v != 1)) {
    if (debug)
      TORCH_WARN("Both fused kernels require query, key and value to have broadcastable ", what, "got Query ", what, q,
                 ", Key ", what, k, ", Value ", what, v, " instead.");
    return false;
  }
  return true;
}

bool check_nested_inputs(const sdp_params& p, bool debug) {
  if (!check_nested_sizes_one(p.query, "query ", debug) || !check_nested_sizes_one(p.key, "key ", debug) ||
      !check_nested_sizes_one(p.value, "value ", debug))
    return false;
  if (!broadcastable(p.query.size(0), p.key.size(0), p.value.size(0), "batch size ", debug)) return false;
  if (!broadcastable(p.query.size(1), p.key.size(1), p.value.size(1), "num heads ", debug)) return false;
  if (!p.query.is_cuda() || !p.key.is_cuda() || !p.value.is_cuda()) {
    if (debug) TORCH_WARN("The flash kernels of this build need all inputs on the HIP device.");
    return false;
  }
  if (!(p.dropout >= 0.0 && p.dropout < 1.0)) {
    if (debug) TORCH_WARN("The flash kernels of this build need 0 <= dropout_p < 1.");
    return false;
  }
  return true;
}

bool check_tensor_shapes(const sdp_params& p, bool debug) {
  if (p.query.dim() != 4 || p.key.dim() != 4 || p.value.dim() != 4) {
    if (debug)
      TORCH_WARN("Both fused kernels requires query, key and value to be 4 dimensional, but got Query dim: ",
                 p.query.dim(), ", Key dim: ", p.key.dim(), ", Value dim: ", p.value.dim(), " instead.");
    return false;
  }
  return true;
}

bool check_batch_size_and_num_heads(const sdp_params& p, bool debug) {
  const bool same_batch = p.query.size(0) == p.key.size(0) && p.query.size(0) == p.value.size(0);
  const int64_t hq = p.query.size(1), hk = p.key.size(1), hv = p.value.size(1);
  const bool heads_ok = p.enable_gqa ? (hk == hv && hk > 0 && hq % hk == 0) : (hq == hk && hq == hv);
  if (!same_batch || !heads_ok) {
    if (debug)
      TORCH_WARN(
          "For dense inputs, both fused kernels require query, key and value to have the same batch_size and "
          "num_heads. ",
          "Query.sizes(): ", p.query.sizes(), ", Key sizes(): ", p.key.sizes(), ", Value sizes(): ", p.value.sizes(),
          " instead. To broadcast dense inputs, try using unsqueeze and expand_to before passing them into the "
          "kernel.",
          p.enable_gqa ? " With enable_gqa the number of query heads must be a multiple of the number of key/value heads."
                       : "");
    return false;
  }
  return true;
}

bool check_for_attn_mask(const sdp_params& p, bool debug) {
  if (p.attn_mask.has_value() && p.attn_mask->defined()) {
    if (debug) TORCH_WARN("Flash Attention does not support non-null attn_mask.");
    return false;
  }
  return true;
}

bool check_head_dim_size(const sdp_params& p, bool debug) {
  const int64_t dq = p.query.size(-1), dk = p.key.size(-1), dv = p.value.size(-1);
  if (!(dq == dk && dq == dv && dq <= 256 && dq >= 8 && dq % 8 == 0)) {
    if (debug)
      TORCH_WARN("Flash attention requires q,k,v to have the same last dimension, at most 256.",
                 " Flash attention requires last dimension of inputs to be divisible by 8.", " Got Query.size(-1): ", dq,
                 ", Key.size(-1): ", dk, ", Value.size(-1): ", dv, " instead.");
    return false;
  }
  return true;
}

bool check_nonzero_sequence_lengths(const sdp_params& p, bool debug) {
  if (p.query.size(-2) == 0 || p.key.size(-2) == 0 || p.query.size(0) == 0 || p.query.size(1) == 0) {
    if (debug) TORCH_WARN("Both fused kernels do not support zero seq_len_q or seq_len_kv.");
    return false;
  }
  if (p.key.size(-2) != p.value.size(-2)) {
    if (debug) TORCH_WARN("Key and Value must have the same sequence length.");
    return false;
  }
  return true;
}

bool check_last_dim_stride_equals_1(const sdp_params& p, bool debug) {
  if (p.query.stride(-1) != 1 || p.key.stride(-1) != 1 || p.value.stride(-1) != 1) {
    if (debug)
      TORCH_WARN("Both fused kernels require the last dimension of the input to have stride 1. ",
                 "Got Query.stride(-1): ", p.query.stride(-1), ", Key.stride(-1): ", p.key.stride(-1),
                 ", Value.stride(-1): ", p.value.stride(-1), " instead.");
    return false;
  }
  return true;
}

bool check_tensor_dtype(const sdp_params& p, bool debug) {
  const auto dt = p.query.scalar_type();
  if (!(dt == p.key.scalar_type() && dt == p.value.scalar_type() && (dt == at::kHalf || dt == at::kBFloat16))) {
    if (debug)
      TORCH_WARN("Expected query, key and value to all be of dtype: {Half, BFloat16}. Got ", "Query dtype: ",
                 p.query.dtype(), ", Key dtype: ", p.key.dtype(), ", and Value dtype: ", p.value.dtype(), " instead.");
    return false;
  }
  return true;
}

// Not in the reference: what this build's flash kernels do not implement, and the one place where the flash
// convention differs from F.scaled_dot_product_attention's definition.
bool check_this_build(const sdp_params& p, bool debug) {
  if (!(p.dropout >= 0.0 && p.dropout < 1.0)) {
    if (debug) TORCH_WARN("The flash kernels of this build need 0 <= dropout_p < 1.");
    return false;
  }
  if (p.is_causal && p.query.size(-2) != p.key.size(-2)) {
    // flash kernels align the causal mask to the bottom-right corner, F.scaled_dot_product_attention documents the
    // top-left one; they agree only for square problems
    if (debug)
      TORCH_WARN("Flash attention with is_causal=True needs seq_len_q == seq_len_kv to match "
                 "scaled_dot_product_attention's top-left aligned mask. Got seq_len_q: ", p.query.size(-2),
                 ", seq_len_kv: ", p.key.size(-2), ".");
    return false;
  }
  if (!p.query.is_cuda() || !p.key.is_cuda() || !p.value.is_cuda()) {
    if (debug) TORCH_WARN("The flash kernels of this build need all inputs on the HIP device.");
    return false;
  }
  return true;
}

bool use_flash_attention(const sdp_params& p, bool debug) {
  if (has_nested_inputs(p)) {
    // (sdp_utils.cpp:97-147: the general constraints, then the nested ones; the causal alignment of ragged sequences
    // is the packed op's bottom-right one, as in PyTorch's own nested path)
    constexpr std::array<bool (*)(const sdp_params&, bool), 6> nested{
        check_runtime_disabled_flash, check_tensor_shapes, check_for_attn_mask,
        check_head_dim_size,          check_tensor_dtype,  check_nested_inputs};
    for (auto c : nested)
      if (!c(p, debug)) return false;
    return true;
  }
  constexpr std::array<bool (*)(const sdp_params&, bool), 9> constraints{
      check_runtime_disabled_flash,   check_tensor_shapes, check_batch_size_and_num_heads,
      check_for_attn_mask,            check_head_dim_size, check_nonzero_sequence_lengths,
      check_last_dim_stride_equals_1, check_tensor_dtype,  check_this_build};
  for (auto c : constraints)
    if (!c(p, debug)) return false;
  return true;
}

bool check_runtime_disabled_mem_efficient(const sdp_params&, bool debug) {
  if (!at::globalContext().userEnabledMemEfficientSDP()) {
    if (debug) TORCH_WARN("Memory Efficient attention has been runtime disabled.");
    return false;
  }
  return true;
}

bool check_head_dim_size_mem_efficient(const sdp_params& p, bool debug) {
  const int64_t dq = p.query.size(-1), dk = p.key.size(-1), dv = p.value.size(-1);
  if (!(dq == dk && dq == dv && dq <= 256 && dq >= 8 && dq % 8 == 0)) {
    if (debug)
      TORCH_WARN("Mem efficient attention requires query.size(-1)==key.size(-1)==value.size(-1), at most 256.",
                 " Mem efficient attention requires last dimension of Q/V to be divisible by 8.",
                 " Got Query.size(-1): ", dq, ", Key.size(-1): ", dk, ", Value.size(-1): ", dv, " instead.");
    return false;
  }
  return true;
}

// Not in the reference: what the mem-efficient entry points of this build need beyond the shared constraints.
bool check_this_build_mem_efficient(const sdp_params& p, bool debug) {
  if (p.attn_mask.has_value() && p.attn_mask->defined()) {
    const auto mt = p.attn_mask->scalar_type();
    if ((mt != at::kBool && mt != p.query.scalar_type()) || p.attn_mask->dim() > 4 || !p.attn_mask->is_cuda() ||
        p.attn_mask->is_nested()) {
      if (debug) TORCH_WARN("attn_mask must be a boolean mask or have the dtype of query, at most 4 dimensions, on the HIP device.");
      return false;
    }
  }
  if (!p.query.is_cuda() || !p.key.is_cuda() || !p.value.is_cuda()) {
    if (debug) TORCH_WARN("The mem-efficient kernels of this build need all inputs on the HIP device.");
    return false;
  }
  return true;
}

// use_mem_efficient_attention, sdp_utils.cpp:76-95
bool use_mem_efficient_attention(const sdp_params& p, bool debug) {
  if (has_nested_inputs(p)) {
    constexpr std::array<bool (*)(const sdp_params&, bool), 8> nested{
        check_runtime_disabled_mem_efficient, check_requires_grad_and_nested, check_tensor_shapes,
        check_head_dim_size_mem_efficient,    check_tensor_dtype,             check_nested_inputs,
        check_nested_same_structure,          check_this_build_mem_efficient};
    for (auto c : nested)
      if (!c(p, debug)) return false;
    return true;
  }
  constexpr std::array<bool (*)(const sdp_params&, bool), 9> constraints{
      check_runtime_disabled_mem_efficient, check_requires_grad_and_nested, check_tensor_shapes, check_batch_size_and_num_heads,
      check_head_dim_size_mem_efficient, check_nonzero_sequence_lengths, check_last_dim_stride_equals_1,
      check_tensor_dtype, check_this_build_mem_efficient};
  for (auto c : constraints)
    if (!c(p, debug)) return false;
  return true;
}

SDPBackend select_sdp_backend(const sdp_params& p, std::optional<double> scale) {
  auto& ctx = at::globalContext();
  if (!ctx.userEnabledMathSDP() && !ctx.userEnabledFlashSDP() && !ctx.userEnabledMemEfficientSDP() &&
      !ctx.userEnabledCuDNNSDP())
    return SDPBackend::error;
  // flash first, then mem-efficient (attn_mask, top-left causal on non-square problems), as the reference's default
  // order (sdp_utils.cpp:9-12)
  if (use_flash_attention(p, /*debug=*/false)) return SDPBackend::flash_attention;
  if (use_mem_efficient_attention(p, /*debug=*/false)) return SDPBackend::efficient_attention;
  // Not eligible here.  Of PyTorch's own backends only the math one is left for HIP tensors: its flash and
  // mem-efficient choices would land on this build's registered ops again, and the cuDNN backend does not exist in a
  // ROCm build.  The choice is made here, from the flags as they are: nothing process-wide is changed while another
  // host thread may be selecting a backend too.
  if (ctx.userEnabledMathSDP()) return SDPBackend::math;
  // Only fused kernels are enabled and they cannot take these inputs: say why, as the reference does
  // (sdp_utils.cpp:135-146).
  TORCH_WARN("Memory efficient kernel not used because:");
  use_mem_efficient_attention(p, /*debug=*/true);
  TORCH_WARN("Flash attention kernel not used because:");
  use_flash_attention(p, /*debug=*/true);
  TORCH_CHECK(false, "No available kernel.  Aborting execution.");
  return SDPBackend::error;
}

}  // namespace sdp

int64_t fused_sdp_choice(const at::Tensor& query, const at::Tensor& key, const at::Tensor& value,
                         const std::optional<at::Tensor>& attn_mask, double dropout_p, bool is_causal,
                         std::optional<double> scale, bool enable_gqa) {
  const sdp::sdp_params params{query, key, value, attn_mask, dropout_p, is_causal, enable_gqa};
  const auto backend = sdp::select_sdp_backend(params, scale);
  TORCH_CHECK(backend != sdp::SDPBackend::error,
              "No viable backend for scaled_dot_product_attention was found. ",
              "This is likely due to turning off both the math kernel and the fused kernels.");
  return static_cast<int64_t>(backend);
}

std::string mem_efficient_refusal_reason(const at::Tensor& query, const at::Tensor& key, const at::Tensor& value,
                                         const std::optional<at::Tensor>& attn_mask, double dropout_p, bool is_causal,
                                         bool enable_gqa) {
  const sdp::sdp_params p{query, key, value, attn_mask, dropout_p, is_causal, enable_gqa};
  if (sdp::use_mem_efficient_attention(p, false)) return "";
  c10::WarningUtils::WarnAlways always(true);
  struct Collect : c10::WarningHandler {
    std::string text;
    void process(const c10::Warning& w) override { text += w.msg(); }
  } collect;
  c10::WarningUtils::WarningHandlerGuard guard(&collect);
  sdp::use_mem_efficient_attention(p, true);
  return collect.text.empty() ? "refused" : collect.text;
}

// Why the flash kernels would refuse these inputs ("" if they take them); used by the tests and for diagnostics.
std::string flash_refusal_reason(const at::Tensor& query, const at::Tensor& key, const at::Tensor& value,
                                 const std::optional<at::Tensor>& attn_mask, double dropout_p, bool is_causal,
                                 bool enable_gqa) {
  const sdp::sdp_params p{query, key, value, attn_mask, dropout_p, is_causal, enable_gqa};
  if (sdp::use_flash_attention(p, false)) return "";
  c10::WarningUtils::WarnAlways always(true);
  struct Collect : c10::WarningHandler {
    std::string text;
    void process(const c10::Warning& w) override { text += w.msg(); }
  } collect;
  c10::WarningUtils::WarningHandlerGuard guard(&collect);
  sdp::use_flash_attention(p, true);
  return collect.text.empty() ? "refused" : collect.text;
}

namespace {
// F.scaled_dot_product_attention asks the stub's CUDA slot for HIP tensors (the reference fills the PrivateUse1 slot,
// _fused_sdp_choice.cpp:75-77).
struct InstallChoice {
  InstallChoice() { at::native::_fused_sdp_choice_stub.set_cuda_dispatch_ptr(&fused_sdp_choice); }
} install_choice;
}  // namespace

}  // namespace torch_mlu_amd

// torch._fused_sdp_choice(...) called directly (as the reference's tests do) is an operator call and does not pass
// through the stub.  The operator's own HIP kernel is kept — it is the fallback above — and this selector sits one
// dispatch key higher.
TORCH_LIBRARY_IMPL(aten, AutogradCUDA, m) {
  m.impl("_fused_sdp_choice", TORCH_FN(torch_mlu_amd::fused_sdp_choice));
}

TORCH_LIBRARY_FRAGMENT(torch_mlu_amd, m) {
  m.def(
      "_flash_refusal_reason(Tensor query, Tensor key, Tensor value, Tensor? attn_mask=None, float dropout_p=0.0, "
      "bool is_causal=False, bool enable_gqa=False) -> str",
      &torch_mlu_amd::flash_refusal_reason);
  m.def(
      "_mem_efficient_refusal_reason(Tensor query, Tensor key, Tensor value, Tensor? attn_mask=None, float dropout_p=0.0, "
      "bool is_causal=False, bool enable_gqa=False) -> str",
      &torch_mlu_amd::mem_efficient_refusal_reason);
}
