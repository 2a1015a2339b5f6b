// ATen extension: registers `_scaled_dot_product_flash_attention` and `_flash_attention_forward` for HIP tensors
// and hands them to the C-ABI launcher in libfa_fwd.so.
//
// Host-side mirror of torch_mlu's op layer for this path:
//   cnnl__scaled_dot_product_flash_attention  torch_mlu/csrc/aten/operators/cnnl/transformers/attention.cpp:48-159
//   cnnl__flash_attention_forward             torch_mlu/csrc/aten/operators/cnnl/transformers/attention.cpp:161-203
//   mha_varlen_fwd (validation + launch)      torch_mlu/csrc/aten/operators/cnnl/internal/FlashAttention_internal.cpp:57-267
//   generated dispatcher wrapper              codegen/dest/gen_external_mlu.py:483-549 (device guard)
//   registration                              codegen/templates/RegisterMLU.cpp:185-187 (TORCH_LIBRARY_IMPL)
//
// Differences from the reference, all forced by the installed PyTorch or by the no-copy design:
//   * the schemas are the installed PyTorch's (optional cum_seq; window and alibi arguments that must be unset;
//     seqused_k = per-sequence fill level of a KV cache, honoured); the tuple positions and meanings are the
//     reference's (codegen/mlu_functions.yaml:1313,1315);
//   * Q/K/V are never copied: their strides go to the launcher (the reference makes up to three transposing
//     copies at attention.cpp:124-129);
//   * Hq may be a multiple of Hkv at the dense op too (the inner launcher already allowed it,
//     FlashAttention_internal.cpp:122-124);
//   * LSE is returned as [B, Hq, Sq] (dense) / [Hq, total_q] (packed) without the pad-to-16 of
//     FlashAttention_internal.cpp:261-265, which is what the installed PyTorch's shape contract says.
#include <ATen/ATen.h>
#include <ATen/NestedTensorImpl.h>
#include <ATen/native/nested/NestedTensorUtils.h>
#include <ATen/hip/HIPContext.h>
#include <ATen/hip/HIPGeneratorImpl.h>
#include <c10/hip/HIPGraphsC10Utils.h>
#include <ATen/hip/impl/HIPCachingAllocatorMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/InferenceMode.h>
#include <c10/core/DeviceGuard.h>
#include <c10/util/Logging.h>
#include <torch/library.h>

#include <atomic>
#include <cmath>
#include <cstring>
#include <limits>
#include <map>
#include <mutex>
#include <tuple>

#include "fa_bwd.h"
#include "fa_fwd.h"

namespace torch_mlu_amd {

namespace {

std::atomic<int64_t> g_launches{0};  // how many times this extension enqueued the HIP kernels (test hook)

// sdp::calculate_scale, torch_mlu/csrc/aten/operators/cnnl/transformers/sdp_utils.h:40-47, then narrowed to float
// as at attention.cpp:174-175.
float resolve_scale(const at::Tensor& query, std::optional<double> scale) {
  const double s = scale.has_value() ? *scale : 1.0 / std::sqrt(static_cast<double>(query.size(-1)));
  return static_cast<float>(s);
}

struct Packed {
  const at::Tensor* cu_q;
  const at::Tensor* cu_k;
  int64_t max_q, max_k;
};

// The checks of mha_varlen_fwd (FlashAttention_internal.cpp:73-127) in the reference's order and wording.
// `dense` inputs are [B, S, H, D] views, packed ones [T, H, D].
void check_inputs(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const Packed* pk, bool require_device) {
  const auto q_dtype = q.scalar_type();
  TORCH_CHECK(q_dtype == at::kHalf || q_dtype == at::kBFloat16, "FlashAttention only support fp16 and bf16 data type");
  TORCH_CHECK(k.scalar_type() == q_dtype, "query and key must have the same dtype");
  TORCH_CHECK(v.scalar_type() == q_dtype, "query and value must have the same dtype");
  if (pk) {
    TORCH_CHECK(pk->cu_q->scalar_type() == at::kInt, "cu_seqlens_q must have dtype int32");
    TORCH_CHECK(pk->cu_k->scalar_type() == at::kInt, "cu_seqlens_k must have dtype int32");
  }
  if (require_device) {
    TORCH_CHECK(q.is_cuda(), "Input tensor must be on HIP device");
    TORCH_CHECK(k.is_cuda(), "Input tensor must be on HIP device");
    TORCH_CHECK(v.is_cuda(), "Input tensor must be on HIP device");
    if (pk) {
      TORCH_CHECK(pk->cu_q->is_cuda(), "cu_seqlens_q must be on HIP device");
      TORCH_CHECK(pk->cu_k->is_cuda(), "cu_seqlens_k must be on HIP device");
    }
    TORCH_CHECK(k.device() == q.device() && v.device() == q.device(), "Input tensors must be on the same device");
  }
  TORCH_CHECK(q.dim() == (pk ? 3 : 4) && k.dim() == q.dim() && v.dim() == q.dim(),
              pk ? "packed query, key and value must have shape (total, num_heads, head_size)"
                 : "query, key and value must have shape (batch_size, seqlen, num_heads, head_size)");
  TORCH_CHECK(q.stride(-1) == 1, "Input tensor must have contiguous last dimension");
  TORCH_CHECK(k.stride(-1) == 1, "Input tensor must have contiguous last dimension");
  TORCH_CHECK(v.stride(-1) == 1, "Input tensor must have contiguous last dimension");
  if (pk) {
    TORCH_CHECK(pk->cu_q->is_contiguous(), "cu_seqlens_q must be contiguous");
    TORCH_CHECK(pk->cu_k->is_contiguous(), "cu_seqlens_k must be contiguous");
  }
  const int64_t batch = pk ? pk->cu_q->numel() - 1 : q.size(0);
  const int64_t heads = q.size(-2), heads_k = k.size(-2), head_size = q.size(-1);
  TORCH_CHECK(batch > 0, "batch size must be positive");
  TORCH_CHECK(head_size <= 256, "FlashAttention forward only supports head dimension at most 256");
  TORCH_CHECK(head_size % 8 == 0 && head_size > 0, "FlashAttention forward only supports head dimensions that are a multiple of 8");
  TORCH_CHECK(heads_k > 0 && heads % heads_k == 0, "Number of heads in key/value must divide number of heads in query");
  TORCH_CHECK(k.size(-1) == head_size && v.size(-1) == head_size, "query, key and value must have the same head dimension");
  TORCH_CHECK(v.size(-2) == heads_k, "key and value must have the same number of heads");
  if (pk) {
    TORCH_CHECK(pk->cu_q->dim() == 1, "cu_seqlens_q must have shape (batch_size + 1)");
    TORCH_CHECK(pk->cu_k->dim() == 1 && pk->cu_k->numel() == batch + 1, "cu_seqlens_k must have shape (batch_size + 1)");
    TORCH_CHECK(k.size(0) == v.size(0), "Key and Value must have the same sequence length");
    TORCH_CHECK(pk->max_q >= 0 && pk->max_k >= 0, "max_seqlen must be non-negative");
  } else {
    TORCH_CHECK(k.size(0) == batch && v.size(0) == batch, "query, key and value must have the same batch size");
    TORCH_CHECK(k.size(1) == v.size(1), "Key and Value must have the same sequence length");
  }
}

// 16-byte vector access needs 8-element-aligned rows, and the kernels address the rows of a tile with 32-bit byte
// offsets, so the sequence stride ([.., S, H, D]: dimension -3) must stay below 32 MiB / 128 rows; anything else gets
// one copy (never hit by dense layouts).
at::Tensor aligned_or_copy(const at::Tensor& t) {
  bool ok = reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 == 0;
  for (int64_t i = 0; i + 1 < t.dim(); ++i) ok = ok && (t.size(i) == 1 || (t.stride(i) % 8 == 0 && t.stride(i) >= 0));
  if (t.dim() >= 3 && t.size(-3) > 1) ok = ok && t.stride(-3) * 2 <= (int64_t)(0xffffffffLL / 128);
  if (ok) return t;
  TORCH_WARN_ONCE("flash attention: input rows are not 16-byte aligned (or lie more than 32 MiB apart); making one contiguous copy");
  return t.contiguous();
}

void fill_strides(const at::Tensor& t, bool packed, int64_t& sb, int64_t& ss, int64_t& sh) {
  if (packed) {
    sb = 0; ss = t.stride(0); sh = t.stride(1);
  } else {
    sb = t.stride(0); ss = t.stride(1); sh = t.stride(2);
  }
  // a size-1 dimension may carry any stride; keep it harmless for the launcher's alignment rule
  if (!packed && t.size(0) == 1) sb = 0;
  if (t.size(packed ? 0 : 1) == 1) ss = 0;
  if (t.size(packed ? 1 : 2) == 1) sh = 0;
}

}  // namespace

// One (seed, offset) pair of the default generator's Philox state for a call with dropout, taken under the generator's
// mutex (FlashAttention_internal.cpp:198-210).  The increment only has to keep later consumers off this offset.
// `seqused_k` / `seqlen_k`: int32 [batch] on the device.  The backward ops have no such argument, so a call that will
// be differentiated is refused here rather than differentiated wrongly later.
static at::Tensor checked_seqused_k(const at::Tensor& t, int64_t batch, const at::Tensor& q, const at::Tensor& k,
                                    const at::Tensor& v, const char* name) {
  TORCH_CHECK(t.scalar_type() == at::kInt, name, " must have dtype int32");
  TORCH_CHECK(t.is_cuda(), name, " must be on HIP device");
  TORCH_CHECK(t.dim() == 1 && t.size(0) == batch, name, " must have shape (batch_size)");
  TORCH_CHECK(!(at::GradMode::is_enabled() && (q.requires_grad() || k.requires_grad() || v.requires_grad())), name,
              " is for inference: the backward ops cannot take it");
  return t.contiguous();
}

// The generator's Philox state, advanced under its mutex (FlashAttention_internal.cpp:198-210).  Outside graph
// capture the two numbers are known here; during capture the generator hands out device pointers that it refills
// before every replay (the reference's generator does the same, framework/generator/generator_impl.cpp:264-292), and
// the kernel reads them when it runs: seed = *seed_ptr, offset = *offset_ptr + the intra-graph offset.
static void take_philox_state(int64_t seqlen_q, int64_t seqlen_k, fa_fwd_params& p) {
  auto* gen = at::get_generator_or_default<at::CUDAGeneratorImpl>(std::nullopt, at::cuda::detail::getDefaultCUDAGenerator());
  std::lock_guard<std::mutex> lock(gen->mutex_);
  const uint64_t increment = 4 * static_cast<uint64_t>((seqlen_q * seqlen_k + 1023) / 1024 + 1);
  const at::PhiloxCudaState st = gen->philox_cuda_state(increment);
  if (st.captured_) {
    p.philox_seed = 0;
    p.philox_offset = st.offset_intragraph_;
    p.philox_seed_ptr = st.seed_.ptr;
    p.philox_offset_ptr = st.offset_.ptr;
  } else {
    p.philox_seed = st.seed_.val;
    p.philox_offset = st.offset_.val;
  }
}

// ---- _flash_attention_forward ---------------------------------------------------------------------------------
// cnnl__flash_attention_forward, attention.cpp:161-203.  cum_seq given: packed [T, H, D] inputs (the reference's
// only mode); absent: dense [B, S, H, D] inputs (installed-PyTorch extension of the schema).
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor> flash_attention_forward(
    const at::Tensor& query, const at::Tensor& key, const at::Tensor& value,
    const std::optional<at::Tensor>& cum_seq_q, const std::optional<at::Tensor>& cum_seq_k, int64_t max_q,
    int64_t max_k, double dropout_p, bool is_causal, bool return_debug_mask, std::optional<double> scale,
    std::optional<int64_t> window_size_left, std::optional<int64_t> window_size_right,
    const std::optional<at::Tensor>& seqused_k, const std::optional<at::Tensor>& alibi_slopes) {
  const bool packed = cum_seq_q.has_value() && cum_seq_q->defined();
  TORCH_CHECK(packed == (cum_seq_k.has_value() && cum_seq_k->defined()),
              "cum_seq_q and cum_seq_k must be given together");
  TORCH_CHECK(dropout_p >= 0.0 && dropout_p < 1.0, "flash attention forward: dropout_p must be in [0, 1), got ", dropout_p);
  TORCH_CHECK(!window_size_left.has_value() || *window_size_left < 0, "flash attention forward: sliding window is not supported");
  TORCH_CHECK(!window_size_right.has_value() || *window_size_right < 0 || (is_causal && *window_size_right == 0),
              "flash attention forward: sliding window is not supported");
  const bool has_used = seqused_k.has_value() && seqused_k->defined();
  TORCH_CHECK(!(alibi_slopes.has_value() && alibi_slopes->defined()), "flash attention forward: alibi_slopes is not supported");

  Packed pk{packed ? &*cum_seq_q : nullptr, packed ? &*cum_seq_k : nullptr, max_q, max_k};
  check_inputs(query, key, value, packed ? &pk : nullptr, /*require_device=*/true);

  // HIP tensors carry the "cuda" device type in PyTorch-ROCm: the generic guard resolves to the HIP implementation
  const c10::OptionalDeviceGuard guard(query.device());
  const float softmax_scale = resolve_scale(query, scale);

  const at::Tensor q = aligned_or_copy(query), k = aligned_or_copy(key), v = aligned_or_copy(value);
  // out = empty_like(query) over a contiguous query in the reference (attention.cpp:176): dense [B,S,H,D] storage
  at::Tensor output = at::empty(q.sizes(), q.options());
  const int64_t batch = packed ? cum_seq_q->numel() - 1 : q.size(0);
  const int64_t heads = q.size(-2), head_size = q.size(-1);
  const int64_t seqlen_q = packed ? max_q : q.size(1);
  const int64_t seqlen_k = packed ? max_k : k.size(1);
  const int64_t total_q = packed ? q.size(0) : batch * seqlen_q;
  // kernel-side LSE buffer: [Hq, total_q] packed (FlashAttention_internal.cpp:129), [B, Hq, Sq] dense
  at::Tensor lse = packed ? at::empty({heads, total_q}, q.options().dtype(at::kFloat))
                          : at::empty({batch, heads, seqlen_q}, q.options().dtype(at::kFloat));
  TORCH_CHECK(seqlen_q <= INT32_MAX && seqlen_k <= INT32_MAX && batch <= INT32_MAX, "sequence length too large");

  fa_fwd_params p{};
  p.q = q.data_ptr(); p.k = k.data_ptr(); p.v = v.data_ptr(); p.out = output.data_ptr();
  p.lse = lse.data_ptr<float>();
  p.cu_seqlens_q = packed ? cum_seq_q->data_ptr<int32_t>() : nullptr;
  p.cu_seqlens_k = packed ? cum_seq_k->data_ptr<int32_t>() : nullptr;
  fill_strides(q, packed, p.q_stride_b, p.q_stride_s, p.q_stride_h);
  fill_strides(k, packed, p.k_stride_b, p.k_stride_s, p.k_stride_h);
  fill_strides(v, packed, p.v_stride_b, p.v_stride_s, p.v_stride_h);
  fill_strides(output, packed, p.o_stride_b, p.o_stride_s, p.o_stride_h);
  if (packed) {
    p.lse_stride_b = 0; p.lse_stride_h = lse.stride(0); p.lse_stride_s = lse.stride(1);
  } else {
    p.lse_stride_b = lse.stride(0); p.lse_stride_h = lse.stride(1); p.lse_stride_s = lse.stride(2);
  }
  p.batch = static_cast<int32_t>(batch);
  p.heads_q = static_cast<int32_t>(heads);
  p.heads_k = static_cast<int32_t>(k.size(-2));
  p.seqlen_q = static_cast<int32_t>(seqlen_q);
  p.seqlen_k = static_cast<int32_t>(seqlen_k);
  p.head_dim = static_cast<int32_t>(head_size);
  p.scale = softmax_scale;
  p.dtype = q.scalar_type() == at::kBFloat16 ? FA_DTYPE_BF16 : FA_DTYPE_FP16;
  p.is_causal = is_causal ? 1 : 0;
  p.kernel = FA_KERNEL_AUTO;
  p.num_splits = 0;
  at::Tensor used;  // per-sequence count of the key rows that exist (a KV cache filled to different lengths)
  if (has_used) {
    used = checked_seqused_k(*seqused_k, batch, query, key, value, "seqused_k");
    p.seqused_k = used.data_ptr<int32_t>();
  }

  // p == 0: the reference returns two uninitialised 0-d int64 tensors (FlashAttention_internal.cpp:211-213); p > 0:
  // the generator's Philox state, advanced under its mutex (:198-210) — here the kernel stores the two numbers into
  // the slots, which live on the device as the installed PyTorch's backward expects.
  at::Tensor seed_t = at::empty({}, q.options().dtype(at::kLong));
  at::Tensor offset_t = at::empty({}, q.options().dtype(at::kLong));
  at::Tensor debug_attn_mask = at::empty({0}, q.options());
  if (dropout_p > 0.0) {
    take_philox_state(seqlen_q, seqlen_k, p);
    p.dropout_p = static_cast<float>(dropout_p);
    p.rng_seed_out = seed_t.data_ptr<int64_t>();
    p.rng_offset_out = offset_t.data_ptr<int64_t>();
    if (return_debug_mask) {
      // [B, H, max_q, max_k], > 0 where kept (the reference: zeros filled by the kernel, :141-146; its tests use
      // `mask > 0`, test_scaled_dot_product_attention.py:1049-1050)
      debug_attn_mask = at::zeros({batch, heads, seqlen_q, seqlen_k}, q.options());
      p.dropout_mask = debug_attn_mask.data_ptr();
    }
  }

  if (total_q > 0) {
    // workspace: stream-ordered caching allocator, as the reference does (FlashAttention_internal.cpp:215-230)
    const size_t ws_bytes = fa_fwd_workspace_bytes(&p);
    at::Tensor ws;
    if (ws_bytes) ws = at::empty({static_cast<int64_t>(ws_bytes)}, q.options().dtype(at::kByte));
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(q.device().index()).stream();
    const int rc = fa_fwd_launch(&p, ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, stream);
    TORCH_CHECK(rc == FA_OK, "fa_fwd_launch failed: ", fa_fwd_error_string(rc), " (rc=", rc, ")");
    g_launches.fetch_add(1, std::memory_order_relaxed);
  }

  // return_debug_mask only has an effect with dropout (attention.cpp:178-199)
  return std::make_tuple(output, lse, seed_t, offset_t, debug_attn_mask);
}

namespace {

// Uniform prefix sums arange(0, (B+1) S, S) as the reference fabricates on every call (attention.cpp:109-119).
// They are immutable, so one copy per (device, B, S) is kept.  A miss enqueues one arange on the current stream and
// records an event behind it; a later call on another stream makes that stream wait for the event (a device-side
// dependency) — the host never waits.  The cached tensor is built outside inference mode and without a gradient
// history, so that a first call under torch.inference_mode() cannot leave a tensor behind that autograd refuses to
// save later.  While a HIP graph is being captured the cache is bypassed (no event, no allocation that outlives the
// capture).  At most kCuSeqlensCacheEntries entries are kept; the least recently used one is dropped first.
constexpr size_t kCuSeqlensCacheEntries = 256;

struct CuSeqlensEntry {
  at::Tensor t;
  hipEvent_t ready = nullptr;   // recorded behind the arange on `stream`
  hipStream_t stream = nullptr;
  uint64_t last_use = 0;
};

at::Tensor uniform_cu_seqlens(int64_t batch, int64_t seqlen, const at::Tensor& like) {
  const auto opts = like.options().dtype(at::kInt);
  auto make = [&] { return at::arange(0, (batch + 1) * seqlen, seqlen > 0 ? seqlen : 1, opts); };
  if (seqlen == 0) return at::zeros({batch + 1}, opts);
  if (c10::hip::currentStreamCaptureStatusMayInitCtx() != c10::hip::CaptureStatus::None) return make();
  static std::mutex mu;
  static std::map<std::tuple<int, int64_t, int64_t>, CuSeqlensEntry> cache;
  static uint64_t tick = 0;
  const int dev = static_cast<int>(like.device().index());
  const auto cur = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(dev);
  const auto key = std::make_tuple(dev, batch, seqlen);
  std::lock_guard<std::mutex> lock(mu);
  auto it = cache.find(key);
  if (it == cache.end()) {
    if (cache.size() >= kCuSeqlensCacheEntries) {
      auto victim = cache.begin();
      for (auto e = cache.begin(); e != cache.end(); ++e)
        if (e->second.last_use < victim->second.last_use) victim = e;
      // tensors handed out earlier keep the storage alive; the event is only needed by streams that have not used
      // this entry yet, and no such use can start once the entry is gone
      if (victim->second.ready) (void)hipEventDestroy(victim->second.ready);
      cache.erase(victim);
    }
    CuSeqlensEntry e;
    {
      c10::InferenceMode no_inference(false);
      at::AutoGradMode no_grad(false);
      e.t = make();
    }
    e.stream = cur.stream();
    if (hipEventCreateWithFlags(&e.ready, hipEventDisableTiming) != hipSuccess || hipEventRecord(e.ready, e.stream) != hipSuccess) {
      (void)hipGetLastError();
      if (e.ready) (void)hipEventDestroy(e.ready);
      return e.t;  // not cached: the tensor is only known to be ready on this stream
    }
    it = cache.emplace(key, std::move(e)).first;
  } else if (it->second.stream != cur.stream()) {
    // device-side wait; free once the arange has completed
    (void)hipStreamWaitEvent(cur.stream(), it->second.ready, 0);
    // the storage was allocated on another stream: tell the caching allocator about this one, so that the block is
    // not reused under a reader of this stream after the entry has been dropped
    c10::hip::HIPCachingAllocatorMasqueradingAsCUDA::recordStreamMasqueradingAsCUDA(it->second.t.storage().data_ptr(), cur);
  }
  it->second.last_use = ++tick;
  return it->second.t;
}

}  // namespace

// ---- _scaled_dot_product_flash_attention ----------------------------------------------------------------------
// cnnl__scaled_dot_product_flash_attention, attention.cpp:48-159.
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, c10::SymInt, c10::SymInt, at::Tensor, at::Tensor, at::Tensor>
scaled_dot_product_flash_attention(const at::Tensor& query, const at::Tensor& key, const at::Tensor& value,
                                   double dropout_p, bool is_causal, bool return_debug_mask,
                                   std::optional<double> scale) {
  C10_LOG_API_USAGE_ONCE("torch.sdpa.flash_attention");  // attention.cpp:67
  // attention.cpp:70-100
  TORCH_CHECK(query.dim() == 4 && key.dim() == 4 && value.dim() == 4,
              "query, key and value must be 4-dimensional (batch, num_heads, seq_len, head_dim)");
  TORCH_CHECK(query.size(0) == key.size(0) && query.size(0) == value.size(0),
              "query, key and value must have the same batch size");
  TORCH_CHECK(key.size(2) == value.size(2), "Key and Value must have the same sequence length");
  TORCH_CHECK(key.size(1) == value.size(1), "key and value must have the same number of heads");
  // relaxed from equality (attention.cpp:82-83) to the divisibility the launcher already accepts
  TORCH_CHECK(key.size(1) > 0 && query.size(1) % key.size(1) == 0,
              "Number of heads in key/value must divide number of heads in query");
  TORCH_CHECK(query.size(3) == key.size(3), "query and key must have the same head dimension");

  const int64_t batch_size = query.size(0);
  const int64_t max_seqlen_batch_q = query.size(2);
  const int64_t max_seqlen_batch_k = key.size(2);

  // [B,H,S,D] -> [B,S,H,D] views; no contiguous copies (attention.cpp:105-107 without :124-129)
  const at::Tensor q_t = query.transpose(1, 2);
  const at::Tensor k_t = key.transpose(1, 2);
  const at::Tensor v_t = value.transpose(1, 2);

  auto [attention, log_sumexp, philox_seed, philox_offset, debug_attn_mask] = at::_flash_attention_forward(
      q_t, k_t, v_t, std::nullopt, std::nullopt, max_seqlen_batch_q, max_seqlen_batch_k, dropout_p, is_causal,
      return_debug_mask, scale, std::nullopt, std::nullopt, std::nullopt, std::nullopt);

  const at::Tensor cumulative_sequence_length_q = uniform_cu_seqlens(batch_size, max_seqlen_batch_q, query);
  const at::Tensor cumulative_sequence_length_k = uniform_cu_seqlens(batch_size, max_seqlen_batch_k, query);

  // [B,S,H,D] storage returned as the [B,H,S,D] view (attention.cpp:146-148)
  attention = attention.transpose(1, 2);
  return std::make_tuple(attention, log_sumexp, cumulative_sequence_length_q, cumulative_sequence_length_k,
                         c10::SymInt(max_seqlen_batch_q), c10::SymInt(max_seqlen_batch_k), philox_seed,
                         philox_offset, debug_attn_mask);
}

// ---- _flash_attention_backward --------------------------------------------------------------------------------
// cnnl__flash_attention_backward, attention.cpp:305-348, and the checks of mha_varlen_bwd
// (FlashAttention_internal.cpp:288-366).  3-D inputs: packed [T, H, D] with cum_seq (the reference's only mode);
// 4-D inputs: dense [B, S, H, D] views (cum_seq ignored), which is how the dense wrapper below calls it.
std::tuple<at::Tensor, at::Tensor, at::Tensor> flash_attention_backward(
    const at::Tensor& grad_out, const at::Tensor& query, const at::Tensor& key, const at::Tensor& value,
    const at::Tensor& out, const at::Tensor& logsumexp, const at::Tensor& cum_seq_q, const at::Tensor& cum_seq_k,
    int64_t max_q, int64_t max_k, double dropout_p, bool is_causal, const at::Tensor& philox_seed,
    const at::Tensor& philox_offset, std::optional<double> scale, std::optional<int64_t> window_size_left,
    std::optional<int64_t> window_size_right) {
  TORCH_CHECK(dropout_p >= 0.0 && dropout_p < 1.0, "flash attention backward: dropout_p must be in [0, 1), got ", dropout_p);
  if (dropout_p > 0.0)
    TORCH_CHECK(philox_seed.defined() && philox_offset.defined() && philox_seed.is_cuda() && philox_offset.is_cuda() &&
                    philox_seed.scalar_type() == at::kLong && philox_offset.scalar_type() == at::kLong &&
                    philox_seed.numel() == 1 && philox_offset.numel() == 1,
                "flash attention backward: philox_seed and philox_offset must be the int64 device scalars the forward "
                "returned");
  TORCH_CHECK(!window_size_left.has_value() || *window_size_left < 0, "flash attention backward: sliding window is not supported");
  TORCH_CHECK(!window_size_right.has_value() || *window_size_right < 0 || (is_causal && *window_size_right == 0),
              "flash attention backward: sliding window is not supported");
  const bool packed = query.dim() == 3;
  if (packed) TORCH_CHECK(cum_seq_q.defined() && cum_seq_k.defined(), "packed inputs need cum_seq_q and cum_seq_k");
  Packed pk{packed ? &cum_seq_q : nullptr, packed ? &cum_seq_k : nullptr, max_q, max_k};
  check_inputs(query, key, value, packed ? &pk : nullptr, /*require_device=*/true);
  TORCH_CHECK(grad_out.scalar_type() == query.scalar_type(), "query and dout must have the same dtype");
  TORCH_CHECK(out.scalar_type() == query.scalar_type(), "query and out must have the same dtype");
  TORCH_CHECK(grad_out.sizes() == query.sizes() && out.sizes() == query.sizes(), "dout and out must have the shape of query");
  TORCH_CHECK(logsumexp.scalar_type() == at::kFloat && logsumexp.is_cuda(), "logsumexp must be a float32 tensor on the device");
  TORCH_CHECK(query.size(-1) <= 256, "FlashAttention backward only supports head dimension at most 256");  // :355-357

  const c10::OptionalDeviceGuard guard(query.device());
  const float softmax_scale = resolve_scale(query, scale);
  auto fix = [](const at::Tensor& t) { return t.stride(-1) == 1 ? aligned_or_copy(t) : t.contiguous(); };
  const at::Tensor q = aligned_or_copy(query), k = aligned_or_copy(key), v = aligned_or_copy(value);
  const at::Tensor dout = fix(grad_out), o = fix(out);  // the reference makes both contiguous (attention.cpp:324-325)
  at::Tensor dq = at::empty(q.sizes(), q.options());
  at::Tensor dk = at::empty(k.sizes(), k.options());
  at::Tensor dv = at::empty(v.sizes(), v.options());

  const int64_t batch = packed ? cum_seq_q.numel() - 1 : q.size(0);
  const int64_t heads = q.size(-2);
  const int64_t seqlen_q = packed ? max_q : q.size(1);
  const int64_t seqlen_k = packed ? max_k : k.size(1);
  const int64_t total_q = packed ? q.size(0) : batch * seqlen_q;
  if (packed) {
    TORCH_CHECK(logsumexp.dim() == 2 && logsumexp.size(0) == heads && logsumexp.size(1) == total_q,
                "logsumexp must have shape (num_heads, total_q)");
  } else {
    TORCH_CHECK(logsumexp.dim() == 3 && logsumexp.size(0) == batch && logsumexp.size(1) == heads &&
                    logsumexp.size(2) >= seqlen_q,
                "logsumexp must have shape (batch_size, num_heads, seqlen_q)");
  }

  fa_bwd_params p{};
  p.q = q.data_ptr(); p.k = k.data_ptr(); p.v = v.data_ptr(); p.out = o.data_ptr(); p.dout = dout.data_ptr();
  p.lse = logsumexp.data_ptr<float>();
  p.dq = dq.data_ptr(); p.dk = dk.data_ptr(); p.dv = dv.data_ptr();
  p.cu_seqlens_q = packed ? cum_seq_q.data_ptr<int32_t>() : nullptr;
  p.cu_seqlens_k = packed ? cum_seq_k.data_ptr<int32_t>() : nullptr;
  fill_strides(q, packed, p.q_stride_b, p.q_stride_s, p.q_stride_h);
  fill_strides(k, packed, p.k_stride_b, p.k_stride_s, p.k_stride_h);
  fill_strides(v, packed, p.v_stride_b, p.v_stride_s, p.v_stride_h);
  fill_strides(o, packed, p.o_stride_b, p.o_stride_s, p.o_stride_h);
  fill_strides(dout, packed, p.do_stride_b, p.do_stride_s, p.do_stride_h);
  fill_strides(dq, packed, p.dq_stride_b, p.dq_stride_s, p.dq_stride_h);
  fill_strides(dk, packed, p.dk_stride_b, p.dk_stride_s, p.dk_stride_h);
  fill_strides(dv, packed, p.dv_stride_b, p.dv_stride_s, p.dv_stride_h);
  if (packed) {
    p.lse_stride_b = 0; p.lse_stride_h = logsumexp.stride(0); p.lse_stride_s = logsumexp.stride(1);
  } else {
    p.lse_stride_b = logsumexp.stride(0); p.lse_stride_h = logsumexp.stride(1); p.lse_stride_s = logsumexp.stride(2);
  }
  p.batch = static_cast<int32_t>(batch);
  p.heads_q = static_cast<int32_t>(heads);
  p.heads_k = static_cast<int32_t>(k.size(-2));
  p.seqlen_q = static_cast<int32_t>(seqlen_q);
  p.seqlen_k = static_cast<int32_t>(seqlen_k);
  p.head_dim = static_cast<int32_t>(q.size(-1));
  p.total_q = total_q;
  p.scale = softmax_scale;
  p.dtype = q.scalar_type() == at::kBFloat16 ? FA_DTYPE_BF16 : FA_DTYPE_FP16;
  p.is_causal = is_causal ? 1 : 0;
  if (dropout_p > 0.0) {
    p.dropout_p = static_cast<float>(dropout_p);
    p.philox_seed = philox_seed.data_ptr<int64_t>();
    p.philox_offset = philox_offset.data_ptr<int64_t>();
  }

  if (total_q == 0 || k.numel() == 0) {
    dq.zero_(); dk.zero_(); dv.zero_();
    return std::make_tuple(dq, dk, dv);
  }
  const size_t ws_bytes = fa_bwd_workspace_bytes(&p);
  at::Tensor ws = at::empty({static_cast<int64_t>(ws_bytes > 0 ? ws_bytes : 16)}, q.options().dtype(at::kByte));
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(q.device().index()).stream();
  const int rc = fa_bwd_launch(&p, ws.data_ptr(), ws_bytes, stream);
  TORCH_CHECK(rc == FA_OK, "fa_bwd_launch failed: ", fa_fwd_error_string(rc), " (rc=", rc, ")");
  g_launches.fetch_add(1, std::memory_order_relaxed);
  return std::make_tuple(dq, dk, dv);
}

// ---- _scaled_dot_product_flash_attention_backward -------------------------------------------------------------
// cnnl__scaled_dot_product_flash_attention_backward, attention.cpp:205-303 — without its contiguous copies.
std::tuple<at::Tensor, at::Tensor, at::Tensor> scaled_dot_product_flash_attention_backward(
    const at::Tensor& grad_out, const at::Tensor& query, const at::Tensor& key, const at::Tensor& value,
    const at::Tensor& out, const at::Tensor& logsumexp, const at::Tensor& cum_seq_q, const at::Tensor& cum_seq_k,
    int64_t max_q, int64_t max_k, double dropout_p, bool is_causal, const at::Tensor& philox_seed,
    const at::Tensor& philox_offset, std::optional<double> scale) {
  if (!grad_out.defined()) return std::make_tuple(at::Tensor{}, at::Tensor{}, at::Tensor{});  // attention.cpp:222-224
  TORCH_CHECK(query.dim() == 4 && key.dim() == 4 && value.dim() == 4 && grad_out.dim() == 4,
              "query, key, value and grad_out must be 4-dimensional (batch, num_heads, seq_len, head_dim)");
  TORCH_CHECK(query.size(0) == grad_out.size(0) && query.size(0) == key.size(0) && query.size(0) == value.size(0),
              "query, key, value and grad_out must have the same batch size");
  TORCH_CHECK(key.size(2) == value.size(2), "Key and Value must have the same sequence length");
  TORCH_CHECK(query.size(2) == grad_out.size(2) && query.size(1) == grad_out.size(1), "grad_out must have the shape of query");
  TORCH_CHECK(query.size(3) == key.size(3) && value.size(3) == grad_out.size(3),
              "query, key, value and grad_out must have the same head dimension");
  auto [grad_q, grad_k, grad_v] = at::_flash_attention_backward(
      grad_out.transpose(1, 2), query.transpose(1, 2), key.transpose(1, 2), value.transpose(1, 2),
      out.transpose(1, 2), logsumexp, cum_seq_q, cum_seq_k, max_q, max_k, dropout_p, is_causal, philox_seed,
      philox_offset, scale, std::nullopt, std::nullopt);
  // [B,S,H,D] storage returned as [B,H,S,D] views (attention.cpp:297-302)
  return std::make_tuple(grad_q.transpose(1, 2), grad_k.transpose(1, 2), grad_v.transpose(1, 2));
}

namespace {
// cu_seqlens of the mem-efficient ops: int32 [batch + 1] on the device (attention.cpp:433-443,455-465 and their messages)
void check_efficient_cu_seqlens(const at::Tensor& cu_q, const at::Tensor& cu_k, int64_t batch) {
  TORCH_CHECK(cu_q.scalar_type() == at::kInt, "cu_seqlens_q must have dtype int32");
  TORCH_CHECK(cu_q.is_cuda(), "cu_seqlens_q must be on HIP device");
  TORCH_CHECK(cu_q.dim() == 1 && cu_q.size(0) == batch + 1, "cu_seqlens_q must have shape (batch_size + 1)");
  TORCH_CHECK(cu_k.scalar_type() == at::kInt, "cu_seqlens_k must have dtype int32");
  TORCH_CHECK(cu_k.is_cuda(), "cu_seqlens_k must be on HIP device");
  TORCH_CHECK(cu_k.dim() == 1 && cu_k.size(0) == batch + 1, "cu_seqlens_k must have shape (batch_size + 1)");
  TORCH_CHECK(cu_q.is_contiguous() && cu_k.is_contiguous(), "cu_seqlens must be contiguous");
}
// A [B, S, H, D] tensor whose rows can be addressed by their index in the flattened [B * S] view (one copy if not)
at::Tensor flattenable(const at::Tensor& t) {
  return (t.size(0) <= 1 || t.stride(0) == t.size(1) * t.stride(1)) ? t : t.contiguous();
}
// The bias as a [B, H, Sq, Sk] view (stride 0 where broadcast) that meets the kernels' alignment rule: groups of 4
// keys 8-byte aligned.  If the caller's does not, one copy of the un-broadcast bias with rows padded to a multiple of
// 8 columns is made (the reference always copies: cnnl_contiguous, attention.cpp:660-663).
at::Tensor bias_for_kernels(const at::Tensor& bias, at::ScalarType dt, int64_t B, int64_t Hq, int64_t Sq, int64_t Sk) {
  TORCH_CHECK(bias.scalar_type() == dt, "bias must have the same dtype as query");
  TORCH_CHECK(bias.is_cuda(), "bias must be on HIP device");
  TORCH_CHECK(bias.dim() <= 4, "bias must have at most 4 dimensions");
  at::Tensor bias_e = bias.expand({B, Hq, Sq, Sk});
  const bool ok = Sk == 0 || (bias_e.stride(3) == 1 && bias_e.stride(0) % 4 == 0 && bias_e.stride(1) % 4 == 0 &&
                              bias_e.stride(2) % 4 == 0 && reinterpret_cast<uintptr_t>(bias_e.data_ptr()) % 8 == 0);
  if (!ok) {
    const int64_t Skp = (Sk + 7) / 8 * 8;
    at::Tensor b4 = bias;
    while (b4.dim() < 4) b4 = b4.unsqueeze(0);
    at::Tensor padded = at::empty({b4.size(0), b4.size(1), b4.size(2), Skp}, b4.options());
    padded.narrow(3, 0, Sk).copy_(b4.expand({b4.size(0), b4.size(1), b4.size(2), Sk}));
    bias_e = padded.narrow(3, 0, Sk).expand({B, Hq, Sq, Sk});
  }
  return bias_e;
}
}  // namespace

// ---- _efficient_attention_forward -------------------------------------------------------------------------------
// cnnl__efficient_attention_forward (attention.cpp:390-508) + mem_eff_fwd (FlashAttention_internal.cpp:485-690):
// inputs [B, S, H, D], optional additive bias broadcastable to [B, H, Sq, Skv], custom_mask_type 0 (none),
// 1 (causal from the top-left corner) or 2 (causal from the bottom-right corner).  No contiguous copies of q/k/v.
// Returned as the installed PyTorch's schema asks: output [B, Sq, H, D] (the dense wrapper transposes it),
// logsumexp [B, H, Sq] (or [B, H, 0] without compute_log_sumexp), philox slots, and the two maximum lengths.
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, c10::SymInt, c10::SymInt> efficient_attention_forward(
    const at::Tensor& query, const at::Tensor& key, const at::Tensor& value, const std::optional<at::Tensor>& bias,
    const std::optional<at::Tensor>& cu_seqlens_q, const std::optional<at::Tensor>& cu_seqlens_k,
    std::optional<c10::SymInt> max_seqlen_q, std::optional<c10::SymInt> max_seqlen_k, double dropout_p,
    int64_t custom_mask_type, bool compute_log_sumexp, std::optional<double> scale,
    const std::optional<at::Tensor>& seqlen_k, std::optional<int64_t> window_size) {
  // the reference's checks, in its order (attention.cpp:405-423)
  TORCH_CHECK(query.dim() == 4 && key.dim() == 4 && value.dim() == 4, "query, key and value must be 4-dimensional "
              "(batch, seq_len, num_heads, head_dim)");
  TORCH_CHECK(query.size(0) == key.size(0) && query.size(0) == value.size(0), "query, key and value must have the same batch size");
  TORCH_CHECK(key.size(1) == value.size(1), "key and value must have the same sequence length");
  TORCH_CHECK(key.size(2) == value.size(2) && key.size(2) > 0 && query.size(2) % key.size(2) == 0,
              "Number of heads in key/value must divide number of heads in query");
  TORCH_CHECK(query.size(3) == key.size(3), "query and key must have the same head dimension");
  TORCH_CHECK(value.size(3) == query.size(3), "this build needs value.size(-1) == query.size(-1)");
  // cu_seqlens (attention.cpp:431-466): offsets of the sequences in the rows of the [B * S, H, D] view of the inputs
  const bool packed = cu_seqlens_q.has_value() && cu_seqlens_q->defined();
  TORCH_CHECK(packed == (cu_seqlens_k.has_value() && cu_seqlens_k->defined()), "cu_seqlens_q and cu_seqlens_k must be given together");
  // A second packed convention, the installed PyTorch's own (what its nested-tensor path passes): batch 1, all
  // sequences' rows one after the other in [1, total, H, D] tensors, cu_seqlens of (number of sequences + 1) entries
  // and the two maximum lengths.  A bias is then [sequences, H, max_seqlen_q, max_seqlen_k], indexed by sequence and by
  // the row / key position inside the sequence.
  const bool ragged = packed && query.size(0) == 1 && cu_seqlens_q->dim() == 1 && cu_seqlens_q->size(0) != 2;
  if (ragged) {
    TORCH_CHECK(max_seqlen_q.has_value() && max_seqlen_k.has_value(),
                "cu_seqlens with batch size 1 need max_seqlen_q and max_seqlen_k");
    TORCH_CHECK(cu_seqlens_q->size(0) >= 2, "cu_seqlens_q must have at least two entries");
    check_efficient_cu_seqlens(*cu_seqlens_q, *cu_seqlens_k, cu_seqlens_q->size(0) - 1);
  } else if (packed) {
    check_efficient_cu_seqlens(*cu_seqlens_q, *cu_seqlens_k, query.size(0));
  }
  TORCH_CHECK(!window_size.has_value() || *window_size <= 0, "efficient attention forward: sliding window is not supported");
  TORCH_CHECK(dropout_p >= 0.0 && dropout_p < 1.0, "efficient attention forward: dropout_p must be in [0, 1), got ", dropout_p);
  TORCH_CHECK(custom_mask_type >= 0 && custom_mask_type <= 2, "custom_mask_type must be 0, 1 or 2");
  // mem_eff_fwd's checks (FlashAttention_internal.cpp:500-527)
  const auto dt = query.scalar_type();
  TORCH_CHECK(dt == at::kHalf || dt == at::kBFloat16, "FlashAttention only support fp16 and bf16 data type");
  TORCH_CHECK(key.scalar_type() == dt, "query and key must have the same dtype");
  TORCH_CHECK(value.scalar_type() == dt, "query and value must have the same dtype");
  TORCH_CHECK(query.is_cuda() && key.is_cuda() && value.is_cuda(), "Input tensor must be on HIP device");
  TORCH_CHECK(query.stride(-1) == 1 && key.stride(-1) == 1 && value.stride(-1) == 1,
              "Input tensor must have contiguous last dimension");
  const int64_t B = query.size(0), Sq = query.size(1), Hq = query.size(2), D = query.size(3);
  const int64_t Sk = key.size(1), Hk = key.size(2);
  TORCH_CHECK(B > 0, "batch size must be positive");
  TORCH_CHECK(D <= 256, "FlashAttention forward only supports head dimension at most 256");
  TORCH_CHECK(D % 8 == 0, "head dimension must be a multiple of 8");
  TORCH_CHECK(Sq <= INT32_MAX && Sk <= INT32_MAX && B <= INT32_MAX, "sequence length too large");

  const c10::OptionalDeviceGuard guard(query.device());
  const float softmax_scale = resolve_scale(query, scale);
  at::Tensor q = aligned_or_copy(query), k = aligned_or_copy(key), v = aligned_or_copy(value);
  if (packed) {  // rows are addressed by their index in the flattened [B * S] view
    q = flattenable(q); k = flattenable(k); v = flattenable(v);
  }
  // packed: rows outside every sequence are never written; logsumexp is the kernel's raw [H, B * Sq] buffer, as the
  // reference returns it (FlashAttention_internal.cpp:599-606,689)
  at::Tensor output = packed ? at::zeros({B, Sq, Hq, D}, q.options()) : at::empty({B, Sq, Hq, D}, q.options());
  at::Tensor lse = packed ? at::full({Hq, B * Sq}, std::numeric_limits<float>::infinity(), q.options().dtype(at::kFloat))
                          : at::empty({B, Hq, Sq}, q.options().dtype(at::kFloat));

  // what the kernels see as (batch, seqlen_q, seqlen_k): the tensors' own, or the ragged convention's
  const int64_t nseq = ragged ? cu_seqlens_q->size(0) - 1 : B;
  const int64_t kSq = ragged ? max_seqlen_q->expect_int() : Sq, kSk = ragged ? max_seqlen_k->expect_int() : Sk;
  TORCH_CHECK(kSq >= 0 && kSk >= 0 && kSq <= INT32_MAX && kSk <= INT32_MAX && nseq <= INT32_MAX, "sequence length too large");
  at::Tensor bias_e;
  if (bias.has_value() && bias->defined()) bias_e = bias_for_kernels(*bias, dt, nseq, Hq, kSq, kSk);

  fa_fwd_params p{};
  p.q = q.data_ptr(); p.k = k.data_ptr(); p.v = v.data_ptr(); p.out = output.data_ptr();
  p.lse = lse.data_ptr<float>();
  fill_strides(q, false, p.q_stride_b, p.q_stride_s, p.q_stride_h);
  fill_strides(k, false, p.k_stride_b, p.k_stride_s, p.k_stride_h);
  fill_strides(v, false, p.v_stride_b, p.v_stride_s, p.v_stride_h);
  fill_strides(output, false, p.o_stride_b, p.o_stride_s, p.o_stride_h);
  if (packed) {
    p.cu_seqlens_q = cu_seqlens_q->data_ptr<int32_t>();
    p.cu_seqlens_k = cu_seqlens_k->data_ptr<int32_t>();
    p.lse_stride_b = 0; p.lse_stride_h = lse.stride(0); p.lse_stride_s = lse.stride(1);
  } else {
    p.lse_stride_b = lse.stride(0); p.lse_stride_h = lse.stride(1); p.lse_stride_s = lse.stride(2);
  }
  p.batch = static_cast<int32_t>(nseq);
  p.heads_q = static_cast<int32_t>(Hq);
  p.heads_k = static_cast<int32_t>(Hk);
  p.seqlen_q = static_cast<int32_t>(kSq);
  p.seqlen_k = static_cast<int32_t>(kSk);
  p.head_dim = static_cast<int32_t>(D);
  p.scale = softmax_scale;
  p.dtype = dt == at::kBFloat16 ? FA_DTYPE_BF16 : FA_DTYPE_FP16;
  p.is_causal = custom_mask_type == 1 ? FA_MASK_CAUSAL_TOP_LEFT
                                      : (custom_mask_type == 2 ? FA_MASK_CAUSAL_BOTTOM_RIGHT : FA_MASK_NONE);
  p.kernel = FA_KERNEL_AUTO;
  at::Tensor used;
  if (seqlen_k.has_value() && seqlen_k->defined()) {
    used = checked_seqused_k(*seqlen_k, nseq, query, key, value, "seqlen_k");
    p.seqused_k = used.data_ptr<int32_t>();
  }
  if (bias_e.defined() && kSk > 0) {
    p.bias = bias_e.data_ptr();
    p.bias_stride_b = bias_e.stride(0); p.bias_stride_h = bias_e.stride(1); p.bias_stride_q = bias_e.stride(2);
  }
  // the two Philox numbers of a call with dropout live on the device, stored there by the kernel (as in the flash op)
  at::Tensor seed_t = at::empty({}, q.options().dtype(at::kLong));
  at::Tensor offset_t = at::empty({}, q.options().dtype(at::kLong));
  if (dropout_p > 0.0) {
    take_philox_state(kSq, kSk, p);
    p.dropout_p = static_cast<float>(dropout_p);
    p.rng_seed_out = seed_t.data_ptr<int64_t>();
    p.rng_offset_out = offset_t.data_ptr<int64_t>();
  }
  if (B * Sq * Hq > 0) {
    const size_t ws_bytes = fa_fwd_workspace_bytes(&p);
    at::Tensor ws;
    if (ws_bytes) ws = at::empty({static_cast<int64_t>(ws_bytes)}, q.options().dtype(at::kByte));
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(q.device().index()).stream();
    const int rc = fa_fwd_launch(&p, ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, stream);
    TORCH_CHECK(rc == FA_OK, "fa_fwd_launch failed: ", fa_fwd_error_string(rc), " (rc=", rc, ")");
    g_launches.fetch_add(1, std::memory_order_relaxed);
  }
  if (!compute_log_sumexp) lse = packed ? at::empty({Hq, 0}, q.options().dtype(at::kFloat)) : at::empty({B, Hq, 0}, q.options().dtype(at::kFloat));
  return std::make_tuple(output, lse, seed_t, offset_t, c10::SymInt(kSq), c10::SymInt(kSk));
}

// ---- _scaled_dot_product_efficient_attention -------------------------------------------------------------------
// cnnl__scaled_dot_product_efficient_attention, attention.cpp:350-388: [B, H, S, D] in, transposes, causal from the
// top-left corner (:368-370), output returned as the [B, H, Sq, D] view of [B, Sq, H, D] storage.
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor> scaled_dot_product_efficient_attention(
    const at::Tensor& query, const at::Tensor& key, const at::Tensor& value, const std::optional<at::Tensor>& attn_bias,
    bool compute_log_sumexp, double dropout_p, bool is_causal, std::optional<double> scale) {
  TORCH_CHECK(query.dim() == 4 && key.dim() == 4 && value.dim() == 4,
              "query, key and value must be 4-dimensional (batch, num_heads, seq_len, head_dim)");
  auto [out, lse, seed, offset, mq, mk] = efficient_attention_forward(
      query.transpose(1, 2), key.transpose(1, 2), value.transpose(1, 2), attn_bias, std::nullopt, std::nullopt,
      std::nullopt, std::nullopt, dropout_p, is_causal ? 1 : 0, compute_log_sumexp, scale, std::nullopt, std::nullopt);
  (void)mq;
  (void)mk;
  return std::make_tuple(out.transpose(1, 2), lse, seed, offset);
}

// ---- _scaled_dot_product_efficient_attention on nested (ragged) tensors, inference ------------------------------
// The reference prefers its mem-efficient kernels for nested inputs and accepts them there without gradients
// (sdp_utils.cpp:22-24,82-87).  PyTorch's own nested-tensor wrapper of this op drops the attn_bias, so nested inputs
// with an attn_mask get this one: query / key / value are nested [B, H, S*, D] views of [B, S*, H, D] data (what
// F.scaled_dot_product_attention is given), packed here into [1, total, H, D] buffers with cu_seqlens from the nested
// sizes and handed to the packed op above; attn_bias is dense, broadcastable to [B, H, max S_q, max S_k], indexed from
// each sequence's first row and key.
namespace {
struct PackedNested {
  at::Tensor buf;    // [1, total, H, D]
  at::Tensor cu;     // int32 [B + 1] on the device
  at::Tensor sizes;  // the nested sizes of the [B, S*, H, D] tensor
  int64_t max_len;
};
PackedNested pack_nested(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_nested() && t.dim() == 4, name, " must be a nested tensor of 4 dimensions (batch, num_heads, seq_len, head_dim)");
  const at::Tensor c = t.transpose(1, 2).contiguous();  // [B, S*, H, D], rows of all sequences one after the other
  const auto* impl = at::native::get_nested_tensor_impl(c);
  const at::Tensor sizes = impl->get_nested_sizes();  // int64 [B, 3] on the CPU: (S_b, H, D)
  const int64_t B = sizes.size(0);
  TORCH_CHECK(B > 0 && sizes.size(1) == 3, name, ": unexpected nested structure");
  const auto sz = sizes.accessor<int64_t, 2>();
  const int64_t H = sz[0][1], D = sz[0][2];
  std::vector<int32_t> cu(B + 1, 0);
  int64_t total = 0, mx = 0;
  for (int64_t b = 0; b < B; ++b) {
    TORCH_CHECK(sz[b][1] == H && sz[b][2] == D, name, ": ragged num_heads or head_dim are not supported");
    total += sz[b][0];
    mx = std::max(mx, sz[b][0]);
    TORCH_CHECK(total <= INT32_MAX, "sequence length too large");
    cu[b + 1] = static_cast<int32_t>(total);
  }
  const at::Tensor buffer = impl->get_buffer();
  TORCH_CHECK(buffer.numel() == total * H * D, name, ": unexpected nested storage");
  at::Tensor cu_t = at::empty({B + 1}, at::TensorOptions().dtype(at::kInt).pinned_memory(true));
  std::memcpy(cu_t.data_ptr<int32_t>(), cu.data(), sizeof(int32_t) * (B + 1));
  return {buffer.view({1, total, H, D}), cu_t.to(t.device(), /*non_blocking=*/true), sizes, mx};
}
}  // namespace

std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor> scaled_dot_product_efficient_attention_nested(
    const at::Tensor& query, const at::Tensor& key, const at::Tensor& value, const std::optional<at::Tensor>& attn_bias,
    bool compute_log_sumexp, double dropout_p, bool is_causal, std::optional<double> scale) {
  TORCH_CHECK(query.is_nested() && key.is_nested() && value.is_nested(),
              "nested scaled_dot_product_attention needs query, key and value to be nested tensors");
  TORCH_CHECK(!(attn_bias.has_value() && attn_bias->defined() && attn_bias->is_nested()), "attn_mask must be a dense tensor");
  const PackedNested q = pack_nested(query, "query"), k = pack_nested(key, "key"), v = pack_nested(value, "value");
  TORCH_CHECK(q.cu.size(0) == k.cu.size(0) && at::equal(k.sizes.select(1, 0), v.sizes.select(1, 0)),
              "query, key and value must hold the same number of sequences, and key and value sequences of equal lengths");
  auto [out, lse, seed, offset, mq, mk] = efficient_attention_forward(
      q.buf, k.buf, v.buf, attn_bias, q.cu, k.cu, c10::SymInt(q.max_len), c10::SymInt(k.max_len), dropout_p,
      is_causal ? 1 : 0, compute_log_sumexp, scale, std::nullopt, std::nullopt);
  (void)mq;
  (void)mk;
  // [1, total, H, D] -> nested [B, S*, H, D] -> the [B, H, S*, D] view the dense wrapper returns too
  const at::Tensor out_nt = at::native::wrap_buffer(out.view({-1}), q.sizes);
  return std::make_tuple(out_nt.transpose(1, 2), lse, seed, offset);
}

// ---- _efficient_attention_backward ----------------------------------------------------------------------------
// cnnl__efficient_attention_backward (attention.cpp:579-727) + mem_eff_bwd (FlashAttention_internal.cpp:692-906):
// inputs [B, S, H, D], the forward's bias and mask type, logsumexp [B, H, Sq].  No contiguous copies of q/k/v.
// grad_bias: the reference allocates it (empty_like(bias) when bias_requires_grad, otherwise an uninitialised
// [B*H, Sq, Sk], attention.cpp:664-671) but never passes it to the vendor call, so its contents are undefined there;
// here it is computed when bias_requires_grad, in the shape of `bias`, and left undefined otherwise.
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor> efficient_attention_backward(
    const at::Tensor& grad_out_, const at::Tensor& query, const at::Tensor& key, const at::Tensor& value,
    const std::optional<at::Tensor>& bias, const at::Tensor& out, const std::optional<at::Tensor>& cu_seqlens_q,
    const std::optional<at::Tensor>& cu_seqlens_k, int64_t max_seqlen_q, int64_t max_seqlen_k,
    const at::Tensor& logsumexp, double dropout_p, const at::Tensor& philox_seed, const at::Tensor& philox_offset,
    int64_t custom_mask_type, bool bias_requires_grad, std::optional<double> scale,
    std::optional<int64_t> num_splits_key, std::optional<int64_t> window_size, bool shared_storage_dqdkdv) {
  (void)max_seqlen_q; (void)max_seqlen_k; (void)num_splits_key;
  if (!grad_out_.defined()) return std::make_tuple(at::Tensor{}, at::Tensor{}, at::Tensor{}, at::Tensor{});  // :599-601
  // the reference's shape checks (attention.cpp:602-625)
  TORCH_CHECK(query.dim() == 4 && grad_out_.dim() == 4 && key.dim() == 4 && value.dim() == 4 && out.dim() == 4,
              "grad_out, query, key, value and out must be 4-dimensional (batch, seq_len, num_heads, head_dim)");
  TORCH_CHECK(query.size(0) == grad_out_.size(0) && query.size(0) == key.size(0) && query.size(0) == value.size(0),
              "grad_out, query, key and value must have the same batch size");
  TORCH_CHECK(key.size(1) == value.size(1), "key and value must have the same sequence length");
  TORCH_CHECK(query.size(1) == grad_out_.size(1), "query and grad_out must have the same sequence length");
  TORCH_CHECK(key.size(2) == value.size(2) && key.size(2) > 0 && query.size(2) % key.size(2) == 0,
              "Number of heads in key/value must divide number of heads in query");
  TORCH_CHECK(query.size(2) == grad_out_.size(2), "query and grad_out must have the same number of heads");
  TORCH_CHECK(query.size(3) == key.size(3), "query and key must have the same head dimension");
  TORCH_CHECK(value.size(3) == grad_out_.size(3) && value.size(3) == query.size(3),
              "this build needs value.size(-1) == query.size(-1) == grad_out.size(-1)");
  TORCH_CHECK(out.sizes() == grad_out_.sizes(), "out must have the shape of grad_out");
  const bool packed = cu_seqlens_q.has_value() && cu_seqlens_q->defined();
  TORCH_CHECK(packed == (cu_seqlens_k.has_value() && cu_seqlens_k->defined()), "cu_seqlens_q and cu_seqlens_k must be given together");
  if (packed) check_efficient_cu_seqlens(*cu_seqlens_q, *cu_seqlens_k, query.size(0));
  TORCH_CHECK(!window_size.has_value() || *window_size <= 0, "efficient attention backward: sliding window is not supported");
  TORCH_CHECK(dropout_p >= 0.0 && dropout_p < 1.0, "efficient attention backward: dropout_p must be in [0, 1), got ", dropout_p);
  if (dropout_p > 0.0)
    TORCH_CHECK(philox_seed.defined() && philox_offset.defined() && philox_seed.is_cuda() && philox_offset.is_cuda() &&
                    philox_seed.scalar_type() == at::kLong && philox_offset.scalar_type() == at::kLong &&
                    philox_seed.numel() == 1 && philox_offset.numel() == 1,
                "efficient attention backward: philox_seed and philox_offset must be the int64 device scalars the "
                "forward returned");
  TORCH_CHECK(custom_mask_type >= 0 && custom_mask_type <= 2, "custom_mask_type must be 0, 1 or 2");
  // mem_eff_bwd's checks (FlashAttention_internal.cpp:714-758)
  const auto dt = query.scalar_type();
  TORCH_CHECK(dt == at::kHalf || dt == at::kBFloat16, "FlashAttention only support fp16 and bf16 data type");
  TORCH_CHECK(key.scalar_type() == dt, "query and key must have the same dtype");
  TORCH_CHECK(value.scalar_type() == dt, "query and value must have the same dtype");
  TORCH_CHECK(out.scalar_type() == dt, "query and out must have the same dtype");
  TORCH_CHECK(grad_out_.scalar_type() == dt, "query and dout must have the same dtype");
  TORCH_CHECK(query.is_cuda() && key.is_cuda() && value.is_cuda(), "Input tensor must be on HIP device");
  TORCH_CHECK(out.is_cuda(), "out tensor must be on HIP device");
  TORCH_CHECK(grad_out_.is_cuda(), "dout tensor must be on HIP device");
  TORCH_CHECK(logsumexp.is_cuda() && logsumexp.scalar_type() == at::kFloat, "softmax_lse tensor must be a float32 tensor on HIP device");
  TORCH_CHECK(query.stride(-1) == 1 && key.stride(-1) == 1 && value.stride(-1) == 1,
              "Input tensor must have contiguous last dimension");
  const int64_t B = query.size(0), Sq = query.size(1), Hq = query.size(2), D = query.size(3);
  const int64_t Sk = key.size(1), Hk = key.size(2);
  TORCH_CHECK(B > 0, "batch size must be positive");
  TORCH_CHECK(D <= 256, "FlashAttention backward only supports head dimension at most 256");
  TORCH_CHECK(D % 8 == 0, "head dimension must be a multiple of 8");
  TORCH_CHECK(Sq <= INT32_MAX && Sk <= INT32_MAX && B <= INT32_MAX, "sequence length too large");
  if (packed) {
    TORCH_CHECK(logsumexp.dim() == 2 && logsumexp.size(0) == Hq && logsumexp.size(1) == B * Sq,
                "logsumexp must have shape (num_heads, batch_size * seqlen_q): call the forward with compute_log_sumexp");
  } else {
    TORCH_CHECK(logsumexp.dim() == 3 && logsumexp.size(0) == B && logsumexp.size(1) == Hq && logsumexp.size(2) >= Sq,
                "logsumexp must have shape (batch_size, num_heads, seqlen_q): call the forward with compute_log_sumexp");
  }

  const c10::OptionalDeviceGuard guard(query.device());
  const float softmax_scale = resolve_scale(query, scale);
  auto fix = [](const at::Tensor& t) { return t.stride(-1) == 1 ? aligned_or_copy(t) : t.contiguous(); };
  at::Tensor q = aligned_or_copy(query), k = aligned_or_copy(key), v = aligned_or_copy(value);
  at::Tensor dout = fix(grad_out_), o = fix(out);  // the reference makes both contiguous (attention.cpp:646-650)
  if (packed) {
    q = flattenable(q); k = flattenable(k); v = flattenable(v); dout = flattenable(dout); o = flattenable(o);
  }
  at::Tensor dq, dk, dv;
  if (packed) {  // rows outside every sequence get no gradient
    TORCH_CHECK(!shared_storage_dqdkdv, "shared_storage_dqdkdv is not supported together with cu_seqlens");
    dq = at::zeros({B, Sq, Hq, D}, q.options());
    dk = at::zeros({B, Sk, Hk, D}, q.options());
    dv = at::zeros({B, Sk, Hk, D}, q.options());
  } else if (shared_storage_dqdkdv) {  // one [B, S, 3, H, D] allocation, the three gradients as its slices
    TORCH_CHECK(Sq == Sk && Hq == Hk, "shared_storage_dqdkdv needs query and key of the same shape");
    at::Tensor chunk = at::empty({B, Sq, 3, Hq, D}, q.options());
    dq = chunk.select(2, 0); dk = chunk.select(2, 1); dv = chunk.select(2, 2);
  } else {
    dq = at::empty({B, Sq, Hq, D}, q.options());
    dk = at::empty({B, Sk, Hk, D}, q.options());
    dv = at::empty({B, Sk, Hk, D}, q.options());
  }
  const bool has_bias = bias.has_value() && bias->defined();
  at::Tensor bias_e, dbias;
  if (has_bias) bias_e = bias_for_kernels(*bias, dt, B, Hq, Sq, Sk);
  const bool want_dbias = has_bias && bias_requires_grad;
  if (want_dbias)  // rows padded to a multiple of 8 columns: every row start 16-byte aligned; packed: only the part
                   // inside each sequence is written
    dbias = (packed ? at::zeros({B, Hq, Sq, (Sk + 7) / 8 * 8}, q.options())
                    : at::empty({B, Hq, Sq, (Sk + 7) / 8 * 8}, q.options())).narrow(3, 0, Sk);

  fa_bwd_params p{};
  p.q = q.data_ptr(); p.k = k.data_ptr(); p.v = v.data_ptr(); p.out = o.data_ptr(); p.dout = dout.data_ptr();
  p.lse = logsumexp.data_ptr<float>();
  p.dq = dq.data_ptr(); p.dk = dk.data_ptr(); p.dv = dv.data_ptr();
  fill_strides(q, false, p.q_stride_b, p.q_stride_s, p.q_stride_h);
  fill_strides(k, false, p.k_stride_b, p.k_stride_s, p.k_stride_h);
  fill_strides(v, false, p.v_stride_b, p.v_stride_s, p.v_stride_h);
  fill_strides(o, false, p.o_stride_b, p.o_stride_s, p.o_stride_h);
  fill_strides(dout, false, p.do_stride_b, p.do_stride_s, p.do_stride_h);
  fill_strides(dq, false, p.dq_stride_b, p.dq_stride_s, p.dq_stride_h);
  fill_strides(dk, false, p.dk_stride_b, p.dk_stride_s, p.dk_stride_h);
  fill_strides(dv, false, p.dv_stride_b, p.dv_stride_s, p.dv_stride_h);
  if (packed) {
    p.cu_seqlens_q = cu_seqlens_q->data_ptr<int32_t>();
    p.cu_seqlens_k = cu_seqlens_k->data_ptr<int32_t>();
    p.total_q = B * Sq;
    p.lse_stride_b = 0; p.lse_stride_h = logsumexp.stride(0); p.lse_stride_s = logsumexp.stride(1);
  } else {
    p.lse_stride_b = logsumexp.stride(0); p.lse_stride_h = logsumexp.stride(1); p.lse_stride_s = logsumexp.stride(2);
  }
  p.batch = static_cast<int32_t>(B);
  p.heads_q = static_cast<int32_t>(Hq);
  p.heads_k = static_cast<int32_t>(Hk);
  p.seqlen_q = static_cast<int32_t>(Sq);
  p.seqlen_k = static_cast<int32_t>(Sk);
  p.head_dim = static_cast<int32_t>(D);
  p.scale = softmax_scale;
  p.dtype = dt == at::kBFloat16 ? FA_DTYPE_BF16 : FA_DTYPE_FP16;
  p.is_causal = custom_mask_type == 1 ? FA_MASK_CAUSAL_TOP_LEFT
                                      : (custom_mask_type == 2 ? FA_MASK_CAUSAL_BOTTOM_RIGHT : FA_MASK_NONE);
  if (dropout_p > 0.0) {
    p.dropout_p = static_cast<float>(dropout_p);
    p.philox_seed = philox_seed.data_ptr<int64_t>();
    p.philox_offset = philox_offset.data_ptr<int64_t>();
  }
  if (has_bias && Sk > 0) {
    p.bias = bias_e.data_ptr();
    p.bias_stride_b = bias_e.stride(0); p.bias_stride_h = bias_e.stride(1); p.bias_stride_q = bias_e.stride(2);
    if (want_dbias) {
      p.dbias = dbias.data_ptr();
      p.dbias_stride_b = dbias.stride(0); p.dbias_stride_h = dbias.stride(1); p.dbias_stride_q = dbias.stride(2);
    }
  }
  if (B * Sq * Hq == 0 || Sk == 0) {
    dq.zero_(); dk.zero_(); dv.zero_();
    if (want_dbias) dbias.zero_();
  } else {
    const size_t ws_bytes = fa_bwd_workspace_bytes(&p);
    at::Tensor ws = at::empty({static_cast<int64_t>(ws_bytes > 0 ? ws_bytes : 16)}, q.options().dtype(at::kByte));
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(q.device().index()).stream();
    const int rc = fa_bwd_launch(&p, ws.data_ptr(), ws_bytes, stream);
    TORCH_CHECK(rc == FA_OK, "fa_bwd_launch failed: ", fa_fwd_error_string(rc), " (rc=", rc, ")");
    g_launches.fetch_add(1, std::memory_order_relaxed);
  }
  at::Tensor grad_bias;
  if (want_dbias) {  // in the shape the caller's bias has: what was broadcast is summed
    grad_bias = dbias;
    if (bias->sizes() != dbias.sizes()) grad_bias = at::sum_to(dbias, bias->sizes());
  }
  return std::make_tuple(dq, dk, dv, grad_bias);
}

// ---- _scaled_dot_product_efficient_attention_backward ---------------------------------------------------------
// cnnl__scaled_dot_product_efficient_attention_backward, attention.cpp:510-577: [B, H, S, D] in and out, causal from
// the top-left corner (:547-549), the bias gradient asked for by grad_input_mask[3].
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor> scaled_dot_product_efficient_attention_backward(
    const at::Tensor& grad_out_, const at::Tensor& query, const at::Tensor& key, const at::Tensor& value,
    const at::Tensor& attn_bias, const at::Tensor& out, const at::Tensor& logsumexp, const at::Tensor& philox_seed,
    const at::Tensor& philox_offset, double dropout_p, std::array<bool, 4> grad_input_mask, bool is_causal,
    std::optional<double> scale) {
  if (!grad_out_.defined()) return std::make_tuple(at::Tensor{}, at::Tensor{}, at::Tensor{}, at::Tensor{});
  TORCH_CHECK(query.dim() == 4 && key.dim() == 4 && value.dim() == 4 && grad_out_.dim() == 4 && out.dim() == 4,
              "grad_out, query, key, value and out must be 4-dimensional (batch, num_heads, seq_len, head_dim)");
  std::optional<at::Tensor> kernel_bias;  // an undefined tensor means "no bias" (attention.cpp:536-541)
  if (attn_bias.defined()) kernel_bias = attn_bias;
  auto [grad_q, grad_k, grad_v, grad_bias] = efficient_attention_backward(
      grad_out_.transpose(1, 2), query.transpose(1, 2), key.transpose(1, 2), value.transpose(1, 2), kernel_bias,
      out.transpose(1, 2), std::nullopt, std::nullopt, query.size(2), key.size(2), logsumexp, dropout_p, philox_seed,
      philox_offset, is_causal ? 1 : 0, grad_input_mask[3], scale, std::nullopt, std::nullopt, false);
  return std::make_tuple(grad_q.transpose(1, 2), grad_k.transpose(1, 2), grad_v.transpose(1, 2), grad_bias);
}

// ---- test hooks -----------------------------------------------------------------------------------------------
int64_t launch_count() { return g_launches.load(std::memory_order_relaxed); }

// Runs only the launcher's input checks; with require_device == false they can be exercised on CPU tensors.
void validate_flash_inputs(const at::Tensor& query, const at::Tensor& key, const at::Tensor& value,
                           const std::optional<at::Tensor>& cum_seq_q, const std::optional<at::Tensor>& cum_seq_k,
                           int64_t max_q, int64_t max_k, bool require_device) {
  const bool packed = cum_seq_q.has_value() && cum_seq_q->defined();
  TORCH_CHECK(packed == (cum_seq_k.has_value() && cum_seq_k->defined()), "cum_seq_q and cum_seq_k must be given together");
  Packed pk{packed ? &*cum_seq_q : nullptr, packed ? &*cum_seq_k : nullptr, max_q, max_k};
  check_inputs(query, key, value, packed ? &pk : nullptr, require_device);
}

}  // namespace torch_mlu_amd

// HIP tensors carry the CUDA dispatch key in PyTorch-ROCm; registering here replaces PyTorch's own kernels for
// the two ops (the dispatcher prints one "overriding a previously registered kernel" warning per op).
TORCH_LIBRARY_IMPL(aten, NestedTensorCUDA, m) {
  m.impl("_scaled_dot_product_efficient_attention",
         TORCH_FN(torch_mlu_amd::scaled_dot_product_efficient_attention_nested));
}

TORCH_LIBRARY_IMPL(aten, CUDA, m) {
  m.impl("_scaled_dot_product_flash_attention", TORCH_FN(torch_mlu_amd::scaled_dot_product_flash_attention));
  m.impl("_flash_attention_forward", TORCH_FN(torch_mlu_amd::flash_attention_forward));
  m.impl("_scaled_dot_product_flash_attention_backward",
         TORCH_FN(torch_mlu_amd::scaled_dot_product_flash_attention_backward));
  m.impl("_flash_attention_backward", TORCH_FN(torch_mlu_amd::flash_attention_backward));
  m.impl("_scaled_dot_product_efficient_attention", TORCH_FN(torch_mlu_amd::scaled_dot_product_efficient_attention));
  m.impl("_efficient_attention_forward", TORCH_FN(torch_mlu_amd::efficient_attention_forward));
  m.impl("_scaled_dot_product_efficient_attention_backward",
         TORCH_FN(torch_mlu_amd::scaled_dot_product_efficient_attention_backward));
  m.impl("_efficient_attention_backward", TORCH_FN(torch_mlu_amd::efficient_attention_backward));
}

TORCH_LIBRARY(torch_mlu_amd, m) {
  m.def("_launch_count() -> int", &torch_mlu_amd::launch_count);
  m.def(
      "_validate_flash_inputs(Tensor query, Tensor key, Tensor value, Tensor? cum_seq_q, Tensor? cum_seq_k, "
      "int max_q, int max_k, bool require_device) -> ()",
      &torch_mlu_amd::validate_flash_inputs);
  // the same two entry points under a private namespace, so that a test can call this build's implementation
  // by name no matter what else is registered for the aten ops
  m.def(
      "_flash_attention_forward(Tensor query, Tensor key, Tensor value, Tensor? cum_seq_q, Tensor? cum_seq_k, "
      "int max_q, int max_k, float dropout_p, bool is_causal, bool return_debug_mask, *, float? scale=None, "
      "int? window_size_left=None, int? window_size_right=None, Tensor? seqused_k=None, Tensor? alibi_slopes=None) "
      "-> (Tensor, Tensor, Tensor, Tensor, Tensor)",
      &torch_mlu_amd::flash_attention_forward);
}
