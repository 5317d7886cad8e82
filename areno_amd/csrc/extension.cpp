// PyTorch-ROCm binding of libareno_hip.so: at::Tensor checks -> C ABI (include/areno_hip.h).
//
// Mirrors the reference's pybind surface for this path (areno/accel/csrc/extension.cpp:180-184):
//   areno_paged_causal_attention_decode_forward, areno_varlen_causal_attention_forward
// with the same TORCH_CHECK contract as its host launchers (areno/accel/csrc/attention.cu:813-861,
// 926-1020): device / contiguity / rank / dtype / shape agreement, current device guard, launch on the
// current stream, fresh output tensor, per-call workspace from the caching allocator.  The extra
// entry points (cache write, paged prefill, scales) are this build's extension of the path.

#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include "../../include/areno_hip.h"

namespace {

int dtype_code(const at::Tensor& t, const char* op, const char* name) {
  switch (t.scalar_type()) {
    case at::kFloat: return ARENO_DT_F32;
    case at::kHalf: return ARENO_DT_F16;
    case at::kBFloat16: return ARENO_DT_BF16;
    case at::kChar: return ARENO_DT_I8;
    case at::kFloat8_e4m3fn: return ARENO_DT_FP8_E4M3;
    default: TORCH_CHECK(false, op, " ", name, " has unsupported dtype ", t.scalar_type());
  }
  return -1;
}

void check_status(int status, const char* op) {
  TORCH_CHECK(status == ARENO_OK, op, " failed: ", areno_hip_status_string(status), " (", areno_hip_last_error(), ")");
}

// ROCm builds of PyTorch expose HIP devices under the "cuda" device type; these are its own
// stream / guard accessors for that arrangement.
void* current_stream(const at::Tensor& t) {
  return static_cast<void*>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream());
}

areno_paged_cache describe_cache(const at::Tensor& k_cache, const at::Tensor& v_cache,
                                 const c10::optional<at::Tensor>& k_scale, const c10::optional<at::Tensor>& v_scale,
                                 const char* op) {
  TORCH_CHECK(k_cache.is_cuda(), op, " k_cache must be CUDA");
  TORCH_CHECK(v_cache.is_cuda(), op, " v_cache must be CUDA");
  TORCH_CHECK(k_cache.is_contiguous(), op, " k_cache must be contiguous");
  TORCH_CHECK(v_cache.is_contiguous(), op, " v_cache must be contiguous");
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4, op, " cache tensors must be 4D");
  TORCH_CHECK(k_cache.scalar_type() == v_cache.scalar_type(), op, " cache dtype mismatch");
  TORCH_CHECK(k_cache.size(0) == v_cache.size(0) && k_cache.size(1) == v_cache.size(1), op,
              " cache block shape mismatch");
  TORCH_CHECK(k_cache.size(2) == v_cache.size(2), op, " cache head mismatch");
  TORCH_CHECK(k_cache.size(3) == v_cache.size(3), op, " cache head dim mismatch");
  areno_paged_cache c;
  c.k = k_cache.data_ptr();
  c.v = v_cache.data_ptr();
  c.k_scale = nullptr;
  c.v_scale = nullptr;
  c.num_blocks = k_cache.size(0);
  c.block_size = static_cast<int32_t>(k_cache.size(1));
  c.kv_heads = static_cast<int32_t>(k_cache.size(2));
  c.head_dim = static_cast<int32_t>(k_cache.size(3));
  c.cache_dtype = dtype_code(k_cache, op, "k_cache");
  c.scale_dtype = ARENO_DT_F32;
  const bool quantized = c.cache_dtype == ARENO_DT_I8 || c.cache_dtype == ARENO_DT_FP8_E4M3;
  TORCH_CHECK(quantized == (k_scale.has_value() && v_scale.has_value()), op,
              " k_scale and v_scale are required for int8/float8_e4m3fn caches and forbidden otherwise");
  if (quantized) {
    const at::Tensor& ks = *k_scale;
    const at::Tensor& vs = *v_scale;
    TORCH_CHECK(ks.is_cuda() && vs.is_cuda(), op, " scales must be CUDA");
    TORCH_CHECK(ks.is_contiguous() && vs.is_contiguous(), op, " scales must be contiguous");
    TORCH_CHECK(ks.scalar_type() == vs.scalar_type(), op, " scale dtype mismatch");
    TORCH_CHECK(ks.scalar_type() == at::kHalf || ks.scalar_type() == at::kFloat, op, " scales must be fp16 or fp32");
    TORCH_CHECK(ks.dim() == 3 && vs.dim() == 3, op, " scales must be shaped (num_blocks, block_size, kv_heads)");
    for (int i = 0; i < 3; ++i) {
      TORCH_CHECK(ks.size(i) == k_cache.size(i) && vs.size(i) == k_cache.size(i), op, " scale shape mismatch");
    }
    c.k_scale = ks.data_ptr();
    c.v_scale = vs.data_ptr();
    c.scale_dtype = ks.scalar_type() == at::kHalf ? ARENO_DT_F16 : ARENO_DT_F32;
  }
  return c;
}

at::Tensor paged_decode_forward_impl(at::Tensor q, at::Tensor k_update, at::Tensor v_update, at::Tensor k_cache,
                                     at::Tensor v_cache, at::Tensor block_table, at::Tensor cache_seqlens,
                                     int64_t window_left, int64_t num_splits, double softmax_scale,
                                     c10::optional<at::Tensor> k_scale, c10::optional<at::Tensor> v_scale,
                                     int64_t prefix_group_rows, c10::optional<at::Tensor> shared_prefix_lens,
                                     const areno_decode_plan* plan) {
  const char* op = "areno_paged_causal_attention_decode";
  TORCH_CHECK(q.is_cuda(), op, " q must be CUDA");
  TORCH_CHECK(k_update.is_cuda(), op, " k_update must be CUDA");
  TORCH_CHECK(v_update.is_cuda(), op, " v_update must be CUDA");
  TORCH_CHECK(block_table.is_cuda(), op, " block_table must be CUDA");
  TORCH_CHECK(cache_seqlens.is_cuda(), op, " cache_seqlens must be CUDA");
  TORCH_CHECK(q.is_contiguous(), op, " q must be contiguous");
  TORCH_CHECK(k_update.is_contiguous(), op, " k_update must be contiguous");
  TORCH_CHECK(v_update.is_contiguous(), op, " v_update must be contiguous");
  TORCH_CHECK(block_table.is_contiguous(), op, " block_table must be contiguous");
  TORCH_CHECK(cache_seqlens.is_contiguous(), op, " cache_seqlens must be contiguous");
  TORCH_CHECK(q.dim() == 3, op, " q must be shaped (batch, heads, head_dim)");
  TORCH_CHECK(k_update.dim() == 3 && v_update.dim() == 3, op, " updates must be 3D");
  TORCH_CHECK(block_table.dim() == 2, op, " block_table must be 2D");
  TORCH_CHECK(cache_seqlens.dim() == 1, op, " cache_seqlens must be 1D");
  const areno_paged_cache cache = describe_cache(k_cache, v_cache, k_scale, v_scale, op);
  const bool quantized = cache.k_scale != nullptr;
  if (!quantized) {
    TORCH_CHECK(q.scalar_type() == k_cache.scalar_type(), op, " dtype mismatch");
  } else {
    TORCH_CHECK(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16, op,
                " q must be fp16 or bf16 with a quantized cache");
  }
  TORCH_CHECK(k_update.scalar_type() == q.scalar_type() && v_update.scalar_type() == q.scalar_type(), op,
              " update dtype mismatch");
  TORCH_CHECK(block_table.scalar_type() == at::kInt, op, " block_table must be int32");
  TORCH_CHECK(cache_seqlens.scalar_type() == at::kInt, op, " cache_seqlens must be int32");
  TORCH_CHECK(q.size(0) == block_table.size(0) && q.size(0) == cache_seqlens.size(0), op, " batch mismatch");
  TORCH_CHECK(k_update.size(0) == q.size(0) && v_update.size(0) == q.size(0), op, " update batch mismatch");
  TORCH_CHECK(k_update.size(1) == k_cache.size(2) && v_update.size(1) == v_cache.size(2), op, " update head mismatch");
  TORCH_CHECK(q.size(2) == k_cache.size(3) && q.size(2) == v_cache.size(3), op, " head dim mismatch");
  TORCH_CHECK(k_update.size(2) == k_cache.size(3) && v_update.size(2) == v_cache.size(3), op,
              " update head dim mismatch");
  TORCH_CHECK(q.size(1) % k_cache.size(2) == 0, op, " q heads must be divisible by kv heads");
  TORCH_CHECK(num_splits >= 1, op, " num_splits must be >= 1");

  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(q));
  auto out = at::empty_like(q);
  if (q.size(0) == 0) return out;
  const int32_t* shared_ptr = nullptr;
  int32_t group_rows = 0;
  if (shared_prefix_lens.has_value()) {
    const at::Tensor& sl = *shared_prefix_lens;
    TORCH_CHECK(prefix_group_rows >= 1 && q.size(0) % prefix_group_rows == 0, op,
                " batch must be a multiple of prefix_group_rows");
    TORCH_CHECK(sl.is_cuda() && sl.is_contiguous() && sl.scalar_type() == at::kInt && sl.dim() == 1 &&
                    sl.size(0) == q.size(0) / prefix_group_rows,
                op, " shared_prefix_lens must be a CUDA int32 (batch / prefix_group_rows,) tensor");
    shared_ptr = sl.data_ptr<int32_t>();
    group_rows = static_cast<int32_t>(prefix_group_rows);
  }
  const size_t ws_bytes = areno_hip_paged_decode_grouped_workspace_bytes(
      static_cast<int32_t>(q.size(0)), static_cast<int32_t>(q.size(1)), cache.kv_heads, cache.head_dim,
      cache.block_size, static_cast<int32_t>(block_table.size(1)), static_cast<int32_t>(num_splits), group_rows);
  TORCH_CHECK(ws_bytes > 0, op, " invalid shapes for the split-KV workspace");
  auto workspace = at::empty({static_cast<int64_t>(ws_bytes)}, q.options().dtype(at::kByte));
  const int status = areno_hip_paged_decode_planned(
      &cache, q.data_ptr(), k_update.data_ptr(), v_update.data_ptr(), out.data_ptr(), dtype_code(q, op, "q"),
      static_cast<int32_t>(q.size(0)), static_cast<int32_t>(q.size(1)), block_table.data_ptr<int32_t>(),
      static_cast<int32_t>(block_table.size(1)), cache_seqlens.data_ptr<int32_t>(), static_cast<int32_t>(window_left),
      static_cast<int32_t>(num_splits), static_cast<float>(softmax_scale), group_rows, shared_ptr, plan,
      workspace.data_ptr(), ws_bytes, ARENO_STAGE_ALL, current_stream(q));
  check_status(status, op);
  return out;
}

at::Tensor paged_decode_forward_scaled(at::Tensor q, at::Tensor k_update, at::Tensor v_update, at::Tensor k_cache,
                                       at::Tensor v_cache, at::Tensor block_table, at::Tensor cache_seqlens,
                                       int64_t window_left, int64_t num_splits, double softmax_scale,
                                       c10::optional<at::Tensor> k_scale, c10::optional<at::Tensor> v_scale,
                                       int64_t prefix_group_rows, c10::optional<at::Tensor> shared_prefix_lens) {
  return paged_decode_forward_impl(q, k_update, v_update, k_cache, v_cache, block_table, cache_seqlens, window_left,
                                   num_splits, softmax_scale, k_scale, v_scale, prefix_group_rows, shared_prefix_lens,
                                   nullptr);
}

// A per-step plan of the decode op (areno_hip_paged_decode_plan): the host-side description and the device buffer it
// points into, kept alive together.
struct DecodePlan {
  areno_decode_plan plan;
  at::Tensor buffer;
};

std::shared_ptr<DecodePlan> paged_decode_plan(at::Tensor block_table, at::Tensor cache_seqlens, at::Tensor k_cache,
                                              at::Tensor v_cache, c10::optional<at::Tensor> k_scale,
                                              c10::optional<at::Tensor> v_scale, int64_t q_dtype_code, int64_t q_heads,
                                              int64_t window_left, bool with_update, int64_t prefix_group_rows,
                                              c10::optional<at::Tensor> shared_prefix_lens,
                                              c10::optional<at::Tensor> buffer) {
  const char* op = "areno_paged_decode_plan";
  TORCH_CHECK(block_table.is_cuda() && cache_seqlens.is_cuda(), op, " block_table and cache_seqlens must be CUDA");
  TORCH_CHECK(block_table.is_contiguous() && cache_seqlens.is_contiguous(), op, " tensors must be contiguous");
  TORCH_CHECK(block_table.dim() == 2 && cache_seqlens.dim() == 1, op, " expects block_table 2D and cache_seqlens 1D");
  TORCH_CHECK(block_table.scalar_type() == at::kInt && cache_seqlens.scalar_type() == at::kInt, op,
              " block_table and cache_seqlens must be int32");
  TORCH_CHECK(block_table.size(0) == cache_seqlens.size(0), op, " batch mismatch");
  TORCH_CHECK(q_dtype_code == ARENO_DT_F16 || q_dtype_code == ARENO_DT_BF16 || q_dtype_code == ARENO_DT_F32, op,
              " q dtype must be fp16, bf16 or fp32");
  const areno_paged_cache cache = describe_cache(k_cache, v_cache, k_scale, v_scale, op);
  TORCH_CHECK(q_heads > 0 && q_heads % cache.kv_heads == 0, op, " q heads must be divisible by kv heads");
  const int32_t batch = static_cast<int32_t>(block_table.size(0));
  const int32_t* shared_ptr = nullptr;
  int32_t group_rows = 0;
  if (shared_prefix_lens.has_value()) {
    const at::Tensor& sl = *shared_prefix_lens;
    TORCH_CHECK(prefix_group_rows >= 1 && batch % prefix_group_rows == 0, op,
                " batch must be a multiple of prefix_group_rows");
    TORCH_CHECK(sl.is_cuda() && sl.is_contiguous() && sl.scalar_type() == at::kInt && sl.dim() == 1 &&
                    sl.size(0) == batch / prefix_group_rows,
                op, " shared_prefix_lens must be a CUDA int32 (batch / prefix_group_rows,) tensor");
    shared_ptr = sl.data_ptr<int32_t>();
    group_rows = static_cast<int32_t>(prefix_group_rows);
  }
  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(block_table));
  auto holder = std::make_shared<DecodePlan>();
  const size_t bytes = areno_hip_paged_decode_plan_bytes(batch > 0 ? batch : 1);
  if (buffer.has_value()) {
    TORCH_CHECK(buffer->is_cuda() && buffer->is_contiguous() && buffer->scalar_type() == at::kByte &&
                    static_cast<size_t>(buffer->numel()) >= bytes,
                op, " buffer must be a contiguous CUDA uint8 tensor of at least ", bytes, " bytes");
    holder->buffer = *buffer;
  } else {
    holder->buffer = at::empty({static_cast<int64_t>(bytes)}, block_table.options().dtype(at::kByte));
  }
  const int status = areno_hip_paged_decode_plan(
      &holder->plan, holder->buffer.data_ptr(), static_cast<size_t>(holder->buffer.numel()), &cache,
      static_cast<int32_t>(q_dtype_code), batch, static_cast<int32_t>(q_heads), block_table.data_ptr<int32_t>(),
      static_cast<int32_t>(block_table.size(1)), cache_seqlens.data_ptr<int32_t>(), static_cast<int32_t>(window_left),
      with_update ? 1 : 0, group_rows, shared_ptr, current_stream(block_table));
  check_status(status, op);
  return holder;
}

at::Tensor paged_decode_forward_planned(at::Tensor q, at::Tensor k_update, at::Tensor v_update, at::Tensor k_cache,
                                        at::Tensor v_cache, at::Tensor block_table, at::Tensor cache_seqlens,
                                        int64_t window_left, int64_t num_splits, double softmax_scale,
                                        c10::optional<at::Tensor> k_scale, c10::optional<at::Tensor> v_scale,
                                        int64_t prefix_group_rows, c10::optional<at::Tensor> shared_prefix_lens,
                                        std::shared_ptr<DecodePlan> plan) {
  TORCH_CHECK(plan != nullptr, "areno_paged_causal_attention_decode: plan is None");
  return paged_decode_forward_impl(q, k_update, v_update, k_cache, v_cache, block_table, cache_seqlens, window_left,
                                   num_splits, softmax_scale, k_scale, v_scale, prefix_group_rows, shared_prefix_lens,
                                   &plan->plan);
}

// Reference signature (extension.cpp:184 in the reference).
at::Tensor paged_decode_forward(at::Tensor q, at::Tensor k_update, at::Tensor v_update, at::Tensor k_cache,
                                at::Tensor v_cache, at::Tensor block_table, at::Tensor cache_seqlens,
                                int64_t window_left, int64_t num_splits, double softmax_scale) {
  return paged_decode_forward_impl(q, k_update, v_update, k_cache, v_cache, block_table, cache_seqlens, window_left,
                                   num_splits, softmax_scale, c10::nullopt, c10::nullopt, 0, c10::nullopt, nullptr);
}

at::Tensor varlen_forward(at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor cu_seqlens, int64_t window_left,
                          double softmax_scale) {
  const char* op = "areno_varlen_causal_attention";
  TORCH_CHECK(q.is_cuda(), op, " q must be CUDA");
  TORCH_CHECK(k.is_cuda(), op, " k must be CUDA");
  TORCH_CHECK(v.is_cuda(), op, " v must be CUDA");
  TORCH_CHECK(cu_seqlens.is_cuda(), op, " cu_seqlens must be CUDA");
  TORCH_CHECK(q.is_contiguous(), op, " q must be contiguous");
  TORCH_CHECK(k.is_contiguous(), op, " k must be contiguous");
  TORCH_CHECK(v.is_contiguous(), op, " v must be contiguous");
  TORCH_CHECK(cu_seqlens.is_contiguous(), op, " cu_seqlens must be contiguous");
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3, op, " expects 3D q/k/v");
  TORCH_CHECK(cu_seqlens.dim() == 1, op, " cu_seqlens must be 1D");
  TORCH_CHECK(cu_seqlens.scalar_type() == at::kInt, op, " cu_seqlens must be int32");
  TORCH_CHECK(q.scalar_type() == k.scalar_type() && q.scalar_type() == v.scalar_type(), op, " dtype mismatch");
  TORCH_CHECK(q.size(0) == k.size(0) && q.size(0) == v.size(0), op, " token count mismatch");
  TORCH_CHECK(k.size(1) == v.size(1), op, " key/value head mismatch");
  TORCH_CHECK(q.size(1) % k.size(1) == 0, op, " q heads must be divisible by kv heads");
  TORCH_CHECK(q.size(2) == k.size(2) && q.size(2) == v.size(2), op, " head dim mismatch");
  TORCH_CHECK(cu_seqlens.size(0) >= 2, op, " cu_seqlens must contain at least one sequence");
  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(q));
  auto out = at::empty_like(q);
  const size_t ws_bytes =
      areno_hip_prefill_workspace_bytes(static_cast<int32_t>(k.size(1)), static_cast<int32_t>(q.size(2)));
  auto workspace = at::empty({static_cast<int64_t>(ws_bytes)}, q.options().dtype(at::kByte));
  const int status = areno_hip_varlen_attention(
      q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), dtype_code(q, op, "q"), q.size(0),
      static_cast<int32_t>(q.size(1)), static_cast<int32_t>(k.size(1)), static_cast<int32_t>(q.size(2)),
      cu_seqlens.data_ptr<int32_t>(), static_cast<int32_t>(cu_seqlens.size(0) - 1), static_cast<int32_t>(window_left),
      static_cast<float>(softmax_scale), workspace.data_ptr(), ws_bytes, current_stream(q));
  check_status(status, op);
  return out;
}

void cache_write(at::Tensor k, at::Tensor v, at::Tensor k_cache, at::Tensor v_cache, at::Tensor block_ids,
                 at::Tensor block_offsets, c10::optional<at::Tensor> k_scale, c10::optional<at::Tensor> v_scale) {
  const char* op = "areno_paged_cache_write";
  TORCH_CHECK(k.is_cuda() && v.is_cuda(), op, " k and v must be CUDA");
  TORCH_CHECK(block_ids.is_cuda() && block_offsets.is_cuda(), op, " block ids/offsets must be CUDA");
  TORCH_CHECK(k.is_contiguous() && v.is_contiguous(), op, " k and v must be contiguous");
  TORCH_CHECK(block_ids.is_contiguous() && block_offsets.is_contiguous(), op, " block ids/offsets must be contiguous");
  TORCH_CHECK(k.dim() == 3 && v.dim() == 3, op, " expects k/v shaped (tokens, kv_heads, head_dim)");
  TORCH_CHECK(block_ids.dim() == 1 && block_offsets.dim() == 1, op, " block ids/offsets must be 1D");
  TORCH_CHECK(block_ids.scalar_type() == at::kLong && block_offsets.scalar_type() == at::kLong, op,
              " block ids/offsets must be int64");
  TORCH_CHECK(k.scalar_type() == v.scalar_type(), op, " dtype mismatch");
  const areno_paged_cache cache = describe_cache(k_cache, v_cache, k_scale, v_scale, op);
  if (cache.k_scale == nullptr) TORCH_CHECK(k.scalar_type() == k_cache.scalar_type(), op, " dtype mismatch");
  TORCH_CHECK(k.size(0) == v.size(0) && k.size(0) == block_ids.size(0) && k.size(0) == block_offsets.size(0), op,
              " token count mismatch");
  TORCH_CHECK(k.size(1) == k_cache.size(2) && v.size(1) == v_cache.size(2), op, " head mismatch");
  TORCH_CHECK(k.size(2) == k_cache.size(3) && v.size(2) == v_cache.size(3), op, " head dim mismatch");
  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(k));
  const int status =
      areno_hip_cache_write(&cache, k.data_ptr(), v.data_ptr(), dtype_code(k, op, "k"), k.size(0),
                            block_ids.data_ptr<int64_t>(), block_offsets.data_ptr<int64_t>(), current_stream(k));
  check_status(status, op);
}

at::Tensor paged_varlen_forward(at::Tensor q, at::Tensor k_cache, at::Tensor v_cache, at::Tensor block_table,
                                at::Tensor cu_seqlens_q, at::Tensor context_lens, int64_t window_left,
                                double softmax_scale, c10::optional<at::Tensor> k_scale,
                                c10::optional<at::Tensor> v_scale) {
  const char* op = "areno_paged_varlen_causal_attention";
  TORCH_CHECK(q.is_cuda() && block_table.is_cuda() && cu_seqlens_q.is_cuda() && context_lens.is_cuda(), op,
              " tensors must be CUDA");
  TORCH_CHECK(q.is_contiguous() && block_table.is_contiguous() && cu_seqlens_q.is_contiguous() &&
                  context_lens.is_contiguous(),
              op, " tensors must be contiguous");
  TORCH_CHECK(q.dim() == 3, op, " q must be shaped (tokens, heads, head_dim)");
  TORCH_CHECK(block_table.dim() == 2 && cu_seqlens_q.dim() == 1 && context_lens.dim() == 1, op,
              " expects block_table 2D, cu_seqlens_q 1D, context_lens 1D");
  TORCH_CHECK(block_table.scalar_type() == at::kInt && cu_seqlens_q.scalar_type() == at::kInt &&
                  context_lens.scalar_type() == at::kInt,
              op, " block_table, cu_seqlens_q and context_lens must be int32");
  const areno_paged_cache cache = describe_cache(k_cache, v_cache, k_scale, v_scale, op);
  if (cache.k_scale == nullptr) {
    TORCH_CHECK(q.scalar_type() == k_cache.scalar_type(), op, " dtype mismatch");
  } else {
    TORCH_CHECK(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16, op,
                " q must be fp16 or bf16 with a quantized cache");
  }
  TORCH_CHECK(cu_seqlens_q.size(0) >= 2, op, " cu_seqlens_q must contain at least one sequence");
  TORCH_CHECK(context_lens.size(0) == cu_seqlens_q.size(0) - 1 && block_table.size(0) == context_lens.size(0), op,
              " sequence count mismatch");
  TORCH_CHECK(q.size(2) == k_cache.size(3), op, " head dim mismatch");
  TORCH_CHECK(q.size(1) % k_cache.size(2) == 0, op, " q heads must be divisible by kv heads");
  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(q));
  auto out = at::empty_like(q);
  const size_t ws_bytes = areno_hip_prefill_workspace_bytes(cache.kv_heads, cache.head_dim);
  auto workspace = at::empty({static_cast<int64_t>(ws_bytes)}, q.options().dtype(at::kByte));
  const int status = areno_hip_paged_varlen_prefill(
      &cache, q.data_ptr(), out.data_ptr(), dtype_code(q, op, "q"), q.size(0), static_cast<int32_t>(q.size(1)),
      static_cast<int32_t>(context_lens.size(0)), block_table.data_ptr<int32_t>(),
      static_cast<int32_t>(block_table.size(1)), cu_seqlens_q.data_ptr<int32_t>(), context_lens.data_ptr<int32_t>(),
      static_cast<int32_t>(window_left), static_cast<float>(softmax_scale), workspace.data_ptr(), ws_bytes,
      current_stream(q));
  check_status(status, op);
  return out;
}

// The rotary rows of a step's tokens (areno_hip_rope_rows): float32 (tokens, 2, head_dim), rounded for `like`'s dtype.
at::Tensor rope_rows(at::Tensor positions, at::Tensor cos, at::Tensor sin, at::Tensor like) {
  const char* op = "areno_rope_rows";
  TORCH_CHECK(positions.is_cuda() && cos.is_cuda() && sin.is_cuda(), op, " tensors must be CUDA");
  TORCH_CHECK(positions.is_contiguous() && cos.is_contiguous() && sin.is_contiguous(), op, " tensors must be contiguous");
  TORCH_CHECK(positions.dim() == 1 && positions.scalar_type() == at::kLong, op, " positions must be int64 (tokens,)");
  TORCH_CHECK(cos.dim() == 2 && cos.sizes() == sin.sizes() && cos.scalar_type() == at::kFloat &&
                  sin.scalar_type() == at::kFloat,
              op, " cos/sin must be float32 (max_position, head_dim)");
  TORCH_CHECK(like.scalar_type() == at::kHalf || like.scalar_type() == at::kBFloat16, op,
              " the activation dtype must be fp16 or bf16");
  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(positions));
  auto rows = at::empty({positions.size(0), 2, cos.size(1)}, cos.options());
  const int status = areno_hip_rope_rows(rows.data_ptr<float>(), positions.data_ptr<int64_t>(), cos.data_ptr<float>(),
                                         sin.data_ptr<float>(), positions.size(0), static_cast<int32_t>(cos.size(1)),
                                         static_cast<int32_t>(cos.size(0)), dtype_code(like, op, "like"),
                                         current_stream(positions));
  check_status(status, op);
  return rows;
}

// Where the fused front step takes its rotary values from: the tables and the tokens' positions, or the prepared rows.
struct RotarySource {
  const int64_t* positions = nullptr;
  const float* cos = nullptr;
  const float* sin = nullptr;
  int32_t max_pos = 0;
  const float* rows = nullptr;
};

std::vector<at::Tensor> qk_rope_write_common(const char* op, const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                             const RotarySource& rotary, const c10::optional<at::Tensor>& q_weight,
                                             const c10::optional<at::Tensor>& k_weight, double eps,
                                             const c10::optional<at::Tensor>& k_cache,
                                             const c10::optional<at::Tensor>& v_cache,
                                             const c10::optional<at::Tensor>& block_ids,
                                             const c10::optional<at::Tensor>& block_offsets,
                                             const c10::optional<at::Tensor>& k_scale,
                                             const c10::optional<at::Tensor>& v_scale) {
  auto weight_ptr = [&](const c10::optional<at::Tensor>& w, const char* name) -> const float* {
    if (!w.has_value()) return nullptr;
    TORCH_CHECK(w->is_cuda() && w->is_contiguous() && w->scalar_type() == at::kFloat && w->dim() == 1 &&
                    w->size(0) == q.size(2),
                op, " ", name, " must be a CUDA float32 (head_dim,) tensor");
    return w->data_ptr<float>();
  };
  const float* qw = weight_ptr(q_weight, "q_weight");
  const float* kw = weight_ptr(k_weight, "k_weight");
  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(q));
  auto q_out = at::empty_like(q);
  auto k_out = at::empty_like(k);
  areno_paged_cache cache = {};
  const areno_paged_cache* cache_ptr = nullptr;
  const int64_t* ids = nullptr;
  const int64_t* offs = nullptr;
  if (k_cache.has_value()) {
    TORCH_CHECK(v_cache.has_value() && block_ids.has_value() && block_offsets.has_value(), op,
                " a cache write needs v_cache, cache_block_ids and cache_block_offsets");
    cache = describe_cache(*k_cache, *v_cache, k_scale, v_scale, op);
    TORCH_CHECK(block_ids->is_cuda() && block_offsets->is_cuda() && block_ids->is_contiguous() &&
                    block_offsets->is_contiguous() && block_ids->scalar_type() == at::kLong &&
                    block_offsets->scalar_type() == at::kLong && block_ids->dim() == 1 &&
                    block_ids->size(0) == q.size(0) && block_offsets->sizes() == block_ids->sizes(),
                op, " block ids/offsets must be int64 (tokens,)");
    TORCH_CHECK(k.size(1) == k_cache->size(2) && k.size(2) == k_cache->size(3), op, " cache geometry mismatch");
    cache_ptr = &cache;
    ids = block_ids->data_ptr<int64_t>();
    offs = block_offsets->data_ptr<int64_t>();
  }
  const int32_t dtype = dtype_code(q, op, "q");
  const int32_t hq = static_cast<int32_t>(q.size(1)), hkv = static_cast<int32_t>(k.size(1));
  const int32_t d = static_cast<int32_t>(q.size(2));
  const int status =
      rotary.rows != nullptr
          ? areno_hip_qk_norm_rope_cache_write_rows(cache_ptr, q.data_ptr(), k.data_ptr(), v.data_ptr(), q_out.data_ptr(),
                                                    k_out.data_ptr(), dtype, q.size(0), hq, hkv, d, rotary.rows, qw, kw,
                                                    static_cast<float>(eps), ids, offs, current_stream(q))
          : areno_hip_qk_norm_rope_cache_write(cache_ptr, q.data_ptr(), k.data_ptr(), v.data_ptr(), q_out.data_ptr(),
                                               k_out.data_ptr(), dtype, q.size(0), hq, hkv, d, rotary.positions,
                                               rotary.cos, rotary.sin, rotary.max_pos, qw, kw, static_cast<float>(eps),
                                               ids, offs, current_stream(q));
  check_status(status, op);
  return {q_out, k_out};
}

void check_qkv_rows(const char* op, const at::Tensor& q, const at::Tensor& k, const at::Tensor& v) {
  TORCH_CHECK(q.is_cuda() && k.is_cuda() && v.is_cuda(), op, " tensors must be CUDA");
  TORCH_CHECK(q.is_contiguous() && k.is_contiguous() && v.is_contiguous(), op, " tensors must be contiguous");
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3, op, " expects q/k/v shaped (tokens, heads, head_dim)");
  TORCH_CHECK(q.scalar_type() == k.scalar_type() && q.scalar_type() == v.scalar_type(), op, " dtype mismatch");
  TORCH_CHECK(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16, op, " q/k/v must be fp16 or bf16");
  TORCH_CHECK(k.sizes() == v.sizes(), op, " k/v shape mismatch");
  TORCH_CHECK(q.size(0) == k.size(0) && q.size(2) == k.size(2), op, " q and k/v disagree on tokens or head_dim");
}

std::vector<at::Tensor> qk_norm_rope_cache_write(at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor positions,
                                                 at::Tensor cos, at::Tensor sin, c10::optional<at::Tensor> q_weight,
                                                 c10::optional<at::Tensor> k_weight, double eps,
                                                 c10::optional<at::Tensor> k_cache, c10::optional<at::Tensor> v_cache,
                                                 c10::optional<at::Tensor> block_ids,
                                                 c10::optional<at::Tensor> block_offsets,
                                                 c10::optional<at::Tensor> k_scale, c10::optional<at::Tensor> v_scale) {
  const char* op = "areno_qk_norm_rope_cache_write";
  check_qkv_rows(op, q, k, v);
  TORCH_CHECK(positions.is_cuda() && cos.is_cuda() && sin.is_cuda(), op, " tensors must be CUDA");
  TORCH_CHECK(positions.is_contiguous() && cos.is_contiguous() && sin.is_contiguous(), op, " tensors must be contiguous");
  TORCH_CHECK(positions.dim() == 1 && positions.size(0) == q.size(0) && positions.scalar_type() == at::kLong, op,
              " positions must be int64 (tokens,)");
  TORCH_CHECK(cos.dim() == 2 && cos.sizes() == sin.sizes() && cos.size(1) == q.size(2) &&
                  cos.scalar_type() == at::kFloat && sin.scalar_type() == at::kFloat,
              op, " cos/sin must be float32 (max_position, head_dim)");
  RotarySource rotary;
  rotary.positions = positions.data_ptr<int64_t>();
  rotary.cos = cos.data_ptr<float>();
  rotary.sin = sin.data_ptr<float>();
  rotary.max_pos = static_cast<int32_t>(cos.size(0));
  return qk_rope_write_common(op, q, k, v, rotary, q_weight, k_weight, eps, k_cache, v_cache, block_ids, block_offsets,
                              k_scale, v_scale);
}

std::vector<at::Tensor> qk_norm_rope_cache_write_rows(at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor rope_rows,
                                                      c10::optional<at::Tensor> q_weight,
                                                      c10::optional<at::Tensor> k_weight, double eps,
                                                      c10::optional<at::Tensor> k_cache,
                                                      c10::optional<at::Tensor> v_cache,
                                                      c10::optional<at::Tensor> block_ids,
                                                      c10::optional<at::Tensor> block_offsets,
                                                      c10::optional<at::Tensor> k_scale,
                                                      c10::optional<at::Tensor> v_scale) {
  const char* op = "areno_qk_norm_rope_cache_write";
  check_qkv_rows(op, q, k, v);
  TORCH_CHECK(rope_rows.is_cuda() && rope_rows.is_contiguous() && rope_rows.scalar_type() == at::kFloat &&
                  rope_rows.dim() == 3 && rope_rows.size(0) == q.size(0) && rope_rows.size(1) == 2 &&
                  rope_rows.size(2) == q.size(2),
              op, " rope_rows must be a contiguous CUDA float32 (tokens, 2, head_dim) tensor");
  RotarySource rotary;
  rotary.rows = rope_rows.data_ptr<float>();
  return qk_rope_write_common(op, q, k, v, rotary, q_weight, k_weight, eps, k_cache, v_cache, block_ids, block_offsets,
                              k_scale, v_scale);
}

// ---- device-resident block tables ------------------------------------------------------------------------------------
// state tensors of one pool: table [max_rows, max_blocks], row_blocks [max_rows], free_ring [num_blocks], state [4],
// all int32 on one device
areno_block_tables describe_tables(const at::Tensor& table, const at::Tensor& row_blocks, const at::Tensor& free_ring,
                                   const at::Tensor& state, int64_t block_size, const char* op) {
  for (const at::Tensor* t : {&table, &row_blocks, &free_ring, &state}) {
    TORCH_CHECK(t->is_cuda() && t->is_contiguous() && t->scalar_type() == at::kInt, op,
                " block-table state must be contiguous CUDA int32 tensors");
    TORCH_CHECK(t->device() == table.device(), op, " block-table state must live on one device");
  }
  TORCH_CHECK(table.dim() == 2 && row_blocks.dim() == 1 && row_blocks.size(0) == table.size(0) && free_ring.dim() == 1 &&
                  state.dim() == 1 && state.size(0) == 4,
              op, " block-table state has the wrong shape");
  TORCH_CHECK(block_size > 0 && table.size(0) > 0 && table.size(1) > 0 && free_ring.size(0) > 0, op,
              " block-table sizes must be positive");
  areno_block_tables bt;
  bt.table = table.data_ptr<int32_t>();
  bt.row_blocks = row_blocks.data_ptr<int32_t>();
  bt.free_ring = free_ring.data_ptr<int32_t>();
  bt.state = state.data_ptr<int32_t>();
  bt.max_rows = static_cast<int32_t>(table.size(0));
  bt.max_blocks = static_cast<int32_t>(table.size(1));
  bt.num_blocks = static_cast<int32_t>(free_ring.size(0));
  bt.block_size = static_cast<int32_t>(block_size);
  return bt;
}

void check_rows(const at::Tensor& rows, const at::Tensor& like, const char* op) {
  TORCH_CHECK(rows.is_cuda() && rows.device() == like.device() && rows.is_contiguous() &&
                  rows.scalar_type() == at::kLong && rows.dim() == 1,
              op, " rows must be a contiguous CUDA int64 vector on the tables' device");
}

void check_counts(const at::Tensor& v, int64_t n, const at::Tensor& like, const char* op, const char* name) {
  TORCH_CHECK(v.is_cuda() && v.device() == like.device() && v.is_contiguous() && v.scalar_type() == at::kInt &&
                  v.dim() == 1 && v.size(0) == n,
              op, " ", name, " must be a contiguous CUDA int32 vector of ", n, " entries");
}

void block_tables_init(at::Tensor table, at::Tensor row_blocks, at::Tensor free_ring, at::Tensor state,
                       int64_t block_size) {
  const char* op = "areno_block_tables_init";
  const areno_block_tables bt = describe_tables(table, row_blocks, free_ring, state, block_size, op);
  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(table));
  check_status(areno_hip_block_tables_init(&bt, current_stream(table)), op);
}

// decode = false: amounts are token counts the rows must hold; decode = true: the positions the rows write next
void block_tables_reserve(at::Tensor table, at::Tensor row_blocks, at::Tensor free_ring, at::Tensor state,
                          int64_t block_size, at::Tensor rows, at::Tensor amounts, bool decode) {
  const char* op = decode ? "areno_block_tables_ensure_decode" : "areno_block_tables_reserve";
  const areno_block_tables bt = describe_tables(table, row_blocks, free_ring, state, block_size, op);
  check_rows(rows, table, op);
  check_counts(amounts, rows.size(0), table, op, decode ? "next_positions" : "token_counts");
  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(table));
  const int32_t n = static_cast<int32_t>(rows.size(0));
  const int status =
      decode ? areno_hip_block_tables_ensure_decode(&bt, rows.data_ptr<int64_t>(), amounts.data_ptr<int32_t>(), n,
                                                    current_stream(table))
             : areno_hip_block_tables_reserve(&bt, rows.data_ptr<int64_t>(), amounts.data_ptr<int32_t>(), n,
                                              current_stream(table));
  check_status(status, op);
}

void block_tables_release(at::Tensor table, at::Tensor row_blocks, at::Tensor free_ring, at::Tensor state,
                          int64_t block_size, at::Tensor rows) {
  const char* op = "areno_block_tables_release";
  const areno_block_tables bt = describe_tables(table, row_blocks, free_ring, state, block_size, op);
  check_rows(rows, table, op);
  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(table));
  check_status(areno_hip_block_tables_release(&bt, rows.data_ptr<int64_t>(), static_cast<int32_t>(rows.size(0)),
                                              current_stream(table)),
               op);
}

at::Tensor block_tables_gather(at::Tensor table, at::Tensor row_blocks, at::Tensor free_ring, at::Tensor state,
                               int64_t block_size, at::Tensor rows, bool pad_scratch,
                               c10::optional<at::Tensor> out_opt) {
  const char* op = "areno_block_tables_gather";
  const areno_block_tables bt = describe_tables(table, row_blocks, free_ring, state, block_size, op);
  check_rows(rows, table, op);
  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(table));
  at::Tensor out = out_opt.has_value() ? *out_opt : at::empty({rows.size(0), table.size(1)}, table.options());
  TORCH_CHECK(out.is_cuda() && out.device() == table.device() && out.is_contiguous() && out.scalar_type() == at::kInt &&
                  out.dim() == 2 && out.size(0) == rows.size(0) && out.size(1) == table.size(1),
              op, " out must be a contiguous CUDA int32 (rows, max_blocks) tensor");
  check_status(areno_hip_block_tables_gather(&bt, rows.data_ptr<int64_t>(), static_cast<int32_t>(rows.size(0)),
                                             pad_scratch ? ARENO_PAD_SCRATCH_BLOCK : ARENO_PAD_LAST_BLOCK,
                                             out.data_ptr<int32_t>(), current_stream(table)),
               op);
  return out;
}

at::Tensor block_tables_decode_step(at::Tensor table, at::Tensor row_blocks, at::Tensor free_ring, at::Tensor state,
                                    int64_t block_size, at::Tensor rows, at::Tensor next_positions, bool pad_scratch,
                                    c10::optional<at::Tensor> out_opt) {
  const char* op = "areno_block_tables_decode_step";
  const areno_block_tables bt = describe_tables(table, row_blocks, free_ring, state, block_size, op);
  check_rows(rows, table, op);
  check_counts(next_positions, rows.size(0), table, op, "next_positions");
  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(table));
  at::Tensor out = out_opt.has_value() ? *out_opt : at::empty({rows.size(0), table.size(1)}, table.options());
  TORCH_CHECK(out.is_cuda() && out.device() == table.device() && out.is_contiguous() && out.scalar_type() == at::kInt &&
                  out.dim() == 2 && out.size(0) == rows.size(0) && out.size(1) == table.size(1),
              op, " out must be a contiguous CUDA int32 (rows, max_blocks) tensor");
  check_status(areno_hip_block_tables_decode_step(
                   &bt, rows.data_ptr<int64_t>(), next_positions.data_ptr<int32_t>(), static_cast<int32_t>(rows.size(0)),
                   pad_scratch ? ARENO_PAD_SCRATCH_BLOCK : ARENO_PAD_LAST_BLOCK, out.data_ptr<int32_t>(),
                   current_stream(table)),
               op);
  return out;
}

std::vector<at::Tensor> block_tables_prefill_slots(at::Tensor table, at::Tensor row_blocks, at::Tensor free_ring,
                                                   at::Tensor state, int64_t block_size, at::Tensor rows,
                                                   at::Tensor cursors, at::Tensor cu_seqlens, int64_t tokens) {
  const char* op = "areno_block_tables_prefill_slots";
  const areno_block_tables bt = describe_tables(table, row_blocks, free_ring, state, block_size, op);
  check_rows(rows, table, op);
  check_counts(cursors, rows.size(0), table, op, "cursors");
  check_counts(cu_seqlens, rows.size(0) + 1, table, op, "cu_seqlens");
  TORCH_CHECK(tokens >= 0, op, " negative token count");
  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(table));
  const auto opts = table.options().dtype(at::kLong);
  at::Tensor ids = at::empty({tokens}, opts), offs = at::empty({tokens}, opts), pos = at::empty({tokens}, opts);
  check_status(areno_hip_block_tables_prefill_slots(
                   &bt, rows.data_ptr<int64_t>(), cursors.data_ptr<int32_t>(), cu_seqlens.data_ptr<int32_t>(),
                   static_cast<int32_t>(rows.size(0)), tokens, ids.data_ptr<int64_t>(), offs.data_ptr<int64_t>(),
                   pos.data_ptr<int64_t>(), current_stream(table)),
               op);
  return {ids, offs, pos};
}

// Backward of the varlen / dense ops.  q / grad_out / out: (Tq, Hq, D); k / v: (Tk, Hkv, D); returns fp32 gradients
// like the reference's launchers (attention.cu:786-811, 898-925 there), or, with `grads_in_input_dtype`, the same
// sums rounded once to the inputs' type by the kernels (what the reference's autograd functions make of the fp32
// gradients with a cast each).
std::vector<at::Tensor> attention_backward(at::Tensor grad_out, at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor out,
                                           at::Tensor cu_q, c10::optional<at::Tensor> cu_k,
                                           c10::optional<at::Tensor> context_lens, int64_t window_left,
                                           double softmax_scale, bool grads_in_input_dtype) {
  const char* op = "areno_attention_backward";
  for (const at::Tensor* t : {&grad_out, &q, &k, &v, &out}) {
    TORCH_CHECK(t->is_cuda(), op, " tensors must be CUDA");
    TORCH_CHECK(t->is_contiguous(), op, " tensors must be contiguous");
    TORCH_CHECK(t->dim() == 3, op, " expects 3D tensors (tokens, heads, head_dim)");
    TORCH_CHECK(t->scalar_type() == q.scalar_type(), op, " dtype mismatch");
  }
  TORCH_CHECK(grad_out.sizes() == q.sizes() && out.sizes() == q.sizes(), op, " grad/out shape mismatch");
  TORCH_CHECK(k.sizes() == v.sizes(), op, " key/value shape mismatch");
  TORCH_CHECK(q.size(1) % k.size(1) == 0, op, " q heads must be divisible by kv heads");
  TORCH_CHECK(q.size(2) == k.size(2), op, " head dim mismatch");
  auto check_i32 = [&](const at::Tensor& t, int64_t n, const char* name) {
    TORCH_CHECK(t.is_cuda() && t.is_contiguous() && t.scalar_type() == at::kInt && t.dim() == 1 && t.size(0) == n, op,
                " ", name, " must be a contiguous CUDA int32 vector of ", n, " entries");
  };
  TORCH_CHECK(cu_q.dim() == 1 && cu_q.size(0) >= 2, op, " cu_seqlens must contain at least one sequence");
  const int64_t num_seqs = cu_q.size(0) - 1;
  check_i32(cu_q, num_seqs + 1, "cu_seqlens_q");
  if (cu_k.has_value()) check_i32(*cu_k, num_seqs + 1, "cu_seqlens_k");
  if (context_lens.has_value()) check_i32(*context_lens, num_seqs, "context_lens");
  const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device_of(q));
  const auto fopts = grads_in_input_dtype ? q.options() : q.options().dtype(at::kFloat);
  const int32_t grad_dtype = grads_in_input_dtype ? dtype_code(q, op, "q") : static_cast<int32_t>(ARENO_DT_F32);
  at::Tensor dq = at::empty(q.sizes(), fopts), dk = at::empty(k.sizes(), fopts), dv = at::empty(v.sizes(), fopts);
  const size_t ws_bytes = areno_hip_attention_backward_workspace_bytes(q.size(0), static_cast<int32_t>(q.size(1)));
  at::Tensor workspace = at::empty({static_cast<int64_t>(ws_bytes)}, q.options().dtype(at::kByte));
  const int status = areno_hip_attention_backward_typed(
      grad_out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), dq.data_ptr(), dk.data_ptr(),
      dv.data_ptr(), grad_dtype, dtype_code(q, op, "q"), q.size(0), k.size(0),
      static_cast<int32_t>(q.size(1)), static_cast<int32_t>(k.size(1)), static_cast<int32_t>(q.size(2)),
      cu_q.data_ptr<int32_t>(), cu_k.has_value() ? cu_k->data_ptr<int32_t>() : nullptr,
      context_lens.has_value() ? context_lens->data_ptr<int32_t>() : nullptr, static_cast<int32_t>(num_seqs),
      static_cast<int32_t>(window_left), static_cast<float>(softmax_scale), workspace.data_ptr(), ws_bytes,
      current_stream(q));
  check_status(status, op);
  return {dq, dk, dv};
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("areno_paged_causal_attention_decode_forward", &paged_decode_forward,
        "ARENO paged causal attention decode forward");
  m.def("areno_varlen_causal_attention_forward", &varlen_forward, "ARENO varlen causal attention forward");
  m.def("areno_paged_causal_attention_decode_forward_scaled", &paged_decode_forward_scaled,
        "paged decode forward with optional int8/fp8 cache scales");
  pybind11::class_<DecodePlan, std::shared_ptr<DecodePlan>>(m, "DecodePlan")
      .def_property_readonly("units", [](const DecodePlan& p) { return p.plan.units; })
      .def_property_readonly("items", [](const DecodePlan& p) { return p.plan.items; })
      .def_property_readonly("batch", [](const DecodePlan& p) { return p.plan.batch; })
      .def_property_readonly("buffer", [](const DecodePlan& p) { return p.buffer; });
  m.def("areno_paged_decode_plan", &paged_decode_plan, "work list of a decode step, built once for all its layers");
  m.def("areno_paged_causal_attention_decode_forward_planned", &paged_decode_forward_planned,
        "paged decode forward with a per-step plan");
  m.def("areno_paged_cache_write", &cache_write, "quantize-and-scatter KV cache write");
  m.def("areno_rope_rows", &rope_rows, "rotary rows of a step's tokens, rounded for an activation dtype");
  m.def("areno_qk_norm_rope_cache_write_rows", &qk_norm_rope_cache_write_rows,
        "QK norm + rotary + cache write from prepared rotary rows");
  m.def("areno_paged_varlen_causal_attention_forward", &paged_varlen_forward,
        "causal varlen prefill over paged (optionally quantized) KV");
  m.def("areno_qk_norm_rope_cache_write", &qk_norm_rope_cache_write,
        "QK RMSNorm + rotary embedding + quantizing KV cache write in one pass");
  m.def("areno_block_tables_init", &block_tables_init, "device-resident block tables: all pages free");
  m.def("areno_block_tables_reserve", &block_tables_reserve, "device-resident block tables: pages for prefill / decode");
  m.def("areno_block_tables_release", &block_tables_release, "device-resident block tables: give rows' pages back");
  m.def("areno_block_tables_gather", &block_tables_gather, "device-resident block tables: padded table of rows");
  m.def("areno_block_tables_decode_step", &block_tables_decode_step,
        "device-resident block tables: pages for the next decode position, then the padded table");
  m.def("areno_block_tables_prefill_slots", &block_tables_prefill_slots,
        "device-resident block tables: page id, slot and position of packed prefill tokens");
  m.def("areno_attention_backward", &attention_backward, "gradients of the varlen / dense causal attention ops");
  m.def("abi_version", &areno_hip_abi_version, "C ABI version of libareno_hip.so");
}
