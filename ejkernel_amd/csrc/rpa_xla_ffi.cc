// XLA FFI handlers over the C ABI of librpa_mi355x.so, for hosts that call the ops from JAX.
//
// They play the role the reference's own native custom call plays for its Triton kernels:
// ejkernel/callib/_triton_call.py:738-757 lowers to jax.ffi with api_version 2 and registers the target for platform
// "rocm".  This file needs the XLA FFI headers that ship inside jaxlib (jax.ffi.include_dir()); it is compiled by
// ejkernel_amd/jax_ffi.py only where JAX is installed and is not part of the default build.
//
// Handlers (operands | results | attributes):
//   RpaFwd           queries, kv_pages, context_lens, block_tables, query_start_loc, num_seqs [, sinks] | out, scratch |
//                    softmax_scale f32, logits_soft_cap f32 (0 = none), sliding_window i32 (0 = none), compute i32,
//                    num_queries_per_block, num_kv_pages_per_block, num_warps, num_stages i32
//   RpaV3            queries, keys, values, kv_cache, kv_lens, block_tables, query_start_loc, distribution |
//                    out, kv_cache (the caller aliases it to operand 3: the reference donates the cache,
//                    ejkernel/kernels/_xla/ragged_page_attention_v3/_kernel.py:110-126), scratch |
//                    softmax_scale, logits_soft_cap, q_scale, k_scale, v_scale f32 (0 = none), sliding_window i32
//   RpaPageAttn      query, key_cache, value_cache, context_lens, block_tables | out, scratch | attn_scale f32
//   RpaRaggedDecode  query, key, value, sequence_start, sequence_end [, softmax_aux] | out, scratch |
//                    softmax_scale, logits_soft_cap f32, window_left i32 (< 0 = none)
//
// Scratch memory: every handler has one more result than its op, a byte buffer of the size the matching
// rpa_*_workspace_bytes function names (the Python wrapper declares it and drops it), so XLA owns and places the
// scratch and a handler allocates nothing, frees nothing and never synchronises: it enqueues the kernel that clears
// the ticket region (XLA's buffers arrive uninitialised and are reused between calls) and then the op, on the stream
// XLA hands over.  That is all a command buffer capture may contain.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "../../include/rpa_mi355x.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

static ffi::Error Invalid(const std::string& msg) { return ffi::Error(ffi::ErrorCode::kInvalidArgument, msg); }
static ffi::Error Failed(const std::string& msg) { return ffi::Error(ffi::ErrorCode::kInternal, msg); }

namespace {
// Points the launch at the scratch result and clears its tickets on the stream.
ffi::Error UseScratch(hipStream_t stream, ffi::Result<ffi::AnyBuffer>& scratch, uint64_t need, void** workspace,
                      uint64_t* workspace_bytes) {
  const uint64_t have = static_cast<uint64_t>(scratch->size_bytes());
  if (have < need) return Invalid("the scratch result is smaller than the op's workspace (declare rpa_*_workspace_bytes bytes)");
  if ((reinterpret_cast<uintptr_t>(scratch->untyped_data()) & 255u) != 0) return Invalid("the scratch result is not 256-byte aligned");
  if (rpa_workspace_init(scratch->untyped_data(), have, stream) != RPA_OK) return Failed(rpa_last_error());
  *workspace = scratch->untyped_data();
  *workspace_bytes = have;
  return ffi::Error::Success();
}

int DtypeOf(ffi::DataType t) {
  if (t == ffi::BF16) return RPA_DTYPE_BF16;
  if (t == ffi::F32) return RPA_DTYPE_F32;
  if (t == ffi::F8E4M3FN) return RPA_DTYPE_FP8_E4M3;
  if (t == ffi::F8E5M2) return RPA_DTYPE_FP8_E5M2;
  return -1;
}
}  // namespace

// ---------------------------------------------------------------------------------------------- ragged_page_attention
static ffi::Error RpaFwdImpl(hipStream_t stream, ffi::AnyBuffer queries, ffi::AnyBuffer kv_pages,
                             ffi::Buffer<ffi::S32> context_lens, ffi::Buffer<ffi::S32> block_tables,
                             ffi::Buffer<ffi::S32> query_start_loc, ffi::Buffer<ffi::S32> num_seqs,
                             ffi::RemainingArgs rest, ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> scratch,
                             float softmax_scale, float logits_soft_cap, int32_t sliding_window, int32_t compute,
                             int32_t num_queries_per_block, int32_t num_kv_pages_per_block, int32_t num_warps,
                             int32_t num_stages) {
  const auto qd = queries.dimensions();
  const auto kd = kv_pages.dimensions();
  const auto bd = block_tables.dimensions();
  if (qd.size() != 3 || kd.size() != 4 || bd.size() != 2) return Invalid("rank mismatch in ragged_page_attention operands");
  if (queries.element_type() != kv_pages.element_type()) return Invalid("queries and kv_pages must have one dtype");
  RpaParams p = {};
  p.dtype = DtypeOf(queries.element_type());
  if (p.dtype != RPA_DTYPE_BF16 && p.dtype != RPA_DTYPE_F32) return Invalid("queries must be bfloat16 or float32");
  p.queries = queries.untyped_data();
  p.kv_pages = kv_pages.untyped_data();
  p.context_lens = context_lens.typed_data();
  p.block_tables = block_tables.typed_data();
  p.query_start_loc = query_start_loc.typed_data();
  p.num_seqs = num_seqs.typed_data();
  p.out = out->untyped_data();
  p.total_tokens = static_cast<int32_t>(qd[0]);
  p.num_q_heads = static_cast<int32_t>(qd[1]);
  p.head_dim = static_cast<int32_t>(qd[2]);
  p.num_pages = static_cast<int32_t>(kd[0]);
  p.page_size = static_cast<int32_t>(kd[1]);
  p.num_kv_heads = static_cast<int32_t>(kd[2] / 2);
  p.max_num_seqs = static_cast<int32_t>(bd[0]);
  p.pages_per_seq = static_cast<int32_t>(bd[1]);
  if (rest.size() > 0) {  // optional sink logits, fp32 [num_q_heads, num_sinks]
    auto sinks = rest.get<ffi::Buffer<ffi::F32>>(0);
    if (!sinks.has_value()) return Invalid("sinks must be float32 [num_q_heads, num_sinks]");
    p.sinks = sinks->typed_data();
    p.num_sinks = static_cast<int32_t>(sinks->dimensions().back());
  }
  p.softmax_scale = softmax_scale;
  p.logits_soft_cap = logits_soft_cap;
  p.sliding_window = sliding_window;
  p.compute = compute;
  p.num_queries_per_block = num_queries_per_block;
  p.num_kv_pages_per_block = num_kv_pages_per_block;
  p.num_warps = num_warps;
  p.num_stages = num_stages;
  if (ffi::Error e = UseScratch(stream, scratch, rpa_workspace_bytes(&p), &p.workspace, &p.workspace_bytes); e.failure()) return e;
  if (rpa_fwd_launch(&p, stream) != RPA_OK) return Invalid(rpa_last_error());
  return ffi::Error::Success();
}

XLA_FFI_DEFINE_HANDLER_SYMBOL(RpaFwd, RpaFwdImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()          // queries
                                  .Arg<ffi::AnyBuffer>()          // kv_pages
                                  .Arg<ffi::Buffer<ffi::S32>>()   // context_lens
                                  .Arg<ffi::Buffer<ffi::S32>>()   // block_tables
                                  .Arg<ffi::Buffer<ffi::S32>>()   // query_start_loc
                                  .Arg<ffi::Buffer<ffi::S32>>()   // num_seqs
                                  .RemainingArgs()                // [sinks]
                                  .Ret<ffi::AnyBuffer>()          // out
                                  .Ret<ffi::AnyBuffer>()          // scratch
                                  .Attr<float>("softmax_scale")
                                  .Attr<float>("logits_soft_cap")
                                  .Attr<int32_t>("sliding_window")
                                  .Attr<int32_t>("compute")
                                  .Attr<int32_t>("num_queries_per_block")
                                  .Attr<int32_t>("num_kv_pages_per_block")
                                  .Attr<int32_t>("num_warps")
                                  .Attr<int32_t>("num_stages"));

// ------------------------------------------------------------------------------------------- ragged_page_attention_v3
static ffi::Error RpaV3Impl(hipStream_t stream, ffi::AnyBuffer queries, ffi::AnyBuffer keys, ffi::AnyBuffer values,
                            ffi::AnyBuffer kv_cache, ffi::Buffer<ffi::S32> kv_lens, ffi::Buffer<ffi::S32> block_tables,
                            ffi::Buffer<ffi::S32> query_start_loc, ffi::Buffer<ffi::S32> distribution,
                            ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> cache_out,
                            ffi::Result<ffi::AnyBuffer> scratch, float softmax_scale, float logits_soft_cap, float q_scale, float k_scale, float v_scale, int32_t sliding_window) {
  const auto qd = queries.dimensions();
  const auto kd = keys.dimensions();
  const auto cd = kv_cache.dimensions();  // [pages, page_size, 2 * kv heads / packing, packing, aligned head_dim]
  if (qd.size() != 3 || kd.size() != 3 || cd.size() != 5 || distribution.element_count() != 3)
    return Invalid("rank mismatch in ragged_page_attention_v3 operands");
  if (keys.element_type() != kv_cache.element_type() || values.element_type() != kv_cache.element_type())
    return Invalid("keys, values and kv_cache must have one dtype");
  // The cache is donated: the caller aliases result 1 to operand 3, and the update happens in place.  Without the
  // alias XLA hands over a second buffer, and the rows the call does not write would be missing from it.
  if (cache_out->untyped_data() != kv_cache.untyped_data())
    return Invalid("kv_cache must be aliased to the second result (input_output_aliases={3: 1})");
  RpaV3Params v = {};
  RpaParams& p = v.attn;
  p.dtype = DtypeOf(queries.element_type());
  v.cache_dtype = DtypeOf(kv_cache.element_type());
  if ((p.dtype != RPA_DTYPE_BF16 && p.dtype != RPA_DTYPE_F32) || v.cache_dtype < 0) return Invalid("unsupported dtype");
  p.queries = queries.untyped_data();
  p.kv_pages = cache_out->untyped_data();
  p.context_lens = kv_lens.typed_data();
  p.block_tables = block_tables.typed_data();
  p.query_start_loc = query_start_loc.typed_data();
  p.num_seqs = distribution.typed_data() + 2;  // distribution[-1] (_kernel.py:195)
  p.out = out->untyped_data();
  p.total_tokens = static_cast<int32_t>(qd[0]);
  p.num_q_heads = static_cast<int32_t>(qd[1]);
  p.head_dim = static_cast<int32_t>(qd[2]);
  p.num_kv_heads = static_cast<int32_t>(kd[1]);
  p.num_pages = static_cast<int32_t>(cd[0]);
  p.page_size = static_cast<int32_t>(cd[1]);
  p.max_num_seqs = static_cast<int32_t>(kv_lens.element_count());
  p.pages_per_seq = p.max_num_seqs > 0 ? static_cast<int32_t>(block_tables.element_count() / p.max_num_seqs) : 0;
  p.softmax_scale = softmax_scale;
  p.logits_soft_cap = logits_soft_cap;
  p.sliding_window = sliding_window;
  p.compute = p.dtype == RPA_DTYPE_F32 ? RPA_COMPUTE_F32 : RPA_COMPUTE_BF16;
  p.q_scale = q_scale;
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  p.flags = RPA_FLAG_FP32_LOGITS;
  v.new_keys = keys.untyped_data();
  v.new_values = values.untyped_data();
  v.cache_head_dim = static_cast<int32_t>(cd[4]);
  v.cache_combined_heads = static_cast<int32_t>(cd[2] * cd[3]);
  if (ffi::Error e = UseScratch(stream, scratch, rpa_v3_workspace_bytes(&v), &p.workspace, &p.workspace_bytes); e.failure()) return e;
  if (rpa_v3_launch(&v, stream) != RPA_OK) return Invalid(rpa_last_error());
  return ffi::Error::Success();
}

XLA_FFI_DEFINE_HANDLER_SYMBOL(RpaV3, RpaV3Impl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()          // queries
                                  .Arg<ffi::AnyBuffer>()          // keys
                                  .Arg<ffi::AnyBuffer>()          // values
                                  .Arg<ffi::AnyBuffer>()          // kv_cache (donated)
                                  .Arg<ffi::Buffer<ffi::S32>>()   // kv_lens
                                  .Arg<ffi::Buffer<ffi::S32>>()   // block_tables
                                  .Arg<ffi::Buffer<ffi::S32>>()   // query_start_loc
                                  .Arg<ffi::Buffer<ffi::S32>>()   // distribution
                                  .Ret<ffi::AnyBuffer>()          // out
                                  .Ret<ffi::AnyBuffer>()          // kv_cache, aliased to operand 3
                                  .Ret<ffi::AnyBuffer>()          // scratch
                                  .Attr<float>("softmax_scale")
                                  .Attr<float>("logits_soft_cap")
                                  .Attr<float>("q_scale")
                                  .Attr<float>("k_scale")
                                  .Attr<float>("v_scale")
                                  .Attr<int32_t>("sliding_window"));

// ------------------------------------------------------------------------------------------------------ page_attention
static ffi::Error RpaPageAttnImpl(hipStream_t stream, ffi::AnyBuffer query, ffi::AnyBuffer key_cache,
                                  ffi::AnyBuffer value_cache, ffi::Buffer<ffi::S32> context_lens,
                                  ffi::Buffer<ffi::S32> block_tables, ffi::Result<ffi::AnyBuffer> out,
                                  ffi::Result<ffi::AnyBuffer> scratch, float attn_scale) {
  const auto qd = query.dimensions();
  const auto kd = key_cache.dimensions();
  const auto bd = block_tables.dimensions();
  if (qd.size() != 3 || kd.size() != 4 || bd.size() != 2) return Invalid("rank mismatch in page_attention operands");
  RpaPageAttnParams p = {};
  p.dtype = DtypeOf(query.element_type());
  if (p.dtype != RPA_DTYPE_BF16 && p.dtype != RPA_DTYPE_F32) return Invalid("query must be bfloat16 or float32");
  p.compute = p.dtype == RPA_DTYPE_F32 ? RPA_COMPUTE_F32 : RPA_COMPUTE_BF16;
  p.query = query.untyped_data();
  p.key_cache = key_cache.untyped_data();
  p.value_cache = value_cache.untyped_data();
  p.context_lens = context_lens.typed_data();
  p.block_tables = block_tables.typed_data();
  p.out = out->untyped_data();
  p.num_seqs = static_cast<int32_t>(qd[0]);
  p.num_q_heads = static_cast<int32_t>(qd[1]);
  p.head_dim = static_cast<int32_t>(qd[2]);
  p.num_blocks = static_cast<int32_t>(kd[0]);
  p.num_kv_heads = static_cast<int32_t>(kd[1]);
  p.block_size = static_cast<int32_t>(kd[2]);
  p.max_blocks = static_cast<int32_t>(bd[1]);
  p.attn_scale = attn_scale;
  if (ffi::Error e = UseScratch(stream, scratch, rpa_page_attention_workspace_bytes(&p), &p.workspace, &p.workspace_bytes); e.failure()) return e;
  if (rpa_page_attention_launch(&p, stream) != RPA_OK) return Invalid(rpa_last_error());
  return ffi::Error::Success();
}

XLA_FFI_DEFINE_HANDLER_SYMBOL(RpaPageAttn, RpaPageAttnImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()          // query
                                  .Arg<ffi::AnyBuffer>()          // key_cache
                                  .Arg<ffi::AnyBuffer>()          // value_cache
                                  .Arg<ffi::Buffer<ffi::S32>>()   // context_lens
                                  .Arg<ffi::Buffer<ffi::S32>>()   // block_tables
                                  .Ret<ffi::AnyBuffer>()          // out
                                  .Ret<ffi::AnyBuffer>()          // scratch
                                  .Attr<float>("attn_scale"));

// ---------------------------------------------------------------------------------------------- ragged_decode_attention
static ffi::Error RpaRaggedDecodeImpl(hipStream_t stream, ffi::AnyBuffer query, ffi::AnyBuffer key, ffi::AnyBuffer value,
                                      ffi::Buffer<ffi::S32> sequence_start, ffi::Buffer<ffi::S32> sequence_end,
                                      ffi::RemainingArgs rest, ffi::Result<ffi::AnyBuffer> out,
                                      ffi::Result<ffi::AnyBuffer> scratch, float softmax_scale, float logits_soft_cap,
                                      int32_t window_left) {
  const auto qd = query.dimensions();
  const auto kd = key.dimensions();
  if (qd.size() != 3 || kd.size() != 4) return Invalid("rank mismatch in ragged_decode_attention operands");
  RpaRaggedDecodeParams p = {};
  p.dtype = DtypeOf(query.element_type());
  if (p.dtype != RPA_DTYPE_BF16 && p.dtype != RPA_DTYPE_F32) return Invalid("query must be bfloat16 or float32");
  p.compute = p.dtype == RPA_DTYPE_F32 ? RPA_COMPUTE_F32 : RPA_COMPUTE_BF16;
  p.query = query.untyped_data();
  p.key = key.untyped_data();
  p.value = value.untyped_data();
  p.sequence_start = sequence_start.typed_data();
  p.sequence_end = sequence_end.typed_data();
  p.out = out->untyped_data();
  p.batch = static_cast<int32_t>(qd[0]);
  p.num_q_heads = static_cast<int32_t>(qd[1]);
  p.head_dim = static_cast<int32_t>(qd[2]);
  p.seq_len = static_cast<int32_t>(kd[1]);
  p.num_kv_heads = static_cast<int32_t>(kd[2]);
  p.softmax_scale = softmax_scale;
  p.logits_soft_cap = logits_soft_cap;
  p.window_left = window_left;
  if (rest.size() > 0) {  // softmax_aux, fp32 [aux_rows, num_sinks]
    auto aux = rest.get<ffi::Buffer<ffi::F32>>(0);
    if (!aux.has_value() || aux->dimensions().size() != 2) return Invalid("softmax_aux must be float32 [rows, num_sinks]");
    p.softmax_aux = aux->typed_data();
    p.aux_rows = static_cast<int32_t>(aux->dimensions()[0]);
    p.num_sinks = static_cast<int32_t>(aux->dimensions()[1]);
  }
  if (ffi::Error e = UseScratch(stream, scratch, rpa_ragged_decode_workspace_bytes(&p), &p.workspace, &p.workspace_bytes); e.failure()) return e;
  if (rpa_ragged_decode_launch(&p, stream) != RPA_OK) return Invalid(rpa_last_error());
  return ffi::Error::Success();
}

XLA_FFI_DEFINE_HANDLER_SYMBOL(RpaRaggedDecode, RpaRaggedDecodeImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()          // query
                                  .Arg<ffi::AnyBuffer>()          // key
                                  .Arg<ffi::AnyBuffer>()          // value
                                  .Arg<ffi::Buffer<ffi::S32>>()   // sequence_start
                                  .Arg<ffi::Buffer<ffi::S32>>()   // sequence_end
                                  .RemainingArgs()                // [softmax_aux]
                                  .Ret<ffi::AnyBuffer>()          // out
                                  .Ret<ffi::AnyBuffer>()          // scratch
                                  .Attr<float>("softmax_scale")
                                  .Attr<float>("logits_soft_cap")
                                  .Attr<int32_t>("window_left"));
