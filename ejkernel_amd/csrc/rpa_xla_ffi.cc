// XLA FFI handler over the C ABI of librpa_mi355x.so, for hosts that call the op from JAX.
//
// It plays the role the reference's own native custom call plays for its Triton kernels:
// ejkernel/callib/_triton_call.py:738-757 lowers to jax.ffi with api_version 2 and
// registers the target for platform "rocm".  This file needs the XLA FFI headers that ship
// inside jaxlib (jax.ffi.include_dir()); it is compiled by ejkernel_amd/jax_ffi.py only
// where JAX is installed and is not part of the default build.
//
// Operands:  queries, kv_pages, context_lens, block_tables, query_start_loc, num_seqs [, sinks]
// Results:   out (same shape/dtype as queries), workspace (u8[rpa_workspace_bytes], owned by XLA)
// Attributes: softmax_scale f32, logits_soft_cap f32 (0 = none), sliding_window i32 (0 = none),
//             compute i32 (RPA_COMPUTE_*), num_queries_per_block, num_kv_pages_per_block, num_warps,
//             num_stages i32, has_sinks i32.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "../../include/rpa_mi355x.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

static ffi::Error Invalid(const std::string& msg) { return ffi::Error(ffi::ErrorCode::kInvalidArgument, msg); }

static ffi::Error RpaFwdImpl(hipStream_t stream, ffi::AnyBuffer queries, ffi::AnyBuffer kv_pages,
                             ffi::Buffer<ffi::S32> context_lens, ffi::Buffer<ffi::S32> block_tables,
                             ffi::Buffer<ffi::S32> query_start_loc, ffi::Buffer<ffi::S32> num_seqs,
                             ffi::RemainingArgs rest, ffi::Result<ffi::AnyBuffer> out,
                             ffi::Result<ffi::AnyBuffer> workspace, float softmax_scale, float logits_soft_cap,
                             int32_t sliding_window, int32_t compute, int32_t num_queries_per_block,
                             int32_t num_kv_pages_per_block, int32_t num_warps, int32_t num_stages) {
  const auto qd = queries.dimensions();
  const auto kd = kv_pages.dimensions();
  const auto bd = block_tables.dimensions();
  if (qd.size() != 3 || kd.size() != 4 || bd.size() != 2) return Invalid("rank mismatch in ragged_page_attention operands");
  if (queries.element_type() != kv_pages.element_type()) return Invalid("queries and kv_pages must have one dtype");
  RpaParams p = {};
  if (queries.element_type() == ffi::BF16) p.dtype = RPA_DTYPE_BF16;
  else if (queries.element_type() == ffi::F32) p.dtype = RPA_DTYPE_F32;
  else return Invalid("queries must be bfloat16 or float32");
  p.queries = queries.untyped_data();
  p.kv_pages = kv_pages.untyped_data();
  p.context_lens = context_lens.typed_data();
  p.block_tables = block_tables.typed_data();
  p.query_start_loc = query_start_loc.typed_data();
  p.num_seqs = num_seqs.typed_data();
  p.out = out->untyped_data();
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
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
  // XLA hands over uninitialised result buffers: the tickets at the head of the workspace are cleared on the
  // same stream before every launch (a fill kernel inside rpa_workspace_init when XLA captures command buffers).
  int rc = rpa_workspace_init(p.workspace, p.workspace_bytes, stream);
  if (rc == RPA_OK) rc = rpa_fwd_launch(&p, stream);
  if (rc != RPA_OK) return Invalid(rpa_last_error());
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
                                  .Ret<ffi::AnyBuffer>()          // workspace
                                  .Attr<float>("softmax_scale")
                                  .Attr<float>("logits_soft_cap")
                                  .Attr<int32_t>("sliding_window")
                                  .Attr<int32_t>("compute")
                                  .Attr<int32_t>("num_queries_per_block")
                                  .Attr<int32_t>("num_kv_pages_per_block")
                                  .Attr<int32_t>("num_warps")
                                  .Attr<int32_t>("num_stages"));
