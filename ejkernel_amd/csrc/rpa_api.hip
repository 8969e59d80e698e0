// C ABI of librpa_mi355x.so: argument validation and kernel selection.
//
// Validation mirrors what the reference enforces before its kernels run:
// ejkernel/kernels/_pallas/tpu/ragged_page_attention/_pallas_impl_fwd.py:177-230
// (static_validate_inputs) and the named-dimension checks of
// ejkernel/kernels/_xla/ragged_page_attention/_interface.py:26-47.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <mutex>

#include "rpa_host.h"

namespace rpa {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// The kernels fetch rows in 16-byte pieces wherever a row is a multiple of 16 bytes (every shape the MFMA path takes);
// rows that are not go through the scalar kernel, element by element.
static uint32_t data_alignment(const RpaParams& p) {
  const uint32_t esize = p.dtype == RPA_DTYPE_BF16 ? 2u : 4u;
  return (static_cast<uint64_t>(p.head_dim) * esize) % 16 == 0 ? 16u : esize;
}
static bool aligned_to(const void* ptr, uint32_t bytes) { return (reinterpret_cast<uintptr_t>(ptr) & (bytes - 1)) == 0; }
static bool data_aligned(const RpaParams& p, const void* ptr) { return aligned_to(ptr, data_alignment(p)); }

static int validate(const RpaParams& p, bool need_pointers, bool one_token_per_seq = false, bool contiguous = false) {
  if (p.total_tokens < 0 || p.num_q_heads <= 0 || p.num_kv_heads <= 0 || p.head_dim <= 0 || p.page_size <= 0 ||
      p.num_pages <= 0 || p.max_num_seqs <= 0 || p.pages_per_seq <= 0 || p.num_sinks < 0)
    return fail(RPA_ERR_INVALID_ARGUMENT, "non-positive dimension in RpaParams");
  if (p.num_q_heads % p.num_kv_heads != 0)
    return fail(RPA_ERR_INVALID_ARGUMENT, "num_q_heads=%d must be divisible by num_kv_heads=%d", p.num_q_heads,
                p.num_kv_heads);
  if (p.sliding_window < 0) return fail(RPA_ERR_INVALID_ARGUMENT, "sliding_window=%d must be positive", p.sliding_window);
  if (p.dtype != RPA_DTYPE_BF16 && p.dtype != RPA_DTYPE_F32) return fail(RPA_ERR_INVALID_ARGUMENT, "unknown dtype %d", p.dtype);
  if (p.compute != RPA_COMPUTE_BF16 && p.compute != RPA_COMPUTE_F32)
    return fail(RPA_ERR_INVALID_ARGUMENT, "unknown compute mode %d", p.compute);
  if (!(p.softmax_scale == p.softmax_scale)) return fail(RPA_ERR_INVALID_ARGUMENT, "softmax_scale is NaN");
  if (!(p.logits_soft_cap == p.logits_soft_cap)) return fail(RPA_ERR_INVALID_ARGUMENT, "logits_soft_cap is NaN");
  if (!(p.q_scale >= 0.f) || !(p.k_scale >= 0.f) || !(p.v_scale >= 0.f))
    return fail(RPA_ERR_INVALID_ARGUMENT, "q_scale / k_scale / v_scale must be positive (0 = absent)");
  if (need_pointers) {
    if (!p.queries || !p.kv_pages || !p.context_lens || (!contiguous && !p.block_tables) || !p.out ||
        (!one_token_per_seq && (!p.query_start_loc || !p.num_seqs)))
      return fail(RPA_ERR_INVALID_ARGUMENT, "null device pointer in RpaParams");
    if (p.num_sinks > 0 && !p.sinks) return fail(RPA_ERR_INVALID_ARGUMENT, "num_sinks=%d but sinks is null", p.num_sinks);
    if (!data_aligned(p, p.queries) || !data_aligned(p, p.kv_pages) || !data_aligned(p, p.out))
      return fail(RPA_ERR_INVALID_ARGUMENT, "queries, the cache and out must be aligned to %u bytes", data_alignment(p));
    if (!aligned_to(p.context_lens, 4) || !aligned_to(p.block_tables, 4) || !aligned_to(p.query_start_loc, 4) ||
        !aligned_to(p.num_seqs, 4) || !aligned_to(p.sinks, 4))
      return fail(RPA_ERR_INVALID_ARGUMENT, "int32 / fp32 arrays must be aligned to 4 bytes");
  }
  return RPA_OK;
}

// Clears the ticket region with a kernel rather than hipMemsetAsync, so the call may be recorded into a HIP graph.
__global__ void zero_fill_kernel(uint4* dst, size_t n16) {
  for (size_t k = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; k < n16;
       k += static_cast<size_t>(gridDim.x) * blockDim.x)
    dst[k] = make_uint4(0u, 0u, 0u, 0u);
}

int device_cu_count() {
  static std::atomic<int> cache[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
  int n = cache[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cache[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

}  // namespace rpa

extern "C" {

int rpa_abi_version(void) { return RPA_ABI_VERSION; }

const char* rpa_last_error(void) { return rpa::g_err; }

uint64_t rpa_workspace_bytes(const RpaParams* dims) {
  if (dims == nullptr || rpa::validate(*dims, false) != RPA_OK) return 0;
  rpa::WorkspaceLayout wl;
  rpa::tiled_workspace_layout(*dims, &wl);
  return wl.total_bytes;
}

int rpa_kernel_path(const RpaParams* dims) {
  if (dims == nullptr || rpa::validate(*dims, false) != RPA_OK) return -1;
  return rpa::tiled_supported(*dims) ? 1 : 0;
}

int rpa_workspace_init(void* workspace, uint64_t workspace_bytes, void* hip_stream) {
  // Only the split tickets need a defined value; they sit at the head of the workspace and every launch
  // leaves them at zero again.
  if (workspace == nullptr) return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "workspace is null");
  const uint64_t n = workspace_bytes < rpa::kWorkspaceTicketBytes ? workspace_bytes : rpa::kWorkspaceTicketBytes;
  if ((reinterpret_cast<uintptr_t>(workspace) & 15u) != 0) return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "workspace must be 16-byte aligned");
  if (n >= 16) {
    hipLaunchKernelGGL(rpa::zero_fill_kernel, dim3(64), dim3(256), 0, static_cast<hipStream_t>(hip_stream),
                       static_cast<uint4*>(workspace), static_cast<size_t>(n / 16));
    if (hipGetLastError() != hipSuccess) return rpa::fail(RPA_ERR_LAUNCH, "clearing the workspace tickets failed");
  }
  return RPA_OK;
}

namespace rpa {
static int dispatch(const RpaParams& p, const KvLayout& kv, bool tiled, hipStream_t stream, const PreState& pre = PreState());
}

// ---- rpa_fwd_launch_static: the forward pass for callers that cannot allocate.
//
// The kernels' scratch (split tickets, prefill queue counters, partial attention states of split (sequence, kv head)s)
// lives in a file-scope device array instead of a caller-supplied workspace.  Every GPU the library runs on holds its
// own copy of the array until the process ends; its address on a GPU comes from hipGetSymbolAddress, looked up once per
// device with that device current, and that pointer -- never the array's name, which in host code is only a handle --
// is what the kernels receive.
namespace rpa {
constexpr uint64_t kStaticScratchBytes = 34ull << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static std::mutex g_scratch_mu;
static std::atomic<void*> g_scratch_ptr[64];  // per device; null until the first call there

// Address of this device's copy of `scratch`; the first call on a device looks it up.  Nothing is enqueued: the
// tickets and queue counters at the head of the array are zero when the code object is loaded (a zero-initialised
// device variable) and every launch leaves them at zero again, and no other part of the array needs an initial
// value (a partial state is written before the ticket that publishes it).  So a first call made under stream capture
// records the attention kernel and nothing else, and first calls on two streams cannot reset each other's tickets.
// The lookup itself may load the code object: make the first call on a device outside any capture.
static int static_scratch(void** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail(RPA_ERR_LAUNCH, "hipGetDevice failed or device index above 63");
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
      const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess || p == nullptr)
        return fail(RPA_ERR_LAUNCH, "hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
      g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
  }
  *out = p;
  return RPA_OK;
}
}  // namespace rpa

uint64_t rpa_static_scratch_bytes(void) { return rpa::kStaticScratchBytes; }

int rpa_fwd_launch_static(const RpaParams* params, void* hip_stream) {
  if (params == nullptr) return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "params is null");
  RpaParams p = *params;
  int rc = rpa::validate(p, true);
  if (rc != RPA_OK) return rc;
  const bool tiled = rpa::tiled_supported(p);
  p.workspace = nullptr;
  p.workspace_bytes = 0;
  if (tiled) {
    const uint64_t need = rpa_workspace_bytes(&p);
    if (need > rpa::kStaticScratchBytes)
      return rpa::fail(RPA_ERR_WORKSPACE,
                       "this shape needs %llu bytes of scratch, the static scratch of rpa_fwd_launch_static holds %llu: "
                       "use rpa_fwd_launch with a workspace",
                       (unsigned long long)need, (unsigned long long)rpa::kStaticScratchBytes);
    void* ptr = nullptr;
    rc = rpa::static_scratch(&ptr);
    if (rc != RPA_OK) return rc;
    p.workspace = ptr;
    p.workspace_bytes = rpa::kStaticScratchBytes;
  }
  return rpa::dispatch(p, rpa::interleaved_layout(p), tiled, static_cast<hipStream_t>(hip_stream));
}

int rpa_fwd_launch(const RpaParams* params, void* hip_stream) {
  if (params == nullptr) return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "params is null");
  const RpaParams& p = *params;
  int rc = rpa::validate(p, true);
  if (rc != RPA_OK) return rc;
  return rpa::dispatch(p, rpa::interleaved_layout(p), rpa::tiled_supported(p), static_cast<hipStream_t>(hip_stream));
}

static RpaParams page_attention_params(const RpaPageAttnParams& a) {
  RpaParams p = {};
  p.queries = a.query;
  p.kv_pages = a.key_cache;
  p.context_lens = a.context_lens;
  p.block_tables = a.block_tables;
  p.query_start_loc = nullptr;  // sequence s owns row s
  p.num_seqs = nullptr;         // all of them are present
  p.out = a.out;
  p.workspace = a.workspace;
  p.workspace_bytes = a.workspace_bytes;
  p.total_tokens = a.num_seqs;
  p.max_num_seqs = a.num_seqs;
  p.num_q_heads = a.num_q_heads;
  p.num_kv_heads = a.num_kv_heads;
  p.head_dim = a.head_dim;
  p.page_size = a.block_size;
  p.num_pages = a.num_blocks;
  p.pages_per_seq = a.max_blocks;
  p.softmax_scale = a.attn_scale;
  p.dtype = a.dtype;
  p.compute = a.compute;
  p.flags = a.flags & (RPA_FLAG_FORCE_GENERIC | RPA_FLAG_FP32_LOGITS);
  return p;
}

// One query token per sequence: the tiled kernel runs without prefill tiles (which assume the interleaved cache).
static bool page_attention_tiled(const RpaParams& p) { return rpa::tiled_supported(p); }

uint64_t rpa_page_attention_workspace_bytes(const RpaPageAttnParams* dims) {
  if (dims == nullptr) return 0;
  const RpaParams p = page_attention_params(*dims);
  return rpa_workspace_bytes(&p);
}

int rpa_page_attention_launch(const RpaPageAttnParams* params, void* hip_stream) {
  if (params == nullptr) return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "params is null");
  const RpaParams p = page_attention_params(*params);
  int rc = rpa::validate(p, true, true);
  if (rc != RPA_OK) return rc;
  if (!params->value_cache) return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "null device pointer in RpaPageAttnParams");
  if (!rpa::data_aligned(p, params->value_cache)) return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "value_cache is not aligned like key_cache must be");
  const uint32_t esize = p.dtype == RPA_DTYPE_BF16 ? 2u : 4u;
  rpa::KvLayout kv;
  kv.k_base = static_cast<const char*>(params->key_cache);
  kv.v_base = static_cast<const char*>(params->value_cache);
  kv.stride_b = p.head_dim * esize;
  kv.head_b = static_cast<uint32_t>(p.page_size) * kv.stride_b;
  kv.page_b = static_cast<uint64_t>(p.num_kv_heads) * kv.head_b;
  kv.contiguous = 0;
  kv.capacity = rpa::paged_capacity(p);
  if (static_cast<uint64_t>(p.page_size) * p.head_dim * esize > 0xffffffffull)
    return rpa::fail(RPA_ERR_UNSUPPORTED, "a cache block of one head exceeds 4 GiB");
  return rpa::dispatch(p, kv, page_attention_tiled(p), static_cast<hipStream_t>(hip_stream));
}

static RpaParams ragged_decode_params(const RpaRaggedDecodeParams& a) {
  RpaParams p = {};
  p.queries = a.query;
  p.kv_pages = a.key;
  p.context_lens = a.sequence_end;  // the query sits at sequence_end - 1 and sees keys below sequence_end
  p.kv_start = a.sequence_start;
  p.block_tables = nullptr;         // contiguous caches: sequence b is "page" b
  p.query_start_loc = nullptr;
  p.num_seqs = nullptr;
  p.out = a.out;
  p.workspace = a.workspace;
  p.workspace_bytes = a.workspace_bytes;
  p.total_tokens = a.batch;
  p.max_num_seqs = a.batch;
  p.num_q_heads = a.num_q_heads;
  p.num_kv_heads = a.num_kv_heads;
  p.head_dim = a.head_dim;
  int page = 4;  // a power of two that holds a whole sequence, so the slot inside the "page" is the position
  while (page < a.seq_len && page < (1 << 30)) page <<= 1;
  p.page_size = page;
  p.num_pages = a.batch;
  p.pages_per_seq = 1;
  p.softmax_scale = a.softmax_scale;
  p.logits_soft_cap = a.logits_soft_cap;
  p.sliding_window = a.window_left >= 0 ? a.window_left + 1 : 0;  // k >= pos - left  <=>  k > pos - (left + 1)
  p.dtype = a.dtype;
  p.compute = a.compute;
  p.flags = a.flags & RPA_FLAG_FORCE_GENERIC;
  return p;
}

// With sinks the workspace continues behind the attention kernels' part: the sink keys' attention state per
// (sequence, query head) and the first position left for the attention kernels per sequence.
struct SinkWorkspace {
  uint64_t base, pre_o_off, pre_ml_off, start_off, total;
};
static SinkWorkspace sink_workspace(const RpaRaggedDecodeParams& a, const RpaParams& p) {
  SinkWorkspace w;
  const uint64_t rows = static_cast<uint64_t>(a.batch) * a.num_q_heads;
  w.base = (rpa_workspace_bytes(&p) + 255) & ~255ull;
  w.pre_o_off = w.base;
  w.pre_ml_off = w.pre_o_off + ((rows * a.head_dim * 4 + 255) & ~255ull);
  w.start_off = w.pre_ml_off + ((rows * 8 + 255) & ~255ull);
  w.total = w.start_off + ((static_cast<uint64_t>(a.batch) * 4 + 255) & ~255ull);
  return w;
}

uint64_t rpa_ragged_decode_workspace_bytes(const RpaRaggedDecodeParams* dims) {
  if (dims == nullptr || dims->seq_len <= 0 || dims->batch <= 0 || dims->num_q_heads <= 0 || dims->head_dim <= 0) return 0;
  const RpaParams p = ragged_decode_params(*dims);
  if (dims->num_sinks > 0) return sink_workspace(*dims, p).total;
  return rpa_workspace_bytes(&p);
}

int rpa_ragged_decode_launch(const RpaRaggedDecodeParams* params, void* hip_stream) {
  if (params == nullptr) return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "params is null");
  if (params->seq_len <= 0) return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "seq_len=%d must be positive", params->seq_len);
  RpaParams p = ragged_decode_params(*params);
  int rc = rpa::validate(p, true, true, true);
  if (rc != RPA_OK) return rc;
  if (!params->value || !params->sequence_start)
    return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "null device pointer in RpaRaggedDecodeParams");
  if (!rpa::data_aligned(p, params->value) || !rpa::aligned_to(params->sequence_start, 4) || !rpa::aligned_to(params->softmax_aux, 4))
    return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "value is not aligned like key must be, or an int32 / fp32 array is not aligned to 4 bytes");
  const uint32_t esize = p.dtype == RPA_DTYPE_BF16 ? 2u : 4u;
  rpa::KvLayout kv;
  kv.k_base = static_cast<const char*>(params->key);
  kv.v_base = static_cast<const char*>(params->value);
  kv.head_b = p.head_dim * esize;
  kv.stride_b = static_cast<uint32_t>(p.num_kv_heads) * kv.head_b;
  kv.page_b = static_cast<uint64_t>(params->seq_len) * kv.stride_b;
  kv.contiguous = 1;
  kv.capacity = params->seq_len;
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  const bool tiled = page_attention_tiled(p);
  if (params->num_sinks == 0) return rpa::dispatch(p, kv, tiled, stream);

  const int G = p.num_q_heads / p.num_kv_heads;
  if (params->num_sinks < 0 || params->num_sinks > RPA_MAX_SINK_KEYS)
    return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "num_sinks=%d must lie in [0, %d]", params->num_sinks, RPA_MAX_SINK_KEYS);
  if (!params->softmax_aux) return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "num_sinks=%d but softmax_aux is null", params->num_sinks);
  if (params->aux_rows != 1 && params->aux_rows != G)
    return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "aux_rows=%d must be 1 or num_q_heads / num_kv_heads = %d", params->aux_rows, G);
  const SinkWorkspace w = sink_workspace(*params, p);
  if (p.workspace == nullptr || p.workspace_bytes < w.total)
    return rpa::fail(RPA_ERR_WORKSPACE, "workspace of %llu bytes is too small, rpa_ragged_decode_workspace_bytes() asks for %llu",
                     (unsigned long long)p.workspace_bytes, (unsigned long long)w.total);
  if (tiled) {
    // the attention kernel walks the sink keys itself, in the wavefront that finishes each (sequence, kv head)
    rpa::PreState sinks;
    sinks.sink_aux = params->softmax_aux;
    sinks.sink_n = params->num_sinks;
    sinks.sink_rows = params->aux_rows;
    sinks.sink_limit = params->seq_len;
    return rpa::dispatch(p, kv, true, stream, sinks);
  }
  // the scalar kernel: a pre-pass accumulates the sink keys into an attention state that it merges into every row
  char* ws = static_cast<char*>(p.workspace);
  rpa::SinkKeyArgs sk;
  sk.aux = params->softmax_aux;
  sk.num_sinks = params->num_sinks;
  sk.aux_rows = params->aux_rows;
  sk.seq_len = params->seq_len;
  sk.pre_o = reinterpret_cast<float*>(ws + w.pre_o_off);
  sk.pre_ml = reinterpret_cast<float*>(ws + w.pre_ml_off);
  sk.main_start = reinterpret_cast<int32_t*>(ws + w.start_off);
  rc = rpa::launch_sink_keys(p, kv, sk, stream);
  if (rc == RPA_ERR_UNSUPPORTED) return rpa::fail(rc, "head_dim=%d exceeds the supported maximum of 512", p.head_dim);
  if (rc != RPA_OK) return rpa::fail(rc, "sink key launch failed: %s", hipGetErrorString(hipGetLastError()));
  p.kv_start = sk.main_start;
  p.workspace_bytes = w.base;
  rpa::PreState pre;
  pre.o = sk.pre_o;
  pre.ml = sk.pre_ml;
  return rpa::dispatch(p, kv, tiled, stream, pre);
}

namespace rpa {
static int dispatch(const RpaParams& p, const KvLayout& kv, bool tiled, hipStream_t stream, const PreState& pre) {
  int rc;
  if (tiled) {
    rc = rpa::launch_tiled(p, kv, stream, pre);
    if (rc == RPA_ERR_WORKSPACE)
      return rpa::fail(rc, "workspace of %llu bytes is too small, rpa_workspace_bytes() asks for %llu",
                       (unsigned long long)p.workspace_bytes, (unsigned long long)rpa_workspace_bytes(&p));
    if (rc != RPA_OK) return rpa::fail(rc, "kernel launch failed: %s", hipGetErrorString(hipGetLastError()));
    return RPA_OK;
  }
  rc = rpa::launch_generic(p, kv, stream, pre);
  if (rc == RPA_ERR_UNSUPPORTED) return rpa::fail(rc, "head_dim=%d exceeds the supported maximum of 512", p.head_dim);
  if (rc != RPA_OK) return rpa::fail(rc, "kernel launch failed: %s", hipGetErrorString(hipGetLastError()));
  return RPA_OK;
}
}  // namespace rpa

uint64_t rpa_v3_workspace_bytes(const RpaV3Params* dims) {
  if (dims == nullptr) return 0;
  const uint64_t base = rpa_workspace_bytes(&dims->attn);
  if (base == 0 || (dims->cache_dtype != RPA_DTYPE_FP8_E4M3 && dims->cache_dtype != RPA_DTYPE_FP8_E5M2)) return base;
  const uint64_t rows = static_cast<uint64_t>(dims->attn.total_tokens > 0 ? dims->attn.total_tokens : 0) * dims->attn.num_q_heads;
  // behind the kernels' part: the row statistics, then the logits kept between the two launches (if any)
  return ((base + 255) & ~255ull) + ((rows * 8 + 255) & ~255ull) + ((rpa::logit_stash_bytes(dims->attn) + 255) & ~255ull);
}

int rpa_v3_launch(const RpaV3Params* params, void* hip_stream) {
  if (params == nullptr) return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "params is null");
  RpaV3Params v = *params;
  v.attn.flags |= RPA_FLAG_FP32_LOGITS;
  int rc = rpa::validate(v.attn, true);
  if (rc != RPA_OK) return rc;
  if (!v.new_keys || !v.new_values) return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "null new_keys / new_values");
  if (!rpa::aligned_to(v.new_keys, 16) || !rpa::aligned_to(v.new_values, 16) || !rpa::aligned_to(v.attn.kv_pages, 16))
    return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "new_keys, new_values and the cache must be aligned to 16 bytes");
  if (v.attn.num_sinks != 0) return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "ragged_page_attention_v3 has no sinks");
  const bool fp8 = v.cache_dtype == RPA_DTYPE_FP8_E4M3 || v.cache_dtype == RPA_DTYPE_FP8_E5M2;
  if (!fp8 && v.cache_dtype != v.attn.dtype)
    return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "cache_dtype=%d: the cache has the dtype of the queries (%d) or is RPA_DTYPE_FP8_E4M3 / RPA_DTYPE_FP8_E5M2",
                     v.cache_dtype, v.attn.dtype);
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  const uint32_t esize = fp8 ? 1u : v.attn.dtype == RPA_DTYPE_BF16 ? 2u : 4u;
  const int chd = v.cache_head_dim > 0 ? v.cache_head_dim : v.attn.head_dim;  // elements per cache row
  if (chd < v.attn.head_dim || (static_cast<uint64_t>(chd) * esize) % 16 != 0)
    return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "cache_head_dim=%d: rows hold head_dim=%d elements at least and are a multiple of 16 bytes",
                     v.cache_head_dim, v.attn.head_dim);
  const int chx2 = v.cache_combined_heads > 0 ? v.cache_combined_heads : 2 * v.attn.num_kv_heads;  // heads per cache token
  if (chx2 < 2 * v.attn.num_kv_heads)
    return rpa::fail(RPA_ERR_INVALID_ARGUMENT, "cache_combined_heads=%d: a cache token holds 2 * num_kv_heads = %d rows at least",
                     v.cache_combined_heads, 2 * v.attn.num_kv_heads);
  if (fp8) {
    if (v.attn.dtype != RPA_DTYPE_BF16 || v.attn.compute != RPA_COMPUTE_BF16)
      return rpa::fail(RPA_ERR_UNSUPPORTED, "an 8-bit cache takes bf16 queries and RPA_COMPUTE_BF16");
    if (!rpa::tiled_supported(v.attn))
      return rpa::fail(RPA_ERR_UNSUPPORTED,
                       "an 8-bit cache runs on the MFMA kernel only (head_dim a multiple of 16 in 64..256, page_size a power of two >= 4, "
                       "no RPA_FLAG_FORCE_GENERIC)");
    const uint64_t need = rpa_v3_workspace_bytes(&v);
    if (v.attn.workspace == nullptr || v.attn.workspace_bytes < need)
      return rpa::fail(RPA_ERR_WORKSPACE, "workspace of %llu bytes is too small, rpa_v3_workspace_bytes() asks for %llu",
                       (unsigned long long)v.attn.workspace_bytes, (unsigned long long)need);
  }
  // Everything that can fail is checked before the cache is touched: a rejected call leaves the cache as it was.
  if (!fp8 && rpa::tiled_supported(v.attn)) {
    const uint64_t need = rpa_workspace_bytes(&v.attn);
    if (v.attn.workspace == nullptr || v.attn.workspace_bytes < need)
      return rpa::fail(RPA_ERR_WORKSPACE, "workspace of %llu bytes is too small, rpa_v3_workspace_bytes() asks for %llu",
                       (unsigned long long)v.attn.workspace_bytes, (unsigned long long)need);
  }
  if (v.attn.head_dim > 512 || (static_cast<uint64_t>(v.attn.head_dim) * (fp8 ? 1 : v.attn.dtype == RPA_DTYPE_BF16 ? 2 : 4)) % 16 != 0)
    return rpa::fail(RPA_ERR_UNSUPPORTED, "head_dim=%d: rows must be a multiple of 16 bytes and head_dim at most 512", v.attn.head_dim);
  rc = rpa::launch_kv_cache_update(v, stream);
  if (rc == RPA_ERR_UNSUPPORTED)
    return rpa::fail(rc, "head_dim=%d rows are not a multiple of 16 bytes", v.attn.head_dim);
  if (rc != RPA_OK) return rpa::fail(rc, "cache update launch failed: %s", hipGetErrorString(hipGetLastError()));
  if (!fp8 && chd == v.attn.head_dim && chx2 == 2 * v.attn.num_kv_heads) return rpa_fwd_launch(&v.attn, hip_stream);

  // 8-bit elements or padded rows: the cache is addressed through its own strides (K row of head j at combined
  // head 2j, its V row at 2j + 1, chd elements each)
  const RpaParams& p = v.attn;
  rpa::KvLayout kv;
  kv.k_base = static_cast<const char*>(p.kv_pages);
  kv.v_base = kv.k_base + static_cast<size_t>(chd) * esize;
  kv.stride_b = static_cast<uint32_t>(chx2) * chd * esize;
  kv.page_b = static_cast<uint64_t>(p.page_size) * kv.stride_b;
  kv.head_b = 2u * chd * esize;
  kv.contiguous = 0;
  kv.capacity = rpa::paged_capacity(p);
  if (!fp8) return rpa::dispatch(p, kv, rpa::tiled_supported(p), stream);
  const uint64_t base = (rpa_workspace_bytes(&p) + 255) & ~255ull;
  float* stats = reinterpret_cast<float*>(static_cast<char*>(p.workspace) + base);
  const uint64_t stats_bytes = (static_cast<uint64_t>(p.total_tokens > 0 ? p.total_tokens : 0) * p.num_q_heads * 8 + 255) & ~255ull;
  float* logits = rpa::logit_stash_bytes(p) != 0 ? reinterpret_cast<float*>(static_cast<char*>(p.workspace) + base + stats_bytes) : nullptr;
  RpaParams q = p;
  q.workspace_bytes = base;
  rc = rpa::launch_tiled_fp8(q, kv, v.cache_dtype == RPA_DTYPE_FP8_E5M2 ? 2 : 1, stats, logits, stream);
  if (rc != RPA_OK) return rpa::fail(rc, "kernel launch failed: %s", hipGetErrorString(hipGetLastError()));
  return RPA_OK;
}

}  // extern "C"
