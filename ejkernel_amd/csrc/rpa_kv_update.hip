// Cache update of ragged_page_attention_v3 (rows of the cache may be longer than head_dim: the padding of an updated
// token is zeroed, as the reference's scatter of merge_kv's zero-padded rows does): token t of sequence s (t in [q_start, q_start + q_len)) is the key /
// value at position kv_len - q_len + (t - q_start) of that sequence, and its rows go to
// cache[block_tables[s, pos / page], pos % page, 2j | 2j + 1, :] for every kv head j
// (ejkernel/kernels/_xla/ragged_page_attention_v3/_kernel.py:44-57 merge_kv, :207-218 update).
// One workgroup per token; the 16-byte pieces of its K and V rows are spread over the threads.  Pure copy: the
// element type only sets the row length in bytes.
#include "rpa_device.h"
#include "rpa_host.h"

namespace rpa {

__global__ __launch_bounds__(256) void kv_cache_update_kernel(RpaParams p, const char* __restrict__ new_k,
                                                              const char* __restrict__ new_v, int row_bytes, int dst_row_bytes,
                                                              int dst_heads) {
  const int t = blockIdx.x;
  int nseq = p.num_seqs[0];
  nseq = nseq < 0 ? 0 : (nseq > p.max_num_seqs ? p.max_num_seqs : nseq);
  if (t >= batch_rows(p, nseq)) return;
  const int s = find_seq(p.query_start_loc, nseq, t);
  const SeqMeta sm = seq_meta(p, paged_capacity(p), s);
  if (t < sm.q0 || t >= sm.q0 + sm.q_len) return;
  const int pos = sm.kv_len - sm.q_len + (t - sm.q0);
  if (pos < 0 || pos >= sm.kv_len) return;
  int page = p.block_tables[static_cast<size_t>(s) * p.pages_per_seq + pos / p.page_size];
  page = page < 0 ? 0 : (page >= p.num_pages ? p.num_pages - 1 : page);
  const size_t tok = static_cast<size_t>(page) * p.page_size + pos % p.page_size;
  char* dst = static_cast<char*>(const_cast<void*>(p.kv_pages)) + tok * dst_heads * dst_row_bytes;
  const size_t src_off = static_cast<size_t>(t) * p.num_kv_heads * row_bytes;
  // The whole token record is written: the new K / V rows, and zeros in what merge_kv pads them with (row tails
  // beyond head_dim, combined heads beyond 2 * num_kv_heads) -- the reference scatters the padded rows.
  const int pieces_per_row = row_bytes / 16, dst_pieces = dst_row_bytes / 16, n = dst_heads * dst_pieces;
  for (int k = threadIdx.x; k < n; k += blockDim.x) {
    const int row = k / dst_pieces, piece = k - row * dst_pieces;  // row = combined head 2j (K) or 2j + 1 (V)
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (row < 2 * p.num_kv_heads && piece < pieces_per_row)
      v = *reinterpret_cast<const uint4*>(((row & 1) ? new_v : new_k) + src_off + static_cast<size_t>(row >> 1) * row_bytes + 16 * piece);
    *reinterpret_cast<uint4*>(dst + static_cast<size_t>(row) * dst_row_bytes + 16 * piece) = v;
  }
}

int launch_kv_cache_update(const RpaV3Params& v, hipStream_t stream) {
  const RpaParams& p = v.attn;
  if (p.total_tokens == 0) return RPA_OK;
  const int esize = v.cache_dtype == RPA_DTYPE_FP8_E4M3 || v.cache_dtype == RPA_DTYPE_FP8_E5M2 ? 1 : v.cache_dtype == RPA_DTYPE_BF16 ? 2 : 4;
  const int row_bytes = p.head_dim * esize;
  const int dst_row_bytes = (v.cache_head_dim > 0 ? v.cache_head_dim : p.head_dim) * esize;
  const int dst_heads = v.cache_combined_heads > 0 ? v.cache_combined_heads : 2 * p.num_kv_heads;
  if (row_bytes % 16 != 0 || dst_row_bytes % 16 != 0 || dst_row_bytes < row_bytes || dst_heads < 2 * p.num_kv_heads) return RPA_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kv_cache_update_kernel, dim3(p.total_tokens), dim3(256), 0, stream, p,
                     static_cast<const char*>(v.new_keys), static_cast<const char*>(v.new_values), row_bytes, dst_row_bytes, dst_heads);
  return hipGetLastError() == hipSuccess ? RPA_OK : RPA_ERR_LAUNCH;
}

}  // namespace rpa
