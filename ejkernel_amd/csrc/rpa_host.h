// Host-side declarations shared by the translation units of librpa_mi355x.so.
#pragma once

#include <hip/hip_runtime.h>

#include "../../include/rpa_mi355x.h"

namespace rpa {

// Where the K and V rows of (page, slot, kv head) live, in bytes.  ragged_page_attention interleaves K and V of a
// head inside one token record; page_attention keeps two caches of [blocks, kv heads, block, head_dim].
struct KvLayout {
  const char* k_base;
  const char* v_base;
  uint64_t page_b;    // between pages
  uint32_t stride_b;  // between the tokens of a page
  uint32_t head_b;    // between the kv heads of a token
  int32_t contiguous; // 1: no block table, sequence s is page s (page_b = bytes between sequences, slot = position)
  int32_t capacity;   // tokens one sequence can address: pages_per_seq * page_size, or the contiguous cache's seq_len
};
__host__ __device__ inline int32_t paged_capacity(const RpaParams& p) {
  const int64_t c = static_cast<int64_t>(p.pages_per_seq) * p.page_size;
  return c > 0x7fffffff ? 0x7fffffff : static_cast<int32_t>(c);
}
inline KvLayout interleaved_layout(const RpaParams& p) {
  const uint32_t esize = p.dtype == RPA_DTYPE_BF16 ? 2u : 4u;
  KvLayout l;
  l.k_base = static_cast<const char*>(p.kv_pages);
  l.v_base = l.k_base + static_cast<size_t>(p.head_dim) * esize;
  l.stride_b = 2u * p.num_kv_heads * p.head_dim * esize;
  l.page_b = static_cast<uint64_t>(p.page_size) * l.stride_b;
  l.head_b = 2u * p.head_dim * esize;
  l.contiguous = 0;
  l.capacity = paged_capacity(p);
  return l;
}

// Attention state -- row maximum, row sum, unnormalised output -- that an earlier kernel accumulated over keys
// outside the range the attention kernels walk.  It is merged into a row like one more part of a split key range,
// before the row is normalised.  Honoured where a sequence has one query token: the wave-level decode loop and the
// scalar kernel, not the prefill tiles.
struct PreState {
  const float* o = nullptr;   // [tokens, num_q_heads, head_dim]
  const float* ml = nullptr;  // [tokens, num_q_heads, 2]: maximum (-inf if no key), sum
  // Or, instead of a state from an earlier kernel (tiled kernel only): the sink keys of ragged_decode_attention
  // themselves.  The attention kernel then starts `sink_n` keys after kv_start[s] and the wavefront that finishes a
  // (sequence, kv head) walks the keys [kv_start[s], kv_start[s] + sink_n) below `sink_limit` itself, with
  // sink_aux[row][t] added to the logit of absolute position t < sink_n (_xla_impl_fwd.py:71-75, :98-134).
  const float* sink_aux = nullptr;  // [sink_rows, sink_n]
  int32_t sink_n = 0, sink_rows = 1, sink_limit = 0;
};

// Sink keys of ragged_decode_attention (_xla_impl_fwd.py:71-75, :98-134): accumulates, per (sequence, query head),
// the keys at positions [kv_start[s], kv_start[s] + num_sinks) below seq_len into `pre_o` / `pre_ml`, with
// softmax_aux[row][t] added to the logit of absolute position t < num_sinks, and writes kv_start[s] + num_sinks to
// `main_start`, the first position left for the attention kernels.
struct SinkKeyArgs {
  const float* aux;
  int32_t num_sinks, aux_rows, seq_len;
  float* pre_o;
  float* pre_ml;
  int32_t* main_start;
};
int launch_sink_keys(const RpaParams& p, const KvLayout& kv, const SinkKeyArgs& sk, hipStream_t stream);

// Each returns RPA_OK or a negative RPA_ERR_* code; all of them only enqueue on `stream`.
int launch_generic(const RpaParams& p, const KvLayout& kv, hipStream_t stream, const PreState& pre = PreState());
// Writes the new tokens' K/V rows into the paged cache (ragged_page_attention_v3, _kernel.py:207-218).
int launch_kv_cache_update(const RpaV3Params& v, hipStream_t stream);

// Tiled MFMA path (bf16, head_dim 128 or 256, page_size a multiple of 4).
constexpr int kTiledMaxSeqs = 1024;        // entries of a schedule array in LDS; larger batches keep every 2nd, 4th, ...
constexpr int kTiledMaxSchedShift = 4;     // sequence's start there: up to 16384 sequences
inline int sched_shift_for(int max_num_seqs) {
  int k = 0;
  while (((max_num_seqs + (1 << k) - 1) >> k) > kTiledMaxSeqs) ++k;
  return k;
}
constexpr int kTiledMaxWgsPerCu = 4;        // persistent grid = compute units x this, at most

constexpr uint64_t kWorkspaceTicketBytes = 1u << 20;  // head of the workspace, cleared by rpa_workspace_init
// The last 512 words of the ticket region hold the counters of the prefill queues, each in a 64-byte line of its
// own (counters that share a line queue up behind each other where the atomics execute): the ticket counter of queue
// x at word 16 x, the count of XCDs whose workgroups have all left at word 128, and at word 144 + 16 x the count of
// workgroups of XCD x that have left.  The split tickets, one word per (sequence, kv head), lie below them.
constexpr uint32_t kQueueCounterIndex = (1u << 20) / 4 - 512;
constexpr uint32_t kQueueStride = 16, kQueueExitIndex = 128, kQueueXcdExitIndex = 144;

struct WorkspaceLayout {
  uint64_t counters_bytes;                   // split tickets at offset 0
  uint64_t partial_o_off, partial_o_bytes;   // fp32 [slots][16][head_dim]
  uint64_t partial_ml_off, partial_ml_bytes; // fp32 [slots][16][2] (row max, row sum)
  uint64_t total_bytes;
};

bool tiled_supported(const RpaParams& p);
void tiled_workspace_layout(const RpaParams& p, WorkspaceLayout* wl);
int launch_tiled(const RpaParams& p, const KvLayout& kv, hipStream_t stream, const PreState& pre = PreState());
// The same for an 8-bit cache described by `kv` (kv_elem 1 = e4m3, 2 = e5m2): two launches, row statistics into
// `stats` [total_tokens, num_q_heads, 2] and then the attention (RPA_FLAG_FP32_LOGITS arithmetic, no sinks).
// `logits` (null, or logit_stash_bytes(p) bytes): where the statistics launch leaves its logits for the second launch.
int launch_tiled_fp8(const RpaParams& p, const KvLayout& kv, int kv_elem, float* stats, float* logits, hipStream_t stream);
// Bytes of fp32 logits a two-launch call on an 8-bit cache keeps between its launches, 0 where it does not (batches
// that run on prefill tiles, or more than kLogitStashMaxBytes).
uint64_t logit_stash_bytes(const RpaParams& p);

// Compute units of the current device (cached per device).
int device_cu_count();

// Records the calling thread's error message and returns `code`.
int fail(int code, const char* fmt, ...);

}  // namespace rpa
