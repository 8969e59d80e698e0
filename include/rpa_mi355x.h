/*
 * rpa_mi355x.h -- C ABI of the MI355X (gfx950) ragged paged attention forward.
 *
 * This is the boundary a foreign-function binding targets.  It replaces the backend
 * entry point the reference registers for this operation,
 *   ejkernel/kernels/_xla/ragged_page_attention/_interface.py:25-109
 * (reached from ejkernel/modules/operations/ragged_page_attention.py:540-641), and is
 * shaped like the reference's own native precedent, a custom call that receives device
 * buffers plus a stream (ejkernel/callib/_triton_call.py:738-757).
 *
 * Conventions
 *  - Every pointer in RpaParams is a DEVICE pointer owned by the caller.
 *  - rpa_fwd_launch only enqueues work on the given HIP stream: it never allocates,
 *    frees, or synchronises, and may be called from several host threads at once.
 *  - All functions return 0 on success and a negative RPA_ERR_* code on failure;
 *    rpa_last_error() gives the message of the calling thread's last failure.
 */
#ifndef RPA_MI355X_H_
#define RPA_MI355X_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RPA_ABI_VERSION 6

/* element type of queries / kv_pages / out */
#define RPA_DTYPE_BF16 0
#define RPA_DTYPE_F32 1
#define RPA_DTYPE_FP8_E4M3 2 /* OCP e4m3 (finite, no infinities; jnp.float8_e4m3fn): cache of rpa_v3_launch only */
#define RPA_DTYPE_FP8_E5M2 3 /* OCP e5m2 (jnp.float8_e5m2): cache of rpa_v3_launch only */

/* arithmetic mode */
#define RPA_COMPUTE_BF16 0 /* bf16 MFMA contractions, fp32 online softmax, reference rounding points */
#define RPA_COMPUTE_F32 1  /* everything in fp32 (page-gather exactness check) */

#define RPA_OK 0
#define RPA_ERR_INVALID_ARGUMENT (-1)
#define RPA_ERR_UNSUPPORTED (-2)
#define RPA_ERR_WORKSPACE (-3)
#define RPA_ERR_LAUNCH (-4)

#define RPA_MAX_SINK_KEYS 64 /* most sink positions rpa_ragged_decode_launch accepts (num_sinks) */

/* rpa_fwd_launch flags */
#define RPA_FLAG_FORCE_GENERIC 1u /* route every sequence through the scalar fp32 kernel */
#define RPA_FLAG_FP32_LOGITS 2u   /* the arithmetic of ragged_page_attention_v3 (_kernel.py:228-262): q enters the   */
                                  /* contraction unscaled, logits stay fp32 and are scaled after it, probabilities  */
                                  /* are rounded to the cache dtype before P V                                      */
#define RPA_FLAG_PREFILL_TILES 4u /* long chunks run as 128-row workgroup tiles whatever the size of the batch (by   */
                                  /* default batches of up to 20480 (token, query head) rows run them as 16-row      */
                                  /* wave-level items, which fills the device better when the tiles would be few)    */
#define RPA_FLAG_PIPE_TILES 8u    /* head_dim 128: prefill tiles of 256 rows, one workgroup per compute unit, key loop  */
                                  /* software-pipelined (by default chosen for batches of long chunks: at least 128    */
                                  /* query tokens per sequence on average); implies RPA_FLAG_PREFILL_TILES            */
#define RPA_FLAG_PLAIN_TILES 16u  /* never those: prefill tiles of 128 rows, two workgroups per compute unit          */
#define RPA_FLAG_NO_LOGIT_STASH 32u /* rpa_v3_launch with an 8-bit cache: both launches read K.  By default, batches  */
                                  /* of up to 20480 (token, query head) rows keep the first launch's fp32 logits in   */
                                  /* the workspace (4 bytes per row and position a block-table row can hold, 2 GiB   */
                                  /* at most: rpa_v3_workspace_bytes counts them) and the second launch reads those   */
                                  /* instead of K -- the same numbers, bit for bit                                    */

typedef struct RpaParams {
  /* ---- device buffers (argument names follow ragged_page_attention.py:540-547).  queries, kv_pages and out are   */
  /* aligned to 16 bytes (to the element where head_dim * sizeof(element) is not a multiple of 16), the int32 and   */
  /* fp32 arrays to 4; a misaligned pointer is RPA_ERR_INVALID_ARGUMENT ---- */
  const void* queries;         /* [total_tokens, num_q_heads, head_dim]                      */
  const void* kv_pages;        /* [num_pages, page_size, 2*num_kv_heads, head_dim]; K of kv   */
                               /* head j at combined index 2j, V at 2j+1                      */
  const int32_t* context_lens; /* [max_num_seqs]  kv length incl. the current query tokens    */
  const int32_t* block_tables; /* [max_num_seqs, pages_per_seq] physical page of logical page */
  const int32_t* query_start_loc; /* [max_num_seqs + 1] cumulative query lengths             */
  const int32_t* num_seqs;     /* [1] sequences actually present                              */
  const float* sinks;          /* [num_q_heads, num_sinks] fp32 sink logits, or NULL          */
  void* out;                   /* [total_tokens, num_q_heads, head_dim], same dtype as queries */
  void* workspace;             /* >= rpa_workspace_bytes() bytes, 256-byte aligned, or NULL   */
  uint64_t workspace_bytes;

  /* ---- static shape ---- */
  int32_t total_tokens;
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t head_dim;
  int32_t page_size;
  int32_t num_pages;
  int32_t max_num_seqs;
  int32_t pages_per_seq;
  int32_t num_sinks;

  /* ---- scalars ---- */
  float softmax_scale;    /* multiplies q . k                                   */
  float logits_soft_cap;  /* cap * tanh(x / cap); 0 = disabled                  */
  int32_t sliding_window; /* keys with pos > q_pos - window are kept; 0 = none  */
  int32_t dtype;          /* RPA_DTYPE_*                                        */
  int32_t compute;        /* RPA_COMPUTE_*                                      */

  /* ---- tile hints, 0 = library default.  They carry the fields of RaggedPageAttentionConfig                       */
  /*      (modules/operations/configs.py:242-258), which the reference hands to its backends                        */
  /*      (modules/operations/ragged_page_attention.py:299-318).  The library sees static, possibly padded shapes   */
  /*      only (total_tokens and max_num_seqs are upper bounds, the lengths live on the device), so its own choice  */
  /*      of kernel instantiation goes by those; a caller that knows its batch names the shape here.  Hints never   */
  /*      change which rows are computed, only how the work is cut.                                                  */
  int32_t num_queries_per_block;  /* query rows of a sequence per tile: 1..16 = the wave-level loop alone (decode     */
                                  /* steps and short chunks; by default batches of up to 20480 (token, query head)   */
                                  /* rows); 17..128 = 128-row workgroup tiles for long chunks; above 128 = 256-row    */
                                  /* software-pipelined tiles where they exist (head_dim 128, no soft cap, pages of   */
                                  /* 16 tokens or more; by default at least 128 tokens per max_num_seqs and block     */
                                  /* tables for 1024 keys or more; where the shapes do not say, the device picks      */
                                  /* them from 512 keys per query row on, by the batch's average), 128-row            */
                                  /* tiles otherwise.  RPA_FLAG_PREFILL_TILES / PIPE_TILES / PLAIN_TILES come first.  */
                                  /* With few rows (total_tokens x num_q_heads up to 34816) the 128-row tiles' key     */
                                  /* ranges are cut over idle workgroups when tiles are few: one long chunk alone.     */
  int32_t num_kv_pages_per_block; /* the least stretch of a sequence, in pages, that one streaming wavefront takes     */
                                  /* before a small batch is spread over more wavefronts (split-K granularity;        */
                                  /* default: 2 tiles of 32 keys, more for long sequences -- and one workgroup per     */
                                  /* (sequence, kv head), merged in LDS, for a decode batch of at most 512 of them     */
                                  /* with up to 1024 keys each, which a value here switches off)                      */
  int32_t num_warps;              /* accepted, ignored: workgroups have 4 wavefronts                                   */
  int32_t num_stages;             /* accepted, ignored: 2 LDS stages in the 128-row tile, 4 in the pipelined one      */
  uint32_t flags;                 /* RPA_FLAG_*                                       */

  /* ---- quantisation scales of ragged_page_attention_v3 (_kernel.py:221-226,232-235,258-259); 0 = absent.   */
  /*      q is divided by q_scale before the contraction, logits are multiplied by k_scale * q_scale, the      */
  /*      output by v_scale.  Only v_scale is honoured without RPA_FLAG_FP32_LOGITS.                           */
  float q_scale;
  float k_scale;
  float v_scale;

  /* ---- [max_num_seqs] first key position a sequence may attend to (sequence_start of ragged_decode_attention,   */
  /*      _xla/ragged_decode_attention/_xla_impl_fwd.py:55-58), or NULL for 0.                                   */
  const int32_t* kv_start;
} RpaParams;

/*
 * ragged_page_attention_v3: write the new tokens' K/V rows into the paged cache, then attend over it.
 * Replaces ejkernel/kernels/_xla/ragged_page_attention_v3/_interface.py:25-96 (program: _kernel.py:127-318).
 * The cache has the layout of kv_pages above, which is what merge_kv (_kernel.py:44-57) produces when head_dim
 * is a multiple of 128: [num_pages, page_size, 2*num_kv_heads / packing, packing, head_dim]; cache_head_dim below
 * covers the other head_dims.
 */
typedef struct RpaV3Params {
  RpaParams attn;         /* kv_pages = the cache, updated in place; context_lens = kv_lens (they include the new  */
                          /* tokens); num_seqs = &distribution[2]; RPA_FLAG_FP32_LOGITS is implied                 */
  const void* new_keys;   /* [total_tokens, num_kv_heads, head_dim], dtype of the cache                            */
  const void* new_values; /* [total_tokens, num_kv_heads, head_dim]                                                */
  int32_t cache_dtype;    /* dtype of the cache and of the new rows: attn.dtype, or RPA_DTYPE_FP8_E4M3 / _E5M2 with */
                          /* bf16 queries.  An 8-bit cache follows the program's casts (_kernel.py:249-254, :279):  */
                          /* with q_scale, q / q_scale is rounded to the query dtype, clipped to the 8-bit type's   */
                          /* finite range (+-448 / +-57344) and cast to it; the normalised probabilities are cast   */
                          /* to it before P V.  It runs as two launches (row                                        */
                          /* maximum and sum, then the attention) on the MFMA kernel only, and needs                */
                          /* rpa_v3_workspace_bytes() of workspace.                                                 */
  int32_t cache_head_dim; /* elements per cache row: align_to(head_dim, 128) as merge_kv pads it (_kernel.py:44-57), or 0  */
                          /* for head_dim.  With padded rows (head_dim 64 in rows of 128) the cache is                 */
                          /* [num_pages, page_size, 2*num_kv_heads / packing, packing, cache_head_dim]; the padding    */
                          /* is never read, and zeroed in the token records the update writes (the reference scatters  */
                          /* merge_kv's zero-padded rows).                                                              */
  int32_t cache_combined_heads; /* combined K/V heads per cache token: 2*num_kv_heads rounded up to a multiple of the    */
                          /* packing as merge_kv pads them (an odd num_kv_heads under an 8-bit cache), or 0 for         */
                          /* 2*num_kv_heads.  The padding heads are never read, and zeroed in the records the update writes. */
  int32_t reserved;       /* 0 */
} RpaV3Params;

/* Bytes of workspace rpa_fwd_launch needs for these static dims (pointers are ignored). */
uint64_t rpa_workspace_bytes(const RpaParams* dims);

/* Which kernels rpa_fwd_launch runs for these static dims, dtypes and flags (pointers are ignored): 1 = the MFMA
 * kernels, 0 = the scalar kernel -- fp32 inputs or compute, head_dim below 64, above 256 or no multiple of 16,
 * page_size below 4 or no power of two, more than 16384 sequences, RPA_FLAG_FORCE_GENERIC: exact, and some fifty
 * times slower on a decode batch -- and -1 for dims the launch would reject.  No counterpart in the reference, whose
 * registry names the backend it picked; a caller can warn, as the Python layer does, or choose another shape. */
int rpa_kernel_path(const RpaParams* dims);

/* Clears the counters at the head of a freshly allocated workspace (enqueue only).
 * A launch leaves them cleared again, so this is needed once per allocation. */
int rpa_workspace_init(void* workspace, uint64_t workspace_bytes, void* hip_stream);

/* Enqueues the forward pass on `hip_stream` (a hipStream_t; NULL = default stream). */
int rpa_fwd_launch(const RpaParams* params, void* hip_stream);

/*
 * rpa_fwd_launch for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  `workspace` / `workspace_bytes` of
 * the params are ignored: the kernels' scratch (split tickets, queue counters, partial attention states) is a
 * device array inside the library, rpa_static_scratch_bytes() = 34 MiB per GPU, held until the process ends.  The
 * call allocates and frees nothing and never synchronises; results are those of rpa_fwd_launch, bit for bit.
 * Shapes whose rpa_workspace_bytes() exceeds the array are rejected with RPA_ERR_WORKSPACE (head_dim 256 on the
 * MFMA kernel, today).  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU, on
 * whatever streams, race -- serialise them (one stream, or events between streams).  The call may be captured in a
 * HIP graph (it records the attention kernel and nothing else); make the first call on a device outside any capture,
 * since looking up the array's address may load the library's code object.
 */
uint64_t rpa_static_scratch_bytes(void);
int rpa_fwd_launch_static(const RpaParams* params, void* hip_stream);

/* Bytes of workspace rpa_v3_launch needs (rpa_workspace_bytes() of `attn`; with an 8-bit cache also the row
 * statistics and, unless RPA_FLAG_NO_LOGIT_STASH is set, the logits kept between its two launches). */
uint64_t rpa_v3_workspace_bytes(const RpaV3Params* dims);

/* Enqueues the cache update (token t of sequence s goes to position kv_len - q_len + (t - q_start) of s) and then
 * the forward pass, both on `hip_stream`.  Sequences whose block tables share a page that one of them writes see
 * the written rows (the reference updates and attends sequence by sequence). */
int rpa_v3_launch(const RpaV3Params* params, void* hip_stream);

/*
 * page_attention: one query token per sequence over a key cache and a value cache of
 * [num_blocks, num_kv_heads, block_size, head_dim].  Replaces the backend entry
 * ejkernel/kernels/_xla/page_attention/_interface.py:25-115 (program: _xla_impl_fwd.py:22-101), reached from
 * ejkernel/modules/operations/page_attention.py:364-383.  A key at position k of sequence s is kept iff
 * k < context_lens[s]; a sequence without keys yields zeros.
 */
typedef struct RpaPageAttnParams {
  const void* query;           /* [num_seqs, num_q_heads, head_dim]                          */
  const void* key_cache;       /* [num_blocks, num_kv_heads, block_size, head_dim]           */
  const void* value_cache;     /* [num_blocks, num_kv_heads, block_size, head_dim]           */
  const int32_t* context_lens; /* [num_seqs]                                                 */
  const int32_t* block_tables; /* [num_seqs, max_blocks]                                     */
  void* out;                   /* [num_seqs, num_q_heads, head_dim], dtype of query          */
  void* workspace;             /* >= rpa_page_attention_workspace_bytes() bytes, cleared once with rpa_workspace_init */
  uint64_t workspace_bytes;
  int32_t num_seqs;
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t head_dim;
  int32_t block_size;
  int32_t num_blocks;
  int32_t max_blocks;
  float attn_scale;            /* multiplies q (rounded to the query dtype, as `query * attn_scale` is) */
  int32_t dtype;               /* RPA_DTYPE_*                                                */
  int32_t compute;             /* RPA_COMPUTE_*                                              */
  uint32_t flags;              /* RPA_FLAG_FORCE_GENERIC, RPA_FLAG_FP32_LOGITS               */
} RpaPageAttnParams;

uint64_t rpa_page_attention_workspace_bytes(const RpaPageAttnParams* dims);
int rpa_page_attention_launch(const RpaPageAttnParams* params, void* hip_stream);

/*
 * ragged_decode_attention: one query token per sequence over contiguous caches key / value
 * [batch, seq_len, num_kv_heads, head_dim]; sequence b attends to positions [sequence_start[b], sequence_end[b])
 * from the query position sequence_end[b] - 1, optionally only to the last window_left + 1 of them.  Replaces the
 * backend entry ejkernel/kernels/_xla/ragged_decode_attention/_interface.py:26-121 (program:
 * _xla_impl_fwd.py:25-364), reached from ejkernel/modules/operations/ragged_decode_attention.py.
 *
 * Attention sinks as that program defines them (softmax_aux, _xla_impl_fwd.py:71-75 and :98-134): with num_sinks > 0
 * the keys at positions [sequence_start[b], sequence_start[b] + num_sinks) below seq_len are always visible, whatever
 * sequence_end and the window say, and a key at absolute position t < num_sinks has softmax_aux[row][t] added to its
 * logit (after the soft cap).  aux_rows is 1 (one vector for every head) or num_q_heads / num_kv_heads (row g for
 * the g-th query head of every kv head, which is how the program broadcasts a two-dimensional softmax_aux).
 */
typedef struct RpaRaggedDecodeParams {
  const void* query;             /* [batch, num_q_heads, head_dim]                */
  const void* key;               /* [batch, seq_len, num_kv_heads, head_dim]      */
  const void* value;             /* [batch, seq_len, num_kv_heads, head_dim]      */
  const int32_t* sequence_start; /* [batch]                                       */
  const int32_t* sequence_end;   /* [batch]                                       */
  void* out;                     /* [batch, num_q_heads, head_dim]                */
  void* workspace;               /* >= rpa_ragged_decode_workspace_bytes() bytes, cleared once with rpa_workspace_init */
  uint64_t workspace_bytes;
  int32_t batch;
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t head_dim;
  int32_t seq_len;
  float softmax_scale;
  float logits_soft_cap;         /* 0 = disabled                                  */
  int32_t window_left;           /* keys at positions >= query position - window_left are kept; < 0 = no window */
  int32_t dtype;                 /* RPA_DTYPE_*                                   */
  int32_t compute;               /* RPA_COMPUTE_*                                 */
  uint32_t flags;                /* RPA_FLAG_FORCE_GENERIC                        */
  const float* softmax_aux;      /* [aux_rows, num_sinks] fp32, or null           */
  int32_t num_sinks;             /* 0 = no sinks; at most RPA_MAX_SINK_KEYS       */
  int32_t aux_rows;              /* 1 or num_q_heads / num_kv_heads               */
} RpaRaggedDecodeParams;

uint64_t rpa_ragged_decode_workspace_bytes(const RpaRaggedDecodeParams* dims);
int rpa_ragged_decode_launch(const RpaRaggedDecodeParams* params, void* hip_stream);

/* Message for the calling thread's most recent failure ("" if none). */
const char* rpa_last_error(void);

/* RPA_ABI_VERSION the library was built with. */
int rpa_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* RPA_MI355X_H_ */
