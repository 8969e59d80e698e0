// Device-side helpers shared by the ragged paged attention kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/rpa_mi355x.h"

namespace rpa {

constexpr int kWave = 64;

typedef uint16_t bf16_t;  // raw bfloat16 bits

__device__ __forceinline__ float bf16_to_f32(bf16_t b) { return __uint_as_float(static_cast<uint32_t>(b) << 16); }

// Round-to-nearest-even fp32 -> bf16 bits (NaN stays NaN).
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<bf16_t>((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<bf16_t>(u >> 16);
}

// fp32 value rounded to the nearest bf16, kept as fp32.
__device__ __forceinline__ float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

template <typename T>
struct Elem;
template <>
struct Elem<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <>
struct Elem<bf16_t> {
  static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void store(bf16_t* p, float v) { *p = f32_to_bf16(v); }
};

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

// Largest s in [0, n) with cu[s] <= row (cu is non-decreasing, cu[0] == 0 <= row).
__device__ __forceinline__ int find_seq(const int32_t* __restrict__ cu, int n, int row) {
  int lo = 0, hi = n;  // invariant: cu[lo] <= row, answer in [lo, hi)
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (cu[mid] <= row) lo = mid; else hi = mid;
  }
  return lo;
}

// Ragged metadata with the one-token-per-sequence case folded in: a null query_start_loc means sequence s owns
// exactly row s, a null num_seqs means every one of the max_num_seqs sequences is present (page_attention).
__device__ __forceinline__ int seq_count(const RpaParams& p) {
  int n = p.num_seqs != nullptr ? p.num_seqs[0] : p.max_num_seqs;
  return n < 0 ? 0 : (n > p.max_num_seqs ? p.max_num_seqs : n);
}
__device__ __forceinline__ int q_start_of(const RpaParams& p, int s) {
  return p.query_start_loc != nullptr ? p.query_start_loc[s] : s;
}
__device__ __forceinline__ int kv_start_of(const RpaParams& p, int s) {
  return p.kv_start != nullptr ? max(p.kv_start[s], 0) : 0;
}
__device__ __forceinline__ int seq_of_row(const RpaParams& p, int nseq, int row) {
  return p.query_start_loc != nullptr ? find_seq(p.query_start_loc, nseq, row) : row;
}

// Query rows and key count of sequence s as every kernel uses them: clipped to what the buffers hold, so that
// malformed device metadata can neither read nor write out of bounds.  Row ranges are clipped to
// [0, total_tokens] (a start above its end gives an empty sequence) and the key count to [0, kv_capacity], the
// tokens one sequence's block-table row (or contiguous cache) can address.  The reference's XLA program is safe on
// such input because XLA clamps every dynamic index; its Pallas path rejects it up front
// (ejkernel/kernels/_pallas/tpu/ragged_page_attention/_pallas_impl_fwd.py:124-174: q_len <= kv_len,
// pages_per_seq >= ceil(kv_len / page), cu_q_lens[num_seqs] <= total tokens).
struct SeqMeta {
  int q0, q_len, kv_len;
};
__device__ __forceinline__ int clip_row(const RpaParams& p, int r) { return min(max(r, 0), p.total_tokens); }
__device__ __forceinline__ SeqMeta seq_meta(const RpaParams& p, int kv_capacity, int s) {
  SeqMeta m;
  m.q0 = clip_row(p, q_start_of(p, s));
  m.q_len = max(clip_row(p, q_start_of(p, s + 1)) - m.q0, 0);
  m.kv_len = min(max(p.context_lens[s], 0), kv_capacity);
  return m;
}
// Rows of the ragged batch (rows from here on are written as zeros).
__device__ __forceinline__ int batch_rows(const RpaParams& p, int nseq) { return clip_row(p, q_start_of(p, nseq)); }

}  // namespace rpa
