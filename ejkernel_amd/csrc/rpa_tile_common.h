// Types and helpers shared by the wave-level (decode) and workgroup-level (prefill) attention loops.
#pragma once

#include "rpa_device.h"
#include "rpa_host.h"

namespace rpa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;
typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;

constexpr int kWgThreads = 256;
constexpr int kWgWaves = kWgThreads / kWave;
constexpr float kLog2e = 1.4426950408889634f;

struct TileArgs {
  RpaParams p;
  KvLayout kv;        // K / V addressing of the decode loop (prefill tiles assume the interleaved layout)
  int page_shift;     // log2(page_size)
  int uniform_page;   // page_size >= 16: a 16-token sub-tile lies in one page
  int decode_grid;    // mixed batches: the workgroups from this one on take the decode stream first
  int stream_grid;    // workgroups that take part when the batch has no prefill tiles
  int sched_shift;    // the schedule arrays hold every (1 << sched_shift)-th sequence's start (0: every sequence)
  int min_share_tiles; // small batches: tiles per streaming wavefront before more wavefronts are used
  int item_pad_tiles;  // empty positions every (sequence, kv head) adds to the decode stream (the cost of a part in tiles)
  int even_xcd_permille;  // share of the decode stream given to the workgroups on even XCDs, in 1/1000
  int phase_mode;     // mixed batches: 4 = upper half of the grid streams, prefill tiles from queues; 0..3 = static
                      // split, streaming first on no / upper-half / odd / odd-octet workgroups
  uint32_t* counters; // split tickets [max_num_seqs * num_kv_heads], then the queue counters; zero between launches
  float* partial_o;   // [2 * wavefronts of the grid][16][D]
  float* partial_ml;  // [2 * wavefronts of the grid][16][2]
  float* stats;       // row maximum and row sum per (token, query head) of a two-launch call (null otherwise)
  float* logits;      // two-launch call: the first launch's logits, [token][kv head][logit_pitch / 4][query head of the
                      // kv head][4] (null: K is read twice)
  uint32_t logit_pitch;  // keys per (token, query head) of `logits`: a multiple of 64 that covers a block-table row
  PreState pre;       // state accumulated by an earlier kernel, merged by the wave-level loop (null: none)
  // head_dim 64, instantiation without prefill tiles: a wave-level item covers two kv heads (2 j, 2 j + 1) at once.
  // The 128-wide loop then reads, per token, [K of head 2j | K of head 2j+1] as one K row and the two V rows as one V
  // row -- in the interleaved cache 512 contiguous bytes per token instead of two visits of 256 -- with the query
  // rows of the first head zero in the second half of the contraction and vice versa; every row keeps the half of the
  // output that belongs to its head.
  int pair;
  // Which of two launches of one call does the work, decided on the device, where the lengths are: 0 = this launch
  // (the host has decided), 1 = this launch holds the 128-row prefill tiles, 2 = this one the pipelined 256-row
  // tiles.  With 1 or 2 every workgroup weighs the batch's prefill work against its decode stream the same way and
  // the launch that is not picked ends there.
  int select;
  // A batch of few, short decode sequences: up to how many tiles a (sequence, kv head) may have for the batch to run
  // one workgroup per (sequence, kv head), its four wavefronts merging through LDS (0 = never).
  int wg_item_tiles;
  // Kernels for few sequences (kFew): from how many parts per (sequence, kv head) on, were it cut by wavefront, the decode
  // stream is cut by workgroup: a workgroup's share of a (sequence, kv head) is walked by its four wavefronts, a quarter
  // each, and merged in LDS, so a (sequence, kv head) has a quarter of the parts that go through memory (0 = never).
  int wg_unit_parts;
  // A launch of few prefill tiles and nothing else: into how many runs of key tiles a tile's key range may be cut, a
  // workgroup each, so that the tiles of one long chunk fill the device (0 or 1 = never; 128-row tiles only).  The
  // parts' states lie in partial_o / partial_ml (tile_parts_cap of them fit) and a tile's ticket is the word
  // counters[tile_ticket_base + tile].
  int tile_split, tile_parts_cap, tile_ticket_base;
  int tile_stream_slots_half;  // slots of the decode stream's partial states that fit in the lower half
  uint32_t tile_state_o_half, tile_state_ml_half;  // bytes: half of partial_o and of partial_ml (a launch with a decode stream)
};

// How the softmax scale enters.  Reference arithmetic of ragged_page_attention (kMimic): q is multiplied by the
// bf16 scale and rounded to bf16 before the contraction.  Arithmetic of ragged_page_attention_v3 (!kMimic): q
// enters as it is (divided by q_scale and rounded, if given) and the fp32 logits are multiplied by
// softmax_scale * k_scale * q_scale.
template <bool kMimic>
__device__ __forceinline__ float q_operand(float x, const RpaParams& p, float mimic_scale) {
  if (kMimic) return x * mimic_scale;
  return p.q_scale > 0.f ? x / p.q_scale : x;
}
__device__ __forceinline__ float logit_scale(const RpaParams& p) {
  return p.softmax_scale * (p.k_scale > 0.f ? p.k_scale : 1.f) * (p.q_scale > 0.f ? p.q_scale : 1.f);
}
__device__ __forceinline__ float out_scale(const RpaParams& p) { return p.v_scale > 0.f ? p.v_scale : 1.f; }

// Split of the decode stream over the wavefronts of the grid, in two regions that are each cut evenly: workers
// [0, h) share the first n_a tiles, workers [h, ...) the rest.  Within a region the first `rem` workers take
// q + 1 tiles and the others q.  The caller chooses n_a so that every non-empty share lies in front of every
// empty one: the merge of a split (sequence, kv head) counts on a part from each worker between its first and last.
struct Shares {
  int h, n_a, q_a, rem_a, q_b, rem_b;
  __device__ __forceinline__ void set(int total, int n_workers, int first_region_workers, int first_region_tiles) {
    h = first_region_workers;
    n_a = first_region_tiles;
    const int nb = n_workers - h;
    q_a = h > 0 ? n_a / h : 0;
    rem_a = n_a - q_a * h;
    q_b = nb > 0 ? (total - n_a) / nb : 0;
    rem_b = (total - n_a) - q_b * nb;
  }
  __device__ __forceinline__ int begin(int w) const {
    return w < h ? w * q_a + min(w, rem_a) : n_a + (w - h) * q_b + min(w - h, rem_b);
  }
  __device__ __forceinline__ int owner(int x) const {
    if (x < n_a) {
      const int big = rem_a * (q_a + 1);
      return x < big ? x / (q_a + 1) : rem_a + (x - big) / q_a;
    }
    x -= n_a;
    const int big = rem_b * (q_b + 1);
    return h + (x < big ? x / (q_b + 1) : rem_b + (x - big) / q_b);
  }
};

// A wavefront's part of one (sequence, kv head) of the decode stream.
struct Part {
  bool partial;         // the (sequence, kv head) is shared with other wavefronts
  bool in_workgroup = false;  // the four wavefronts of the workgroup hold a quarter of this part each and merge through LDS
  int merger = 0;             // ... into this wavefront, which then stands for the part (kFew kernels; 0 elsewhere)
  bool again = false;         // ... and the workgroup goes on to another part: a second barrier before the K tiles are written anew
  int slot;             // workspace slot of this part
  int first_w, last_w;  // wavefronts sharing it (every one of them holds at least one of its tiles)
  int stream_a;         // stream index of its first tile
  Shares sh;
};

// Workspace slot of wavefront k's part of the (sequence, kv head) starting at stream tile stream_a: a wavefront
// has at most two partial parts, the one its share starts inside (slot 2k) and the one it ends inside (2k + 1).
__device__ __forceinline__ int part_slot(int k, int stream_a, const Shares& sh) {
  return 2 * k + (sh.begin(k) < stream_a ? 1 : 0);
}

struct SeqInfo {
  int q0, q_len, kv_len, rows, n_rt;
  int lo_al, hi;  // key range of the whole sequence, start aligned down to the tile
  int start;      // first key position the sequence may attend to
  bool eligible;  // single row tile with keys: part of the decode stream
};

template <int TT>
__device__ __forceinline__ SeqInfo seq_info(const TileArgs& a, int s, int G) {
  const RpaParams& p = a.p;
  SeqInfo si;
  const SeqMeta sm = seq_meta(p, a.kv.capacity, s);
  si.q0 = sm.q0;
  si.q_len = sm.q_len;
  si.kv_len = sm.kv_len;
  si.rows = si.q_len * G;
  si.n_rt = (si.rows + 15) >> 4;
  const int pos_min = si.kv_len - si.q_len;
  si.start = kv_start_of(p, s) + a.pre.sink_n;  // sink keys, if any, are walked apart from the stream
  int lo = p.sliding_window > 0 ? max(0, pos_min - p.sliding_window + 1) : 0;
  lo = max(lo, si.start);
  si.lo_al = lo & ~(TT - 1);
  si.hi = si.kv_len;
  si.eligible = si.n_rt == 1 && si.hi > si.lo_al;  // a sequence without keys stays an item: its rows become zero
  return si;
}

// Exclusive prefix sum of one int per thread over the workgroup; `total` gets the sum.
__device__ __forceinline__ int block_excl_scan(int v, int* wave_tot, int& total) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  int inc = v;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    int t = __shfl_up(inc, o, kWave);
    if (lane >= o) inc += t;
  }
  __syncthreads();
  if (lane == kWave - 1) wave_tot[wave] = inc;
  __syncthreads();
  int base = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < kWgWaves; ++w) {
    const int t = wave_tot[w];
    if (w < wave) base += t;
    tot += t;
  }
  total = tot;
  return base + inc - v;
}

// N such sums at once behind one pair of barriers (wave_tot: N * kWgWaves ints): v and total are arrays of N,
// base receives the exclusive prefix sums.
template <int N>
__device__ __forceinline__ void block_excl_scan_n(const int (&v)[N], int* wave_tot, int (&base)[N], int (&total)[N]) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  int inc[N];
#pragma unroll
  for (int k = 0; k < N; ++k) inc[k] = v[k];
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const int t = __shfl_up(inc[k], o, kWave);
      if (lane >= o) inc[k] += t;
    }
  }
  __syncthreads();
  if (lane == kWave - 1) {
#pragma unroll
    for (int k = 0; k < N; ++k) wave_tot[N * wave + k] = inc[k];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < N; ++k) {
    int b = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < kWgWaves; ++w) {
      const int t = wave_tot[N * w + k];
      if (w < wave) b += t;
      tot += t;
    }
    total[k] = tot;
    base[k] = b + inc[k] - v[k];
  }
}

// Hardware round-to-nearest-even conversions (v_cvt_pk_bf16_f32): branch-free, NaN stays NaN.
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2_t v;
  v[0] = static_cast<__bf16>(lo);
  v[1] = static_cast<__bf16>(hi);
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ float rbf(float x) { return static_cast<float>(static_cast<__bf16>(x)); }

// tanh through the hardware exp2 and reciprocal: 1 - 2 / (1 + e^(2x)), which saturates correctly for large |x|
// and has an absolute error near 1e-7; below |x| = 1/16, where that would be a large relative error, the odd
// series x (1 - x^2/3 + 2 x^4/15) takes over (relative error < 1e-8 there).  Branch-free.
__device__ __forceinline__ float tanh_fast(float x) {
  const float e = __builtin_amdgcn_exp2f(x * (2.f * kLog2e));
  const float big = fmaf(-2.f, __builtin_amdgcn_rcpf(1.f + e), 1.f);
  const float x2 = x * x;
  const float small = x * fmaf(x2, fmaf(x2, 2.f / 15.f, -1.f / 3.f), 1.f);
  return fabsf(x) < 0.0625f ? small : big;
}
// tanh of a bf16 value whose result the caller rounds to bf16.  Below 1/32 the result rounds back to the argument
// (tanh(y) = y (1 - y^2/3 + ...) and y^2/3 < 3.3e-4 there, a sixth of the smallest relative half-step of bf16, 2^-9),
// so the series of tanh_fast is not needed; from 1/32 up 1 - 2 / (1 + e^(2y)) is accurate to 5e-6 relative.
__device__ __forceinline__ float tanh_of_bf16(float y) {
  const float e = __builtin_amdgcn_exp2f(y * (2.f * kLog2e));
  const float big = fmaf(-2.f, __builtin_amdgcn_rcpf(1.f + e), 1.f);
  return fabsf(y) < 0.03125f ? y : big;
}
// Two values rounded to bf16 with one packed conversion.
__device__ __forceinline__ void rbf2(float& a, float& b) {
  const uint32_t pk = pack_bf16x2(a, b);
  a = __uint_as_float(pk << 16);
  b = __uint_as_float(pk & 0xffff0000u);
}
// cap * tanh(x / cap) with the reference's bf16 rounding after each op (kMimic) or in plain fp32.
template <bool kMimic>
__device__ __forceinline__ float soft_cap(float x, float cap, float inv_cap) {
  if (kMimic) return rbf(rbf(tanh_of_bf16(rbf(x * inv_cap))) * cap);
  return cap * tanh_fast(x * inv_cap);
}
// The same for two logits at once: the roundings share their conversions.
template <bool kMimic>
__device__ __forceinline__ void soft_cap2(float& a, float& b, float cap, float inv_cap) {
  if (kMimic) {
    float ya = a * inv_cap, yb = b * inv_cap;
    rbf2(ya, yb);
    float ta = tanh_of_bf16(ya), tb = tanh_of_bf16(yb);
    rbf2(ta, tb);
    a = ta * cap;
    b = tb * cap;
    rbf2(a, b);
  } else {
    a = cap * tanh_fast(a * inv_cap);
    b = cap * tanh_fast(b * inv_cap);
  }
}

// Reductions over the four lane groups that hold one query row (lanes l, l^16, l^32, l^48), with the gfx950
// lane-swap instructions instead of LDS permutes: swapping a value with itself yields, in every 16-lane row,
// both members of a row pair (then of a half-wave pair).
__device__ __forceinline__ float row_groups_max(float x) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  const float y = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(y), __float_as_uint(y), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float row_groups_sum(float x) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  const float y = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(y), __float_as_uint(y), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

}  // namespace rpa
