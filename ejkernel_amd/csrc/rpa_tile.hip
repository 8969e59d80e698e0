// Ragged paged attention on MFMA: one persistent launch per batch, two workgroups per compute unit.
//
// Rows of a sequence are its (query token, group head) pairs, handled 16 at a time (one MFMA
// tile) per kv head.  Work is discovered on the device from query_start_loc / context_lens /
// num_seqs (the host never reads them) and comes in three kinds:
//   * the decode stream: all sequences with a single row tile form one stream of key tiles
//     ordered by (sequence, kv head, position); every streaming wavefront takes a contiguous
//     share of it, whatever the individual lengths are.  A wavefront whose share covers only
//     part of a (sequence, kv head) writes its partial (m, l, O) to the workspace and takes a
//     ticket; the last part to arrive merges all parts in stream order, so the result does
//     not depend on timing (rpa_decode.h);
//   * wave items: sequences with two to four row tiles, one (sequence, row tile, kv head) per
//     wavefront over the full key range, through the same loop;
//   * prefill tiles: sequences with more rows, one workgroup per tile of 64 * MRT rows, K/V
//     tiles staged through LDS, handed out from per-XCD queues (rpa_prefill.h).
// In a mixed batch the upper half of the grid streams while the lower half starts on the
// prefill tiles; a batch without prefill tiles uses one workgroup per compute unit.
//
// Scores are S^T = K Q^T, outputs O^T = V^T P^T, so every lane owns one query row: the
// online-softmax state and the O rescale are lane-local.
//
// Numerics follow ejkernel/kernels/_xla/ragged_page_attention/_xla_impl_fwd.py:49,119-149
// (template argument kMimic): q is pre-multiplied by the bf16 scale and rounded to bf16,
// decode-loop logits are rounded to bf16, probabilities are bf16, accumulation is fp32.
// With kMimic = false q enters unscaled and the fp32 logits are scaled afterwards
// (ejkernel/kernels/_xla/ragged_page_attention_v3/_kernel.py:228-262).
#include "rpa_device.h"
#include <atomic>

#include "rpa_decode.h"
#include "rpa_prefill.h"
#include "rpa_prefill_pipe.h"

namespace rpa {

constexpr int kWaveItemMaxRowTiles = 4;  // sequences with more 16-row tiles than this use workgroup tiles
constexpr int kMaxMinShareTiles = 16;  // ... and the most the length of the (sequence, kv head)s raises that to
constexpr int kFewHeads = 64;          // (sequence, kv head)s up to which a decode batch takes the kFew instantiation
constexpr int kMinShareTiles = 2;       // tiles per streaming wavefront before more wavefronts are used
constexpr int kQueueRun = 16;            // consecutive prefill tiles that go to the same XCD queue
constexpr int kSortMax = kWgThreads;      // sequences with prefill tiles that are put in order of length (one per thread)
constexpr int kWaveOnlyMaxRows = 20480;   // (token, query head) rows up to which a batch runs without prefill tiles

// Dynamic LDS: three schedule arrays of max_num_seqs + 1 ints, 24 ints of scratch and the sequences with prefill
// tiles in order of length (up to kSortMax ints), then the data region
// shared by the prefill tiles (workgroup) and the decode K tiles (one per wavefront).
__host__ __device__ constexpr int sort_entries(int max_num_seqs) { return max_num_seqs < kSortMax ? max_num_seqs : kSortMax; }
__host__ __device__ constexpr size_t sched_bytes(int max_num_seqs) {
  return ((static_cast<size_t>(3) * (max_num_seqs + 1) + 24 + sort_entries(max_num_seqs)) * sizeof(int) + 15) &
         ~static_cast<size_t>(15);
}

// kWaveOnly: the prefill tiles are compiled out and sequences with many row tiles run as wave-level items too (right
// for every batch, slow for large prefill batches).  That leaves the decode loop a register allocation of its own, about
// 2 % faster on decode batches, and spreads short prefill chunks over more wavefronts, which is why the host picks
// this instantiation for small batches; it is also the one that merges an attention state in a.pre into every row.
// Prefill tiles of the instantiation: four row tiles per wavefront at head_dim 128 select the software-pipelined tile
// of rpa_prefill_pipe.h, which runs one workgroup per compute unit (one wavefront per SIMD, up to 512 registers).
template <int D, int MRT>
constexpr bool kPipeTile = D == 128 && MRT == 4;
// One workgroup per compute unit (one wavefront per SIMD, up to 512 registers) also for the head_dim-256 decode loop
// over a 16-bit cache: at two wavefronts per SIMD its 256 registers spill 65 of the loop's values, and a streaming
// batch runs one workgroup per unit anyway.
template <int D, int MRT, bool kWaveOnly, int kKv>
constexpr bool kWideDecode = D == 256 && kWaveOnly && kKv == 0;
template <int D, int MRT, bool kWaveOnly, int kKv>
constexpr int kWavesPerSimd = kPipeTile<D, MRT> || kWideDecode<D, MRT, kWaveOnly, kKv> ? 1 : 2;

template <int D, int MRT, bool kMimic, int kKv, int kPass, bool kCut>
__device__ __forceinline__ void run_prefill_tile(const TileArgs& a, char* lds, const SeqInfo& si, int s, int j, int qt,
                                                 int split_info = 0) {
  if constexpr (kPipeTile<D, MRT>) {
    static_assert(kKv == 0, "the pipelined tile reads a 16-bit cache");
    prefill_tile_pipe<kMimic>(a, lds, si, s, j, qt, split_info);
  } else {
    prefill_tile<D, MRT, kMimic, kKv, kPass, kCut>(a, lds, si, s, j, qt, split_info);
  }
}

// A wave-uniform value the compiler cannot see through.  The kinds of work of the kernel below sit in one loop over
// its two phases, and out of a loop the compiler hoists every invariant of every kind in front of it -- shares of the
// stream, queue sizes, divisions by run-time values, some eight hundred scalar instructions that a small launch then
// waits two microseconds for whatever it holds.  Sums that enter a section through this stay inside it.
__device__ __forceinline__ int kept_in_place(int x) {
  asm volatile("" : "+s"(x));
  return x;
}

// kFew with kWaveOnly: the instantiation for batches of a few dozen (sequence, kv head)s at most, where the host can
// tell from max_num_seqs; its decode stream is cut by workgroup or by wavefront.  kFew without: the instantiation for
// launches of few prefill tiles (by the static shapes), whose key ranges can be cut over the idle workgroups.
template <int D, int NT, int MRT, bool kMimic, bool kWaveOnly = false, int kKv = 0, int kPass = 0, bool kFew = false>
__global__ __launch_bounds__(kWgThreads) __attribute__((amdgpu_waves_per_eu(kWavesPerSimd<D, MRT, kWaveOnly, kKv>, kWavesPerSimd<D, MRT, kWaveOnly, kKv>)))
void rpa_tile_kernel(TileArgs a) {
  constexpr int DD = D < 128 ? 128 : D;  // head_dim 64: the wave-level loop works 128 wide, prefill tiles 64 wide
  using C = Cfg<DD, NT, kMimic>;
  using PC = PCfg<D, MRT>;
  extern __shared__ __align__(16) char smem[];
  const RpaParams& p = a.p;
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  // items of the wave-level loop: one per kv head, or one per pair of kv heads (TileArgs::pair) with both heads' rows
  const bool pair = kWaveOnly && kKv == 0 && kPass == 0 && a.pair != 0;
  const int G = (pair ? 2 : 1) * (p.num_q_heads / p.num_kv_heads);
  const int item_heads = pair ? p.num_kv_heads / 2 : p.num_kv_heads;
  // Schedule arrays: exclusive prefix sums over the sequences, kept for every K-th sequence (K = 1 for batches of up
  // to kTiledMaxSeqs sequences); the sequences in between are walked when an entry is looked up.
  const int shift = a.sched_shift, K = 1 << shift;
  const int sched_n = (p.max_num_seqs + K - 1) >> shift;
  int* item_start = reinterpret_cast<int*>(smem);   // wave-level items
  int* tile_start = item_start + (sched_n + 1);     // decode stream tiles
  int* wg_start = tile_start + (sched_n + 1);       // workgroup-level prefill tiles
  int* scratch = wg_start + (sched_n + 1);
  int* wg_seq = scratch + 24;                       // sequence of the r-th entry of wg_start, when those are sorted
  char* lds_data = smem + sched_bytes(sched_n);
  char* lds_k = lds_data + wave * C::LDS_PER_WAVE;

  const int nseq = seq_count(p);

  // ---- schedule.  Per sequence: tiles it adds to the decode stream (one row tile, has keys), workgroup tiles
  // (more than kWaveItemMaxRowTiles row tiles), or wave-level items (everything else).
  auto classify = [&](const SeqInfo& si, int& tiles, int& items, int& wg_items) {
    tiles = items = wg_items = 0;
    if (si.eligible) {
      const int per_head = (si.hi - si.lo_al + C::TT - 1) / C::TT;
      tiles = item_heads * (per_head + a.item_pad_tiles);
      // (a kernel without prefill tiles has no use for the third sum: it counts the sequences that are too long for
      // one workgroup per (sequence, kv head) there, and in the upper half those longer than half of that)
      if (kWaveOnly) wg_items = (per_head > a.wg_item_tiles ? 1 : 0) + (2 * per_head > a.wg_item_tiles ? 65536 : 0);
    } else if (!kWaveOnly && si.n_rt > kWaveItemMaxRowTiles) {
      wg_items = p.num_kv_heads * ((si.rows + PC::WGROWS - 1) / PC::WGROWS);
    } else {
      items = item_heads * si.n_rt;
    }
  };
  const int per = (((nseq + kWgThreads - 1) / kWgThreads + K - 1) >> shift) << shift;  // a multiple of K per thread
  const int s_begin = min(tid * per, nseq), s_end = min(s_begin + per, nseq);
  int my_items = 0, my_tiles = 0, my_wg = 0;
  int my_cost = 0;  // TileArgs::select: prefill work in units of 1024 (query row, key) pairs, see below
  int my_rows = 0;  // ... and its (query row, kv head)s
  int my_kv_len = 0;  // length of this thread's last sequence (the sort below: a thread with one sequence need not read it again)
  for (int s = s_begin; s < s_end; ++s) {
    int t, it, wg;
    const SeqInfo si = seq_info<C::TT>(a, s, G);
    classify(si, t, it, wg);
    my_tiles += t;
    my_items += it;
    my_wg += wg;
    my_kv_len = si.kv_len;
    if constexpr (!kWaveOnly && kKv == 0) {
      if ((a.select != 0 || ((kFew || kPipeTile<D, MRT>) && a.tile_split > 1)) && wg > 0) {
        const long long pairs = static_cast<long long>(si.rows) * p.num_kv_heads * max(si.kv_len - si.q_len / 2, 1);
        my_cost += static_cast<int>(min(pairs >> 10, 1ll << 24));
        my_rows += si.rows * p.num_kv_heads;
      }
    }
  }
  // (all four sums behind one pair of barriers: a small launch is a chain of such waits)
  int total_items, total_tiles, total_wg, total_cost, total_rows = 0;
  int item_base, tile_base, wg_base;
  if constexpr (!kWaveOnly && kKv == 0) {
    const int mine[5] = {my_items, my_tiles, my_wg, my_cost, my_rows};
    int base[5], total[5];
    block_excl_scan_n<5>(mine, scratch, base, total);
    item_base = base[0], tile_base = base[1], wg_base = base[2];
    total_items = total[0], total_tiles = total[1], total_wg = total[2];
    total_cost = __builtin_amdgcn_readfirstlane(total[3]);
    total_rows = __builtin_amdgcn_readfirstlane(total[4]);
  } else {
    const int mine[4] = {my_items, my_tiles, my_wg, my_cost};
    int base[4], total[4];
    block_excl_scan_n<4>(mine, scratch, base, total);
    item_base = base[0], tile_base = base[1], wg_base = base[2];
    total_items = total[0], total_tiles = total[1], total_wg = total[2];
    total_cost = __builtin_amdgcn_readfirstlane(total[3]);
  }
  for (int s = s_begin; s < s_end; ++s) {
    int t, it, wg;
    classify(seq_info<C::TT>(a, s, G), t, it, wg);
    if ((s & (K - 1)) == 0) {
      item_start[s >> shift] = item_base;
      tile_start[s >> shift] = tile_base;
      wg_start[s >> shift] = wg_base;
    }
    item_base += it;
    tile_base += t;
    wg_base += wg;
  }
  total_items = __builtin_amdgcn_readfirstlane(total_items);
  total_tiles = __builtin_amdgcn_readfirstlane(total_tiles);
  total_wg = __builtin_amdgcn_readfirstlane(total_wg);
  int n_long = 0;  // kWaveOnly: sequences of the decode stream with more than wg_item_tiles tiles, and (<< 16) with more than half
  if constexpr (kWaveOnly) {
    n_long = total_wg;
    total_wg = 0;
  }
  const int nc = (nseq + K - 1) >> shift;  // entries in use
  if (tid == 0) {
    item_start[nc] = total_items;
    tile_start[nc] = total_tiles;
    wg_start[nc] = total_wg;
  }
  __syncthreads();

  // ---- two launches, one call (TileArgs::select).  The 128-row tiles run beside a streaming workgroup on every
  // compute unit and win where the decode stream sets the time; the pipelined tiles own their units and win where
  // the prefill work does (16 chunks of 512 tokens beside 64 decode sequences: 0.45 against 0.53 ms; beside 240:
  // 1.08 against 0.92 ms).  The host sees padded shapes only, so where it cannot tell it enqueues both kernels and
  // every workgroup of both decides here, from the same sums: prefill work in units of 1024 (query row, key) pairs
  // against the stream's tiles of 32 keys -- 0.6 ns against 3 ns apiece at the rates the two kernels reach, and the
  // pipelined tiles are worth it from seven tenths of the stream's time on.  And from 512 keys per query row on, by the
  // batch's average: a pipelined tile has its compute unit to itself, and what a tile costs besides its keys -- query
  // rows, first fetches, normalising, storing, the next ticket -- is hidden by nothing, where the 128-row tiles have a
  // second workgroup on the unit (32 to 256 chunks of 128 or 256 tokens: the 128-row tiles are 7-20 % faster with up to
  // 450 keys per row on average, the pipelined ones 5-12 % with 770 to 900).
  if constexpr (!kWaveOnly && kKv == 0) {
    if (a.select != 0) {
      const bool pick_pipe = 10ll * total_cost >= 35ll * total_tiles && 2ll * total_cost >= total_rows;
      if ((a.select == 2) != pick_pipe) return;
    }
  }

  // ---- a launch of few prefill tiles -- one chunk of 512 tokens after 2048 is 128 tiles for 512
  // workgroups, each walking 40 key tiles alone: every tile's key range is cut into `key_split` runs, a workgroup each
  // (TileArgs::tile_split), as many as leaves every part a workgroup of its own and four key tiles by the batch's
  // average (total_cost counts 1024 (query row, key) pairs).
  // Workgroups from `dgrid` on begin with the wave-level work (TileArgs::decode_grid).  A launch whose decode stream
  // is a few tiles -- a decode step or two and a handful of short sequences beside the chunks -- keeps no more
  // workgroups from the prefill tiles than that work has wavefronts for: the stream's wavefronts of min_share_tiles
  // tiles each (they are numbered over the even XCDs first, hence twice as many workgroups) and the wave-level items'.
  // A multiple of 8, the same on every XCD.
  int dgrid = a.decode_grid;
  if constexpr (!kWaveOnly) {
    const int stream_waves = total_tiles > 0 ? total_tiles / max(a.min_share_tiles, 1) + 1 : 0;
    const int wave_wgs = (2 * ((stream_waves + kWgWaves - 1) / kWgWaves) + (total_items + kWgWaves - 1) / kWgWaves + 7) & ~7;
    dgrid = __builtin_amdgcn_readfirstlane(max(dgrid, static_cast<int>(gridDim.x) - wave_wgs));
  }
  int key_split = 1;
  bool tiles_beside_stream = false;  // the parts' states then lie in the upper half of the workspace regions
  if constexpr ((kFew || kPipeTile<D, MRT>) && !kWaveOnly && kKv == 0 && kPass == 0) {
    if (a.tile_split > 1 && total_wg > 0 && a.phase_mode == 4 && shift == 0 &&
        a.tile_ticket_base + total_wg <= static_cast<int>(kQueueCounterIndex) && total_wg < (1 << 24) && a.tile_split <= 7) {
      // With a decode stream in the launch the workgroups from decode_grid on stream first and keep their partial
      // states in the lower half of the workspace (two slots per wavefront): the tiles have decode_grid workgroups to
      // begin with and the upper half for their parts.  That needs the stream on half of the grid at most.
      const int grid = static_cast<int>(gridDim.x);
      tiles_beside_stream = total_tiles > 0;
      const bool room = !tiles_beside_stream ||
                        (grid > dgrid && 2 * kWgWaves * (grid - dgrid) <= a.tile_stream_slots_half);
      // (a stream shorter than the tiles' time, by the weights of the two kernels' pick above: the streaming workgroups
      // come to the queues while parts are left, and every workgroup counts)
      const bool short_stream = 10ll * total_cost >= 35ll * total_tiles;
      const int begin = (tiles_beside_stream && !short_stream) || total_items > 0 ? min(grid, dgrid) : grid;
      const int cap = tiles_beside_stream ? a.tile_parts_cap / 2 : a.tile_parts_cap;
      const long long key_tiles = (static_cast<long long>(total_cost) << 10) / (static_cast<long long>(total_wg) * PC::WGROWS * PC::TK);
      if (room) key_split = min(min(a.tile_split, begin / total_wg), min(static_cast<int>(key_tiles / 4), cap / total_wg));
      key_split = __builtin_amdgcn_readfirstlane(max(key_split, 1));
    }
  }

  // ---- prefill order.  Tiles are drawn from the queues in item order and a tile's cost grows with the number of
  // keys it can see, so the longest sequences go first (as in longest-processing-time-first scheduling: the work left
  // for the end is the short tiles).  wg_start is rebuilt over the sequences that have prefill tiles, by descending
  // length; wg_seq names them.  The data region, not yet in use, holds the temporaries.
  int n_sorted = 0;
  if constexpr (!kWaveOnly) {
    // (With no more tiles than workgroups that begin with tiles every tile starts at once and the order is of no
    // consequence: the sort, two microseconds of a launch that takes thirty, is left out.)
    const int begin_with_tiles = static_cast<int>(gridDim.x) > dgrid && (total_tiles > 0 || total_items > 0)
                                     ? dgrid : static_cast<int>(gridDim.x);
    if (total_wg > begin_with_tiles && shift == 0 && a.phase_mode == 4) {
      // (a thread with one sequence -- every thread of a batch of up to 256 -- has its numbers from the first pass:
      // reading the lengths again is two round trips to memory, two microseconds of a launch of a hundred)
      const bool one = s_end - s_begin <= 1;
      int mine = one ? (my_wg > 0) : 0;
      for (int s = s_begin; s < s_end && !one; ++s) {
        int t, it, wg;
        classify(seq_info<C::TT>(a, s, G), t, it, wg);
        mine += wg > 0;
      }
      int n_pf;
      int at = block_excl_scan(mine, scratch, n_pf);
      n_pf = __builtin_amdgcn_readfirstlane(n_pf);
      if (n_pf <= kSortMax) {
        int* t_seq = reinterpret_cast<int*>(lds_data);
        int* t_key = t_seq + kSortMax;
        int* t_cnt = t_key + kSortMax;
        int* o_cnt = t_cnt + kSortMax;
        // (One word ranks an entry: the length, then the earlier entry first.  Lengths from four million keys on rank
        // alike, which no order of tiles cares about.)
        auto rank_key = [](int kv_len, int entry) { return min(kv_len, (1 << 22) - 1) * 512 + (511 - entry); };
        if (one && my_wg > 0) {
          t_seq[at] = s_begin;
          t_key[at] = rank_key(my_kv_len, at);
          t_cnt[at] = my_wg;
        }
        for (int s = s_begin; s < s_end && !one; ++s) {
          int t, it, wg;
          const SeqInfo si = seq_info<C::TT>(a, s, G);
          classify(si, t, it, wg);
          if (wg > 0) {
            t_seq[at] = s;
            t_key[at] = rank_key(si.kv_len, at);
            t_cnt[at] = wg;
            ++at;
          }
        }
        __syncthreads();
        if (tid < n_pf) {
          const int key = t_key[tid];
          // entries that come before this one: the sign bit of a difference, three vector instructions an entry (as
          // comparisons whose masks meet in scalar registers, 256 sequences took 6.7 us to rank)
          int r = 0;
          for (int t = 0; t < n_pf; ++t) r += static_cast<int>(static_cast<uint32_t>(key - t_key[t]) >> 31);
          wg_seq[r] = t_seq[tid];
          o_cnt[r] = t_cnt[tid];
        }
        __syncthreads();
        int tot;
        const int excl = block_excl_scan(tid < n_pf ? o_cnt[tid] : 0, scratch, tot);
        if (tid < n_pf) wg_start[tid] = excl;
        if (tid == 0) wg_start[n_pf] = tot;
        n_sorted = n_pf;
        __syncthreads();
      }
    }
  }

  // ---- rows past the ragged batch are zero.  A caller with padded static shapes has thousands of them (8192 rows
  // allocated for 256 decode tokens are 65 MB of zeros), so they are written where they cost least: by the workgroups
  // that have nothing else to do when there are such, otherwise by every workgroup after its work, when the
  // workgroups that finish early would idle.
  // The loop reads everything it needs afresh from the kernel arguments (through a pointer the compiler cannot see
  // through), so that placing it after the work keeps no value of the schedule alive across the hot loops.
  auto zero_rows_past_batch = [](int first, int stride) {
    typedef const __attribute__((address_space(4))) TileArgs* KernArgs;
    KernArgs ap = (KernArgs)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(ap));
    RpaParams pp;  // the fields the row arithmetic reads
    pp.num_seqs = ap->p.num_seqs;
    pp.query_start_loc = ap->p.query_start_loc;
    pp.max_num_seqs = ap->p.max_num_seqs;
    pp.total_tokens = ap->p.total_tokens;
    const int total_rows = batch_rows(pp, seq_count(pp));
    const int row_u4 = ap->p.num_q_heads * ap->p.head_dim / 8;  // 16-byte pieces per row
    u32x4_t* o4 = static_cast<u32x4_t*>(ap->p.out);
    for (int row = total_rows + first; row < pp.total_tokens; row += stride)
      for (int k = threadIdx.x; k < row_u4; k += kWgThreads)
        __builtin_nontemporal_store(u32x4_t{0u, 0u, 0u, 0u}, &o4[static_cast<size_t>(row) * row_u4 + k]);
  };

  // A batch without prefill tiles is pure streaming: it runs fastest with one workgroup per compute unit, so
  // the second half of the grid (dispatched after every unit has one workgroup) does not stream.
  const int grid_all = static_cast<int>(gridDim.x);
  // A small batch of decode steps runs one workgroup per (sequence, kv head), see below; such a batch may use the
  // whole grid, the streaming ones stop at stream_grid workgroups.
  bool wg_items_mode = false;
  const int n_heads = nseq * item_heads;
  if constexpr (kWaveOnly && kPass == 0 && kKv == 0 && C::NS == 1 && C::LDS_PER_WAVE >= 16 * D * 4 + 128) {
    // A wavefront walks a quarter of its (sequence, kv head): with few of them the longer ones do better cut into
    // more parts over more wavefronts (one sequence of 1024 keys, 8 kv heads: 20.5 us split over the grid, 22.4
    // in this mode; 32 such sequences: 34.4 against 31.3).
    const int too_long = n_heads >= 32 ? (n_long & 0xffff) : (n_long >> 16);
    wg_items_mode = total_tiles > 0 && total_items == 0 && a.wg_item_tiles > 0 && nseq < 65536 && too_long == 0 && n_heads <= grid_all;
  }
  const int grid_wgs = wg_items_mode ? max(n_heads, min(grid_all, a.stream_grid))
                                     : total_wg == 0 ? min(grid_all, a.stream_grid) : grid_all;
  const bool idle_wgs_exist = grid_wgs < grid_all;
  if (static_cast<int>(blockIdx.x) >= grid_wgs) {
    zero_rows_past_batch(static_cast<int>(blockIdx.x) - grid_wgs, grid_all - grid_wgs);
    return;
  }
  // ---- a small batch of short decode sequences: workgroup b takes (sequence, kv head) number b, a quarter of its
  // tiles per wavefront, and the four partial states meet in LDS.  Split over the grid's wavefronts instead, the
  // parts would go through memory: partial state written through, a ticket, the parts read back -- three round trips
  // of a microsecond or two each, which is most of what such a launch takes.  (The block stands in front of
  // everything the other kinds of work set up -- shares, queues, look-ups: some eight hundred scalar instructions that a
  // wavefront alone on its SIMD takes two microseconds to get through.)
  // Decode steps only: a batch that also holds wave-level items (short chunks, sequences without keys) is split the usual way.
  if constexpr (kWaveOnly && kPass == 0 && kKv == 0 && C::NS == 1 && C::LDS_PER_WAVE >= 16 * D * 4 + 128) {
    if (wg_items_mode) {
      const int b = static_cast<int>(blockIdx.x);
      if (b < n_heads) {
        const int s = b / item_heads, j = b - s * item_heads;
        const SeqInfo si = seq_info<C::TT>(a, s, G);
        if (si.eligible) {
          const int per_head = (si.hi - si.lo_al + C::TT - 1) / C::TT;
          const int per_wave = (per_head + kWgWaves - 1) / kWgWaves;
          Part part;
          part.partial = true;   // (no part of the split through memory: first_w = last_w)
          part.first_w = part.last_w = 0;
          part.in_workgroup = true;
          const int lo = si.lo_al + wave * per_wave * C::TT;
          process_item<DD, NT, kMimic, kWaveOnly, kKv, kPass, kFew>(a, lds_k, si, s, j, 0, lo, min(si.hi, lo + per_wave * C::TT), part);
        }
      }
    }
  }
  if (!wg_items_mode) {
  // Largest s in [0, nseq) with start[s] <= x; sequences that add nothing share their successor's start and
  // are skipped because the search keeps the last one that does not exceed x.
  // `kind` says which count the array sums (0 items, 1 stream tiles, 2 prefill tiles); `base` receives start[s].
  auto find = [&](const int* start, int kind, int x, int& base) {
    int lo = 0, hi = nc;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (start[mid] <= x) lo = mid; else hi = mid;
    }
    lo = __builtin_amdgcn_readfirstlane(lo);
    int s = lo << shift;
    int b = __builtin_amdgcn_readfirstlane(start[lo]);
    if (shift > 0) {
      const int s_last = min(s + K, nseq) - 1;
      for (; s < s_last; ++s) {
        int t, it, wg;
        classify(seq_info<C::TT>(a, s, G), t, it, wg);
        const int cnt = __builtin_amdgcn_readfirstlane(kind == 0 ? it : kind == 1 ? t : wg);
        if (x < b + cnt) break;
        b += cnt;
      }
    }
    base = b;
    return s;
  };

  // Prefill tiles are compute-bound and the decode stream is bandwidth-bound, and one workgroup per compute unit
  // already saturates the memory system.  In a mixed batch the second workgroup of every unit (the upper part of
  // the grid) therefore takes the whole decode stream while the first one starts on the prefill tiles at once;
  // prefill tiles are handed out from queues, so the streaming workgroups join in when the stream is done, and
  // whichever kind of work is longer sets the time.  phase_mode 0..3 keep the static split for experiments.
  const bool queued = total_wg > 0 && a.phase_mode == 4;
  const bool split = queued && grid_all > dgrid;
  const bool do_stream = !split || static_cast<int>(blockIdx.x) >= dgrid;
  const int stream_wg0 = split ? dgrid : 0;
  const int stream_wgs = grid_wgs - stream_wg0;
  const int n_workers = stream_wgs * kWgWaves;
  // Workgroup b runs on XCD b % 8.  The XCDs do not stream from memory at the same rate (on MI355X the odd ones
  // are about a tenth slower), so the wavefronts on even XCDs are numbered first and their region of the stream
  // is made larger; with equal shares the slower XCDs would set the time.
  const bool by_xcd = stream_wgs % 8 == 0 && stream_wg0 % 8 == 0;
  int worker = (static_cast<int>(blockIdx.x) - stream_wg0) * kWgWaves + wave;
  if (by_xcd) {
    const int rel = static_cast<int>(blockIdx.x) - stream_wg0, xcd = rel & 7;
    worker = (xcd & 1) * (n_workers / 2) + (((rel >> 3) * 4 + (xcd >> 1)) * kWgWaves + wave);
  }
  const bool stream_first = total_wg > 0 && (a.phase_mode == 1 ? static_cast<int>(blockIdx.x) >= dgrid
                                            : a.phase_mode == 2 ? (blockIdx.x & 1) != 0
                                            : a.phase_mode == 3 ? ((blockIdx.x >> 3) & 1) != 0
                                            : a.phase_mode == 4);
  // (Without prefill tiles there is one phase, and no loop: out of a loop the compiler hoists every invariant of every
  // kind of work in front of it, some eight hundred scalar instructions that a small launch then waits two
  // microseconds for whatever it holds.)
#pragma unroll 1
  for (int phase = kWaveOnly ? 1 : 0; phase < 2; ++phase) {
    if ((phase == 0) != stream_first) {
      if constexpr (!kWaveOnly) {
      // ---- prefill: one item per (sequence, kv head, tile of WGROWS rows), the row tiles of a (sequence, kv head)
      // adjacent in the item order.  Workgroups are dispatched round-robin over the 8 XCDs, each with its own L2:
      // row tiles that share one K/V stream should run at the same time on the same XCD, so that all but the first
      // of them read it from that L2.
      if (queued) {
        const int total_wg_here = kept_in_place(total_wg) * key_split;  // work items: the tiles, or the parts of the tiles
        // Eight queues, one per XCD: aligned runs of kQueueRun consecutive items go to the queues in turn.  A
        // workgroup draws from the queue of its own XCD until that is empty, then from the others.  Within a
        // (sequence, kv head) the late causal tiles (most keys) come first.  The last workgroup to find every
        // queue empty clears the counters for the next launch.
        // Atomics on one word execute one after the other where the XCDs' memory paths meet, a hundred workgroups
        // asking at the same moment wait tens of microseconds, and a batch of a few tiles is all such moments.  So
        // the workgroups that begin with the prefill tiles own the first tickets of their home queue without asking
        // (workgroup b: ticket b / 8), the counters hand out the tickets after those, and a workgroup that leaves
        // its home queue reads all eight counters at once (plain loads, which do not queue up) and asks only where
        // the count says items are left.
        uint32_t* qctr = a.counters + kQueueCounterIndex;
        const int home = blockIdx.x & 7;
        const int n_first = split && (total_tiles > 0 || total_items > 0) ? dgrid : grid_all;  // begin with tiles
        auto owned = [&](int x) { return n_first > x ? (n_first - x + 7) >> 3 : 0; };    // ... and have home queue x
        // items of queue x: its full runs (run r belongs to queue r % 8) and the partial last run if it is x's
        auto items_of = [&](int x) {
          const int runs = total_wg_here / kQueueRun, rem = total_wg_here - runs * kQueueRun;
          return (runs > x ? (runs - x + 7) >> 3 : 0) * kQueueRun + ((runs & 7) == x ? rem : 0);
        };
        // Few items -- every one the first ticket of a workgroup that begins with the tiles: nobody asks a counter,
        // nothing is left to clear, and a workgroup leaves after its tile (three microseconds of a launch of thirty).
        bool every_item_owned = true;
        for (int x = 0; x < 8; ++x) every_item_owned = every_item_owned && owned(x) >= items_of(x);
        int probe = 0;
        bool first = static_cast<int>(blockIdx.x) < n_first;
        while (true) {
          if (every_item_owned && !first) break;
          // counters of the queues in this workgroup's order, read when the home queue is known to be empty
          uint32_t left = 0;  // bit k: the k-th queue in this workgroup's order has items left by its counter
          if (probe > 0 && wave == 0) {
            const int lane = tid & (kWave - 1);
            const int seen = static_cast<int>(__hip_atomic_load(&qctr[kQueueStride * ((home + (lane & 7)) & 7)], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
#pragma unroll
            for (int k = 0; k < 8; ++k) {
              const int x = (home + k) & 7;
              if (__builtin_amdgcn_readlane(seen, k) + owned(x) < items_of(x)) left |= 1u << k;
            }
          }
          if (tid == 0) {
            int res = -1;
            while (probe < 8) {
              const int x = (home + probe) & 7;
              int t = -1;
              if (first) {
                t = static_cast<int>(blockIdx.x) >> 3;
              } else if (probe == 0 || ((left >> probe) & 1u) != 0) {
                t = owned(x) + static_cast<int>(__hip_atomic_fetch_add(&qctr[kQueueStride * x], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
              }
              first = false;
              if (t >= 0) {
                const int cand = ((t / kQueueRun) * 8 + x) * kQueueRun + t % kQueueRun;
                if (cand < total_wg_here) {
                  res = cand;
                  break;
                }
              }
              ++probe;
            }
            scratch[0] = res;
            scratch[1] = probe;
          }
          first = false;
          __syncthreads();
          const int w = __builtin_amdgcn_readfirstlane(scratch[0]);
          probe = __builtin_amdgcn_readfirstlane(scratch[1]);
          __syncthreads();
          if (w < 0) break;
          const int wt = key_split > 1 ? w / key_split : w, part = w - wt * key_split;  // the tile, and which run of its keys
          int s_base, s;
          if (n_sorted > 0) {
            int lo = 0, hi = n_sorted;
            while (hi - lo > 1) {
              const int mid = (lo + hi) >> 1;
              if (wg_start[mid] <= wt) lo = mid; else hi = mid;
            }
            lo = __builtin_amdgcn_readfirstlane(lo);
            s = __builtin_amdgcn_readfirstlane(wg_seq[lo]);
            s_base = __builtin_amdgcn_readfirstlane(wg_start[lo]);
          } else {
            s = find(wg_start, 2, wt, s_base);
          }
          const SeqInfo si = seq_info<C::TT>(a, s, G);
          const int n_qt = (si.rows + PC::WGROWS - 1) / PC::WGROWS;
          // Order inside a sequence: runs of kQueueRun row tiles of one kv head, the runs with the most keys (the late
          // causal tiles) of every kv head before the next shorter ones.  Head by head instead, the longest tiles of
          // the last head would start when most of the prompt is done and finish alone (a tenth of the time of two
          // 8192-token prompts).
          const int local = wt - s_base;
          const int full = n_qt / kQueueRun, per_round = kQueueRun * p.num_kv_heads;
          int j, member;
          if (local < full * per_round) {
            const int c = local / per_round, rem = local - c * per_round;
            j = rem / kQueueRun;
            member = c * kQueueRun + (rem - j * kQueueRun);
          } else {
            const int rem = local - full * per_round, sz = n_qt - full * kQueueRun;
            j = rem / sz;
            member = full * kQueueRun + (rem - j * sz);
          }
          run_prefill_tile<D, MRT, kMimic, kKv, kPass, kFew && !kWaveOnly>(a, lds_data, si, s, j, n_qt - 1 - member,
                                                       key_split > 1 ? (key_split << 28) | (part << 25) | (tiles_beside_stream ? 1 << 24 : 0) | wt : 0);
        }
        // The last workgroup out clears the counters for the next launch; the exit counts are kept per XCD and
        // then over the XCDs, so that the workgroups of a small batch, which all leave at once, do not queue up on one word.
        if (tid == 0 && !every_item_owned) {
          const uint32_t n_home = (static_cast<uint32_t>(grid_all) - home + 7) >> 3;  // workgroups b with b % 8 == home
          const uint32_t gone = __hip_atomic_fetch_add(&qctr[kQueueXcdExitIndex + kQueueStride * home], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (gone == n_home - 1) {
            const uint32_t n_groups = static_cast<uint32_t>(min(grid_all, 8));
            const uint32_t done = __hip_atomic_fetch_add(&qctr[kQueueExitIndex], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (done == n_groups - 1) {
              for (int i = 0; i < 8; ++i) {
                __hip_atomic_store(&qctr[kQueueStride * i], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&qctr[kQueueXcdExitIndex + kQueueStride * i], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              }
              __hip_atomic_store(&qctr[kQueueExitIndex], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
          }
        }
      } else {
        // Static split: numbering the workgroups XCD by XCD keeps the row tiles of one K/V stream on one XCD; within
        // a (sequence, kv head) the row tiles are rotated by the round in which the group starts, so a workgroup
        // meets early (short) and late (long) causal tiles in turn instead of always the same one.
        const int n_xcd = gridDim.x % 8 == 0 ? 8 : 1;
        const int vwg = (blockIdx.x % n_xcd) * (gridDim.x / n_xcd) + blockIdx.x / n_xcd;
        for (int w = vwg; w < total_wg; w += gridDim.x) {
          int base;
          const int s = find(wg_start, 2, w, base);
          const SeqInfo si = seq_info<C::TT>(a, s, G);
          const int n_qt = (si.rows + PC::WGROWS - 1) / PC::WGROWS;
          const int local = w - base;
          const int j = local / n_qt, member = local - j * n_qt;
          const int round0 = (base + j * n_qt) / static_cast<int>(gridDim.x);
          const int qt = (member + 5 * round0) % n_qt;
          run_prefill_tile<D, MRT, kMimic, kKv, kPass, kFew && !kWaveOnly>(a, lds_data, si, s, j, qt);
        }
      }
      // The wave-private K tiles used from here on overlay the prefill stages: wait until every wavefront of the
      // workgroup has finished reading them.
      __syncthreads();
      }
    } else if (do_stream) {
      const int total_items_here = kept_in_place(total_items), total_tiles_here = kept_in_place(total_tiles);
      const int n_workers_here = kept_in_place(n_workers);
      // ---- sequences with a few row tiles: one item per (sequence, row tile, kv head), strided over the wavefronts
      for (int w = worker; w < total_items_here; w += n_workers_here) {
        int s_base;
        const int s = find(item_start, 0, w, s_base);
        const SeqInfo si = seq_info<C::TT>(a, s, G);
        const int local = w - s_base;
        const int j = local % item_heads, rt = local / item_heads;
        const int row_hi = min(rt * 16 + 16, si.rows);
        const int pos_min = si.kv_len - si.q_len + (rt * 16) / G, pos_max = si.kv_len - si.q_len + (row_hi - 1) / G;
        const int range_hi = min(si.kv_len, pos_max + 1);
        const int range_lo = max(p.sliding_window > 0 ? max(0, pos_min - p.sliding_window + 1) : 0, si.start) & ~(C::TT - 1);
        Part part;
        part.partial = false;
        process_item<DD, NT, kMimic, kWaveOnly, kKv, kPass, kFew>(a, lds_k, si, s, j, rt, range_lo, range_hi, part);
      }

      // ---- decode stream: this wavefront's share [x, x_end) of the tiles, cut at (sequence, kv head) boundaries
      if (total_tiles_here > 0) {
        const int total_tiles = total_tiles_here, n_workers = n_workers_here;  // (the section's own copies, see kept_in_place)
        // Few long sequences are cut into dozens of parts each, and the merge of their partial states by one wavefront
        // is what takes the time.  There the stream is cut by workgroup: a workgroup's part of a (sequence, kv head) is
        // walked by its four wavefronts, a quarter each, and merged in LDS by one of them (in turn), which alone takes
        // part in the split through memory: a quarter of the parts, of the tickets and of what the last one reads.
        // One sequence of 32768 keys 47.3 -> 42.3 us, of 131072 keys 116 -> 108 us, two of 8192 keys 35.5 -> 30.9 us;
        // eight of 4096 keys (16 parts each) would lose, 37.4 -> 39.4 us, and are cut by wavefront.  (In an
        // instantiation of its own, kFew: the loop that serves both cuts costs the large batches registers, 2-4 % of
        // their time; elsewhere unit_waves is the constant 1.)
        int unit_waves = 1;
        if constexpr (kFew && kWaveOnly && kPass == 0 && kKv == 0 && C::NS == 1 && C::LDS_PER_WAVE >= 16 * D * 4 + 128) {
          const float avg = static_cast<float>(total_tiles) / static_cast<float>(max(1, nseq * item_heads));
          const int by_len = max(a.min_share_tiles, min(kMaxMinShareTiles, static_cast<int>(__builtin_sqrtf(avg) * (1.f / 3.f))));
          const int share = max(by_len, total_tiles / n_workers);  // tiles per part, cut by wavefront
          if (a.wg_unit_parts > 0 && avg >= static_cast<float>(a.wg_unit_parts) * static_cast<float>(share)) unit_waves = kWgWaves;
        }
        const int n_units = n_workers / unit_waves, unit = worker / unit_waves;
        Shares sh;
        {
          // Weighted regions when every wavefront gets a few tiles at least.  Small batches use fewer wavefronts
          // instead, kMinShareTiles tiles each: a (sequence, kv head) cut into many one-tile parts would spend its
          // time in the merge, which reads the parts one after the other.
          const int q = total_tiles / n_units, half = n_units / 2;
          // With T tiles per (sequence, kv head) cut into P parts a wavefront streams T / P tiles and the merge reads P
          // parts, a few at a time: the sum is smallest near P = 3 sqrt(T), i.e. sqrt(T) / 3 tiles per part.
          int min_share = a.min_share_tiles;
          if constexpr (kWaveOnly) {
            const float avg = static_cast<float>(total_tiles) / static_cast<float>(max(1, nseq * item_heads));
            min_share = max(min_share, min(kMaxMinShareTiles, static_cast<int>(__builtin_sqrtf(avg) * (1.f / 3.f))));
          }
          min_share *= unit_waves;
          if (q >= min_share) {
            const int rem = total_tiles - q * n_units;
            int first_tiles = half * q + min(half, rem);
            if (by_xcd) first_tiles = static_cast<int>(static_cast<long long>(total_tiles) * a.even_xcd_permille / 1000);
            sh.set(total_tiles, n_units, half, first_tiles);
          } else {
            const int n_active = max(1, total_tiles / min_share);
            sh.set(total_tiles, n_active, n_active, total_tiles);  // one evenly cut region; the other wavefronts get nothing
          }
        }
        int x = sh.begin(unit);
        const int x_end = sh.begin(unit + 1);
        int n_parts = 0;
        while (x < x_end) {
          int s_base;
          const int s = find(tile_start, 1, x, s_base);
          const SeqInfo si = seq_info<C::TT>(a, s, G);
          // A (sequence, kv head) occupies its tiles plus item_pad_tiles empty positions in the stream: what a part
          // costs beyond its tiles (its query rows, the first tile's latency, the hand-off of a partial result) is
          // about that many iterations, and without them a wavefront whose share holds many short (sequence, kv
          // head)s finishes tens of microseconds after the others.
          const int per_head = (si.hi - si.lo_al + C::TT - 1) / C::TT;
          const int per_item = per_head + a.item_pad_tiles;
          const int local = x - s_base;
          const int j = local / per_item, t0 = local - j * per_item;
          const int t1 = min(per_item, t0 + (x_end - x));
          if (t0 >= per_head) {  // only the padding of this (sequence, kv head) is left in the share
            x += t1 - t0;
            continue;
          }
          Part part;
          part.stream_a = x - t0;
          part.sh = sh;
          part.first_w = sh.owner(part.stream_a);
          part.last_w = sh.owner(part.stream_a + per_head - 1);
          part.partial = part.first_w != part.last_w;
          part.slot = part_slot(unit, part.stream_a, sh);
          int lo = t0, hi = min(t1, per_head);
          if constexpr (kFew) {
            if (unit_waves > 1) {
              const int per_wave = (hi - lo + kWgWaves - 1) / kWgWaves;
              lo += wave * per_wave;
              hi = min(hi, lo + per_wave);
              part.in_workgroup = true;
              part.merger = n_parts & (kWgWaves - 1);
              part.again = true;
              ++n_parts;
            }
          }
          process_item<DD, NT, kMimic, kWaveOnly, kKv, kPass, kFew>(a, lds_k, si, s, j, 0, si.lo_al + lo * C::TT, min(si.hi, si.lo_al + hi * C::TT), part);
          x += t1 - t0;
        }
      }
    }
  }
  }  // !wg_items_mode
  if (!idle_wgs_exist) zero_rows_past_batch(static_cast<int>(blockIdx.x), static_cast<int>(gridDim.x));
}

// ----------------------------------------------------------------------------- host side

// Experiment knobs (RPA_TUNE_* environment variables), read once per process on the first launch: a launch costs
// no getenv calls, and a setenv in another host thread cannot race with one.
struct Tune {
  int wgs_per_cu;          // RPA_TUNE_WGS_PER_CU: workgroups of the persistent grid per compute unit (1..kTiledMaxWgsPerCu)
  int decode_wgs_per_cu;   // RPA_TUNE_DECODE_WGS_PER_CU: of these, how many stream a batch without prefill tiles (0 = rule)
  int min_share_tiles;     // RPA_TUNE_MIN_SHARE_TILES
  int item_pad_tiles;      // RPA_TUNE_ITEM_PAD_TILES: empty stream positions per (sequence, kv head)
  int phase_mode;          // RPA_TUNE_PHASE_MODE
  int even_xcd_permille;   // RPA_TUNE_EVEN_XCD_PERMILLE
  int no_mimic;            // RPA_TUNE_NO_MIMIC
  int no_wave_only;        // RPA_TUNE_NO_WAVE_ONLY
  int wave_only_rows;      // RPA_TUNE_WAVE_ONLY_ROWS
  int no_pair64;           // RPA_TUNE_NO_PAIR64: head_dim 64 decodes one kv head per item (experiments)
  int pipe;                // RPA_TUNE_PIPE: 0 = never use the software-pipelined prefill tile (head_dim 128)
  int pipe_stream_wgs;     // RPA_TUNE_PIPE_STREAM_WGS: workgroups (of one per compute unit) that take the decode stream first
  int pipe_min_tokens_per_seq;  // RPA_TUNE_PIPE_MIN_TOKENS_PER_SEQ: average query tokens per sequence from which it is used
  int no_logit_stash;      // RPA_TUNE_NO_LOGIT_STASH: two-launch calls read K in both launches (experiments)
  int device_select;       // RPA_TUNE_DEVICE_SELECT: 0 = never enqueue both tile kernels and let the device pick
  int wg_item_tiles;       // RPA_TUNE_WG_ITEM_TILES: longest (sequence, kv head), in tiles, of a batch that runs one per workgroup
  int tile_split;          // RPA_TUNE_TILE_SPLIT: most runs a prefill tile's key range is cut into when tiles are few
  int wg_unit_parts;       // RPA_TUNE_WG_UNIT_PARTS: parts per (sequence, kv head) from which few sequences are cut by workgroup
};
static const Tune& tune() {
  static const Tune t = [] {
    auto env_int = [](const char* name, int dflt) {
      const char* v = getenv(name);
      return v && *v ? atoi(v) : dflt;
    };
    Tune x;
    x.wgs_per_cu = min(kTiledMaxWgsPerCu, max(1, env_int("RPA_TUNE_WGS_PER_CU", 2)));
    x.decode_wgs_per_cu = max(0, env_int("RPA_TUNE_DECODE_WGS_PER_CU", 0));
    x.min_share_tiles = max(1, env_int("RPA_TUNE_MIN_SHARE_TILES", kMinShareTiles));
    x.item_pad_tiles = min(64, env_int("RPA_TUNE_ITEM_PAD_TILES", -1));  // negative: 128 keys' worth of tiles
    x.phase_mode = env_int("RPA_TUNE_PHASE_MODE", 4);
    x.even_xcd_permille = min(900, env_int("RPA_TUNE_EVEN_XCD_PERMILLE", -1));  // negative: by head_dim, see run_tiled
    x.no_mimic = env_int("RPA_TUNE_NO_MIMIC", 0);
    x.no_wave_only = env_int("RPA_TUNE_NO_WAVE_ONLY", 0);
    x.wave_only_rows = env_int("RPA_TUNE_WAVE_ONLY_ROWS", kWaveOnlyMaxRows);
    x.no_pair64 = env_int("RPA_TUNE_NO_PAIR64", 0);
    x.pipe = env_int("RPA_TUNE_PIPE", 1);
    x.pipe_min_tokens_per_seq = max(1, env_int("RPA_TUNE_PIPE_MIN_TOKENS_PER_SEQ", 128));
    x.pipe_stream_wgs = max(8, env_int("RPA_TUNE_PIPE_STREAM_WGS", 160)) & ~7;
    x.no_logit_stash = env_int("RPA_TUNE_NO_LOGIT_STASH", 0);
    x.device_select = env_int("RPA_TUNE_DEVICE_SELECT", 1);
    x.wg_item_tiles = max(0, env_int("RPA_TUNE_WG_ITEM_TILES", 32));
    x.wg_unit_parts = max(0, env_int("RPA_TUNE_WG_UNIT_PARTS", 32));
    x.tile_split = max(0, env_int("RPA_TUNE_TILE_SPLIT", 4));
    return x;
  }();
  return t;
}

// Workgroups of the persistent grid: two per compute unit (two wavefronts per SIMD, so one wavefront's LDS and
// softmax latency hides behind the other's MFMAs in prefill tiles); the decode stream alone is ~3 % faster with
// one.
static int tiled_grid() { return device_cu_count() * tune().wgs_per_cu; }

bool tiled_supported(const RpaParams& p) {
  if (p.flags & RPA_FLAG_FORCE_GENERIC) return false;
  if (p.dtype != RPA_DTYPE_BF16 || p.compute != RPA_COMPUTE_BF16) return false;
  // 64, 128 and 256 have instantiations of their own width; other multiples of 16 in between run on the next wider one
  if (p.head_dim < 64 || p.head_dim > 256 || p.head_dim % 16 != 0) return false;
  if (p.page_size < 4 || (p.page_size & (p.page_size - 1)) != 0) return false;  // shift/mask page arithmetic
  if (p.max_num_seqs > (kTiledMaxSeqs << kTiledMaxSchedShift)) return false;
  if (static_cast<uint64_t>(p.max_num_seqs) * p.num_kv_heads * 4 > kQueueCounterIndex * 4ull) return false;
  return true;
}

void tiled_workspace_layout(const RpaParams& p, WorkspaceLayout* wl) {
  const uint64_t slots = 2ull * kWgWaves * tiled_grid();  // two partial parts per wavefront at most
  // The ticket region has one size for every shape: a workspace reused across shapes must never hold
  // partial results where another shape keeps its tickets.
  wl->counters_bytes = kWorkspaceTicketBytes;
  wl->partial_o_off = wl->counters_bytes;
  const uint64_t tile_d = p.head_dim <= 128 ? 128 : 256;  // width the kernel works in
  wl->partial_o_bytes = (slots * 16 * tile_d * 4 + 255) & ~static_cast<uint64_t>(255);
  wl->partial_ml_off = wl->partial_o_off + wl->partial_o_bytes;
  wl->partial_ml_bytes = (slots * 16 * 2 * 4 + 255) & ~static_cast<uint64_t>(255);
  wl->total_bytes = wl->partial_ml_off + wl->partial_ml_bytes;
}

// What RaggedPageAttentionConfig.num_queries_per_block (RpaParams::num_queries_per_block) asks for.  The host sees
// padded static shapes only -- total_tokens and max_num_seqs of a serving batch are upper bounds, the lengths live on
// the device -- so a caller that knows its batch names the tile shape here: up to 16 query rows per tile is the
// wave-level loop alone (decode steps, short chunks), up to 128 the 128-row workgroup tiles, more the 256-row
// software-pipelined tiles where they exist (head_dim 128, no soft cap, pages of 16 tokens or more; the 128-row tiles
// otherwise).  0 leaves the choice to the rules below.  RPA_FLAG_* tile flags, when set, come first.
static bool tiles_flagged(const RpaParams& p) { return (p.flags & (RPA_FLAG_PREFILL_TILES | RPA_FLAG_PIPE_TILES)) != 0; }
// +1 the pipelined tile is asked for, -1 it is ruled out, 0 the size rule decides
static int pipe_choice_of(const RpaParams& p) {
  if ((p.flags & RPA_FLAG_PLAIN_TILES) != 0) return -1;
  if ((p.flags & RPA_FLAG_PIPE_TILES) != 0) return 1;
  if (p.num_queries_per_block <= 0) return 0;
  return p.num_queries_per_block > 128 ? 1 : -1;
}

// Small batches -- one query token per sequence by construction, or so few (token, head) rows that prefill tiles
// of 128 rows would leave most of the grid idle -- take the instantiation without prefill tiles: the decode loop
// alone gets a register allocation without spills, and short prefill chunks spread over four times as many
// wavefronts as wave-level items (512 tokens from scratch at 32 heads: 30 us against 65 us with tiles).
static bool wave_only_by_sizes(const RpaParams& p) {
  if (tiles_flagged(p)) return false;
  if (p.num_queries_per_block > 0) return p.num_queries_per_block <= 16;
  return static_cast<int64_t>(p.total_tokens) * p.num_q_heads <= tune().wave_only_rows;
}
static bool small_batch_of(const RpaParams& p) { return p.query_start_loc == nullptr || wave_only_by_sizes(p); }

constexpr uint64_t kLogitStashMaxBytes = 2ull << 30;
static uint32_t logit_pitch_of(const RpaParams& p) {
  const uint64_t cap = static_cast<uint64_t>(p.pages_per_seq > 0 ? p.pages_per_seq : 0) * static_cast<uint64_t>(p.page_size);
  return static_cast<uint32_t>(std::min<uint64_t>((cap + 63) & ~63ull, 1u << 30));
}
uint64_t logit_stash_bytes(const RpaParams& p) {
  // decided by the sizes alone: a size query may come before the pointers are set
  if (tune().no_logit_stash != 0 || p.total_tokens <= 0 || p.num_q_heads <= 0 || !wave_only_by_sizes(p) ||
      (p.flags & RPA_FLAG_NO_LOGIT_STASH) != 0)
    return 0;
  const uint64_t bytes = static_cast<uint64_t>(p.total_tokens) * p.num_q_heads * logit_pitch_of(p) * 4ull;
  return bytes <= kLogitStashMaxBytes ? bytes : 0;
}

template <int D, int NT, int MRT, bool kMimic, bool kWaveOnly = false, int kKv = 0, int kPass = 0, bool kFew = false>
static int launch_cfg(const TileArgs& a, int grid, hipStream_t stream) {
  using C = Cfg<(D < 128 ? 128 : D), NT, kMimic>;
  using PC = PCfg<D, MRT>;
  const size_t data = max(static_cast<size_t>(kWgWaves) * (C::LDS_PER_WAVE + (a.pre.sink_aux != nullptr ? C::SINK_LDS : 0)),
                          static_cast<size_t>(kPipeTile<D, MRT> ? PipeCfg::LDS : PC::LDS));
  const size_t lds = sched_bytes((a.p.max_num_seqs + (1 << a.sched_shift) - 1) >> a.sched_shift) + data;
  // More than 64 KiB of dynamic LDS has to be allowed once per kernel (and device); the call is idempotent.
  static std::atomic<uint64_t> allowed[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
  if (allowed[dev].load(std::memory_order_acquire) < lds) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&rpa_tile_kernel<D, NT, MRT, kMimic, kWaveOnly, kKv, kPass, kFew>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)) != hipSuccess)
      return RPA_ERR_LAUNCH;
    allowed[dev].store(lds, std::memory_order_release);
  }
  hipLaunchKernelGGL((rpa_tile_kernel<D, NT, MRT, kMimic, kWaveOnly, kKv, kPass, kFew>), dim3(grid), dim3(kWgThreads), lds, stream, a);
  return hipGetLastError() == hipSuccess ? RPA_OK : RPA_ERR_LAUNCH;
}

// 8-bit cache (kv_elem 1 = e4m3, 2 = e5m2): the statistics launch, then the attention launch.
template <int D, int NT, int MRT, bool kWaveOnly>
static int launch_two_pass(int kv_elem, const TileArgs& a, int grid, hipStream_t stream) {
  int rc;
  if (kv_elem == 2) {
    rc = launch_cfg<D, NT, MRT, false, kWaveOnly, 2, 1>(a, grid, stream);
    if (rc != RPA_OK) return rc;
    if constexpr (kWaveOnly)
      if (a.logits != nullptr) return launch_cfg<D, NT, MRT, false, kWaveOnly, 2, 3>(a, grid, stream);
    return launch_cfg<D, NT, MRT, false, kWaveOnly, 2, 2>(a, grid, stream);
  }
  rc = launch_cfg<D, NT, MRT, false, kWaveOnly, 1, 1>(a, grid, stream);
  if (rc != RPA_OK) return rc;
  if constexpr (kWaveOnly)
    if (a.logits != nullptr) return launch_cfg<D, NT, MRT, false, kWaveOnly, 1, 3>(a, grid, stream);
  return launch_cfg<D, NT, MRT, false, kWaveOnly, 1, 2>(a, grid, stream);
}

static int launch_tiled_impl(const RpaParams& p, const KvLayout& kv, hipStream_t stream, const PreState& pre, float* stats,
                             int kv_elem = 0, float* logits = nullptr) {
  WorkspaceLayout wl;
  tiled_workspace_layout(p, &wl);
  if (p.workspace == nullptr || p.workspace_bytes < wl.total_bytes) return RPA_ERR_WORKSPACE;
  TileArgs a;
  a.p = p;
  a.kv = kv;
  a.pre = pre;
  a.stats = stats;
  a.logits = nullptr;
  a.logit_pitch = 0;
  a.sched_shift = sched_shift_for(p.max_num_seqs);
  a.min_share_tiles = tune().min_share_tiles;
  // RaggedPageAttentionConfig.num_kv_pages_per_block: the least stretch of a sequence, in pages, that a streaming
  // wavefront takes before a batch is spread over more wavefronts (split-K granularity of small batches)
  if (p.num_kv_pages_per_block > 0) {
    const int64_t keys = static_cast<int64_t>(p.num_kv_pages_per_block) * p.page_size;
    a.min_share_tiles = static_cast<int>(std::min<int64_t>(4096, std::max<int64_t>(1, keys / (p.head_dim > 128 ? 16 : 32))));
  }
  // a part costs about as much as streaming 128 keys: 4 tiles of 32 keys, 8 of 16 (head_dim 256)
  a.item_pad_tiles = tune().item_pad_tiles >= 0 ? tune().item_pad_tiles : (p.head_dim > 128 ? 8 : 4);
  a.page_shift = __builtin_ctz(p.page_size);
  a.uniform_page = p.page_size >= 16;
  a.phase_mode = tune().phase_mode;
  a.pair = 0;
  a.select = 0;
  a.wg_item_tiles = p.num_kv_pages_per_block > 0 ? 0 : tune().wg_item_tiles;  // a caller that names the split gets the split
  a.wg_unit_parts = p.num_kv_pages_per_block > 0 ? 0 : tune().wg_unit_parts;
  {
    // parts of split prefill tiles in the workspace: 64 KiB of accumulators each (128 rows x 128 elements, 256 x 64,
    // 64 x 256) and 8 bytes per row
    WorkspaceLayout wl;
    tiled_workspace_layout(p, &wl);
    const uint64_t rows = p.head_dim <= 64 ? 256 : p.head_dim <= 128 ? 128 : 64;
    a.tile_split = tune().tile_split;
    a.tile_parts_cap = static_cast<int>(std::min<uint64_t>(wl.partial_o_bytes >> 16, wl.partial_ml_bytes / (8 * rows)));
    a.tile_ticket_base = p.max_num_seqs * p.num_kv_heads;
    a.tile_state_o_half = static_cast<uint32_t>((wl.partial_o_bytes / 2) & ~0xffffull);
    a.tile_state_ml_half = static_cast<uint32_t>((wl.partial_ml_bytes / 2) & ~0xffull);
    a.tile_stream_slots_half = kWgWaves * tiled_grid();  // half of the slots of the decode stream's partial states
  }
  // The wavefronts on odd XCDs stream about a tenth slower when all eight compete for memory; per-XCD exit times put the
  // balance at 54.0 % of the stream on the even ones with 256-byte rows and at 54.7 % with 512-byte rows (head_dim 256:
  // even XCDs left at 329 us, odd ones at 338 with 54.0 %; 0.3571 -> 0.3532 ms with 54.7 %).
  a.even_xcd_permille = tune().even_xcd_permille >= 100 ? tune().even_xcd_permille : (p.head_dim > 128 ? 547 : 540);
  // Pure streaming runs fastest with one workgroup per compute unit -- unless a wavefront's loads carry half the
  // bytes (head_dim 64: rows of 128 bytes under 16-byte pieces), when it takes both workgroups to keep as many bytes
  // in flight.
  a.stream_grid = device_cu_count() * (tune().decode_wgs_per_cu > 0 ? tune().decode_wgs_per_cu : p.head_dim == 64 ? 2 : 1);
  a.decode_grid = device_cu_count();
  char* ws = static_cast<char*>(p.workspace);
  a.counters = reinterpret_cast<uint32_t*>(ws);
  a.partial_o = reinterpret_cast<float*>(ws + wl.partial_o_off);
  a.partial_ml = reinterpret_cast<float*>(ws + wl.partial_ml_off);
  const int grid = tiled_grid();
  const bool mimic = (p.flags & RPA_FLAG_FP32_LOGITS) == 0 && tune().no_mimic == 0;
  const bool small_batch = small_batch_of(p);
  // Prefill tiles address one paged cache with a token's K and V rows side by side, [page][slot][combined head][row]
  // (rows may be padded beyond head_dim and tokens beyond 2 * kv heads: the plain tile takes the pitches from the
  // layout; the pipelined tile's instruction stream has the unpadded ones built in); any other layout (two caches, one
  // contiguous cache per sequence) runs through the wave-level loop alone.
  const KvLayout canon = interleaved_layout(p);
  const bool canonical = kv.k_base == canon.k_base && kv.v_base == canon.v_base && kv.stride_b == canon.stride_b &&
                         kv.head_b == canon.head_b && kv.page_b == canon.page_b && kv.contiguous == 0;
  const bool side_by_side = kv.contiguous == 0 && kv.k_base == canon.k_base && kv.v_base > kv.k_base &&
                            static_cast<uint64_t>(kv.v_base - kv.k_base) * 2 == kv.head_b && kv.head_b % 32 == 0 &&
                            kv.stride_b % 16 == 0 && kv.stride_b >= static_cast<uint64_t>(p.num_kv_heads) * kv.head_b &&
                            kv.page_b == static_cast<uint64_t>(p.page_size) * kv.stride_b;
  if (stats != nullptr) {
    // 8-bit cache: row statistics, then the attention with normalised, rounded probabilities.  Batches of decode
    // steps and short chunks run every sequence through the wave-level loop in both launches; a wavefront has half
    // the bytes in flight that it has with a 16-bit cache, so both workgroups of a compute unit stream (0.70 ms
    // against 0.84 ms on 256 x 512..8192 keys).  Batches with long chunks take the instantiation with prefill tiles,
    // as a 16-bit cache does.
    if (!small_batch && side_by_side) {
      if (p.head_dim == 64) return launch_two_pass<64, 2, 4, false>(kv_elem, a, grid, stream);
      if (p.head_dim <= 128) return launch_two_pass<128, 2, 2, false>(kv_elem, a, grid, stream);
      return launch_two_pass<256, 1, 1, false>(kv_elem, a, grid, stream);
    }
    a.stream_grid = device_cu_count() * (tune().decode_wgs_per_cu > 0 ? tune().decode_wgs_per_cu : 2);
    // The statistics launch leaves its logits for the second one, which then reads no K rows: per key, 4 bytes
    // written and 4 read per query head against a K row of head_dim bytes per kv head.
    if (logits != nullptr && logit_stash_bytes(p) != 0) {
      a.logits = logits;
      a.logit_pitch = logit_pitch_of(p);
    }
    return p.head_dim <= 128 ? launch_two_pass<128, 2, 2, true>(kv_elem, a, grid, stream)
                             : launch_two_pass<256, 1, 1, true>(kv_elem, a, grid, stream);
  }
  // A few long chunks and little else -- by the static shapes: 256 tokens or more per max_num_seqs and about as many
  // rows as 256 tiles of 128 at most -- do not fill the device with tiles that each walk their keys alone, and as
  // wave-level items they read K and V once per 16 rows (one chunk of 512 tokens after 2048: 95 us).  They take the
  // 128-row tiles, whose key ranges the device cuts into up to four runs when tiles are few (TileArgs::tile_split):
  // 57 us, 107 against 287 us after 8192 tokens; a chunk with no context at all loses a tenth (32 against 29 us).
  // The same holds for a chunk beside a few decode steps (512 tokens after 8192 with 64 decode steps: 392 us on the
  // wave-level loop, 244 on the tiles): where the rows are few, the token count says that some sequence has hundreds of
  // tokens (224 more tokens than sequences) and the block tables are laid out for long contexts (2048 keys or more --
  // with short ones the wave-level loop is the faster by a tenth or two), the tiles are taken as well.  (Small batches
  // of chunks over heads, lengths and contexts: after up to 1024 keys the two are within a tenth of each other, 16.6
  // against 19.0 us from scratch; after 2048 to 3000 the tiles take 56 us where the wave-level loop takes 73 to 96.)
  const int64_t rows_static = static_cast<int64_t>(p.total_tokens) * p.num_q_heads;
  const bool long_chunks_by_shape = static_cast<int64_t>(p.total_tokens) >= 256ll * p.max_num_seqs ||
                                    (static_cast<int64_t>(p.total_tokens) - p.max_num_seqs >= 224 &&
                                     static_cast<int64_t>(p.pages_per_seq) * p.page_size >= 2048);
  const bool few_long_chunks = p.query_start_loc != nullptr && !tiles_flagged(p) && p.num_queries_per_block <= 0 &&
                               a.tile_split > 1 && tune().no_wave_only == 0 && long_chunks_by_shape &&
                               rows_static <= 32768 + 2048;
  const bool wave_only = pre.ml != nullptr || pre.sink_aux != nullptr || !side_by_side ||
                         (small_batch && !few_long_chunks && tune().no_wave_only == 0);
  if (wave_only) {
    // head_dim 64: two kv heads per item where that keeps a decode token's rows in one 16-row tile
    a.pair = p.head_dim == 64 && p.num_kv_heads % 2 == 0 && 2 * (p.num_q_heads / p.num_kv_heads) <= 16 && pre.ml == nullptr &&
             pre.sink_aux == nullptr && tune().no_pair64 == 0;
    if (a.pair) a.stream_grid = device_cu_count() * (tune().decode_wgs_per_cu > 0 ? tune().decode_wgs_per_cu : 1);
    if (p.head_dim <= 128) {
      // few sequences (what max_num_seqs allows is all the host knows): the instantiation that can also cut the decode
      // stream by workgroup, for the long ones among them
      const int heads = a.pair ? p.num_kv_heads / 2 : p.num_kv_heads;
      if (static_cast<int64_t>(p.max_num_seqs) * heads <= kFewHeads && a.wg_unit_parts > 0)
        return mimic ? launch_cfg<128, 2, 2, true, true, 0, 0, true>(a, grid, stream)
                     : launch_cfg<128, 2, 2, false, true, 0, 0, true>(a, grid, stream);
      return mimic ? launch_cfg<128, 2, 2, true, true>(a, grid, stream) : launch_cfg<128, 2, 2, false, true>(a, grid, stream);
    }
    // head_dim 256: one workgroup per compute unit with the whole register file
    a.stream_grid = device_cu_count();
    return mimic ? launch_cfg<256, 1, 1, true, true>(a, a.stream_grid, stream) : launch_cfg<256, 1, 1, false, true>(a, a.stream_grid, stream);
  }
  // Few rows by the static shapes (about 256 tiles of 128 at most): the instantiations whose tiles' key ranges the device
  // can cut over the idle workgroups (kFew; 128-row tiles).
  const bool cut_kernel = a.tile_split > 1 && static_cast<int64_t>(p.total_tokens) * p.num_q_heads <= 32768 + 2048;
  if (p.head_dim == 64) {
    if (cut_kernel)
      return mimic ? launch_cfg<64, 2, 4, true, false, 0, 0, true>(a, grid, stream) : launch_cfg<64, 2, 4, false, false, 0, 0, true>(a, grid, stream);
    return mimic ? launch_cfg<64, 2, 4, true>(a, grid, stream) : launch_cfg<64, 2, 4, false>(a, grid, stream);
  }
  if (p.head_dim <= 128) {
    // The software-pipelined tile (one workgroup per compute unit) fetches 16 keys per page look-up, has no soft cap
    // and folds a positive logit scale into the exp2 argument.  It pays for batches of long chunks; a batch that mixes
    // chunks with many decode sequences is bound by its decode stream, which needs a streaming workgroup on every
    // compute unit beside the prefill tiles (two workgroups per unit: the plain tile).  The host cannot see the lengths,
    // so it goes by the average number of query tokens per sequence.
    const bool pipe_ok = p.head_dim == 128 && p.page_size >= 16 && p.logits_soft_cap == 0.f &&
                         (mimic || p.softmax_scale * (p.k_scale > 0.f ? p.k_scale : 1.f) * (p.q_scale > 0.f ? p.q_scale : 1.f) > 0.f);
    if (few_long_chunks)
      return mimic ? launch_cfg<128, 2, 2, true, false, 0, 0, true>(a, grid, stream) : launch_cfg<128, 2, 2, false, false, 0, 0, true>(a, grid, stream);
    // (parts of cut 256-row tiles: 128 KiB of accumulators and 2 KiB of row statistics each)
    WorkspaceLayout wl_pipe;
    tiled_workspace_layout(p, &wl_pipe);
    const int pipe_parts_cap = static_cast<int>(std::min<uint64_t>(wl_pipe.partial_o_bytes >> 17, wl_pipe.partial_ml_bytes >> 11));
    const int pipe_choice = pipe_choice_of(p);
    // (block tables for fewer than 1024 keys: no batch in them averages the 512 keys per query row from which the
    // pipelined tiles pay, see the device's pick)
    const bool short_tables = static_cast<int64_t>(p.pages_per_seq) * p.page_size < 1024;
    const bool pipe_wanted = pipe_choice > 0 ||
                             (pipe_choice == 0 && tune().pipe != 0 && !short_tables &&
                              static_cast<int64_t>(p.total_tokens) >= static_cast<int64_t>(tune().pipe_min_tokens_per_seq) * p.max_num_seqs);
    // Neither flag nor hint, and the static shapes do not say "long chunks": the batch may still be one (a serving
    // caller pads total_tokens and max_num_seqs), so both kernels are enqueued and the device picks (TileArgs::select).
    // The launch that is not picked builds the schedule and ends: five microseconds, which a launch of few rows
    // (cut_kernel: every tile starts at once on either kernel) does not get back -- it takes the 128-row tiles
    // (the reference's benchmark shapes of 16 x 16, 16 x 32 and 32 x 16: 32.3 / 39.6 / 32.8 us picked on the device,
    // 29.7 / 36.7 / 26.2 us on the 128-row tiles, 27.3 / 34.7 / 27.9 us on the pipelined ones).
    // (So is a batch of a million rows and more whose shapes say "long chunks": whether they come after long contexts only the
    // device sees, and the unpicked launch is two percent of such a batch at most.)
    if (pipe_choice == 0 && (!pipe_wanted || rows_static >= (1ll << 20)) && !cut_kernel && !short_tables && pipe_ok && canonical &&
        tune().pipe != 0 && tune().device_select != 0) {
      TileArgs b = a;
      a.select = 1;
      int rc = mimic ? launch_cfg<128, 2, 2, true>(a, grid, stream) : launch_cfg<128, 2, 2, false>(a, grid, stream);
      if (rc != RPA_OK) return rc;
      const int g1 = device_cu_count();
      b.select = 2;
      b.tile_parts_cap = pipe_parts_cap;
      b.stream_grid = g1;
      b.decode_grid = max(0, g1 - tune().pipe_stream_wgs);
      return mimic ? launch_cfg<128, 2, 4, true>(b, g1, stream) : launch_cfg<128, 2, 4, false>(b, g1, stream);
    }
    if (pipe_wanted && pipe_ok && canonical) {
      // one workgroup per compute unit; in a mixed batch the last pipe_stream_wgs of them (a multiple of 8: the same
      // number on every XCD) take the decode stream first and join the prefill queues when it is done
      const int g1 = device_cu_count();
      a.tile_parts_cap = pipe_parts_cap;
      a.stream_grid = g1;
      a.decode_grid = max(0, g1 - tune().pipe_stream_wgs);
      return mimic ? launch_cfg<128, 2, 4, true>(a, g1, stream) : launch_cfg<128, 2, 4, false>(a, g1, stream);
    }
    if (cut_kernel)
      return mimic ? launch_cfg<128, 2, 2, true, false, 0, 0, true>(a, grid, stream) : launch_cfg<128, 2, 2, false, false, 0, 0, true>(a, grid, stream);
    return mimic ? launch_cfg<128, 2, 2, true>(a, grid, stream) : launch_cfg<128, 2, 2, false>(a, grid, stream);
  }
  if (cut_kernel)
    return mimic ? launch_cfg<256, 1, 1, true, false, 0, 0, true>(a, grid, stream) : launch_cfg<256, 1, 1, false, false, 0, 0, true>(a, grid, stream);
  return mimic ? launch_cfg<256, 1, 1, true>(a, grid, stream) : launch_cfg<256, 1, 1, false>(a, grid, stream);
}

int launch_tiled(const RpaParams& p, const KvLayout& kv, hipStream_t stream, const PreState& pre) {
  return launch_tiled_impl(p, kv, stream, pre, nullptr);
}
int launch_tiled_fp8(const RpaParams& p, const KvLayout& kv, int kv_elem, float* stats, float* logits, hipStream_t stream) {
  return launch_tiled_impl(p, kv, stream, PreState(), stats, kv_elem, logits);
}

}  // namespace rpa
