// Workgroup-level attention tile for sequences with many rows (prefill chunks).
//
// One workgroup (4 wavefronts) owns WGROWS = 4 * 16 * MRT consecutive rows of one sequence and one
// kv head -- (query token, group head) pairs, so 32 tokens x 4 heads at MRT = 2, G = 4 -- and walks
// the keys those rows can see once.  K and V tiles of TK tokens go from HBM / L2 straight into a
// double-buffered LDS stage with 16-byte direct-to-LDS loads (global_load_lds_dwordx4: no staging
// registers), issued one step ahead.  K rows are stored unpadded with their 16-byte pieces
// XOR-swizzled by the row number (conflict-free ds_read_b128 of the MFMA operand).  The V tile is
// stored by 32-byte column units, the layout the transposing LDS read (ds_read_b64_tr_b16) turns
// into V^T operands directly; at head_dim 256, where a wavefront has 16 rows and the tile is
// LDS-bound, V keeps the row-major layout and is transposed with byte permutes instead.
// Each wavefront computes S^T = K Q^T and O^T += V^T P^T for its own 16 * MRT rows: every K and V
// operand read from LDS feeds MRT MFMAs, Q stays in registers, and each lane owns one row per row
// tile, so the online softmax is lane-local as in the decode loop.  The row sums come from one
// extra MFMA against a vector of ones (they add exactly the bf16 probabilities that enter P V).
// Logits are rounded to bf16 where the reference rounds them (kMimic; _xla_impl_fwd.py:119-124), as in the decode
// loop; the arithmetic of ragged_page_attention_v3 keeps them in fp32.  The K operands of a half are requested one
// half ahead and the barrier that publishes the next tile sits before the last P V of a tile, so
// LDS latency and barrier skew hide behind matrix work.  Halves of a step that lie entirely in a
// wavefront's causal future, left of its window or before the sequence's first visible key are
// skipped.
#pragma once

#include "rpa_tile_common.h"

#ifndef RPA_ROUND_MIN_D
#define RPA_ROUND_MIN_D 64  // smallest head_dim whose prefill tiles round their logits to bf16: all of them (see the key loop)
#endif

namespace rpa {

template <int D, int MRT>
struct PCfg {
  static constexpr int SW = D < 128 ? D : 128;       // width of a slice of head_dim
  static constexpr int NS = D / SW;                  // slices
  static constexpr int CB = SW / 16;                 // MFMA column blocks (16 output elements) per slice
  static constexpr int NKS = D / 32;                 // k-steps of the QK^T contraction
#ifndef RPA_PF_NH
#define RPA_PF_NH 2
#endif
#ifndef RPA_PF_NSTG
#define RPA_PF_NSTG 2
#endif
  static constexpr int NH = D <= 128 ? RPA_PF_NH : 1;  // 32-token halves per step
  static constexpr int TK = 32 * NH;                 // tokens per step
  static constexpr int ROWB = D * 2;                 // LDS bytes per row
  static constexpr int WROWS = 16 * MRT;             // rows per wavefront
  static constexpr int WGROWS = kWgWaves * WROWS;    // rows per workgroup
  static constexpr int TILE_B = TK * ROWB;           // one K (or V) tile: 16 KiB
  static constexpr int NSTG = RPA_PF_NSTG;           // LDS stages: tiles requested ahead of the one in use + 1
  static constexpr int LDS = 2 * NSTG * TILE_B;      // K and V tile per stage
  static constexpr int PR = D / 8;                   // 16-byte pieces per row
  static constexpr int RB = kWave / PR;              // rows one wave-wide load instruction covers
  static constexpr int BLOCKS = TK / RB;             // load instructions per K (or V) tile: 16
  static constexpr int BPW = 2 * BLOCKS / kWgWaves;  // load instructions per wavefront and step
  // V^T operands come from the transposing LDS read (V tile stored by column units) or, where the tile is LDS-bound
  // (16 rows per wavefront at head_dim 256), from 16-byte reads of a row-major tile plus byte permutes: the
  // transposing read moves 8 bytes per lane and takes more LDS time for the same operands.
  static constexpr bool TRV = D <= 128;
  // K rows sit unpadded in LDS with their 16-byte pieces XOR-swizzled by a function of the row number, chosen so
  // that the 16 rows read by one quarter of a wave-wide operand read cover all 64 banks: with 256-byte rows (and
  // longer ones) the row number itself; with 128-byte rows two rows share a bank line, and the row pair number is
  // what has to differ.  The function only depends on the row modulo 16, so sub-tiles are compile-time offsets.
  static __device__ __forceinline__ int swz(int row) { return D == 64 ? (row >> 1) & 7 : row & 15; }
};

constexpr float kLazy = 6.f;  // logits may exceed the softmax reference point by this much before O is rescaled

// kKv / kPass as in the wave-level loop (rpa_decode.h): with an 8-bit cache (kKv 1 = e4m3, 2 = e5m2) the K / V pieces
// of a tile go through registers -- 8 bytes per lane and block, fetched one step ahead like the direct-to-LDS loads of
// the 16-bit cache -- and are widened to bf16 (exactly) on their way into the same LDS layout, so everything after the
// fetch is the 16-bit tile; kPass 1 walks K alone and leaves each row's softmax reference point and its sum of
// exp(logit - point) in TileArgs::stats, kPass 2 forms P = round(exp(logit - point) / sum) in the cache dtype from
// them and accumulates P V with no rescaling.
// kCut: the instantiation that can cut a tile's key range over several workgroups (split_info); it is compiled into
// kernels of their own, for launches of few tiles, because the code that exchanges the runs' states, though it comes
// after the key loop and is seldom run, changes the registers the compiler gives the loop (a third slower on
// every batch in one build, not at all in the next).
template <int D, int MRT, bool kMimic, int kKv = 0, int kPass = 0, bool kCut = false>
__device__ __forceinline__ void prefill_tile(const TileArgs& a, char* __restrict__ lds, const SeqInfo& si, int s, int j,
                                             int qt, int split_info = 0) {
  using C = PCfg<D, MRT>;
  static_assert(kKv == 0 || C::NSTG == 2, "the register stage of an 8-bit cache stands in for one LDS stage ahead");
  static_assert((kKv == 0) == (kPass == 0), "an 8-bit cache runs as two passes, a 16-bit cache as one");
  constexpr uint32_t PB = kKv != 0 ? 8u : 16u;  // bytes of a row piece (eight elements) in the cache
  const RpaParams& p = a.p;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int i = lane & 15, g = lane >> 4;
  const int G = p.num_q_heads / p.num_kv_heads;
  const int W = p.sliding_window;
  const bf16_t* __restrict__ q = static_cast<const bf16_t*>(p.queries);
  bf16_t* __restrict__ out = static_cast<bf16_t*>(p.out);
  const char* kvb = a.kv.k_base;
  // the reference's cap is a weakly typed scalar: it takes the logits' dtype (bf16) before it divides and multiplies
  const float cap = kMimic ? rbf(p.logits_soft_cap) : p.logits_soft_cap;
  const float inv_cap = cap != 0.f ? 1.f / cap : 0.f;
  const int pos0 = si.kv_len - si.q_len;  // position of the sequence's first query token
  // (A head_dim below the instantiation's runs too: q is padded with zeros and the upper part of every K / V row in
  // LDS repeats the lower part -- K: multiplied by zero; V: output elements that are not stored.)
  const int hd = p.head_dim;
  // Pieces (eight elements) of a row that exist in memory: a slot past the last one takes a piece that does exist -- a
  // repeat of the lower ones where their count is a power of two, else the last one.
  const uint32_t npieces = static_cast<uint32_t>(hd / 8);
  const bool pieces_pow2 = (npieces & (npieces - 1)) == 0;
  auto piece_of = [&](uint32_t slot) { return pieces_pow2 ? (slot & (npieces - 1)) : min(slot, npieces - 1); };

  // ---- key range of the workgroup's rows
  const int wg_row_lo = qt * C::WGROWS, wg_row_hi = min(wg_row_lo + C::WGROWS, si.rows);
  const int wg_pos_min = pos0 + wg_row_lo / G, wg_pos_max = pos0 + (wg_row_hi - 1) / G;
  int range_hi = min(si.kv_len, wg_pos_max + 1);
  int range_lo = max(W > 0 ? max(0, wg_pos_min - W + 1) : 0, si.start) & ~(C::TK - 1);
  // A batch of few tiles (TileArgs::tile_split): the key range is cut into `parts` runs of whole key tiles, one
  // workgroup each, whose states meet in the workspace (below).  A run may be empty.
  // split_info (one word, so that one scalar register is what stays alive across the key loop): bits 28..30 the number
  // of runs (0: the range is not cut), 25..27 this workgroup's run, 24 whether the launch also holds a decode stream,
  // 0..23 the tile's number in the launch.
  if (kCut && kPass == 0 && split_info != 0) {
    const int parts = (split_info >> 28) & 7, part = (split_info >> 25) & 7;
    const int n_kt = (max(range_hi - range_lo, 0) + C::TK - 1) / C::TK, per = (n_kt + parts - 1) / parts;
    range_lo = min(range_lo + part * per * C::TK, range_hi);
    range_hi = min(range_hi, range_lo + per * C::TK);
  }
  const int t_last = range_hi - 1;

  // ---- this wavefront's rows: row tile m holds rows w_row_lo + 16 m + i
  const int w_row_lo = wg_row_lo + wave * C::WROWS;
  int pos_n[MRT];
  // Row of the batch and head behind row tile m of this lane.  Needed before and after the key loop, and computed
  // in both places rather than held in registers across it (an opaque zero keeps the compiler from doing so).
  auto row_of = [&](int m, int opaque0, bool& valid, int& head, size_t& q_off) {
    const int R = w_row_lo + 16 * m + i + opaque0;
    valid = R < si.rows;
    const int qi = valid ? R / G : 0;
    head = j * G + (valid ? R - qi * G : 0);
    q_off = (static_cast<size_t>(si.q0 + qi) * p.num_q_heads + head) * hd;
    return qi;
  };
  int t_pos_lo[MRT], t_pos_hi[MRT];  // positions spanned by the valid rows of the row tile (wave-uniform)
  bool t_any[MRT];
  bf16x8_t qreg[MRT][C::NKS];
  const float scale = rbf(p.softmax_scale);
  const float post_scale = logit_scale(p);
  // Without a soft cap the fp32 logit scale is not applied to every logit: maxima and the exp2 argument take it
  // as a factor (it is positive), which costs nothing per key.
  const bool fold_scale = !kMimic && cap == 0.f && post_scale > 0.f;
  const float sf = fold_scale ? post_scale : 1.f, sf_log2e = sf * kLog2e;
#pragma unroll
  for (int m = 0; m < MRT; ++m) {
    bool valid;
    int head;
    size_t q_off;
    const int qi = row_of(m, 0, valid, head, q_off);
    pos_n[m] = valid ? pos0 + qi : -1;
    const int tr_lo = w_row_lo + 16 * m, tr_hi = min(tr_lo + 16, si.rows);
    t_any[m] = tr_hi > tr_lo;
    t_pos_lo[m] = pos0 + tr_lo / G;
    t_pos_hi[m] = pos0 + (max(tr_hi, tr_lo + 1) - 1) / G;
#pragma unroll
    for (int ks = 0; ks < C::NKS; ++ks) {
      u32x4_t raw = {0u, 0u, 0u, 0u};
      if (valid && 32 * ks + 8 * g < hd) raw = *reinterpret_cast<const u32x4_t*>(q + q_off + 32 * ks + 8 * g);
      u32x4_t sc;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float q0 = q_operand<kMimic>(__uint_as_float(raw[e] << 16), p, scale);
        float q1 = q_operand<kMimic>(__uint_as_float(raw[e] & 0xffff0000u), p, scale);
        if constexpr (kKv != 0) {
          if (p.q_scale > 0.f) {
            // q / q_scale in the query dtype, clipped to the cache dtype's range and cast to it (_kernel.py:249-254)
            q0 = fminf(fmaxf(rbf(q0), -fp8_max<kKv>()), fp8_max<kKv>());
            q1 = fminf(fmaxf(rbf(q1), -fp8_max<kKv>()), fp8_max<kKv>());
            round_fp8x2<kKv>(q0, q1);
          }
        }
        sc[e] = pack_bf16x2(q0, q1);
      }
      qreg[m][ks] = __builtin_bit_cast(bf16x8_t, sc);
    }
  }
  // First key of a 32-key half, a0, against per-row-tile thresholds (wave-uniform, fixed for the item):
  //   a0 > act_hi or a0 <= act_lo   the row tile sees none of the half's keys
  //   a0 <= nomask_hi and a0 > nomask_lo   it sees all of them: no per-key mask needed
  int act_hi[MRT], act_lo[MRT], nomask_hi[MRT], nomask_lo[MRT];
#pragma unroll
  for (int m = 0; m < MRT; ++m) {
    act_hi[m] = t_any[m] ? t_pos_hi[m] : -0x7fffffff;
    act_lo[m] = max(W > 0 ? t_pos_lo[m] - W - 31 : -0x7fffffff, si.start - 32);
    nomask_hi[m] = min(t_pos_lo[m] - 31, range_hi - 32);
    nomask_lo[m] = max(W > 0 ? t_pos_hi[m] - W : -0x7fffffff, si.start - 1);
  }
  // One interval test per row tile in the loop: no mask is needed iff clear_lo < a0 <= clear_hi.
  int clear_lo[MRT], clear_hi[MRT];
#pragma unroll
  for (int m = 0; m < MRT; ++m) {
    clear_lo[m] = max(nomask_lo[m], act_lo[m]);
    clear_hi[m] = min(nomask_hi[m], act_hi[m]);
  }
  const int w_pos_hi = pos0 + (min(w_row_lo + C::WROWS, si.rows) - 1) / G;  // < w_pos_lo when the wave has no rows
  const int w_pos_lo = pos0 + w_row_lo / G;
  const bool w_any = w_row_lo < si.rows;
  // Halves that lie entirely in this wavefront's causal future or left of its window are skipped: a half is walked
  // iff w_act_lo < a0 <= w_act_hi.
  const int w_act_hi = w_any ? min(range_hi - 1, w_pos_hi) : -0x7fffffff;
  const int w_act_lo = W > 0 ? w_pos_lo - W - 31 : -0x7fffffff;

  f32x4_t o_acc[MRT][C::NS][C::CB];
  f32x4_t l_acc[MRT];
  // Softmax reference point m per row, kept as the exp2 offset -m log2(e) (0 while the row has seen no key) and
  // as the vote threshold for exp2 arguments: kLazy log2(e) once there is a reference point, -inf before.
  float m_thr[MRT], m_neg[MRT];
  float l32[MRT];    // kPass 1: this lane's part of the row sum, in fp32
  float inv_l[MRT];  // kPass 2: 1 / row sum from the statistics launch
#pragma unroll
  for (int m = 0; m < MRT; ++m) {
    m_thr[m] = -INFINITY;
    m_neg[m] = 0.f;
    l32[m] = 0.f;
    inv_l[m] = 0.f;
    if constexpr (kPass == 2) {
      bool valid;
      int head;
      size_t q_off;
      const int qi = row_of(m, 0, valid, head, q_off);
      if (valid) {
        const size_t idx = static_cast<size_t>(si.q0 + qi) * p.num_q_heads + head;
        const float ms = a.stats[2 * idx], ls = a.stats[2 * idx + 1];
        m_neg[m] = ms == -INFINITY ? 0.f : -ms * kLog2e;
        inv_l[m] = ls > 0.f ? 1.f / ls : 0.f;
      }
    }
    l_acc[m] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
      for (int c = 0; c < C::CB; ++c) o_acc[m][sN][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  // ---- cooperative fetch.  One wave-wide direct-to-LDS load moves a block of RB rows: the LDS side is 1 KiB in
  // lane order, so lane l fills piece slot l % PR of row l / PR and fetches the piece that the swizzle assigns
  // to that slot.  Block-table entries are scalar loads (the rows of a block share a page, except with pages
  // shorter than a block).
  // The cache is [page][slot][combined head][row]: K of kv head j, then its V row, a.kv.head_b bytes per pair; rows
  // may be longer than head_dim and a token may hold more rows than 2 * num_kv_heads (both padded by the caller).
  const uint32_t stride_b = a.kv.stride_b;
  const uint64_t page_b = a.kv.page_b;
  const uint32_t head_off = static_cast<uint32_t>(j) * a.kv.head_b;                   // K row of this kv head inside a token
  const uint32_t v_delta = static_cast<uint32_t>(a.kv.v_base - a.kv.k_base);          // its V row, from the K row
  const const_i32_ptr bt_c = reinterpret_cast<const_i32_ptr>(
      reinterpret_cast<uintptr_t>(p.block_tables + static_cast<size_t>(s) * p.pages_per_seq));
  const int l_row = lane / C::PR, l_slot = lane % C::PR;
  // V blocks are laid out for the transposing operand read instead: [32-byte column unit][row of the block], so the
  // lane that fills LDS bytes [16 l, 16 l + 16) of a block fetches half (l & 1) of unit (l / 2) / RB of row (l / 2) % RB.
  // (Without the transposing read the V tile is laid out like the K tile.)
  // With four rows to a block (256-byte rows) the four 16-lane groups of a transposing read take the same column unit of
  // four consecutive blocks, 1 KiB apart: the same half of the banks, four groups deep where two is the least a
  // 512-byte read takes.  So every second block keeps its units in swapped pairs (unit c at position c ^ 1): odd and even
  // blocks then answer from different halves of the banks.  (With eight rows to a block, 128-byte rows, two groups
  // share a block and the other two the next one: nothing to swap.)
  constexpr bool kSwapUnits = C::TRV && C::RB == 4;
  const int v_row = C::TRV ? (lane >> 1) % C::RB : l_row;
  const uint32_t v_unit = static_cast<uint32_t>((lane >> 1) / C::RB);
  const uint32_t v_src = PB * piece_of(2 * v_unit + (lane & 1));  // byte offset in the row
  const uint32_t v_src_odd = kSwapUnits ? PB * piece_of(2 * (v_unit ^ 1u) + (lane & 1)) : v_src;  // ... in an odd block
  // Wavefront w moves rows [GROUP * w, GROUP * (w + 1)) of the K tile and of the V tile: BPW / 2 blocks each.
  constexpr int HB = C::BPW / 2, GROUP = C::RB * HB;
  uint32_t pre_off[HB];  // per-lane byte offset of K block n inside the group: row part + swizzled piece
#pragma unroll
  for (int n = 0; n < HB; ++n) {
    const int t_local = GROUP * wave + C::RB * n + l_row;
    pre_off[n] = static_cast<uint32_t>(C::RB * n + l_row) * stride_b + PB * piece_of(static_cast<uint32_t>(l_slot ^ C::swz(t_local)));
  }
  const uint32_t v_pre_off = static_cast<uint32_t>(v_row) * stride_b + v_src + v_delta;  // V block 0; block n adds RB rows
  const uint32_t v_pre_off_odd = static_cast<uint32_t>(v_row) * stride_b + v_src_odd + v_delta;
  // (a wavefront's group starts at an even block, so block n of the group is an odd block of the tile iff n is odd)
  static_assert(!kSwapUnits || HB % 2 == 0, "the parity of a block inside its group must be its parity in the tile");
  auto v_src_off = [&](int n) {  // byte offset of this lane's V piece in block n of the group, from the group's first K row
    return C::TRV ? ((n & 1) ? v_pre_off_odd : v_pre_off) + n * C::RB * stride_b : pre_off[n] + v_delta;
  };
  const bool group_in_page = p.page_size >= GROUP;
  // 8-bit cache: this lane's K and V pieces of the tile being fetched, and where they go once widened
  u32x2_t st_k[HB], st_v[HB];
  char* st_dst = lds;
  // One block of a tile: the lane's K piece and V piece, by address or by resource and offset.  16-bit cache: straight
  // into LDS; 8-bit cache: into the register stage.
  auto take = [&](int n, char* dst, const char* k_addr, const char* v_addr) {
    if constexpr (kKv == 0) {
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4_t*>(k_addr), (__attribute__((address_space(3))) void*)(dst + n * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4_t*>(v_addr),
                                       (__attribute__((address_space(3))) void*)(dst + C::TILE_B + n * 1024), 16, 0, 0);
    } else {
      st_k[n] = *reinterpret_cast<const u32x2_t*>(k_addr);
      if constexpr (kPass != 1) st_v[n] = *reinterpret_cast<const u32x2_t*>(v_addr);
    }
  };
  auto fetch_tile = [&](int tile, int buf) {
    const int t_first = tile + GROUP * wave;
    char* dst = lds + 2 * buf * C::TILE_B + HB * wave * 1024;
    if constexpr (kKv != 0) st_dst = dst;
    if (group_in_page && t_first + GROUP - 1 <= t_last) {
      // the whole group lies in one page and inside the range: one block-table entry, one base address
      const int page = min(max(bt_c[t_first >> a.page_shift], 0), p.num_pages - 1);
      const char* sbase = kvb + static_cast<uint64_t>(page) * page_b +
                          static_cast<uint64_t>(t_first & (p.page_size - 1)) * stride_b + head_off;
      // Buffer addressing (scalar base in a resource descriptor, 32-bit per-lane offset): a wavefront is held for
      // about 50 cycles per direct-to-LDS load it issues this way, against about 100 with 64-bit per-lane addresses.
      const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(sbase), 0, 0x7fffffff, 0x00020000);
#pragma unroll
      for (int n = 0; n < HB; ++n) {
        if constexpr (kKv == 0) {
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(dst + n * 1024), 16,
                                                   pre_off[n], 0, 0, 0);
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(dst + C::TILE_B + n * 1024),
                                                   16, v_src_off(n), 0, 0, 0);
        } else {
          st_k[n] = __builtin_amdgcn_raw_buffer_load_b64(rsrc, pre_off[n], 0, 0);
          if constexpr (kPass != 1) st_v[n] = __builtin_amdgcn_raw_buffer_load_b64(rsrc, v_src_off(n), 0, 0);
        }
      }
      return;
    }
    // last tile of the range or small pages: per block, keys past the range repeat the last one (masked)
#pragma unroll
    for (int n = 0; n < HB; ++n) {
      const int t_c = min(t_first + C::RB * n, t_last & ~(C::RB - 1));
      const int t_local = GROUP * wave + C::RB * n + l_row;
      const uint32_t k_piece = PB * piece_of(static_cast<uint32_t>(l_slot ^ C::swz(t_local)));
      const uint32_t v_piece = C::TRV ? ((n & 1) ? v_src_odd : v_src) : k_piece;
      if (C::RB > 4 && p.page_size < C::RB) {
        // pages shorter than a block (pages of 4 tokens under 128-byte rows): every lane looks its own row's page up
        auto row_base = [&](int tok) {
          const int pg = min(max(p.block_tables[static_cast<size_t>(s) * p.pages_per_seq + (tok >> a.page_shift)], 0), p.num_pages - 1);
          return kvb + static_cast<uint64_t>(pg) * page_b + static_cast<uint64_t>(tok & (p.page_size - 1)) * stride_b + head_off;
        };
        take(n, dst, row_base(min(t_c + l_row, t_last)) + k_piece, row_base(min(t_c + v_row, t_last)) + v_piece + v_delta);
        continue;
      }
      const int page = min(max(bt_c[t_c >> a.page_shift], 0), p.num_pages - 1);
      const char* sbase = kvb + static_cast<uint64_t>(page) * page_b +
                          static_cast<uint64_t>(t_c & (p.page_size - 1)) * stride_b + head_off;
      const int tok = min(t_c + l_row, t_last);
      const int v_tok = min(t_c + v_row, t_last);
      take(n, dst, sbase + static_cast<uint32_t>(tok - t_c) * stride_b + k_piece,
           sbase + static_cast<uint32_t>(v_tok - t_c) * stride_b + v_piece + v_delta);
    }
  };
  // Wait until at most `ahead` later tiles of this wave's direct-to-LDS loads are outstanding (they complete in
  // order); the barrier that follows publishes the oldest tile.  s_waitcnt takes an immediate: vmcnt is bits
  // [3:0] and [15:14]; 0x0F70 leaves the other counters unconstrained.
  // 8-bit cache: the staged pieces (the compiler waits for them) are widened and written where the direct-to-LDS
  // loads would have put them: bytes [16 lane, 16 lane + 16) of each 1 KiB block.  The stage they go to held the tile
  // before the current one, which every wavefront left at the last barrier.
  auto wait_fetch = [&](int ahead) {
    if constexpr (kKv != 0) {
#pragma unroll
      for (int n = 0; n < HB; ++n) {
        *reinterpret_cast<u32x4_t*>(st_dst + n * 1024 + lane * 16) = fp8x8_to_bf16x8<kKv>(st_k[n]);
        if constexpr (kPass != 1)
          *reinterpret_cast<u32x4_t*>(st_dst + C::TILE_B + n * 1024 + lane * 16) = fp8x8_to_bf16x8<kKv>(st_v[n]);
      }
      return;
    }
    static_assert(C::BPW * (C::NSTG - 2) <= 24, "extend the immediates below");
    switch (ahead * C::BPW) {
      case 0: __builtin_amdgcn_s_waitcnt(0x0F70); break;
      case 4: __builtin_amdgcn_s_waitcnt(0x0F74); break;
      case 8: __builtin_amdgcn_s_waitcnt(0x0F78); break;
      case 12: __builtin_amdgcn_s_waitcnt(0x0F7C); break;
      case 16: __builtin_amdgcn_s_waitcnt(0x4F70); break;
      default: __builtin_amdgcn_s_waitcnt(0x4F78); break;  // 24
    }
  };

  const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};  // eight bf16 1.0

  // Per-lane byte offsets of the MFMA operand reads inside a stage, fixed for the whole item: the row part of
  // a later sub-tile or half is a compile-time constant on top of them (the swizzle only uses row & 15).
  int k_off[C::NKS];
#pragma unroll
  for (int ks = 0; ks < C::NKS; ++ks) k_off[ks] = i * C::ROWB + 16 * ((4 * ks + g) ^ C::swz(i));
  // V^T operands come from the transposing 64-bit LDS read: in each group of 16 lanes, lanes 4e..4e+3 point at
  // 16 consecutive elements of row e (8 bytes per lane) and lane x receives element x of rows 0..3.  Rows are the
  // four keys 4g..4g+3 of a 16-key sub-tile, the elements one 32-byte column unit; everything else about the
  // address (half, sub-tile, unit) is a compile-time offset.
  const int v_key = 4 * g + (i >> 2);
  const int v_rd = (v_key / C::RB) * 1024 + (v_key % C::RB) * 32 + 8 * (i & 3);
  // swapped units: this lane group's block is odd iff g is (sub-tiles and halves start at even blocks), and unit c of
  // an odd block sits one unit further on for an even c, one back for an odd c
  const int v_rd_swap = kSwapUnits && (g & 1) ? C::RB * 32 : 0;
  // Row-major V tile: lane (i, g) reads piece i (+ 16 per slice) of rows 4g..4g+3 and transposes in registers.
  int v_off[C::NS][4];
#pragma unroll
  for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
    for (int r = 0; r < 4; ++r) v_off[sN][r] = (4 * g + r) * C::ROWB + 16 * ((i + 16 * sN) ^ (4 * g + r));

  if (range_hi > range_lo) {
    const int n_tiles = (range_hi - range_lo + C::TK - 1) / C::TK;
    __syncthreads();  // every wavefront has left the previous item's tiles
    for (int t = 0; t < min(C::NSTG - 1, n_tiles); ++t) fetch_tile(range_lo + t * C::TK, t);
    wait_fetch(min(n_tiles - 1, C::NSTG - 2));
    __syncthreads();  // publishes tile 0
    if (C::NSTG - 1 < n_tiles) fetch_tile(range_lo + (C::NSTG - 1) * C::TK, C::NSTG - 1);
    // The K operands of a half are requested one half ahead, right before the P V MFMAs of the half in progress,
    // so their LDS latency (and the barrier that publishes the next tile) hides behind matrix work.  At head_dim
    // 256 only the first sub-tile's operands are held that long, for lack of registers; the second sub-tile's are
    // requested when the half starts and land while the first sub-tile's MFMAs run.
    constexpr int KAHEAD = D <= 128 ? 2 : 1;
    u32x4_t kop[2][C::NKS];
    auto load_k_sub = [&](const char* kt_n, int h_n, int u) {
#pragma unroll
      for (int ks = 0; ks < C::NKS; ++ks)
        kop[u][ks] = *reinterpret_cast<const u32x4_t*>(kt_n + (32 * h_n + 16 * u) * C::ROWB + k_off[ks]);
    };
    auto load_k = [&](const char* kt_n, int h_n) {
#pragma unroll
      for (int u = 0; u < KAHEAD; ++u) load_k_sub(kt_n, h_n, u);
    };
    load_k(lds, 0);
    for (int kt_i = 0; kt_i < n_tiles; ++kt_i) {
      const int tile = range_lo + kt_i * C::TK;
      const int buf = kt_i % C::NSTG;
      const char* kt = lds + buf * 2 * C::TILE_B;
      const char* vt = kt + C::TILE_B;
#pragma unroll
      for (int h = 0; h < C::NH; ++h) {
        const int a0 = tile + 32 * h;  // first key of this half
        // halves that lie entirely in this wavefront's causal future or left of its window are skipped
        const bool active = a0 > w_act_lo && a0 <= w_act_hi;
        // V of one slice: with the transposing read, per column unit c the keys 4g..4g+3 of the two sub-tiles (one
        // A operand); otherwise eight 16-byte pieces (rows 4g..4g+3 of the two sub-tiles, piece i)
        u32x4_t vraw[8];
        auto load_v = [&](int sN) {
          if constexpr (C::TRV) {
#pragma unroll
            for (int c = 0; c < C::CB; ++c)
#pragma unroll
              for (int u = 0; u < 2; ++u) {
                const s16x4_t t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(
                    vt + v_rd + ((c & 1) ? -v_rd_swap : v_rd_swap) + ((32 * h + 16 * u) / C::RB) * 1024 + (c + C::CB * sN) * (C::RB * 32)));
                const u32x2_t t2 = __builtin_bit_cast(u32x2_t, t);
                vraw[c][2 * u] = t2[0];
                vraw[c][2 * u + 1] = t2[1];
              }
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              vraw[e] = *reinterpret_cast<const u32x4_t*>(vt + (32 * h + 16 * (e >> 2)) * C::ROWB + v_off[sN][e & 3]);
          }
        };
        constexpr int V_READS = C::TRV ? 2 * C::CB : 8;
        u32x4_t pw[MRT];
        if (active) {
        // S^T = K Q^T for the two 16-key sub-tiles, then the V operands of the first slice are requested: they
        // land during the softmax.  The group barriers pin that order.
        f32x4_t s_acc[MRT][2];
        if constexpr (KAHEAD == 1) {
          load_k_sub(kt, h, 1);
          __builtin_amdgcn_sched_group_barrier(0x100, C::NKS, 0);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
          for (int m = 0; m < MRT; ++m) s_acc[m][u] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < C::NKS; ++ks)
#pragma unroll
            for (int m = 0; m < MRT; ++m)
              s_acc[m][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kop[u][ks]), qreg[m][ks],
                                                                    s_acc[m][u], 0, 0, 0);
        }
        if constexpr (kPass != 1) {
          load_v(0);
          // the V reads issue between the QK MFMAs, in the shadow of the matrix pipe, not after them
          constexpr int N_MFMA = 2 * C::NKS * MRT, PER_READ = N_MFMA / V_READS;
          static_assert(PER_READ >= 1 && PER_READ * V_READS == N_MFMA, "MFMAs per V read");
#pragma unroll
          for (int r = 0; r < V_READS; ++r) {
            __builtin_amdgcn_sched_group_barrier(0x008, PER_READ, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        // online softmax per row tile; this lane: row i of the tile, keys a0 + 16u + 4g + r
#pragma unroll
        for (int m = 0; m < MRT; ++m) {
          float sv[2][4];
#pragma unroll
          for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int r = 0; r < 4; ++r) sv[u][r] = s_acc[m][u][r];
          if (!kMimic && !fold_scale) {  // wave-uniform: only with a soft cap (or a non-positive scale)
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
              for (int r = 0; r < 4; ++r) sv[u][r] *= post_scale;
          }
          if (cap != 0.f) {
            asm volatile("" : "+v"(sv[0][0]));  // keeps the soft cap inside this wave-uniform branch (it is not cheap)
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
              for (int r = 0; r < 4; r += 2) {  // the cap's own bf16 roundings make it sensitive to its input: round that too
                if (kMimic) rbf2(sv[u][r], sv[u][r + 1]);
                soft_cap2<kMimic>(sv[u][r], sv[u][r + 1], cap, inv_cap);
              }
          }
          else if (kMimic && D >= RPA_ROUND_MIN_D) {
            // the reference's logits are bf16 (_xla_impl_fwd.py:119-124): round them, two per conversion (at head_dim 64,
            // whose tiles are bound by vector instructions, that is 13 % of the time; a build with -DRPA_ROUND_MIN_D=128
            // keeps fp32 logits there and lands up to three bf16 steps from the reference on rows of a few keys)
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
              for (int r = 0; r < 4; r += 2) {
                const uint32_t pk = pack_bf16x2(sv[u][r], sv[u][r + 1]);
                sv[u][r] = __uint_as_float(pk << 16);
                sv[u][r + 1] = __uint_as_float(pk & 0xffff0000u);
              }
          }
          // a row tile that sees none of these keys goes through the mask with every key dropped: P = 0
          const bool need_mask = a0 <= clear_lo[m] || a0 > clear_hi[m];
          if (need_mask) {
            int tok0 = a0 + 4 * g;
            asm volatile("" : "+v"(tok0));  // keeps the per-key compares inside this (rare) branch
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const int tok = tok0 + 16 * u + r;
                const bool keep = tok <= pos_n[m] && tok < range_hi && (W <= 0 || tok > pos_n[m] - W) && tok >= si.start;
                sv[u][r] = keep ? sv[u][r] : -INFINITY;
              }
          }
          // exp2 arguments against the current reference point: t = (logit - m) log2(e), with m = 0 while the row has
          // seen no key.  They are arithmetic results, so their maximum needs no canonicalising self-maxima and
          // compiles to three-operand maxima.
          float t[2][4];
#pragma unroll
          for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int r = 0; r < 4; ++r) t[u][r] = fmaf(sv[u][r], sf_log2e, m_neg[m]);
          float tmax = fmaxf(fmaxf(fmaxf(t[0][0], t[0][1]), fmaxf(t[0][2], t[0][3])),
                             fmaxf(fmaxf(t[1][0], t[1][1]), fmaxf(t[1][2], t[1][3])));
          // Lazy rescale: the reference point (the same in the four lanes of a row) only moves when some logit
          // exceeds it by more than kLazy; probabilities then stay below e^kLazy, far inside bf16 / fp32 range.
          // The common case needs no cross-lane step at all: a wave-wide vote on the lane-local maxima, and the t
          // are the exp2 arguments as they stand.  When the point moves up by the row maximum, so do the t.
          if constexpr (kPass == 2) {
            // the reference point and the row sum are fixed: normalised probabilities, rounded to the cache dtype
            // (exactly representable in bf16, which is how they enter P V)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
              float e0 = __builtin_amdgcn_exp2f(t[u][0]) * inv_l[m], e1 = __builtin_amdgcn_exp2f(t[u][1]) * inv_l[m];
              float e2 = __builtin_amdgcn_exp2f(t[u][2]) * inv_l[m], e3 = __builtin_amdgcn_exp2f(t[u][3]) * inv_l[m];
              round_fp8x2<kKv>(e0, e1);
              round_fp8x2<kKv>(e2, e3);
              pw[m][2 * u] = pack_bf16x2(e0, e1);
              pw[m][2 * u + 1] = pack_bf16x2(e2, e3);
            }
            continue;
          }
          if (__builtin_expect(__any(tmax > m_thr[m]), 0)) {
            tmax = row_groups_max(tmax);
            const bool bump = tmax > m_thr[m];  // then tmax is finite
            const float shift = bump ? tmax : 0.f;
            const float alpha = !bump ? 1.f : m_thr[m] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(-tmax);
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
              for (int r = 0; r < 4; ++r) t[u][r] -= shift;
            m_neg[m] -= shift;
            m_thr[m] = bump ? kLazy * kLog2e : m_thr[m];
            if constexpr (kPass == 1) {
              l32[m] *= alpha;
            } else {
              l_acc[m] *= alpha;
#pragma unroll
              for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
                for (int c = 0; c < C::CB; ++c) o_acc[m][sN][c] *= alpha;
            }
          }
          if constexpr (kPass == 1) {
            // statistics only: the sum of the unrounded exponentials, in fp32
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
              for (int r = 0; r < 4; ++r) l32[m] += __builtin_amdgcn_exp2f(t[u][r]);
            continue;
          }
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const float e0 = __builtin_amdgcn_exp2f(t[u][0]), e1 = __builtin_amdgcn_exp2f(t[u][1]);
            const float e2 = __builtin_amdgcn_exp2f(t[u][2]), e3 = __builtin_amdgcn_exp2f(t[u][3]);
            pw[m][2 * u] = pack_bf16x2(e0, e1);
            pw[m][2 * u + 1] = pack_bf16x2(e2, e3);
          }
          l_acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ones),
                                                            __builtin_bit_cast(bf16x8_t, pw[m]), l_acc[m], 0, 0, 0);
        }
        }  // active
        __builtin_amdgcn_sched_barrier(0);
        // ---- K operands of the next half.  At the end of a tile the next one is published first: this wavefront's
        // own part of it has landed (wait_fetch), and after the barrier so has everybody's; the stage of the current
        // tile is refilled right away, so every wavefront must hold its last V operands of that tile in registers
        // by then.  With one slice (head_dim 128) that is the case before the P V MFMAs, which then hide the LDS
        // latency and the barrier; with two slices the second slice's V operands are only read during P V, and the
        // step comes after it.
        auto next_k = [&]() {
          if (h + 1 < C::NH) {
            load_k(kt, h + 1);
          } else if (kt_i + 1 < n_tiles) {
            wait_fetch(min(n_tiles - 2 - kt_i, C::NSTG - 2));
            __syncthreads();
            if (kt_i + C::NSTG < n_tiles) fetch_tile(tile + C::NSTG * C::TK, buf);
            load_k(lds + ((kt_i + 1) % C::NSTG) * 2 * C::TILE_B, 0);
          }
        };
        if constexpr (C::NS == 1) next_k();
        __builtin_amdgcn_sched_barrier(0);
        // O^T += V^T P^T: one A operand per MFMA column block c, used by every row tile
        if (kPass != 1 && active) {
#pragma unroll
          for (int sN = 0; sN < C::NS; ++sN) {
            if (sN > 0) load_v(sN);
#pragma unroll
            for (int c = 0; c < C::CB; ++c) {
              u32x4_t av;
              if constexpr (C::TRV) {
                av = vraw[c];
              } else {
                const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
                for (int hh = 0; hh < 4; ++hh)
                  av[hh] = __builtin_amdgcn_perm(vraw[2 * hh + 1][c >> 1], vraw[2 * hh][c >> 1], sel);
              }
#pragma unroll
              for (int m = 0; m < MRT; ++m)
                o_acc[m][sN][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    __builtin_bit_cast(bf16x8_t, av), __builtin_bit_cast(bf16x8_t, pw[m]), o_acc[m][sN][c], 0, 0, 0);
            }
            if constexpr (!C::TRV) {
              if (sN > 0) __builtin_amdgcn_sched_group_barrier(0x100, 8, 1);
#pragma unroll
              for (int c = 0; c < 8; ++c) {
                __builtin_amdgcn_sched_group_barrier(0x002, 4, 1);    // four byte permutes build one A operand
                __builtin_amdgcn_sched_group_barrier(0x008, MRT, 1);  // its MFMAs
              }
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        if constexpr (C::NS > 1) next_k();
      }
    }
  }

  // ---- a part of a split key range: the state of every row -- reference point, sum, unnormalised output -- goes to
  // the workspace as it sits in registers (accumulator c of row tile m and slice sN of this wavefront: 1 KiB in lane
  // order), the workgroup takes a ticket of its tile, and the one that draws the last ticket adds the parts up in
  // part order (its own included, so the result does not depend on who comes last) and goes on to normalise and
  // store.  Written and read at agent scope like the partial states of the decode stream.
  float m_merged[MRT], l_merged[MRT];
  if constexpr (kCut && kPass == 0) {
    if (split_info != 0) {
      const int parts = (split_info >> 28) & 7, part = (split_info >> 25) & 7;
      int tile_id = split_info & 0xffffff;
      const bool upper = ((split_info >> 24) & 1) != 0;
      // (fresh names for the rows' state: what this seldom-run block does with it should not shape the registers it
      // has in the key loop -- it still does, from one build to the next, which is why the block has instantiations
      // of its own)
#pragma unroll
      for (int m = 0; m < MRT; ++m)
#pragma unroll
        for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
          for (int c = 0; c < C::CB; ++c) asm volatile("" : "+v"(o_acc[m][sN][c]));
#pragma unroll
      for (int m = 0; m < MRT; ++m) {
        asm volatile("" : "+v"(l_acc[m]));
        asm volatile("" : "+v"(m_thr[m]), "+v"(m_neg[m]));
      }
      constexpr int kAgentScope = 16;
      constexpr uint32_t kWaveState = MRT * C::NS * C::CB * 1024, kPartState = kWgWaves * kWaveState;  // bytes
      // (a launch that also holds a decode stream keeps that stream's partial states in the lower half of both
      // regions; the tiles' parts then take the upper half)
      const TileArgs* ap = &a;
      const __amdgpu_buffer_rsrc_t o_rsrc = __builtin_amdgcn_make_buffer_rsrc(
          reinterpret_cast<char*>(ap->partial_o) + (upper ? ap->tile_state_o_half : 0u), 0, 0x7fffffff, 0x00020000);
      float2* ml = reinterpret_cast<float2*>(reinterpret_cast<char*>(ap->partial_ml) + (upper ? ap->tile_state_ml_half : 0u));
      uint32_t* const ticket_words = ap->counters + ap->tile_ticket_base;
      const uint32_t my_part = static_cast<uint32_t>(tile_id * parts + part);
      auto state_off = [&](uint32_t pt, int m, int sN, int c) {
        return static_cast<int>(pt * kPartState + wave * kWaveState + ((m * C::NS + sN) * C::CB + c) * 1024 + lane * 16);
      };
#pragma unroll
      for (int m = 0; m < MRT; ++m) {
#pragma unroll
        for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
          for (int c = 0; c < C::CB; ++c)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, o_acc[m][sN][c]), o_rsrc, state_off(my_part, m, sN, c), 0, kAgentScope);
        if (g == 0) {
          const float m_row = m_thr[m] == -INFINITY ? -INFINITY : -m_neg[m] * (1.f / kLog2e);
          const uint64_t v = static_cast<uint64_t>(__float_as_uint(m_row)) | (static_cast<uint64_t>(__float_as_uint(l_acc[m][0])) << 32);
          __hip_atomic_store(reinterpret_cast<uint64_t*>(ml) + (my_part * kWgWaves + wave) * (16 * MRT) + 16 * m + i, v,
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();  // every wavefront's state has left (and every wavefront is out of the key loop's LDS)
      uint32_t* ctr = ticket_words + tile_id;
      int* flag = reinterpret_cast<int*>(lds);
      if (threadIdx.x == 0)
        *flag = static_cast<int>(__hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
      __syncthreads();
      const int ticket = *flag;
      __syncthreads();  // (the flag's word belongs to the next tile's stage from here on)
      if (ticket != parts - 1) return;
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll
      for (int m = 0; m < MRT; ++m) {
        float M = -INFINITY, L = 0.f;
#pragma unroll
        for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
          for (int c = 0; c < C::CB; ++c) o_acc[m][sN][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        for (int pt = 0; pt < parts; ++pt) {
          const uint32_t src = static_cast<uint32_t>(tile_id * parts + pt);
          const uint64_t v = __hip_atomic_load(reinterpret_cast<const uint64_t*>(ml) + (src * kWgWaves + wave) * (16 * MRT) + 16 * m + i,
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          const float mk = __uint_as_float(static_cast<uint32_t>(v)), lk = __uint_as_float(static_cast<uint32_t>(v >> 32));
          const float m_new = fmaxf(M, mk);
          const float m_use = m_new == -INFINITY ? 0.f : m_new;
          const float keep = __builtin_amdgcn_exp2f((M - m_use) * kLog2e);
          const float w = __builtin_amdgcn_exp2f((mk - m_use) * kLog2e);
          L = L * keep + w * lk;
          M = m_new;
#pragma unroll
          for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
            for (int c = 0; c < C::CB; ++c) {
              const u32x4_t ov = __builtin_amdgcn_raw_buffer_load_b128(o_rsrc, state_off(src, m, sN, c), 0, kAgentScope);
              o_acc[m][sN][c] = o_acc[m][sN][c] * keep + w * __builtin_bit_cast(f32x4_t, ov);
            }
        }
        m_merged[m] = M;
        l_merged[m] = L;
      }
      if (threadIdx.x == 0) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }

  // ---- normalise (with optional sinks) and store
#pragma unroll
  for (int m = 0; m < MRT; ++m) {
    bool valid;
    int head;
    size_t q_off;
    int opaque0 = 0;
    asm volatile("" : "+v"(opaque0));
    row_of(m, opaque0, valid, head, q_off);
    const float l_row1 = kPass == 1 ? row_groups_sum(l32[m]) : 0.f;  // the four lanes of a row, every lane taking part
    if (!valid) continue;
    const float m_row = kCut && kPass == 0 && split_info != 0 ? m_merged[m] : m_thr[m] == -INFINITY ? -INFINITY : -m_neg[m] * (1.f / kLog2e);
    if constexpr (kPass == 1) {
      if (g == 0) {
        float* st = a.stats + 2 * (q_off / hd);  // q_off = ((q0 + qi) * num_q_heads + head) * head_dim
        st[0] = m_row;
        st[1] = l_row1;
      }
      continue;
    }
    const float l_run = kCut && kPass == 0 && split_info != 0 ? l_merged[m] : l_acc[m][0];
    float num_scale = 1.f, denom = l_run;
    if (p.sinks != nullptr && p.num_sinks > 0) {
      const float* __restrict__ sk = p.sinks + static_cast<size_t>(head) * p.num_sinks;
      float smax = -INFINITY;
      for (int k = 0; k < p.num_sinks; ++k) smax = fmaxf(smax, sk[k]);
      const float mt = fmaxf(m_row, smax);
      float ssum = 0.f;
      for (int k = 0; k < p.num_sinks; ++k) ssum += expf(sk[k] - mt);
      num_scale = m_row == -INFINITY ? 0.f : expf(m_row - mt);
      denom = num_scale * l_run + ssum;
    }
    const float inv = kPass == 2 ? out_scale(p) : num_scale * out_scale(p) / fmaxf(denom, 1e-6f);
    bf16_t* orow = out + q_off;
    if constexpr (C::TRV) {
      // MFMA c of a slice holds head_dim elements 16 c + 4 g + r of this lane's row
#pragma unroll
      for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
        for (int c = 0; c < C::CB; ++c) {
          u32x2_t w;
          w[0] = pack_bf16x2(o_acc[m][sN][c][0] * inv, o_acc[m][sN][c][1] * inv);
          w[1] = pack_bf16x2(o_acc[m][sN][c][2] * inv, o_acc[m][sN][c][3] * inv);
          if (128 * sN + 16 * c < hd) *reinterpret_cast<u32x2_t*>(orow + 128 * sN + 16 * c + 4 * g) = w;
        }
    } else {
      // MFMA c of a slice holds head_dim elements 8 (4 g + r) + c of this lane's row
#pragma unroll
      for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          u32x4_t w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = pack_bf16x2(o_acc[m][sN][2 * e][r] * inv, o_acc[m][sN][2 * e + 1][r] * inv);
          if (128 * sN + 32 * g + 8 * r < hd) *reinterpret_cast<u32x4_t*>(orow + 128 * sN + 32 * g + 8 * r) = w;
        }
    }
  }
}

}  // namespace rpa
