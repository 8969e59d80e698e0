// Workgroup-level attention tile for large prefill batches at head_dim 128: one wavefront per SIMD, software-pipelined.
//
// One workgroup (4 wavefronts, the only one on its compute unit: up to 512 registers per lane) owns 256 consecutive
// rows of one (sequence, kv head) -- 64 rows = 4 MFMA row tiles per wavefront, so every K / V operand read from LDS
// feeds four MFMAs -- and walks the keys those rows can see in tiles of 64, fetched into LDS stages as in
// rpa_prefill.h (same layouts: K rows swizzled, V by 32-byte column units for the transposing read).
//
// With one wavefront per SIMD nothing but the wavefront's own instruction order overlaps matrix and vector work, so the
// loop is written as that order.  Per 32-key half h the work is
//     QK(h)   S^T = K Q^T                                   32 MFMAs
//     SM1(h)  exp2 arguments t = s c - m c and their maxima  vector
//     SM2(h)  P = exp2(t) rounded to bf16                    vector
//     PV(h)   row sums and O^T += V^T P^T                    36 MFMAs
// and the stream runs  [QK(h+1) | SM1(h)]  [SM2(h) | PV(h)]: the matrix pipe works on the next half's logits while
// the vector unit prepares this half's softmax, then on this half's P V while the vector unit exponentiates, one row
// tile ahead.  Each "|" is an explicit interleave -- one MFMA, a few vector instructions, fenced by scheduling
// barriers -- because the compiler's own order keeps the two kinds apart.  Both phases are bound by the matrix pipe
// when the interleave holds (512 and 576 cycles of MFMA against about 400 and 460 cycles of vector issue).
// LDS operands are requested one phase ahead (V of half h at the start of [QK|SM1], K of half h+2 at the start of
// [SM2|PV]); the tile that a half needs is published by one barrier per tile, placed between the two phases of a
// tile's first half, and the stage freed by it is refilled at once, NSTG - 1 tiles ahead of its use.
//
// Halves that need per-key masks (causal diagonal, window edge, end of the range, first visible key) or a soft cap
// run the same stream with those steps added (`kGeneral`).  A wavefront stops computing after the last half its rows
// can see and keeps taking part in fetches and barriers; halves left of a wavefront's window but inside the
// workgroup's range are walked with every key masked.
#pragma once

#include <type_traits>

#include "rpa_prefill.h"

namespace rpa {

#ifndef RPA_PP_NSTG
#define RPA_PP_NSTG 4
#endif
#ifndef RPA_PP_ROUND
#define RPA_PP_ROUND 1
#endif

struct PipeCfg {
  static constexpr int D = 128;
  static constexpr int NRG = 2;                     // groups of 32 rows per wavefront (one 32x32 MFMA tile each)
  static constexpr int NKS = D / 16;                // k-steps of the QK^T contraction
  static constexpr int NBLK = D / 32;               // blocks of 32 output elements
  static constexpr int TK = 64;                     // keys per tile (two halves of 32)
  static constexpr int ROWB = D * 2;                // LDS bytes per K row
  static constexpr int WROWS = 32 * NRG;            // rows per wavefront
  static constexpr int WGROWS = kWgWaves * WROWS;   // rows per workgroup: 256
  static constexpr int TILE_B = TK * ROWB;          // one K (or V) tile: 16 KiB
  static constexpr int NSTG = RPA_PP_NSTG;          // LDS stages
  static constexpr int LDS = 2 * NSTG * TILE_B;
  static constexpr int PR = D / 8;                  // 16-byte pieces per row
  static constexpr int RB = kWave / PR;             // rows one wave-wide load covers: 4
  static constexpr int HB = TK / RB / kWgWaves;     // K (and V) load instructions per wavefront and tile: 4
  static constexpr int GROUP = RB * HB;             // rows of the K and of the V tile a wavefront moves: 16
  static constexpr int LOADS = 2 * HB;              // load instructions per wavefront and tile
  // Logits are rounded to bf16 before the softmax where the reference rounds them (_xla_impl_fwd.py:119-124).
  static constexpr bool ROUND = RPA_PP_ROUND != 0;
  static __device__ __forceinline__ int swz(int row) { return row & 15; }
};


typedef __attribute__((ext_vector_type(32))) float f32x32_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;
typedef __attribute__((ext_vector_type(8))) int i32x8_t;

#include "rpa_prefill_pipe_asm.inc"

// What the key loop takes and leaves, each member bound to the registers the instruction stream uses for it
// (register map in gen_prefill_pipe_asm.py).
struct PipeIo {
  f32x32_t o0, o1, o2, o3;  // out: O^T accumulators, row group 0 blocks 0-1, 2-3, row group 1 blocks 0-1, 2-3
  f32x2_t lsum;             // out: row sums of the lane's keys per row group ([0], [1])
  f32x2_t mneg, mthr;       // out: exp2 offset and threshold per row group ([0], [1])
  f32x32_t q0, q1;          // in: Q operands of row group 0, 1
  i32x4_t mspan, rowlo;     // in: per-lane bounds of the visible keys per row group ([0], [1])
  i32x4_t kbase0, kbase1;   // in: LDS addresses of the K operand reads per k-step
  i32x4_t kpiece;           // in: fetch: piece offsets in a K row
  i32x4_t misc;             // in: LDS address of the V^T reads, fetch: row in a K block, in a V block, V piece offset
  float cfac;               // in: factor of the exp2 argument
  i32x8_t s0, s1;           // in: scalars (see the register map)
#ifdef RPA_PP_PROF
  i32x8_t prof;
#endif
};

// Experiment builds (-DRPA_PP_PROF, with an .inc file generated under RPA_PPA_PROF=1): cycle counts of the loop's regions.
#ifdef RPA_PP_PROF
#define RPA_PPA_PROF_OUT , "={s[76:83]}"(R.prof)
#define RPA_PPA_PROF_CLOBBERS , "s84", "s85", "s86", "s87", "s88"
#else
#define RPA_PPA_PROF_OUT
#define RPA_PPA_PROF_CLOBBERS
#endif

#define RPA_PPA_CLOBBERS \
  "v0", "v1", "v2", "v3", "v4", "v5", "v6", "v7", "v8", "v9", "v10", "v11", "v12", "v13", "v14", "v15", "v16", "v17",  \
  "v18", "v19", "v20", "v21", "v22", "v23", "v24", "v25", "v26", "v27", "v28", "v29", "v30", "v31", "v32", "v33",      \
  "v34", "v35", "v36", "v37", "v38", "v39", "v40", "v41", "v42", "v43", "v44", "v45", "v46", "v47", "v48", "v49",      \
  "v50", "v51", "v52", "v53", "v54", "v55", "v56", "v57", "v58", "v59", "v60", "v61", "v62", "v63", "v128", "v129",    \
  "v130", "v131", "v132", "v133", "v134", "v135", "v136", "v137", "v138", "v139", "v140", "v141", "v142", "v143",      \
  "v146", "v152", "v153", "v156", "v157", "v168", "v170", "v171", "v176", "v195", "v196", "v197", "v198", "v199",      \
  "v200", "v201", "v202", "v203", "v204", "v205", "v206", "v207", "v208", "v209", "v210", "v211", "v212", "v213",      \
  "v214", "v215", "v216", "v217", "v218", "v219", "v220", "v221", "v222", "v223", "a128", "a129", "a130", "a131",      \
  "a132", "a133", "a134", "a135", "a136", "a137", "a138", "a139", "a140", "a141", "a142", "a143", "a144", "a145",      \
  "a146", "a147", "a148", "a149", "a150", "a151", "a152", "a153", "a154", "a155", "a156", "a157", "a158", "a159",      \
  "a160", "a161", "a162", "a163", "a164", "a165", "a166", "a167", "a168", "a169", "a170", "a171", "a172", "a173",      \
  "a174", "a175", "a176", "a177", "a178", "a179", "a180", "a181", "a182", "a183", "a184", "a185", "a186", "a187",      \
  "a188", "a189", "a190", "a191", "s52", "s53", "s54", "s55", "s56", "s57", "s58", "s59", "s60", "s61", "s62", "s63",  \
  "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71", "s72", "s73", "s74", "s75", "s89", "s90", "s91", "s92",      \
  "vcc", "scc", "memory"

// The key loop of one tile for one wavefront.  LDS stages 0 and 1 hold the first two K/V tiles (or the only one) and
// have been published by a barrier; the stream runs every later barrier and fetch of the tile itself.
template <bool kRound>
__device__ __forceinline__ void pipe_key_loop(PipeIo& R) {
#define RPA_PPA_OPERANDS                                                                                                  \
  : "={a[0:31]}"(R.o0), "={a[32:63]}"(R.o1), "={a[64:95]}"(R.o2), "={a[96:127]}"(R.o3), "={v[144:145]}"(R.lsum),       \
    "={v[148:149]}"(R.mneg), "={v[172:173]}"(R.mthr) RPA_PPA_PROF_OUT                                                  \
  : "{v[64:95]}"(R.q0), "{v[96:127]}"(R.q1), "{v[160:163]}"(R.mspan), "{v[178:181]}"(R.rowlo), "{v[224:227]}"(R.kbase0), \
    "{v[228:231]}"(R.kbase1), "{v[186:189]}"(R.misc), "{v[190:193]}"(R.kpiece), "{v169}"(R.cfac), "{s[36:43]}"(R.s0),   \
    "{s[44:51]}"(R.s1)                                                                                                 \
  : RPA_PPA_CLOBBERS RPA_PPA_PROF_CLOBBERS
  if constexpr (kRound) asm volatile(RPA_PPA_LOOP_ROUND RPA_PPA_OPERANDS);
  else asm volatile(RPA_PPA_LOOP_PLAIN RPA_PPA_OPERANDS);
#undef RPA_PPA_OPERANDS
}

template <bool kMimic>
__device__ __forceinline__ void prefill_tile_pipe(const TileArgs& a, char* __restrict__ lds, const SeqInfo& si, int s, int j,
                                                  int qt, int split_info = 0) {
  using C = PipeCfg;
  constexpr int NRG = C::NRG;
  const RpaParams& p = a.p;
#ifdef RPA_PP_PROF2
  const uint64_t pt0 = __builtin_readcyclecounter();
  uint32_t prof2_loop = 0, prof2_halves = 0;
#endif
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int i = lane & 31, g = lane >> 5;  // 32x32 MFMA tiles: lane (i, g) owns row i of a row group
  const int G = p.num_q_heads / p.num_kv_heads;
  const int W = p.sliding_window;
  const bf16_t* __restrict__ q = static_cast<const bf16_t*>(p.queries);
  bf16_t* __restrict__ out = static_cast<bf16_t*>(p.out);
  const char* kvb = static_cast<const char*>(p.kv_pages);
  const int pos0 = si.kv_len - si.q_len;  // position of the sequence's first query token
  constexpr int hd = C::D;

  // ---- key range of the workgroup's rows
  const int wg_row_lo = qt * C::WGROWS, wg_row_hi = min(wg_row_lo + C::WGROWS, si.rows);
  const int wg_pos_min = pos0 + wg_row_lo / G, wg_pos_max = pos0 + (wg_row_hi - 1) / G;
  int range_hi = min(si.kv_len, wg_pos_max + 1);
  int range_lo = max(W > 0 ? max(0, wg_pos_min - W + 1) : 0, si.start) & ~(C::TK - 1);
  // A launch of few tiles: the key range is cut into runs of whole key tiles, a workgroup each, whose states meet in the
  // workspace (split_info and the exchange as in rpa_prefill.h; here the key loop is a fixed instruction stream, which
  // what comes after it cannot disturb).  A run may be empty.
  if (split_info != 0) {
    const int parts = (split_info >> 28) & 7, part = (split_info >> 25) & 7;
    const int n_kt = (max(range_hi - range_lo, 0) + C::TK - 1) / C::TK, per = (n_kt + parts - 1) / parts;
    range_lo = min(range_lo + part * per * C::TK, range_hi);
    range_hi = min(range_hi, range_lo + per * C::TK);
  }
  const int t_last = range_hi - 1;

  // ---- this wavefront's rows: row group rg holds rows w_row_lo + 32 rg + i
  const int w_row_lo = wg_row_lo + wave * C::WROWS;
  int pos_n[NRG];
  auto row_of = [&](int rg, int opaque0, bool& valid, int& head, size_t& q_off) {
    const int R = w_row_lo + 32 * rg + i + opaque0;
    valid = R < si.rows;
    const int qi = valid ? R / G : 0;
    head = j * G + (valid ? R - qi * G : 0);
    q_off = (static_cast<size_t>(si.q0 + qi) * p.num_q_heads + head) * hd;
    return qi;
  };
  PipeIo R;
  const float scale = rbf(p.softmax_scale);
  // The fp32 logit scale of the unscaled-q arithmetic is folded into the exp2 argument (the host sends a batch
  // with a soft cap, or with a scale that is not positive, to the plain tile).
  const float sf_log2e = (kMimic ? 1.f : logit_scale(p)) * kLog2e;
  // One interval test per half: no row group of this wavefront needs a per-key mask iff all_lo < a0 <= all_hi.
  int all_lo = -0x7fffffff, all_hi = 0x7fffffff;
#pragma unroll
  for (int rg = 0; rg < NRG; ++rg) {
    bool valid;
    int head;
    size_t q_off;
    const int qi = row_of(rg, 0, valid, head, q_off);
    pos_n[rg] = valid ? pos0 + qi : -1;
    const int tr_lo = w_row_lo + 32 * rg, tr_hi = min(tr_lo + 32, si.rows);
    const bool t_any = tr_hi > tr_lo;
    const int t_pos_lo = pos0 + tr_lo / G, t_pos_hi = pos0 + (max(tr_hi, tr_lo + 1) - 1) / G;
    // the row group sees all 32 keys from a0 on iff nomask_lo < a0 <= nomask_hi (a group without rows never does)
    const int nomask_hi = t_any ? min(t_pos_lo - 31, range_hi - 32) : -0x7fffffff;
    const int nomask_lo = max(W > 0 ? t_pos_hi - W : -0x7fffffff, si.start - 1);
    all_lo = max(all_lo, nomask_lo);
    all_hi = min(all_hi, nomask_hi);
    // Q operands: lane (i, g) holds elements 16 ks + 8 g .. + 7 of its row, scaled as the arithmetic asks
#pragma unroll
    for (int ks = 0; ks < C::NKS; ++ks) {
      u32x4_t raw = {0u, 0u, 0u, 0u};
      if (valid) raw = *reinterpret_cast<const u32x4_t*>(q + q_off + 16 * ks + 8 * g);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float f = __uint_as_float(pack_bf16x2(q_operand<kMimic>(__uint_as_float(raw[e] << 16), p, scale),
                                                    q_operand<kMimic>(__uint_as_float(raw[e] & 0xffff0000u), p, scale)));
        if (rg == 0) R.q0[4 * ks + e] = f;
        else R.q1[4 * ks + e] = f;
      }
    }
  }
  const bool w_any = w_row_lo < si.rows;
  const int w_pos_hi = pos0 + (min(w_row_lo + C::WROWS, si.rows) - 1) / G;
  const int w_act_hi = min(range_hi - 1, w_pos_hi);  // last key this wavefront's rows can see

  // Results of the key loop: O^T accumulators as the 32x32 MFMA leaves them, the lane's part of the row sums, and the
  // softmax reference point m per row as the exp2 offset -m log2(e) and its threshold (-inf: the row saw no key).
  float o_acc[NRG][C::NBLK][16];
  float l_part[NRG], m_thr[NRG], m_neg[NRG];
#pragma unroll
  for (int rg = 0; rg < NRG; ++rg) {
    m_thr[rg] = -INFINITY;
    m_neg[rg] = 0.f;
    l_part[rg] = 0.f;
#pragma unroll
    for (int blk = 0; blk < C::NBLK; ++blk)
#pragma unroll
      for (int k = 0; k < 16; ++k) o_acc[rg][blk][k] = 0.f;
  }

  // ---- cooperative fetch (as in rpa_prefill.h): one wave-wide direct-to-LDS load moves 4 rows; wavefront w moves
  // rows [16 w, 16 w + 16) of the K tile and of the V tile.
  const uint32_t stride_b = static_cast<uint32_t>(2 * p.num_kv_heads * hd) * 2u;
  const uint64_t page_b = static_cast<uint64_t>(p.page_size) * stride_b;
  const const_i32_ptr bt_c = reinterpret_cast<const_i32_ptr>(
      reinterpret_cast<uintptr_t>(p.block_tables + static_cast<size_t>(s) * p.pages_per_seq));
  const int l_row = lane / C::PR, l_slot = lane % C::PR;
  const int v_row = (lane >> 1) % C::RB;
  const uint32_t v_src = 16u * static_cast<uint32_t>(2 * ((lane >> 1) / C::RB) + (lane & 1));  // byte offset in the row
  uint32_t pre_off[C::HB];
#pragma unroll
  for (int n = 0; n < C::HB; ++n) {
    const int t_local = C::GROUP * wave + C::RB * n + l_row;
    pre_off[n] = static_cast<uint32_t>(C::RB * n + l_row) * stride_b + 16u * static_cast<uint32_t>(l_slot ^ C::swz(t_local));
  }
  const uint32_t v_pre_off = static_cast<uint32_t>(v_row) * stride_b + v_src + hd * 2;
  const bool group_in_page = p.page_size >= C::GROUP;
  auto fetch_tile = [&](int tile, int buf) {
    const int t_first = tile + C::GROUP * wave;
    char* dst = lds + 2 * buf * C::TILE_B + C::HB * wave * 1024;
    if (group_in_page && t_first + C::GROUP - 1 <= t_last) {
      const int page = min(max(bt_c[t_first >> a.page_shift], 0), p.num_pages - 1);
      const char* sbase = kvb + static_cast<uint64_t>(page) * page_b +
                          static_cast<uint64_t>(t_first & (p.page_size - 1)) * stride_b + 2 * j * hd * 2;
      const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(sbase), 0, 0x7fffffff, 0x00020000);
#pragma unroll
      for (int n = 0; n < C::HB; ++n) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(dst + n * 1024), 16,
                                                 pre_off[n], 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(dst + C::TILE_B + n * 1024),
                                                 16, v_pre_off + n * C::RB * stride_b, 0, 0, 0);
      }
      return;
    }
    // last tile of the range or small pages: per block, keys past the range repeat the last one (masked)
#pragma unroll
    for (int n = 0; n < C::HB; ++n) {
      const int t_c = min(t_first + C::RB * n, t_last & ~(C::RB - 1));
      const int page = min(max(bt_c[t_c >> a.page_shift], 0), p.num_pages - 1);
      const char* sbase = kvb + static_cast<uint64_t>(page) * page_b +
                          static_cast<uint64_t>(t_c & (p.page_size - 1)) * stride_b + 2 * j * hd * 2;
      const int tok = min(t_c + l_row, t_last);
      const int t_local = C::GROUP * wave + C::RB * n + l_row;
      const uint32_t off = static_cast<uint32_t>(tok - t_c) * stride_b + 16u * static_cast<uint32_t>(l_slot ^ C::swz(t_local));
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4_t*>(sbase + off),
                                       (__attribute__((address_space(3))) void*)(dst + n * 1024), 16, 0, 0);
      const int v_tok = min(t_c + v_row, t_last);
      __builtin_amdgcn_global_load_lds(
          reinterpret_cast<const u32x4_t*>(sbase + static_cast<uint32_t>(v_tok - t_c) * stride_b + v_src + hd * 2),
          (__attribute__((address_space(3))) void*)(dst + C::TILE_B + n * 1024), 16, 0, 0);
    }
  };
  // Wait until at most `tiles_ahead` later tiles of this wavefront's loads are outstanding (they complete in order).
  auto wait_fetch = [&](int tiles_ahead) {
    static_assert(C::LOADS == 8 && C::NSTG >= 3 && C::NSTG <= 4, "extend the immediates below");
    switch (tiles_ahead) {
      case 0: __builtin_amdgcn_s_waitcnt(0x0F70); break;   // vmcnt(0)
      case 1: __builtin_amdgcn_s_waitcnt(0x0F78); break;   // vmcnt(8)
      default: __builtin_amdgcn_s_waitcnt(0x4F70); break;  // vmcnt(16)
    }
  };

  if (range_hi > range_lo) {
    const int n_tiles = (range_hi - range_lo + C::TK - 1) / C::TK;
    // halves this wavefront computes: [0, hb); a half starts at range_lo + 32 * index
    const int hb = __builtin_amdgcn_readfirstlane(
        w_any && w_act_hi >= range_lo ? min(2 * n_tiles, ((w_act_hi - range_lo) >> 5) + 1) : 0);

    const int lds_base = static_cast<int>(reinterpret_cast<uintptr_t>(lds));  // LDS pointers are 32-bit offsets
    // LDS addresses of the operand reads in stage 0.  K, per k-step: lane (i, g) reads the 16-byte piece 2 ks + g of
    // key row i (pieces swizzled by the row, see rpa_prefill.h).  V^T, with the transposing read: in each group of 16
    // lanes, lanes 4e..4e+3 point at 16 consecutive elements (one column unit) of key e of a 4-key block; the groups
    // of a half-wave take the two column units of a block of 32 elements, the half-waves the key blocks g.
#pragma unroll
    for (int ks = 0; ks < C::NKS; ++ks) {
      const int addr = lds_base + i * C::ROWB + 16 * ((2 * ks + g) ^ C::swz(i));
      if (ks < 4) R.kbase0[ks] = addr;
      else R.kbase1[ks - 4] = addr;
    }
    const int x16 = lane & 15;
    R.misc[0] = lds_base + C::TILE_B + g * 1024 + ((lane >> 4) & 1) * 128 + (x16 >> 2) * 32 + 8 * (x16 & 3);
    // fetch: the lane's row in a 4-row block and its 16-byte piece, K (swizzled by the row in the tile) and V
    R.misc[1] = l_row;
    R.misc[2] = v_row;
    R.misc[3] = static_cast<int>(v_src) + hd * 2;
#pragma unroll
    for (int n = 0; n < C::HB; ++n) R.kpiece[n] = 16 * (l_slot ^ C::swz(C::RB * n + l_row));
    // Per-lane bounds of the keys a row group may see (none for a row past the end: an unreachable first key)
    R.rowlo = i32x4_t{0, 0, 0, 0};
    R.mspan = i32x4_t{0, 0, 0, 0};
#pragma unroll
    for (int rg = 0; rg < NRG; ++rg) {
      const int hi = min(pos_n[rg], range_hi - 1);
      const int lo = max(W > 0 ? pos_n[rg] - W + 1 : -0x40000000, si.start);
      R.rowlo[rg] = (hi < lo ? 0x40000000 : lo) - 4 * g;
      R.mspan[rg] = max(hi - lo, 0);
    }
    R.cfac = sf_log2e;
    const uint64_t bt_addr = reinterpret_cast<uint64_t>(p.block_tables + static_cast<size_t>(s) * p.pages_per_seq);
    const uint64_t kv_addr = reinterpret_cast<uint64_t>(kvb) + static_cast<uint64_t>(2 * j * hd * 2);
    auto sgpr = [](int x) { return __builtin_amdgcn_readfirstlane(x); };
    R.s0 = i32x8_t{hb, sgpr(n_tiles), sgpr(range_lo), sgpr(all_lo), sgpr(all_hi), sgpr(t_last), 16 * wave,
                   sgpr(lds_base) + C::HB * wave * 1024};
    R.s1 = i32x8_t{sgpr(static_cast<int>(bt_addr)), sgpr(static_cast<int>(bt_addr >> 32)), sgpr(static_cast<int>(kv_addr)),
                   sgpr(static_cast<int>(kv_addr >> 32)), sgpr(static_cast<int>(stride_b)), sgpr(static_cast<int>(page_b)),
                   sgpr(a.page_shift), sgpr(p.num_pages - 1)};

    __syncthreads();  // every wavefront has left the previous item's tiles
    for (int t = 0; t < min(C::NSTG - 1, n_tiles); ++t) fetch_tile(range_lo + t * C::TK, t);
    wait_fetch(min(n_tiles - 1, C::NSTG - 2));
    __syncthreads();  // publishes tile 0
#ifdef RPA_PP_PROF2
    const uint64_t pl0 = __builtin_readcyclecounter();
#endif
    pipe_key_loop<kMimic && C::ROUND>(R);
#ifdef RPA_PP_PROF2
    prof2_loop = static_cast<uint32_t>(__builtin_readcyclecounter() - pl0);
    prof2_halves = hb;
#endif
#ifdef RPA_PP_PROF
    if ((threadIdx.x & (kWave - 1)) == 0) {
      uint32_t* dst = reinterpret_cast<uint32_t*>(a.partial_o) + (blockIdx.x * kWgWaves + threadIdx.x / kWave) * 16;
      for (int k = 0; k < 8; ++k) dst[k] += static_cast<uint32_t>(R.prof[k]);
      dst[8] += 1;
    }
#endif
#pragma unroll
    for (int rg = 0; rg < NRG; ++rg) {
      l_part[rg] = R.lsum[rg];
      m_neg[rg] = R.mneg[rg];
      m_thr[rg] = R.mthr[rg];
#pragma unroll
      for (int blk = 0; blk < C::NBLK; ++blk)
#pragma unroll
        for (int k = 0; k < 16; ++k) {
          const int idx = 16 * (blk & 1) + k;
          o_acc[rg][blk][k] = rg == 0 ? (blk < 2 ? R.o0[idx] : R.o1[idx]) : (blk < 2 ? R.o2[idx] : R.o3[idx]);
        }
    }
  }

  // ---- a run of a cut key range: state to the workspace, a ticket of the tile, and the workgroup that draws the last
  // one adds the runs up in run order (its own included) and goes on.  Per lane 32 pieces of 16 bytes (row group,
  // block, four accumulators), 1 KiB per piece and wavefront in lane order; per row its reference point and sum.
  float m_merged[NRG], l_merged[NRG];
  if (split_info != 0) {
    const int parts = (split_info >> 28) & 7, part = (split_info >> 25) & 7, tile_id = split_info & 0xffffff;
    const bool upper = ((split_info >> 24) & 1) != 0;
    constexpr int kAgentScope = 16;
    constexpr uint32_t kWaveState = NRG * C::NBLK * 4 * 1024, kPartState = kWgWaves * kWaveState;  // bytes
    const __amdgpu_buffer_rsrc_t o_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<char*>(a.partial_o) + (upper ? a.tile_state_o_half : 0u), 0, 0x7fffffff, 0x00020000);
    uint64_t* ml = reinterpret_cast<uint64_t*>(reinterpret_cast<char*>(a.partial_ml) + (upper ? a.tile_state_ml_half : 0u));
    const uint32_t my_part = static_cast<uint32_t>(tile_id * parts + part);
    auto state_off = [&](uint32_t pt, int rg, int blk, int q4) {
      return static_cast<int>(pt * kPartState + wave * kWaveState + ((rg * C::NBLK + blk) * 4 + q4) * 1024 + lane * 16);
    };
    auto ml_index = [&](uint32_t pt, int rg) { return (pt * kWgWaves + wave) * (32 * NRG) + 32 * rg + i; };
#pragma unroll
    for (int rg = 0; rg < NRG; ++rg) {
#pragma unroll
      for (int blk = 0; blk < C::NBLK; ++blk)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const f32x4_t v = {o_acc[rg][blk][4 * q4], o_acc[rg][blk][4 * q4 + 1], o_acc[rg][blk][4 * q4 + 2], o_acc[rg][blk][4 * q4 + 3]};
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, v), o_rsrc, state_off(my_part, rg, blk, q4), 0, kAgentScope);
        }
      const float l_row = l_part[rg] + __shfl_xor(l_part[rg], 32, kWave);  // the two lanes of a row hold half its keys each
      if (g == 0) {
        const float m_row = m_thr[rg] == -INFINITY ? -INFINITY : -m_neg[rg] * (1.f / kLog2e);
        const uint64_t v = static_cast<uint64_t>(__float_as_uint(m_row)) | (static_cast<uint64_t>(__float_as_uint(l_row)) << 32);
        __hip_atomic_store(ml + ml_index(my_part, rg), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // every wavefront's state has left (and every wavefront is out of the key loop's LDS)
    uint32_t* ctr = a.counters + a.tile_ticket_base + tile_id;
    int* flag = reinterpret_cast<int*>(lds);
    if (threadIdx.x == 0)
      *flag = static_cast<int>(__hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    __syncthreads();
    const int ticket = *flag;
    __syncthreads();  // (the flag's word belongs to the next tile's stage from here on)
    if (ticket != parts - 1) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll
    for (int rg = 0; rg < NRG; ++rg) {
      float M = -INFINITY, L = 0.f;
#pragma unroll
      for (int blk = 0; blk < C::NBLK; ++blk)
#pragma unroll
        for (int k = 0; k < 16; ++k) o_acc[rg][blk][k] = 0.f;
      for (int pt = 0; pt < parts; ++pt) {
        const uint32_t src = static_cast<uint32_t>(tile_id * parts + pt);
        const uint64_t v = __hip_atomic_load(ml + ml_index(src, rg), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const float mk = __uint_as_float(static_cast<uint32_t>(v)), lk = __uint_as_float(static_cast<uint32_t>(v >> 32));
        const float m_new = fmaxf(M, mk);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float keep = __builtin_amdgcn_exp2f((M - m_use) * kLog2e);
        const float w = __builtin_amdgcn_exp2f((mk - m_use) * kLog2e);
        L = L * keep + w * lk;
        M = m_new;
#pragma unroll
        for (int blk = 0; blk < C::NBLK; ++blk)
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            const f32x4_t ov = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(o_rsrc, state_off(src, rg, blk, q4), 0, kAgentScope));
#pragma unroll
            for (int e = 0; e < 4; ++e) o_acc[rg][blk][4 * q4 + e] = o_acc[rg][blk][4 * q4 + e] * keep + w * ov[e];
          }
      }
      m_merged[rg] = M;
      l_merged[rg] = L;
    }
    if (threadIdx.x == 0) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  // ---- normalise (with optional sinks) and store
#pragma unroll
  for (int rg = 0; rg < NRG; ++rg) {
    bool valid;
    int head;
    size_t q_off;
    int opaque0 = 0;
    asm volatile("" : "+v"(opaque0));
    row_of(rg, opaque0, valid, head, q_off);
    float l_run = l_part[rg] + __shfl_xor(l_part[rg], 32, kWave);  // the two lanes of a row hold half its keys each
    if (!valid) continue;
    float m_row = m_thr[rg] == -INFINITY ? -INFINITY : -m_neg[rg] * (1.f / kLog2e);
    if (split_info != 0) {
      l_run = l_merged[rg];
      m_row = m_merged[rg];
    }
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
    const float inv = num_scale * out_scale(p) / fmaxf(denom, 1e-6f);
    bf16_t* orow = out + q_off;
    // register 4 q + r of block blk holds head_dim element 32 blk + 8 q + 4 g + r of this lane's row
#pragma unroll
    for (int blk = 0; blk < C::NBLK; ++blk)
#pragma unroll
      for (int qq = 0; qq < 4; ++qq) {
        u32x2_t w;
        w[0] = pack_bf16x2(o_acc[rg][blk][4 * qq] * inv, o_acc[rg][blk][4 * qq + 1] * inv);
        w[1] = pack_bf16x2(o_acc[rg][blk][4 * qq + 2] * inv, o_acc[rg][blk][4 * qq + 3] * inv);
        *reinterpret_cast<u32x2_t*>(orow + 32 * blk + 8 * qq + 4 * g) = w;
      }
  }
#ifdef RPA_PP_PROF2
  if ((threadIdx.x & (kWave - 1)) == 0) {
    uint32_t* dst = reinterpret_cast<uint32_t*>(a.partial_o) + (blockIdx.x * kWgWaves + threadIdx.x / kWave) * 16;
    dst[0] += static_cast<uint32_t>(__builtin_readcyclecounter() - pt0);
    dst[1] += prof2_loop;
    dst[2] += prof2_halves;
    dst[3] += 1;
    if (dst[4] == 0) dst[4] = static_cast<uint32_t>(pt0);  // start of the first tile
    dst[5] = static_cast<uint32_t>(__builtin_readcyclecounter());  // end of the last
  }
#endif
}

}  // namespace rpa
