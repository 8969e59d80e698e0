// Wave-level attention loop: one wavefront streams a key range of one (sequence, kv head) for up to 16 rows.
#pragma once

#include <type_traits>

#include "rpa_tile_common.h"

namespace rpa {

template <int D, int NT, bool kMimic>
struct Cfg {
  static constexpr int NS = D / 128;        // 128-wide slices of head_dim
  static constexpr int NKS = D / 32;        // k-steps of the QK^T contraction
  static constexpr int TT = 16 * NT;        // tokens per iteration
  static constexpr int NSLOT = 4 * NT;      // tokens each lane fetches per iteration
  static constexpr int ROWB = D * 2 + 32;   // LDS bytes per K row: with a 32-byte pad neither the b128 reads (lane = row) nor
                                            // the b128 writes (lane = piece) meet a bank conflict; with 16 the reads do, two-way
  static constexpr int LDS_PER_WAVE = TT * ROWB;
  static constexpr int SINK_KEYS = 8;                   // sink keys of ragged_decode_attention staged in LDS per wavefront
  static constexpr int SINK_LDS = SINK_KEYS * 2 * D * 2 + 16 * SINK_KEYS * 4;  // their K rows, their V rows, 16 rows of biases
};

// Cache element types (kKv): 0 = the query dtype (bf16); 8-bit floats of the OCP formats: 1 = e4m3 (finite, no
// infinities, largest value 448), 2 = e5m2 (largest finite value 57344).
template <int kKv>
__device__ __forceinline__ auto fp8_pair_lo(uint32_t w) {
  if constexpr (kKv == 2) return __builtin_amdgcn_cvt_pk_f32_bf8(static_cast<int>(w), false);
  else return __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w), false);
}
template <int kKv>
__device__ __forceinline__ auto fp8_pair_hi(uint32_t w) {
  if constexpr (kKv == 2) return __builtin_amdgcn_cvt_pk_f32_bf8(static_cast<int>(w), true);
  else return __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w), true);
}
// Bytes 2 half, 2 half + 1 of a dword as floats (the half must fold to a constant: the instruction encodes it).
template <int kKv>
__device__ __forceinline__ auto fp8_pair(uint32_t w, int half) {
  const auto lo = fp8_pair_lo<kKv>(w);
  const auto hi = fp8_pair_hi<kKv>(w);
  return half ? hi : lo;
}
// Eight 8-bit elements in two dwords -> the same eight values as bf16 in four dwords (exact).
template <int kKv>
__device__ __forceinline__ u32x4_t fp8x8_to_bf16x8(u32x2_t w) {
  u32x4_t o;
#pragma unroll
  for (int d = 0; d < 2; ++d) {
    const auto lo = fp8_pair_lo<kKv>(w[d]);  // bytes 0, 1
    const auto hi = fp8_pair_hi<kKv>(w[d]);  // bytes 2, 3
    o[2 * d] = __builtin_amdgcn_perm(__float_as_uint(lo[1]), __float_as_uint(lo[0]), 0x07060302u);
    o[2 * d + 1] = __builtin_amdgcn_perm(__float_as_uint(hi[1]), __float_as_uint(hi[0]), 0x07060302u);
  }
  return o;
}
// Two floats rounded to the 8-bit type (nearest even; the callers keep them inside its finite range) and back.
template <int kKv>
__device__ __forceinline__ void round_fp8x2(float& a, float& b) {
  if constexpr (kKv == 2) {
    const int w = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, 0, false);
    const auto f = __builtin_amdgcn_cvt_pk_f32_bf8(w, false);
    a = f[0];
    b = f[1];
  } else {
    const int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    const auto f = __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
    a = f[0];
    b = f[1];
  }
}
template <int kKv>
constexpr float fp8_max() { return kKv == 2 ? 57344.f : 448.f; }

// Everything one wavefront needs for one work item.  kWaveOnly: the state in TileArgs::pre, if any, is merged into
// every row (only in the kernel instantiation without prefill tiles, so that the common one keeps its register
// allocation).
// kPass: 0 = attention with the online softmax.  An 8-bit cache takes the reference's rounding of the *normalised*
// probabilities to the cache dtype (ragged_page_attention_v3, _kernel.py:279), which needs the row maximum and sum
// before the first P V product, so it runs as two launches: 1 = row statistics only (maximum and sum of exp over
// the visible keys, written to TileArgs::stats), 2 = P = round(exp(s - m) / l) with m, l from there, O = P V.
// Where TileArgs::logits is given, launch 1 also leaves every logit it computed there (capped and masked, fp32, one
// row of logit_pitch keys per (token, query head)) and the second launch is 3 instead of 2: the same arithmetic on the
// stored logits, with no K rows read, no Q and no first product -- for a decode step that is 8 bytes of logits written
// and read per key and query head against a K row of head_dim bytes per key and kv head.
template <int D, int NT, bool kMimic, bool kWaveOnly = false, int kKv = 0, int kPass = 0, bool kFew = false>
__device__ __forceinline__ void process_item(const TileArgs& a, char* __restrict__ lds_k, const SeqInfo& si, int s,
                                             int j, int rt, int range_lo, int range_hi, const Part& part) {
  using C = Cfg<D, NT, kMimic>;
  const RpaParams& p = a.p;
  const int lane = threadIdx.x & (kWave - 1);
  const int i = lane & 15, g = lane >> 4;
  const bool pair = kWaveOnly && kKv == 0 && kPass == 0 && a.pair != 0;  // two kv heads of head_dim 64 per item
  const int G_head = p.num_q_heads / p.num_kv_heads;
  const int G = pair ? 2 * G_head : G_head;  // query heads of the item: j counts head pairs then
  const bf16_t* __restrict__ q = static_cast<const bf16_t*>(p.queries);
  bf16_t* __restrict__ out = static_cast<bf16_t*>(p.out);
  const int W = p.sliding_window;

  // ---- rows of this tile and their key range
  const int row_lo = rt * 16, row_hi = min(row_lo + 16, si.rows);
  const int qi_min = row_lo / G, qi_max = (row_hi - 1) / G;
  const int pos_min = si.kv_len - si.q_len + qi_min, pos_max = si.kv_len - si.q_len + qi_max;
  // this lane's row
  const int R = row_lo + i;
  const bool row_valid = R < si.rows;
  const int qi = row_valid ? R / G : 0;
  const int hg = row_valid ? R - qi * G : 0;
  const int pos_n = row_valid ? si.kv_len - si.q_len + qi : -1;
  const int head = j * G + hg;
  const int hp = pair && hg >= G_head ? 1 : 0;  // which head of the pair this row belongs to
  // head_dim 64 runs on the 128-wide instantiation: q is padded with zeros, the upper eight 16-byte pieces of a K / V
  // row repeat the lower eight (K: multiplied by zero; V: output elements that are not stored).
  const int hd = p.head_dim;
  const size_t q_row_off = (static_cast<size_t>(si.q0 + qi) * p.num_q_heads + head) * hd;

  // ---- Q^T operands: lane (row i, group g) holds q[row][32 ks + 8 g .. +8], pre-scaled and rounded to bf16
  bf16x8_t qreg[C::NKS];
  {
    const float scale = rbf(p.softmax_scale);
#pragma unroll
    for (int ks = 0; ks < C::NKS; ++ks) {
      u32x4_t raw = {0u, 0u, 0u, 0u};
      if (pair) {
        // contraction index 64 hp .. 64 hp + 63 carries this row's query; the other head's half stays zero
        if (row_valid && (ks >> 1) == hp) raw = *reinterpret_cast<const u32x4_t*>(q + q_row_off + 32 * (ks & 1) + 8 * g);
      } else if (row_valid && 32 * ks + 8 * g < hd) {
        raw = *reinterpret_cast<const u32x4_t*>(q + q_row_off + 32 * ks + 8 * g);
      }
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
      qreg[ks] = __builtin_bit_cast(bf16x8_t, sc);
    }
  }

  const float post_scale = logit_scale(p);
  f32x4_t o_acc[C::NS][8];
#pragma unroll
  for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
    for (int c = 0; c < 8; ++c) o_acc[sN][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  float m_fix = 0.f, inv_l = 0.f;  // kPass == 2: the row's maximum and 1 / sum from the statistics launch
  constexpr bool kNorm = kPass >= 2;    // probabilities normalised with the statistics of an earlier launch
  constexpr bool kStored = kPass == 3;  // ... and the logits of that launch instead of K
  // This lane's stored logits (an absent row repeats the item's first one: read, never written).  A (token, kv head)
  // owns logit_pitch * G floats, laid out [key / 4][query head of the kv head][key % 4]: the 32 keys of a tile and
  // the G rows of a decode token are one contiguous run of 128 G bytes.
  float* lrow = nullptr;
  if constexpr (kPass == 1 || kStored)
    if (a.logits != nullptr)
      lrow = a.logits + (static_cast<size_t>(si.q0 + qi) * p.num_kv_heads + j) * static_cast<size_t>(a.logit_pitch) * G + 4 * hg;
  if constexpr (kNorm) {
    const size_t idx = static_cast<size_t>(si.q0 + qi) * p.num_q_heads + head;
    const float ms = a.stats[2 * idx], ls = a.stats[2 * idx + 1];
    m_fix = ms == -INFINITY ? 0.f : ms;
    inv_l = ls > 0.f ? 1.f / ls : 0.f;
    m_run = 0.f;  // every part carries the same reference point: parts merge by plain addition
    l_run = 0.f;
  }

  const int32_t* __restrict__ bt = p.block_tables + static_cast<size_t>(s) * p.pages_per_seq;
  // Same row through the constant address space: reads with a wave-uniform index become scalar loads, which
  // are counted apart from the vector loads of the K/V stream.  The block table is never written by this kernel.
  const const_i32_ptr bt_c = reinterpret_cast<const_i32_ptr>(reinterpret_cast<uintptr_t>(bt));
  const int t_last = range_hi - 1;
  // the reference's cap is a weakly typed scalar: it takes the logits' dtype (bf16) before it divides and multiplies
  const float cap = kMimic ? rbf(p.logits_soft_cap) : p.logits_soft_cap;
  const float inv_cap = cap != 0.f ? 1.f / cap : 0.f;

  using raw_t = typename std::conditional<kKv != 0, u32x2_t, u32x4_t>::type;  // one lane's piece: eight elements
  constexpr uint32_t PIECE_B = kKv != 0 ? 8u : 16u;
  raw_t kreg[C::NSLOT][C::NS];
  raw_t vbuf0[C::NSLOT][C::NS], vbuf1[C::NSLOT][C::NS];
  f32x4_t sreg[NT];  // kStored: this lane's four logits per sub-tile, requested with the V rows
  // tiles never reach past the pitch (a multiple of 64 that covers every position a block-table row can hold); the
  // clamp only keeps a lane in its row should the metadata be malformed
  auto logit_off = [&](int tile, int u) { return min(tile + 16 * u + 4 * g, static_cast<int>(a.logit_pitch) - 4); };

  // Fetch K and V of the TT tokens starting at `tile`: lane (i, g) takes tokens 16u + 4g + r (u < NT, r < 4),
  // 16-byte piece i (+16 per 128-slice) of each row, so a quarter-wave reads one contiguous row.
  //
  // Fast path (page_size >= 16, tile entirely inside the range): a 16-token sub-tile sits in one page, so the
  // block-table entry is a scalar load (it does not share the vector-memory counter with the K/V stream) and
  // the row address is a scalar base plus one per-lane byte offset that is constant for the whole item.
  // Slow path (last tile of a range, small pages): per-lane page lookup; tokens past the end of the range are
  // replaced by the last valid one (their scores are masked).
  const char* kvb = a.kv.k_base;
  const int64_t v_delta = a.kv.v_base - a.kv.k_base;  // the V row of a (token, head) relative to its K row
  const uint32_t stride_b = a.kv.stride_b;            // bytes between tokens
  const uint64_t page_b = a.kv.page_b;
  const uint32_t head_off = static_cast<uint32_t>(pair ? 2 * j : j) * a.kv.head_b;
  // A head_dim below the instantiation's width: the lanes past the row's last piece fetch a piece that exists (a
  // repeat of the lower half where the piece count is a power of two, which the head pairs count on; else the last
  // one) -- in K it meets the zeros q is padded with, in V it feeds output elements that are not stored.
  const int npieces = hd / 8;
  const int piece = (npieces & (npieces - 1)) == 0 ? (i & (npieces - 1)) : min(i, npieces - 1);  // i itself from head_dim 128 up
  uint32_t slice_off[C::NS];  // this lane's piece of 128-slice sN, from its piece of slice 0
#pragma unroll
  for (int sN = 0; sN < C::NS; ++sN)
    slice_off[sN] = sN == 0 ? 0u : PIECE_B * static_cast<uint32_t>(min(i + 16 * sN, npieces - 1) - piece);
  // this lane's piece inside a token's record; with a head pair, pieces 8..15 are those of the second head
  const uint32_t piece_off = head_off + PIECE_B * static_cast<uint32_t>(piece) + (pair && i >= 8 ? a.kv.head_b : 0u);
  const uint32_t lane_off = static_cast<uint32_t>(4 * g) * stride_b + piece_off;
  auto issue_loads = [&](int tile, raw_t (&kr)[C::NSLOT][C::NS], raw_t (&vr)[C::NSLOT][C::NS]) {
    if constexpr (kStored) {
#pragma unroll
      for (int u = 0; u < NT; ++u)
        sreg[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(lrow + static_cast<size_t>(logit_off(tile, u)) * G));
    }
    if (a.uniform_page && tile + C::TT <= range_hi) {
#pragma unroll
      for (int u = 0; u < NT; ++u) {
        const int t16 = tile + 16 * u;
        int page = a.kv.contiguous ? s : bt_c[t16 >> a.page_shift];
        page = min(max(page, 0), p.num_pages - 1);
        const char* sbase = kvb + static_cast<uint64_t>(page) * page_b +
                            static_cast<uint64_t>(t16 & (p.page_size - 1)) * stride_b;
        // A token's K row, then its V row, each in ascending address order (the two 128-slices of a row one after
        // the other): requests that are neighbours in memory do best as neighbours in time -- at head_dim 256, slice 0
        // of K and V followed by slice 1 of K and V costs 1.8 % (config 4), and all K rows of the four tokens before
        // their V rows 1.5 % there and 4.5 % on config 2.  With two slices the empty statements keep the compiler from
        // regrouping; with one slice its own order is the wanted one, and the statements would only cost (2.5 % on
        // config 5).
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const char* row = sbase + static_cast<uint64_t>(r) * stride_b;
          const char* row_v = row + v_delta;
#pragma unroll
          for (int sN = 0; sN < C::NS; ++sN)
            if (!kStored) kr[4 * u + r][sN] = *reinterpret_cast<const raw_t*>(row + (lane_off + slice_off[sN]));
          if constexpr (C::NS > 1) asm volatile("" ::: "memory");
#pragma unroll
          for (int sN = 0; sN < C::NS; ++sN)
            if (kPass != 1) vr[4 * u + r][sN] = *reinterpret_cast<const raw_t*>(row_v + (lane_off + slice_off[sN]));
          if constexpr (C::NS > 1) asm volatile("" ::: "memory");
        }
      }
      return;
    }
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      const int t4c = min(tile + 16 * u + 4 * g, t_last & ~3);
      const int rlim = min(3, t_last - t4c);
      int page = a.kv.contiguous ? s : bt[t4c >> a.page_shift];
      page = min(max(page, 0), p.num_pages - 1);
      const char* base = kvb + static_cast<uint64_t>(page) * page_b +
                         static_cast<uint64_t>(t4c & (p.page_size - 1)) * stride_b + piece_off;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const char* row = base + static_cast<uint64_t>(min(r, rlim)) * stride_b;
#pragma unroll
        for (int sN = 0; sN < C::NS; ++sN) {
          if (!kStored) kr[4 * u + r][sN] = *reinterpret_cast<const raw_t*>(row + slice_off[sN]);
          if (kPass != 1) vr[4 * u + r][sN] = *reinterpret_cast<const raw_t*>(row + v_delta + slice_off[sN]);
        }
      }
    }
  };

  f32x4_t skeep[NT];    // kPass 1 with stored logits: the last tile's logits, not yet stored
  int skeep_tile = -1;
  auto store_logits = [&]() {
    if (skeep_tile < 0) return;
    if (row_valid && skeep_tile + C::TT <= static_cast<int>(a.logit_pitch)) {
#pragma unroll
      for (int u = 0; u < NT; ++u)
        __builtin_nontemporal_store(skeep[u], reinterpret_cast<f32x4_t*>(lrow + static_cast<size_t>(skeep_tile + 16 * u + 4 * g) * G));
    }
    skeep_tile = -1;
  };
  auto body = [&](int tile, raw_t (&vcur)[C::NSLOT][C::NS], raw_t (&vnext)[C::NSLOT][C::NS]) {
    f32x4_t s_acc[NT];
    if constexpr (kStored) {
#pragma unroll
      for (int u = 0; u < NT; ++u) s_acc[u] = sreg[u];
    }
    // 1. K rows to the wave-private LDS tile: row = token within the tile, 16-byte piece i (+16 per slice)
    if constexpr (!kStored)
#pragma unroll
    for (int u = 0; u < NT; ++u)
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int sN = 0; sN < C::NS; ++sN) {
          // the statistics launch fetches no V: its K rows alternate between the two V buffers, two tiles ahead
          const raw_t kraw = kPass == 1 ? vcur[4 * u + r][sN] : kreg[4 * u + r][sN];
          u32x4_t kw;
          if constexpr (kKv != 0) kw = fp8x8_to_bf16x8<kKv>(kraw);
          else kw = kraw;
          *reinterpret_cast<u32x4_t*>(lds_k + (16 * u + 4 * g + r) * C::ROWB + 16 * (i + 16 * sN)) = kw;
        }
    // The logits of the tile before go out ahead of this iteration's loads: the wait for those loads at the top of the
    // next iteration then finds the stores a whole iteration old (stores and loads leave one counter in order; issued
    // after the loads, a store would be waited for when it has only just left).
    if constexpr (kPass == 1) store_logits();
    // 2. next tile's K and V are requested now, a full iteration before they are needed
    if constexpr (kPass == 1) {
      if (tile + 2 * C::TT < range_hi) issue_loads(tile + 2 * C::TT, vcur, vnext);
    } else {
      if (tile + C::TT < range_hi) issue_loads(tile + C::TT, kreg, vnext);
    }
    // 3. S^T = K Q^T: lane (token i of sub-tile u, group g) reads piece 4 ks + g of its row
    if constexpr (!kStored)
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      s_acc[u] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < C::NKS; ++ks) {
        const u32x4_t kop = *reinterpret_cast<const u32x4_t*>(lds_k + (16 * u + i) * C::ROWB + 16 * (4 * ks + g));
        s_acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kop), qreg[ks], s_acc[u], 0, 0, 0);
      }
    }
    // 4. online softmax; this lane: query row i, tokens tile + 16u + 4g + r
    float sv[NT][4];
    const bool need_mask = (tile + C::TT > range_hi) || (tile + C::TT - 1 > pos_min) || (W > 0 && tile <= pos_max - W) ||
                           tile < si.start;
#pragma unroll
    for (int u = 0; u < NT; ++u)
#pragma unroll
      for (int r = 0; r < 4; ++r) sv[u][r] = kStored ? s_acc[u][r] : kMimic ? rbf(s_acc[u][r]) : s_acc[u][r] * post_scale;
    if (!kStored && cap != 0.f) {
      asm volatile("" : "+v"(sv[0][0]));  // keeps the soft cap inside this wave-uniform branch (it is not cheap)
#pragma unroll
      for (int u = 0; u < NT; ++u)
#pragma unroll
        for (int r = 0; r < 4; r += 2) soft_cap2<kMimic>(sv[u][r], sv[u][r + 1], cap, inv_cap);
    }
    if (!kStored && need_mask) {
#pragma unroll
      for (int u = 0; u < NT; ++u)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int tok = tile + 16 * u + 4 * g + r;
          const bool keep = tok <= pos_n && tok < range_hi && (W <= 0 || tok > pos_n - W) && tok >= si.start;
          sv[u][r] = keep ? sv[u][r] : -INFINITY;
        }
    }
    if constexpr (kPass == 1) {
      // the logits as the next launch needs them, capped and masked; stored by the next iteration
      if (a.logits != nullptr) {
#pragma unroll
        for (int u = 0; u < NT; ++u) skeep[u] = f32x4_t{sv[u][0], sv[u][1], sv[u][2], sv[u][3]};
        skeep_tile = tile;
      }
    }
    uint32_t pw[2 * NT];
    if constexpr (kNorm) {
      // normalised probabilities, rounded to the cache dtype
#pragma unroll
      for (int u = 0; u < NT; ++u) {
        float pv[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) pv[r] = __builtin_amdgcn_exp2f((sv[u][r] - m_fix) * kLog2e) * inv_l;
        round_fp8x2<kKv>(pv[0], pv[1]);
        round_fp8x2<kKv>(pv[2], pv[3]);
        pw[2 * u] = (__float_as_uint(pv[0]) >> 16) | (__float_as_uint(pv[1]) & 0xffff0000u);
        pw[2 * u + 1] = (__float_as_uint(pv[2]) >> 16) | (__float_as_uint(pv[3]) & 0xffff0000u);
      }
    } else {
    float tmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < NT; ++u)
#pragma unroll
      for (int r = 0; r < 4; ++r) tmax = fmaxf(tmax, sv[u][r]);
    tmax = row_groups_max(tmax);
    const float m_new = fmaxf(m_run, tmax);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * kLog2e);
    float psum = 0.f;
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      float pv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float d = sv[u][r] - m_use;
        if (kMimic) d = rbf(d);
        float e = __builtin_amdgcn_exp2f(d * kLog2e);
        if (kPass == 0) e = rbf(e);  // probabilities enter P V as bf16, and the row sum adds the same rounded values
        pv[r] = e;
        psum += e;
      }
      pw[2 * u] = (__float_as_uint(pv[0]) >> 16) | (__float_as_uint(pv[1]) & 0xffff0000u);
      pw[2 * u + 1] = (__float_as_uint(pv[2]) >> 16) | (__float_as_uint(pv[3]) & 0xffff0000u);
    }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (kPass == 0 && __any(alpha != 1.f)) {
#pragma unroll
      for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
        for (int c = 0; c < 8; ++c) o_acc[sN][c] *= alpha;
    }
    }
    if constexpr (kPass == 1) return;  // statistics only: no P V
    // 5. O^T += V^T P^T.  MFMA number c of slice sN yields d = 128 sN + 8 (row of the MFMA) + c; its A operand is
    //    column c of every fetched 8-wide piece, gathered from the token rows by byte permutes.
#pragma unroll
    for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
        uint32_t aw[2 * NT];
#pragma unroll
        for (int h = 0; h < 2 * NT; ++h) {
          if constexpr (kKv != 0) {
            // elements c of the two tokens' pieces: byte c of each piece, widened (bf16 = upper half of the float)
            const auto f1 = fp8_pair<kKv>(vcur[2 * h + 1][sN][c >> 2], (c >> 1) & 1);
            const auto f0 = fp8_pair<kKv>(vcur[2 * h][sN][c >> 2], (c >> 1) & 1);
            aw[h] = __builtin_amdgcn_perm(__float_as_uint(f1[c & 1]), __float_as_uint(f0[c & 1]), 0x07060302u);
          } else {
            aw[h] = __builtin_amdgcn_perm(vcur[2 * h + 1][sN][c >> 1], vcur[2 * h][sN][c >> 1], sel);
          }
        }
        if constexpr (NT == 2) {
          const u32x4_t av = {aw[0], aw[1], aw[2], aw[3]};
          const u32x4_t pvv = {pw[0], pw[1], pw[2], pw[3]};
          o_acc[sN][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                                 __builtin_bit_cast(bf16x8_t, pvv), o_acc[sN][c], 0, 0, 0);
        } else {
          const u32x2_t av = {aw[0], aw[1]};
          const u32x2_t pvv = {pw[0], pw[1]};
          o_acc[sN][c] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4_t, av),
                                                                   __builtin_bit_cast(s16x4_t, pvv), o_acc[sN][c], 0, 0, 0);
        }
      }
  };

  // Sink keys of ragged_decode_attention: the part that starts a (sequence, kv head) also takes the keys
  // [first, first + sink_n) below sink_limit, which are visible whatever the window and the end of the sequence say and
  // carry the row's bias on positions below sink_n (si.start lies behind them, so the stream leaves them out).  Their K
  // and V rows -- the first SINK_KEYS of them -- go straight to this wavefront's LDS now, without registers, and are
  // used after the stream, when they have long arrived: the online softmax simply goes on over them.
  bool sink_part = false;
  int sink_first = 0, sink_keys = 0;
  char* lds_sink = lds_k + (kWgWaves - static_cast<int>(threadIdx.x) / kWave) * C::LDS_PER_WAVE +
                   (static_cast<int>(threadIdx.x) / kWave) * C::SINK_LDS;
  auto sink_row = [&](int t) -> const char* {
    int page = a.kv.contiguous ? s : bt[t >> a.page_shift];
    page = min(max(page, 0), p.num_pages - 1);
    return kvb + static_cast<uint64_t>(page) * page_b + static_cast<uint64_t>(t & (p.page_size - 1)) * stride_b + head_off;
  };
  if constexpr (kWaveOnly && kPass == 0 && kKv == 0) {
    if (a.pre.sink_aux != nullptr && (!(part.partial || part.in_workgroup) || range_lo == si.lo_al)) {
      sink_first = kv_start_of(p, s);
      sink_keys = max(0, min(a.pre.sink_n, a.pre.sink_limit - sink_first));
      sink_part = sink_keys > 0;
      if (sink_part) {
        // one wave-wide load of 16 bytes per lane covers 64 / (hd / 8) whole rows, laid out row after row
        // (a load that covers no whole number of rows spills its tail past the last staged row: the K region and the V
        // region are SINK_KEYS rows of the instantiation's width each, which holds that tail for every head_dim)
        const int pieces = hd >> 3, rows_per = kWave / pieces;
        const int staged = min(sink_keys, C::SINK_KEYS);
        for (int r0 = 0; r0 < staged; r0 += rows_per) {
          const char* src = sink_row(sink_first + min(r0 + lane / pieces, staged - 1)) + 16 * (lane % pieces);
          __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4_t*>(src),
                                           (__attribute__((address_space(3))) void*)(lds_sink + r0 * hd * 2), 16, 0, 0);
          __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4_t*>(src + v_delta),
                                           (__attribute__((address_space(3))) void*)(lds_sink + C::SINK_KEYS * D * 2 + r0 * hd * 2), 16, 0, 0);
        }
        // the biases of those positions for the 16 rows of this row tile, [row][key]: 4 bytes per lane, 8 rows per load
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
          const int rrow = max(min(row_lo + 8 * rr + (lane >> 3), si.rows - 1), 0);  // a row of the item (the last one repeats)
          const int brow = a.pre.sink_rows == 1 ? 0 : rrow % G;               // its query head within the kv head
          const int bt_ = min(sink_first + (lane & 7), a.pre.sink_n - 1);
          __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t*>(a.pre.sink_aux + static_cast<size_t>(brow) * a.pre.sink_n + bt_),
                                           (__attribute__((address_space(3))) void*)(lds_sink + C::SINK_KEYS * 2 * D * 2 + rr * 256), 4, 0, 0);
        }
      }
    }
  }

  if (range_hi > range_lo) {
    if constexpr (kPass == 1) {
      issue_loads(range_lo, vbuf0, vbuf1);
      if (range_lo + C::TT < range_hi) issue_loads(range_lo + C::TT, vbuf1, vbuf0);
    } else {
      issue_loads(range_lo, kreg, vbuf0);
    }
    for (int tile = range_lo; tile < range_hi; tile += 2 * C::TT) {
      body(tile, vbuf0, vbuf1);
      if (tile + C::TT >= range_hi) break;
      body(tile + C::TT, vbuf1, vbuf0);
    }
    if constexpr (kPass == 1) store_logits();
  }

  // ---- row sum across the four lane groups
  if constexpr (!kNorm) l_run = row_groups_sum(l_run);

  if constexpr (kWaveOnly && kPass == 0 && kKv == 0) {
    if (sink_part) {
      // Lane (row i, group g) holds q[32 ks + 8 g ..] and the outputs d = 128 sN + 32 g + 8 r + c: it takes those pieces
      // of a sink key's K and V rows, and the four groups of a row add up their parts of the dot product.
      const int bias_row = a.pre.sink_rows == 1 ? 0 : hg;
      const float* __restrict__ bias = a.pre.sink_aux + static_cast<size_t>(bias_row) * a.pre.sink_n;
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the rows staged in LDS have arrived
      for (int k = 0; k < sink_keys; ++k) {
        const int t = sink_first + k;
        u32x4_t kk[C::NKS], vv[C::NS][4];
#pragma unroll
        for (int ks = 0; ks < C::NKS; ++ks) kk[ks] = u32x4_t{0u, 0u, 0u, 0u};
#pragma unroll
        for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
          for (int r = 0; r < 4; ++r) vv[sN][r] = u32x4_t{0u, 0u, 0u, 0u};
        if (k < C::SINK_KEYS) {
          const char* krow = lds_sink + k * hd * 2;
          const char* vrow = lds_sink + C::SINK_KEYS * D * 2 + k * hd * 2;
#pragma unroll
          for (int ks = 0; ks < C::NKS; ++ks)
            if (32 * ks + 8 * g < hd) kk[ks] = *reinterpret_cast<const u32x4_t*>(krow + 2 * (32 * ks + 8 * g));
#pragma unroll
          for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (128 * sN + 32 * g + 8 * r < hd) vv[sN][r] = *reinterpret_cast<const u32x4_t*>(vrow + 2 * (128 * sN + 32 * g + 8 * r));
        } else {
          // more sinks than the staged ones: from memory, one key at a time
          const char* krow = sink_row(t);
          const char* vrow = krow + v_delta;
#pragma unroll
          for (int ks = 0; ks < C::NKS; ++ks)
            if (32 * ks + 8 * g < hd) kk[ks] = *reinterpret_cast<const u32x4_t*>(krow + 2 * (32 * ks + 8 * g));
#pragma unroll
          for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (128 * sN + 32 * g + 8 * r < hd) vv[sN][r] = *reinterpret_cast<const u32x4_t*>(vrow + 2 * (128 * sN + 32 * g + 8 * r));
        }
        float dot = 0.f;
#pragma unroll
        for (int ks = 0; ks < C::NKS; ++ks) {
          const u32x4_t qq = __builtin_bit_cast(u32x4_t, qreg[ks]);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            dot = fmaf(__uint_as_float(qq[e] << 16), __uint_as_float(kk[ks][e] << 16), dot);
            dot = fmaf(__uint_as_float(qq[e] & 0xffff0000u), __uint_as_float(kk[ks][e] & 0xffff0000u), dot);
          }
        }
        dot += __shfl_xor(dot, 16, kWave);
        dot += __shfl_xor(dot, 32, kWave);
        float sc = kMimic ? rbf(dot) : dot * post_scale;
        if (cap != 0.f) sc = soft_cap<kMimic>(sc, cap, inv_cap);
        if (t < a.pre.sink_n)
          sc += k < C::SINK_KEYS ? *reinterpret_cast<const float*>(lds_sink + C::SINK_KEYS * 2 * D * 2 + (C::SINK_KEYS * i + k) * 4)
                                 : bias[t];
        const float m_new = fmaxf(m_run, sc);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a bias of -inf takes its key out
        const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * kLog2e);
        float d = sc - m_use;
        if (kMimic) d = rbf(d);
        const float e = rbf(__builtin_amdgcn_exp2f(d * kLog2e));
        l_run = l_run * alpha + e;
        m_run = m_new;
#pragma unroll
        for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
          for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
              o_acc[sN][2 * c][r] = fmaf(e, __uint_as_float(vv[sN][r][c] << 16), o_acc[sN][2 * c][r] * alpha);
              o_acc[sN][2 * c + 1][r] = fmaf(e, __uint_as_float(vv[sN][r][c] & 0xffff0000u), o_acc[sN][2 * c + 1][r] * alpha);
            }
      }
    }
  }

  bool merged = false;
  if constexpr (kWaveOnly && kPass == 0 && kKv == 0 && C::NS == 1 && C::LDS_PER_WAVE >= 16 * D * 4 + 128) {
    if (part.in_workgroup) {
      // ---- the four wavefronts of the workgroup hold a quarter of this part each: all but one leave their state in
      // their own K tile (accumulator piece c of row i, lane group g at ((16 c + i) * 4 + g) * 16, then the rows'
      // maxima and sums), the merging one adds them to its own in wavefront order.  Every wavefront of the
      // workgroup comes here, with or without keys, so the barriers are complete.
      const int wv = static_cast<int>(threadIdx.x) / kWave;
      const int merger = kFew ? part.merger : 0;
      constexpr int kState = 16 * D * 4;
      if (wv != merger) {
#pragma unroll
        for (int c = 0; c < 8; ++c) *reinterpret_cast<f32x4_t*>(lds_k + ((16 * c + i) * 4 + g) * 16) = o_acc[0][c];
        if (g == 0) *reinterpret_cast<float2*>(lds_k + kState + 8 * i) = float2{m_run, l_run};
      }
      __syncthreads();
      if (wv != merger) {
        if (kFew && part.again) __syncthreads();  // (the merging wavefront has read the states: the K tiles may be written again)
        return;
      }
#pragma unroll 1
      for (int w = 0; w < kWgWaves; ++w) {
        if (w == wv) continue;
        const char* st = lds_k + (w - wv) * C::LDS_PER_WAVE;
        const float2 ml = *reinterpret_cast<const float2*>(st + kState + 8 * i);
        const float m_new = fmaxf(m_run, ml.x);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float keep = __builtin_amdgcn_exp2f((m_run - m_use) * kLog2e);
        const float wgt = __builtin_amdgcn_exp2f((ml.x - m_use) * kLog2e);
        l_run = l_run * keep + wgt * ml.y;
        m_run = m_new;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          const f32x4_t ov = *reinterpret_cast<const f32x4_t*>(st + ((16 * c + i) * 4 + g) * 16);
          o_acc[0][c] = o_acc[0][c] * keep + wgt * ov;
        }
      }
      if (kFew && part.again) __syncthreads();
      merged = true;
    }
  }
  // (kFew: what a workgroup has merged may still be one of several parts of its (sequence, kv head))
  if (part.partial && !(merged && (!kFew || part.first_w == part.last_w))) {
    // ---- partial to the workspace, then take a ticket; the last part merges all of them in stream order.
    // Who writes, who reads: this wavefront writes its slot; the wavefront that draws the last ticket of the
    // (sequence, kv head) -- any workgroup, usually on another XCD with another L2 -- reads every slot.  Partials are
    // written and read at agent scope (sc1): write-through stores and loads that do not hit in a non-coherent L2 meet
    // in memory-side storage, so no L2 write-back or invalidate is needed around the ticket.  The row statistics and
    // the ticket are relaxed atomics; the accumulators are 16-byte buffer accesses that carry the same scope bit
    // (atomics end at eight bytes, and eight-byte accesses cost a memory burst each: with 8 rows at head_dim 256 they
    // took a tenth of the kernel).  What the hand-off needs beyond that is order: every store of this wavefront must
    // have completed before its ticket increment can be seen.  The explicit s_waitcnt vmcnt(0) below provides that (on
    // gfx9 stores count in vmcnt, and a store leaves the counter when it has been acknowledged by the level its scope
    // bits write through to); the fences beside it only keep the compiler from moving memory operations across.  The
    // reader orders itself by data dependence: its loads are issued after the ticket value has come back and been
    // compared.
    //
    // The accumulators travel as they sit in registers: piece n (= 8 * slice + MFMA number) of row i, lane group g, is
    // the 16 bytes at ((n * 16 + i) * 4 + g) * 16 of the slot, so one store covers 64 contiguous bytes per valid row.
    const size_t slot = static_cast<size_t>(__builtin_amdgcn_readfirstlane(part.slot));
    constexpr int kAgentScope = 16;  // auxiliary bit 4 of a buffer access: sc1, coherent across the device's L2s
    const __amdgpu_buffer_rsrc_t slots_rsrc = __builtin_amdgcn_make_buffer_rsrc(a.partial_o, 0, 0x7fffffff, 0x00020000);
    auto slot_piece = [&](uint32_t sl, int n, int row) -> int {
      return static_cast<int>(sl * static_cast<uint32_t>(16 * D * 4) + static_cast<uint32_t>(((n * 16 + row) * 4 + g) * 16));
    };
    if (row_valid) {
      if constexpr (kPass != 1)
#pragma unroll
        for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
          for (int c = 0; c < 8; ++c)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, o_acc[sN][c]), slots_rsrc,
                                                   slot_piece(static_cast<uint32_t>(slot), sN * 8 + c, i), 0, kAgentScope);
      if (g == 0) {
        const uint64_t v = static_cast<uint64_t>(__float_as_uint(m_run)) | (static_cast<uint64_t>(__float_as_uint(l_run)) << 32);
        __hip_atomic_store(reinterpret_cast<uint64_t*>(a.partial_ml) + slot * 16 + i, v, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    uint32_t* ctr = a.counters + static_cast<size_t>(s) * p.num_kv_heads + j;
    uint32_t ticket = 0;
    if (lane == 0) ticket = __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ticket = __shfl(ticket, 0, kWave);
    if (ticket != static_cast<uint32_t>(part.last_w - part.first_w)) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    float M = -INFINITY, L = 0.f;
    if constexpr (kWaveOnly) {
      // A decode row tile has few rows (one per query head of the group), and a (sequence, kv head) of a small batch is
      // cut into many parts -- 128 for one sequence on 1024 wavefronts -- which this wavefront would read one after
      // the other at one memory latency each.  The lanes of the rows that do not exist take parts instead: with R
      // rows padded to rp = 2^k, lane row i reads row i % rp of part k0 + i / rp, 16 / rp parts at a time (times the
      // chunk), and the lanes of one row add up their sums at the end.
      const int R = row_hi - row_lo;
      const int rp = R <= 1 ? 1 : R <= 2 ? 2 : R <= 4 ? 4 : R <= 8 ? 8 : 16;
      const int pp = 16 / rp;
      const int rrow = i & (rp - 1), sub = i / rp;
      const bool rv = rrow < R;
      constexpr int kChunk = C::NS == 1 ? 2 : 1;
      const uint64_t* ml = reinterpret_cast<const uint64_t*>(a.partial_ml) + rrow;
      // One pass with a reference point of the lane's own that moves as parts come in (the parts' maxima are not read
      // ahead of their sums: that was a memory round trip of its own per 16 parts), and the next chunk's loads are in
      // flight while the current one is added: a merge of 128 parts waits for about three round trips instead of 24.
      float Mi = -INFINITY;
#pragma unroll
      for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
        for (int c = 0; c < 8; ++c) o_acc[sN][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if (rv) {
        const int step = kChunk * pp;
        uint64_t ml_a[kChunk], ml_b[kChunk];
        u32x4_t ov_a[kChunk][C::NS][8], ov_b[kChunk][C::NS][8];
        auto fetch = [&](int k0, uint64_t (&mlv)[kChunk], u32x4_t (&ov)[kChunk][C::NS][8]) {
#pragma unroll
          for (int c = 0; c < kChunk; ++c) {
            const size_t sl = part_slot(min(k0 + c * pp + sub, part.last_w), part.stream_a, part.sh);
            mlv[c] = __hip_atomic_load(ml + sl * 16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if constexpr (kPass != 1)
#pragma unroll
              for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
                for (int cc = 0; cc < 8; ++cc)
                  ov[c][sN][cc] = __builtin_amdgcn_raw_buffer_load_b128(slots_rsrc, slot_piece(static_cast<uint32_t>(sl), sN * 8 + cc, rrow),
                                                                        0, kAgentScope);
          }
        };
        auto take = [&](int k0, const uint64_t (&mlv)[kChunk], const u32x4_t (&ov)[kChunk][C::NS][8]) {
#pragma unroll
          for (int c = 0; c < kChunk; ++c) {
            if (k0 + c * pp + sub > part.last_w) continue;  // past the last part: the load repeated it, it is not added again
            const float mk = __uint_as_float(static_cast<uint32_t>(mlv[c]));
            const float lk = __uint_as_float(static_cast<uint32_t>(mlv[c] >> 32));
            const float m_new = fmaxf(Mi, mk);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            const float keep = __builtin_amdgcn_exp2f((Mi - m_use) * kLog2e);  // 1 while the point stays, 0 for the first part
            const float w = __builtin_amdgcn_exp2f((mk - m_use) * kLog2e);
            L = L * keep + w * lk;
            Mi = m_new;
            if constexpr (kPass != 1)
#pragma unroll
              for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
                for (int cc = 0; cc < 8; ++cc)
#pragma unroll
                  for (int r = 0; r < 4; ++r) o_acc[sN][cc][r] = o_acc[sN][cc][r] * keep + w * __uint_as_float(ov[c][sN][cc][r]);
          }
        };
        fetch(part.first_w, ml_a, ov_a);
        for (int k0 = part.first_w; k0 <= part.last_w; k0 += 2 * step) {
          const bool second = k0 + step <= part.last_w;
          if (second) fetch(k0 + step, ml_b, ov_b);
          take(k0, ml_a, ov_a);
          if (second) {
            if (k0 + 2 * step <= part.last_w) fetch(k0 + 2 * step, ml_a, ov_a);
            take(k0 + step, ml_b, ov_b);
          }
        }
      }
      // the lanes of one row: a common reference point, then sums
      M = Mi;
#pragma unroll
      for (int d = 1; d < 16; d <<= 1)
        if (d >= rp) M = fmaxf(M, __shfl_xor(M, d, kWave));
      {
        const float M_use = M == -INFINITY ? 0.f : M;
        const float to_row = __builtin_amdgcn_exp2f((Mi - M_use) * kLog2e);  // 0 for a lane that took no part
        L *= to_row;
        if constexpr (kPass != 1)
#pragma unroll
          for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
            for (int c = 0; c < 8; ++c) o_acc[sN][c] *= to_row;
      }
#pragma unroll
      for (int d = 1; d < 16; d <<= 1)
        if (d >= rp) {
          L += __shfl_xor(L, d, kWave);
          if constexpr (kPass != 1)
#pragma unroll
          for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
            for (int c = 0; c < 8; ++c)
#pragma unroll
              for (int r = 0; r < 4; ++r) o_acc[sN][c][r] += __shfl_xor(o_acc[sN][c][r], d, kWave);
        }
    } else {
    // The parts are read kMergeChunk at a time (more would take registers from the prefill tile, which shares this
    // kernel): all loads of a chunk are issued before the first is used, so the
    // merge costs one memory latency per chunk instead of two per part.
    constexpr int kMergeChunk = C::NS == 1 ? 2 : 1;
    const uint64_t* ml = reinterpret_cast<const uint64_t*>(a.partial_ml) + i;
    if (row_valid)
      for (int k0 = part.first_w; k0 <= part.last_w; k0 += 2 * kMergeChunk) {
        uint64_t v[2 * kMergeChunk];
#pragma unroll
        for (int c = 0; c < 2 * kMergeChunk; ++c) {
          const int k = min(k0 + c, part.last_w);
          v[c] = __hip_atomic_load(ml + static_cast<size_t>(part_slot(k, part.stream_a, part.sh)) * 16, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int c = 0; c < 2 * kMergeChunk; ++c) M = fmaxf(M, __uint_as_float(static_cast<uint32_t>(v[c])));
      }
    const float M_use = M == -INFINITY ? 0.f : M;
#pragma unroll
    for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
      for (int c = 0; c < 8; ++c) o_acc[sN][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    if (row_valid) {
      for (int k0 = part.first_w; k0 <= part.last_w; k0 += kMergeChunk) {
        uint64_t mlv[kMergeChunk];
        u32x4_t ov[kMergeChunk][C::NS][8];
#pragma unroll
        for (int c = 0; c < kMergeChunk; ++c) {
          const size_t sl = part_slot(min(k0 + c, part.last_w), part.stream_a, part.sh);
          mlv[c] = __hip_atomic_load(ml + sl * 16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if constexpr (kPass != 1)
#pragma unroll
          for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
            for (int cc = 0; cc < 8; ++cc)
              ov[c][sN][cc] = __builtin_amdgcn_raw_buffer_load_b128(slots_rsrc, slot_piece(static_cast<uint32_t>(sl), sN * 8 + cc, i), 0,
                                                                    kAgentScope);
        }
#pragma unroll
        for (int c = 0; c < kMergeChunk; ++c) {
          if (k0 + c > part.last_w) break;  // the tail of the last chunk repeats the last part: not added again
          const float mk = __uint_as_float(static_cast<uint32_t>(mlv[c]));
          const float lk = __uint_as_float(static_cast<uint32_t>(mlv[c] >> 32));
          const float w = __builtin_amdgcn_exp2f((mk - M_use) * kLog2e);
          L += w * lk;
          if constexpr (kPass != 1)
#pragma unroll
          for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
            for (int cc = 0; cc < 8; ++cc)
#pragma unroll
              for (int r = 0; r < 4; ++r) o_acc[sN][cc][r] += w * __uint_as_float(ov[c][sN][cc][r]);
        }
      }
    }
    }
    m_run = M;
    l_run = L;
    if (lane == 0) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  // ---- normalise (with optional sinks) and store
  if (!row_valid) return;
  if constexpr (kPass == 1) {
    if (g == 0) {
      float* st = a.stats + 2 * (static_cast<size_t>(si.q0 + qi) * p.num_q_heads + head);
      st[0] = m_run;
      st[1] = l_run;
    }
    return;
  }
  if (kWaveOnly && kPass == 0 && a.pre.ml != nullptr) {
    // keys an earlier kernel accumulated for this (token, head): one more part
    const size_t idx = static_cast<size_t>(si.q0 + qi) * p.num_q_heads + head;
    const float ms = a.pre.ml[2 * idx], ls = a.pre.ml[2 * idx + 1];
    const float M = fmaxf(m_run, ms);
    const float M_use = M == -INFINITY ? 0.f : M;
    const float w0 = __builtin_amdgcn_exp2f((m_run - M_use) * kLog2e), w1 = __builtin_amdgcn_exp2f((ms - M_use) * kLog2e);
    const float* po = a.pre.o + idx * hd;
#pragma unroll
    for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int d0 = 128 * sN + 32 * g + 8 * r;  // this lane holds d0 .. d0 + 7 of its row in o_acc[sN][0..7][r]
        if (d0 < hd) {
          const f32x4_t x0 = *reinterpret_cast<const f32x4_t*>(po + d0), x1 = *reinterpret_cast<const f32x4_t*>(po + d0 + 4);
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            o_acc[sN][c][r] = w0 * o_acc[sN][c][r] + w1 * x0[c];
            o_acc[sN][c + 4][r] = w0 * o_acc[sN][c + 4][r] + w1 * x1[c];
          }
        }
      }
    l_run = w0 * l_run + w1 * ls;
    m_run = M;
  }
  float num_scale = 1.f, denom = l_run;
  if (p.sinks != nullptr && p.num_sinks > 0) {
    const float* __restrict__ sk = p.sinks + static_cast<size_t>(head) * p.num_sinks;
    float smax = -INFINITY;
    for (int k = 0; k < p.num_sinks; ++k) smax = fmaxf(smax, sk[k]);
    const float mt = fmaxf(m_run, smax);
    float ssum = 0.f;
    for (int k = 0; k < p.num_sinks; ++k) ssum += expf(sk[k] - mt);
    num_scale = m_run == -INFINITY ? 0.f : expf(m_run - mt);
    denom = num_scale * l_run + ssum;
  }
  const float inv = kNorm ? out_scale(p) : num_scale * out_scale(p) / fmaxf(denom, 1e-6f);
  bf16_t* orow = out + q_row_off;
#pragma unroll
  for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      u32x4_t w;
#pragma unroll
      for (int e = 0; e < 4; ++e) w[e] = pack_bf16x2(o_acc[sN][2 * e][r] * inv, o_acc[sN][2 * e + 1][r] * inv);
      const int d0 = 128 * sN + 32 * g + 8 * r;
      if (pair) {
        if ((d0 >> 6) == hp) *reinterpret_cast<u32x4_t*>(orow + (d0 & 63)) = w;  // the half that is this row's head
      } else if (d0 < hd) {
        *reinterpret_cast<u32x4_t*>(orow + d0) = w;
      }
    }
}

}  // namespace rpa
