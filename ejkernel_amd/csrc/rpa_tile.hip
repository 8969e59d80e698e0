// Ragged paged attention on MFMA, one wavefront per work item, one launch per batch.
//
// Work item = (sequence, kv head, 16-row tile of the sequence's (query token, group head)
// rows, split of the key range).  A decode sequence (1-4 query tokens) is a single row
// tile whose key range is split along the sequence; the partial (m, l, O) of each split
// goes to the workspace and the last split to arrive (an atomic ticket per sequence and
// kv head) merges them in split order, so results do not depend on timing.  Work is
// discovered on the device from query_start_loc / context_lens / num_seqs; the host
// never reads them.
//
// Per iteration a wavefront streams TT = 16*NT tokens of its kv head: K and V rows are
// fetched with 16-byte loads in which each quarter-wave reads one whole contiguous row
// (256 B at head_dim 128), one iteration ahead of their use.  K goes through a
// wave-private LDS tile to reach the MFMA operand layout; V is transposed in registers
// (byte permutes).  Scores are S^T = K Q^T, outputs O^T = V^T P^T, so every lane owns one
// query row: the online-softmax state and the O rescale are lane-local, and the row
// maximum needs only two cross-lane steps per iteration.
//
// Numerics follow ejkernel/kernels/_xla/ragged_page_attention/_xla_impl_fwd.py:49,119-149:
// q is pre-multiplied by the bf16 scale and rounded to bf16, logits are rounded to bf16,
// probabilities are bf16, accumulation is fp32.
#include "rpa_device.h"
#include "rpa_host.h"

namespace rpa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

constexpr int kWgThreads = 256;
constexpr int kWgWaves = kWgThreads / kWave;
constexpr float kLog2e = 1.4426950408889634f;

struct TileArgs {
  RpaParams p;
  int target_items;   // upper bound used to size split length (and the workspace)
  int user_chunk;     // tokens per split requested by the caller, 0 = automatic
  int page_shift;     // log2(page_size) or -1
  uint32_t* counters; // [max_num_seqs * num_kv_heads], zero between launches
  float* partial_o;   // [slots][16][D]
  float* partial_ml;  // [slots][16][2]
};

struct SeqInfo {
  int q0, q_len, kv_len, rows, n_rt;
  int lo_al, hi;  // key range of the whole sequence, start aligned down to the tile
  bool eligible;  // single row tile: may be split along the keys
};

template <int TT>
__device__ __forceinline__ SeqInfo seq_info(const RpaParams& p, int s, int G) {
  SeqInfo si;
  si.q0 = p.query_start_loc[s];
  si.q_len = p.query_start_loc[s + 1] - si.q0;
  si.kv_len = p.context_lens[s];
  si.rows = si.q_len > 0 ? si.q_len * G : 0;
  si.n_rt = (si.rows + 15) >> 4;
  si.eligible = si.n_rt == 1;
  const int pos_min = si.kv_len - si.q_len;
  int lo = p.sliding_window > 0 ? max(0, pos_min - p.sliding_window + 1) : 0;
  si.lo_al = lo & ~(TT - 1);
  si.hi = max(si.kv_len, 0);
  return si;
}

__device__ __forceinline__ int n_splits_of(const SeqInfo& si, int chunk) {
  if (!si.eligible) return 1;
  const int span = si.hi - si.lo_al;
  return span <= chunk ? 1 : (span + chunk - 1) / chunk;
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

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return static_cast<uint32_t>(f32_to_bf16(lo)) | (static_cast<uint32_t>(f32_to_bf16(hi)) << 16);
}

template <int D, int NT, bool kMimic>
struct Cfg {
  static constexpr int NS = D / 128;        // 128-wide slices of head_dim
  static constexpr int NKS = D / 32;        // k-steps of the QK^T contraction
  static constexpr int TT = 16 * NT;        // tokens per iteration
  static constexpr int NSLOT = 4 * NT;      // tokens each lane fetches per iteration
  static constexpr int ROWB = D * 2 + 16;   // LDS bytes per K row (16 B pad: conflict-free b128 reads)
  static constexpr int LDS_PER_WAVE = TT * ROWB;
};

// Everything one wavefront needs for one work item.
template <int D, int NT, bool kMimic>
__device__ __forceinline__ void process_item(const TileArgs& a, char* __restrict__ lds_k, const SeqInfo& si, int s,
                                             int j, int rt, int split, int n_splits, int chunk, int slot_base) {
  using C = Cfg<D, NT, kMimic>;
  const RpaParams& p = a.p;
  const int lane = threadIdx.x & (kWave - 1);
  const int i = lane & 15, g = lane >> 4;
  const int G = p.num_q_heads / p.num_kv_heads;
  const bf16_t* __restrict__ q = static_cast<const bf16_t*>(p.queries);
  const bf16_t* __restrict__ kv = static_cast<const bf16_t*>(p.kv_pages);
  bf16_t* __restrict__ out = static_cast<bf16_t*>(p.out);
  const int W = p.sliding_window;

  // ---- rows of this tile and their key range
  const int row_lo = rt * 16, row_hi = min(row_lo + 16, si.rows);
  const int qi_min = row_lo / G, qi_max = (row_hi - 1) / G;
  const int pos_min = si.kv_len - si.q_len + qi_min, pos_max = si.kv_len - si.q_len + qi_max;
  int range_hi = min(si.kv_len, pos_max + 1);
  int range_lo = (W > 0 ? max(0, pos_min - W + 1) : 0) & ~(C::TT - 1);
  if (n_splits > 1) {
    range_lo = si.lo_al + split * chunk;
    range_hi = min(range_hi, range_lo + chunk);
  }
  // this lane's row
  const int R = row_lo + i;
  const bool row_valid = R < si.rows;
  const int qi = row_valid ? R / G : 0;
  const int hg = row_valid ? R - qi * G : 0;
  const int pos_n = row_valid ? si.kv_len - si.q_len + qi : -1;
  const int head = j * G + hg;
  const size_t q_row_off = (static_cast<size_t>(si.q0 + qi) * p.num_q_heads + head) * D;

  // ---- Q^T operands: lane (row i, group g) holds q[row][32 ks + 8 g .. +8], pre-scaled and rounded to bf16
  bf16x8_t qreg[C::NKS];
  {
    const float scale = round_bf16(p.softmax_scale);
#pragma unroll
    for (int ks = 0; ks < C::NKS; ++ks) {
      u32x4_t raw = {0u, 0u, 0u, 0u};
      if (row_valid) raw = *reinterpret_cast<const u32x4_t*>(q + q_row_off + 32 * ks + 8 * g);
      u32x4_t sc;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float lo = __uint_as_float(raw[e] << 16) * scale, hi = __uint_as_float(raw[e] & 0xffff0000u) * scale;
        sc[e] = pack_bf16x2(lo, hi);
      }
      qreg[ks] = __builtin_bit_cast(bf16x8_t, sc);
    }
  }

  f32x4_t o_acc[C::NS][8];
#pragma unroll
  for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
    for (int c = 0; c < 8; ++c) o_acc[sN][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;

  const size_t tok_stride = static_cast<size_t>(2) * p.num_kv_heads * D;  // elements between tokens
  const int32_t* __restrict__ bt = p.block_tables + static_cast<size_t>(s) * p.pages_per_seq;
  const int t_last = range_hi - 1;
  const float cap = p.logits_soft_cap;

  u32x4_t kreg[C::NSLOT][C::NS];
  u32x4_t vbuf0[C::NSLOT][C::NS], vbuf1[C::NSLOT][C::NS];

  // Page ids of this lane's token groups (tokens tile + 16u + 4g .. +3), read one iteration before the rows.
  int pg[NT];
  auto token_group = [&](int tile, int u, int& t4c) {
    t4c = min(tile + 16 * u + 4 * g, t_last & ~3);
  };
  auto load_pages = [&](int tile) {
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      int t4c;
      token_group(tile, u, t4c);
      pg[u] = bt[a.page_shift >= 0 ? (t4c >> a.page_shift) : (t4c / p.page_size)];
    }
  };
  // Fetch K and V of the TT tokens starting at `tile`: lane (i, g) takes tokens 16u + 4g + r (u < NT, r < 4),
  // 16-byte piece i (+16 per 128-slice) of each row, so a quarter-wave reads one contiguous row.  Tokens past
  // the end of the range are replaced by the last valid one (their scores are masked).
  auto issue_loads = [&](int tile, u32x4_t (&kr)[C::NSLOT][C::NS], u32x4_t (&vr)[C::NSLOT][C::NS]) {
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      int t4c;
      token_group(tile, u, t4c);
      const int rlim = min(3, t_last - t4c);
      const int slot = a.page_shift >= 0 ? (t4c & (p.page_size - 1)) : (t4c % p.page_size);
      const int page = min(max(pg[u], 0), p.num_pages - 1);
      const bf16_t* base = kv + (static_cast<size_t>(page) * p.page_size + slot) * tok_stride +
                           static_cast<size_t>(2 * j) * D + 8 * i;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const bf16_t* row = base + static_cast<size_t>(min(r, rlim)) * tok_stride;
#pragma unroll
        for (int sN = 0; sN < C::NS; ++sN) {
          kr[4 * u + r][sN] = *reinterpret_cast<const u32x4_t*>(row + 128 * sN);
          vr[4 * u + r][sN] = *reinterpret_cast<const u32x4_t*>(row + D + 128 * sN);
        }
      }
    }
    load_pages(tile + C::TT);
  };

  auto body = [&](int tile, u32x4_t (&vcur)[C::NSLOT][C::NS], u32x4_t (&vnext)[C::NSLOT][C::NS]) {
    // 1. K rows to the wave-private LDS tile: row = token within the tile, 16-byte piece i (+16 per slice)
#pragma unroll
    for (int u = 0; u < NT; ++u)
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int sN = 0; sN < C::NS; ++sN)
          *reinterpret_cast<u32x4_t*>(lds_k + (16 * u + 4 * g + r) * C::ROWB + 16 * (i + 16 * sN)) = kreg[4 * u + r][sN];
    // 2. next tile's K and V are requested now, a full iteration before they are needed
    if (tile + C::TT < range_hi) issue_loads(tile + C::TT, kreg, vnext);
    // 3. S^T = K Q^T: lane (token i of sub-tile u, group g) reads piece 4 ks + g of its row
    f32x4_t s_acc[NT];
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
    const bool need_mask = (tile + C::TT > range_hi) || (tile + C::TT - 1 > pos_min) || (W > 0 && tile <= pos_max - W);
    float tmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < NT; ++u)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float x = s_acc[u][r];
        if (kMimic) x = round_bf16(x);
        if (cap != 0.f) {
          if (kMimic) x = round_bf16(round_bf16(tanhf(round_bf16(x / cap))) * cap);
          else x = cap * tanhf(x / cap);
        }
        if (need_mask) {
          const int tok = tile + 16 * u + 4 * g + r;
          const bool keep = tok <= pos_n && tok < range_hi && (W <= 0 || tok > pos_n - W);
          x = keep ? x : -INFINITY;
        }
        sv[u][r] = x;
        tmax = fmaxf(tmax, x);
      }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    const float m_new = fmaxf(m_run, tmax);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * kLog2e);
    float psum = 0.f;
    uint32_t pw[2 * NT];
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      float pv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float d = sv[u][r] - m_use;
        if (kMimic) d = round_bf16(d);
        float e = __builtin_amdgcn_exp2f(d * kLog2e);
        e = round_bf16(e);  // probabilities enter P V as bf16, and the row sum adds the same rounded values
        pv[r] = e;
        psum += e;
      }
      pw[2 * u] = (__float_as_uint(pv[0]) >> 16) | (__float_as_uint(pv[1]) & 0xffff0000u);
      pw[2 * u + 1] = (__float_as_uint(pv[2]) >> 16) | (__float_as_uint(pv[3]) & 0xffff0000u);
    }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
        for (int c = 0; c < 8; ++c) o_acc[sN][c] *= alpha;
    }
    // 5. O^T += V^T P^T.  MFMA number c of slice sN yields d = 128 sN + 8 (row of the MFMA) + c; its A operand is
    //    column c of every fetched 8-wide piece, gathered from the token rows by byte permutes.
#pragma unroll
    for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
        uint32_t aw[2 * NT];
#pragma unroll
        for (int h = 0; h < 2 * NT; ++h)
          aw[h] = __builtin_amdgcn_perm(vcur[2 * h + 1][sN][c >> 1], vcur[2 * h][sN][c >> 1], sel);
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

  if (range_hi > range_lo) {
    load_pages(range_lo);
    issue_loads(range_lo, kreg, vbuf0);
    for (int tile = range_lo; tile < range_hi; tile += 2 * C::TT) {
      body(tile, vbuf0, vbuf1);
      if (tile + C::TT >= range_hi) break;
      body(tile + C::TT, vbuf1, vbuf0);
    }
  }

  // ---- row sum across the four lane groups
  l_run += __shfl_xor(l_run, 16, kWave);
  l_run += __shfl_xor(l_run, 32, kWave);

  if (n_splits > 1) {
    // ---- partial to the workspace, then take a ticket; the last split merges all of them in split order
    const size_t slot = static_cast<size_t>(slot_base + split);
    float* po = a.partial_o + (slot * 16 + i) * D;
    if (row_valid) {
#pragma unroll
      for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float* dst = po + 128 * sN + 32 * g + 8 * r;
          *reinterpret_cast<f32x4_t*>(dst) = f32x4_t{o_acc[sN][0][r], o_acc[sN][1][r], o_acc[sN][2][r], o_acc[sN][3][r]};
          *reinterpret_cast<f32x4_t*>(dst + 4) = f32x4_t{o_acc[sN][4][r], o_acc[sN][5][r], o_acc[sN][6][r], o_acc[sN][7][r]};
        }
      if (g == 0) {
        a.partial_ml[(slot * 16 + i) * 2] = m_run;
        a.partial_ml[(slot * 16 + i) * 2 + 1] = l_run;
      }
    }
    __threadfence();
    uint32_t* ctr = a.counters + static_cast<size_t>(s) * p.num_kv_heads + j;
    uint32_t ticket = 0;
    if (lane == 0) ticket = __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    ticket = __shfl(ticket, 0, kWave);
    if (ticket != static_cast<uint32_t>(n_splits - 1)) return;
    __threadfence();
    float M = -INFINITY;
    for (int k = 0; k < n_splits; ++k) {
      const float mk = a.partial_ml[((static_cast<size_t>(slot_base) + k) * 16 + i) * 2];
      M = fmaxf(M, row_valid ? mk : -INFINITY);
    }
    const float M_use = M == -INFINITY ? 0.f : M;
    float L = 0.f;
#pragma unroll
    for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
      for (int c = 0; c < 8; ++c) o_acc[sN][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    if (row_valid) {
      for (int k = 0; k < n_splits; ++k) {
        const size_t sl = static_cast<size_t>(slot_base) + k;
        const float mk = a.partial_ml[(sl * 16 + i) * 2];
        const float lk = a.partial_ml[(sl * 16 + i) * 2 + 1];
        const float w = __builtin_amdgcn_exp2f((mk - M_use) * kLog2e);
        L += w * lk;
        const float* src = a.partial_o + (sl * 16 + i) * D;
#pragma unroll
        for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const f32x4_t x0 = *reinterpret_cast<const f32x4_t*>(src + 128 * sN + 32 * g + 8 * r);
            const f32x4_t x1 = *reinterpret_cast<const f32x4_t*>(src + 128 * sN + 32 * g + 8 * r + 4);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
              o_acc[sN][c][r] += w * x0[c];
              o_acc[sN][c + 4][r] += w * x1[c];
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
  const float inv = num_scale / fmaxf(denom, 1e-6f);
  bf16_t* orow = out + q_row_off;
#pragma unroll
  for (int sN = 0; sN < C::NS; ++sN)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      u32x4_t w;
#pragma unroll
      for (int e = 0; e < 4; ++e) w[e] = pack_bf16x2(o_acc[sN][2 * e][r] * inv, o_acc[sN][2 * e + 1][r] * inv);
      *reinterpret_cast<u32x4_t*>(orow + 128 * sN + 32 * g + 8 * r) = w;
    }
}

template <int D, int NT, bool kMimic>
__global__ __launch_bounds__(kWgThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void rpa_tile_kernel(TileArgs a) {
  using C = Cfg<D, NT, kMimic>;
  extern __shared__ __align__(16) char smem[];
  const RpaParams& p = a.p;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int G = p.num_q_heads / p.num_kv_heads;
  // LDS: [4 waves x K tile][item_start: S+1][slot_start: S+1][scratch 8 ints]
  char* lds_k = smem + wave * C::LDS_PER_WAVE;
  int* item_start = reinterpret_cast<int*>(smem + kWgWaves * C::LDS_PER_WAVE);
  int* slot_start = item_start + (p.max_num_seqs + 1);
  int* scratch = slot_start + (p.max_num_seqs + 1);

  int nseq = p.num_seqs[0];
  nseq = min(max(nseq, 0), p.max_num_seqs);

  // ---- schedule: split length from the batch's total decode keys, then items and partial slots per sequence
  const int per = (nseq + kWgThreads - 1) / kWgThreads;
  const int s_begin = min(tid * per, nseq), s_end = min(s_begin + per, nseq);
  int my_tok = 0;
  for (int s = s_begin; s < s_end; ++s) {
    const SeqInfo si = seq_info<C::TT>(p, s, G);
    if (si.eligible) my_tok += (si.hi - si.lo_al + 63) >> 6;  // in units of 64 keys: no overflow
  }
  int tot64;
  block_excl_scan(my_tok, scratch, tot64);
  long long want = (static_cast<long long>(tot64) * 64 * p.num_kv_heads + a.target_items - 1) / a.target_items;
  int chunk = static_cast<int>(min(want, static_cast<long long>(1) << 30));
  chunk = max(chunk, a.user_chunk > 0 ? a.user_chunk : 4 * C::TT);
  chunk = (chunk + C::TT - 1) & ~(C::TT - 1);

  int my_items = 0, my_slots = 0;
  for (int s = s_begin; s < s_end; ++s) {
    const SeqInfo si = seq_info<C::TT>(p, s, G);
    const int ns = n_splits_of(si, chunk);
    my_items += p.num_kv_heads * si.n_rt * ns;
    my_slots += ns > 1 ? p.num_kv_heads * ns : 0;
  }
  int total_items, total_slots;
  int item_base = block_excl_scan(my_items, scratch, total_items);
  int slot_base = block_excl_scan(my_slots, scratch, total_slots);
  for (int s = s_begin; s < s_end; ++s) {
    const SeqInfo si = seq_info<C::TT>(p, s, G);
    const int ns = n_splits_of(si, chunk);
    item_start[s] = item_base;
    slot_start[s] = slot_base;
    item_base += p.num_kv_heads * si.n_rt * ns;
    slot_base += ns > 1 ? p.num_kv_heads * ns : 0;
  }
  if (tid == 0) item_start[nseq] = total_items;
  __syncthreads();

  // ---- rows past the ragged batch are zero
  {
    const int total_rows = p.query_start_loc[nseq];
    const int row_u4 = p.num_q_heads * D / 8;  // 16-byte pieces per row
    u32x4_t* o4 = static_cast<u32x4_t*>(p.out);
    for (int row = total_rows + blockIdx.x; row < p.total_tokens; row += gridDim.x)
      for (int k = tid; k < row_u4; k += kWgThreads) o4[static_cast<size_t>(row) * row_u4 + k] = u32x4_t{0u, 0u, 0u, 0u};
  }

  // ---- items, strided over all wavefronts of the grid
  const int n_waves = gridDim.x * kWgWaves;
  for (int w = blockIdx.x * kWgWaves + wave; w < total_items; w += n_waves) {
    int lo = 0, hi = nseq;  // largest s with item_start[s] <= w
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (item_start[mid] <= w) lo = mid; else hi = mid;
    }
    const int s = lo;
    const SeqInfo si = seq_info<C::TT>(p, s, G);
    const int ns = n_splits_of(si, chunk);
    int local = w - item_start[s];
    const int j = local % p.num_kv_heads;
    local /= p.num_kv_heads;
    const int split = local % ns;
    const int rt = local / ns;
    process_item<D, NT, kMimic>(a, lds_k, si, s, j, rt, split, ns, chunk, slot_start[s] + j * ns);
  }
}

// ----------------------------------------------------------------------------- host side

static int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  return v && *v ? atoi(v) : dflt;
}

bool tiled_supported(const RpaParams& p) {
  if (p.flags & RPA_FLAG_FORCE_GENERIC) return false;
  if (p.dtype != RPA_DTYPE_BF16 || p.compute != RPA_COMPUTE_BF16) return false;
  if (p.head_dim != 128 && p.head_dim != 256) return false;
  if (p.page_size % 4 != 0) return false;
  if (p.max_num_seqs > kTiledMaxSeqs) return false;
  if (static_cast<uint64_t>(p.max_num_seqs) * p.num_kv_heads * 4 > kWorkspaceTicketBytes) return false;
  return true;
}

void tiled_workspace_layout(const RpaParams& p, WorkspaceLayout* wl) {
  const uint64_t n_ctr = static_cast<uint64_t>(p.max_num_seqs) * p.num_kv_heads;
  const uint64_t slots = static_cast<uint64_t>(kTiledTargetItems) + n_ctr;
  // The ticket region has one size for every shape: a workspace reused across shapes must never hold
  // partial results where another shape keeps its tickets.
  wl->counters_bytes = kWorkspaceTicketBytes;
  wl->partial_o_off = wl->counters_bytes;
  wl->partial_o_bytes = (slots * 16 * p.head_dim * 4 + 255) & ~static_cast<uint64_t>(255);
  wl->partial_ml_off = wl->partial_o_off + wl->partial_o_bytes;
  wl->partial_ml_bytes = (slots * 16 * 2 * 4 + 255) & ~static_cast<uint64_t>(255);
  wl->total_bytes = wl->partial_ml_off + wl->partial_ml_bytes;
}

template <int D, int NT, bool kMimic>
static int launch_cfg(const TileArgs& a, int grid, hipStream_t stream) {
  using C = Cfg<D, NT, kMimic>;
  const size_t lds = static_cast<size_t>(kWgWaves) * C::LDS_PER_WAVE + (2 * (a.p.max_num_seqs + 1) + 8) * sizeof(int);
  hipLaunchKernelGGL((rpa_tile_kernel<D, NT, kMimic>), dim3(grid), dim3(kWgThreads), lds, stream, a);
  return hipGetLastError() == hipSuccess ? RPA_OK : RPA_ERR_LAUNCH;
}

int launch_tiled(const RpaParams& p, hipStream_t stream) {
  WorkspaceLayout wl;
  tiled_workspace_layout(p, &wl);
  if (p.workspace == nullptr || p.workspace_bytes < wl.total_bytes) return RPA_ERR_WORKSPACE;
  TileArgs a;
  a.p = p;
  a.target_items = min(kTiledTargetItems, max(64, env_int("RPA_TUNE_TARGET_ITEMS", kTiledTargetItems)));
  a.user_chunk = p.num_kv_pages_per_block > 0 ? p.num_kv_pages_per_block * p.page_size : 0;
  a.page_shift = (p.page_size & (p.page_size - 1)) == 0 ? __builtin_ctz(p.page_size) : -1;
  char* ws = static_cast<char*>(p.workspace);
  a.counters = reinterpret_cast<uint32_t*>(ws);
  a.partial_o = reinterpret_cast<float*>(ws + wl.partial_o_off);
  a.partial_ml = reinterpret_cast<float*>(ws + wl.partial_ml_off);
  const int grid = device_cu_count() * max(1, env_int("RPA_TUNE_WGS_PER_CU", 2));
  const bool mimic = env_int("RPA_TUNE_NO_MIMIC", 0) == 0;
  if (p.head_dim == 128) return mimic ? launch_cfg<128, 2, true>(a, grid, stream) : launch_cfg<128, 2, false>(a, grid, stream);
  return mimic ? launch_cfg<256, 1, true>(a, grid, stream) : launch_cfg<256, 1, false>(a, grid, stream);
}

}  // namespace rpa
