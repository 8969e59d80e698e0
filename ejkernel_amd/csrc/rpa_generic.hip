// Scalar fp32 ragged paged attention: one wavefront per (query row, kv head).
//
// This is the exactness kernel: any head_dim, page_size and dtype, no MFMA, fp32
// accumulation throughout.  It proves the page-table walk, the K/V de-interleave, the
// GQA mapping and the causal / window / kv_len masks, and it is the fallback for shapes
// the tiled kernels do not cover.  Semantics follow the reference's XLA implementation,
// ejkernel/kernels/_xla/ragged_page_attention/_xla_impl_fwd.py:39-201 (mask :128-136,
// soft cap :125-126, sinks :161-172, denominator clamp :174), except that key blocks
// lying entirely outside a sliding window are skipped instead of producing NaN.
#include "rpa_device.h"
#include "rpa_host.h"

namespace rpa {

constexpr int kMaxElemsPerLane = 8;  // head_dim <= 512

template <typename T, bool kBf16Compute>
__global__ __launch_bounds__(kWave) void rpa_generic_kernel(RpaParams p, KvLayout kvl, PreState pre) {
  extern __shared__ float q_lds[];  // [head_dim] scaled query row of the current head
  const int row = blockIdx.x;
  const int j = blockIdx.y;
  const int lane = threadIdx.x;
  const int D = p.head_dim;
  const int G = p.num_q_heads / p.num_kv_heads;
  const T* __restrict__ q = static_cast<const T*>(p.queries);
  T* __restrict__ out = static_cast<T*>(p.out);

  const int nseq = seq_count(p);
  const int total = batch_rows(p, nseq);
  const size_t row_base = (static_cast<size_t>(row) * p.num_q_heads + static_cast<size_t>(j) * G) * D;
  const int s = row < total ? seq_of_row(p, nseq, row) : 0;
  const SeqMeta sm = seq_meta(p, kvl.capacity, row < total ? s : 0);
  // rows past the ragged batch are defined as zero (so are rows that malformed row offsets leave without a sequence)
  if (row >= total || row < sm.q0 || row >= sm.q0 + sm.q_len) {
    for (int i = lane; i < G * D; i += kWave) Elem<T>::store(out + row_base + i, 0.f);
    return;
  }
  const int q_len = sm.q_len;
  const int kv_len = sm.kv_len;
  const int pos = kv_len - q_len + (row - sm.q0);
  const int hi = min(pos + 1, kv_len);
  const int lo = max(p.sliding_window > 0 ? max(0, pos - p.sliding_window + 1) : 0, kv_start_of(p, s));

  const bool t_is_bf16 = sizeof(T) == 2;
  // RPA_FLAG_FP32_LOGITS: q enters the dot product unscaled (divided by q_scale and rounded to the storage type, if
  // given), the fp32 logit is multiplied by softmax_scale * k_scale * q_scale, probabilities are rounded to the
  // storage type before P V (ragged_page_attention_v3, _kernel.py:221-262).
  const bool v3 = (p.flags & RPA_FLAG_FP32_LOGITS) != 0;
  const float scale = t_is_bf16 ? round_bf16(p.softmax_scale) : p.softmax_scale;
  const float post = p.softmax_scale * (p.k_scale > 0.f ? p.k_scale : 1.f) * (p.q_scale > 0.f ? p.q_scale : 1.f);
  const float o_scale = p.v_scale > 0.f ? p.v_scale : 1.f;
  // the reference's cap is a weakly typed scalar: it takes the logits' dtype before it divides and multiplies
  const float cap = kBf16Compute && !v3 ? round_bf16(p.logits_soft_cap) : p.logits_soft_cap;
  const int32_t* __restrict__ bt = p.block_tables + static_cast<size_t>(s) * p.pages_per_seq;

  for (int g = 0; g < G; ++g) {
    const int h = j * G + g;
    __syncthreads();
    for (int d = lane; d < D; d += kWave) {
      float v = Elem<T>::load(q + (static_cast<size_t>(row) * p.num_q_heads + h) * D + d);
      if (v3) {
        if (p.q_scale > 0.f) {
          v = v / p.q_scale;
          if (t_is_bf16) v = round_bf16(v);
        }
      } else {
        v *= scale;
        if (t_is_bf16 || kBf16Compute) v = round_bf16(v);
      }
      q_lds[d] = v;
    }
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[kMaxElemsPerLane];
#pragma unroll
    for (int e = 0; e < kMaxElemsPerLane; ++e) acc[e] = 0.f;

    for (int t0 = lo; t0 < hi; t0 += kWave) {
      const int t = t0 + lane;
      const bool valid = t < hi;
      const int tc = valid ? t : hi - 1;
      const int page = min(max(kvl.contiguous ? s : bt[tc / p.page_size], 0), p.num_pages - 1);
      const size_t k_off = static_cast<size_t>(page) * kvl.page_b + static_cast<size_t>(tc % p.page_size) * kvl.stride_b +
                           static_cast<size_t>(j) * kvl.head_b;  // bytes from the K (or V) base
      const T* __restrict__ kp = reinterpret_cast<const T*>(kvl.k_base + k_off);
      float sc = 0.f;
      for (int d = 0; d < D; ++d) {
        float kvv = Elem<T>::load(kp + d);
        if (kBf16Compute && !t_is_bf16) kvv = round_bf16(kvv);
        sc = fmaf(q_lds[d], kvv, sc);
      }
      if (v3) sc *= post;
      else if (kBf16Compute) sc = round_bf16(sc);
      if (cap != 0.f) {
        if (kBf16Compute && !v3) {
          sc = round_bf16(round_bf16(tanhf(round_bf16(sc / cap))) * cap);
        } else {
          sc = cap * tanhf(sc / cap);
        }
      }
      if (!valid) sc = -INFINITY;
      const float m_new = fmaxf(m, wave_max(sc));
      float pr;
      if (v3) {
        pr = valid ? expf(sc - m_new) : 0.f;
        if (t_is_bf16) pr = round_bf16(pr);
      } else if (kBf16Compute) {
        pr = valid ? round_bf16(expf(round_bf16(sc - m_new))) : 0.f;
      } else {
        pr = valid ? expf(sc - m_new) : 0.f;
      }
      const float alpha = expf(m - m_new);  // m == -inf on the first tile -> 0
      l = l * alpha + wave_sum(pr);
      m = m_new;
#pragma unroll
      for (int e = 0; e < kMaxElemsPerLane; ++e) acc[e] *= alpha;
      const int n_in_tile = min(kWave, hi - t0);
      const uint32_t off_lo = static_cast<uint32_t>(k_off), off_hi = static_cast<uint32_t>(k_off >> 32);
      for (int tt = 0; tt < n_in_tile; ++tt) {
        const float p_tt = __shfl(pr, tt, kWave);
        const size_t o = (static_cast<size_t>(__shfl(off_hi, tt, kWave)) << 32) | __shfl(off_lo, tt, kWave);
        const T* __restrict__ vp = reinterpret_cast<const T*>(kvl.v_base + o);
#pragma unroll
        for (int e = 0; e < kMaxElemsPerLane; ++e) {
          const int d = lane + e * kWave;
          if (d < D) {
            float vv = Elem<T>::load(vp + d);
            if (kBf16Compute && !t_is_bf16) vv = round_bf16(vv);
            acc[e] = fmaf(p_tt, vv, acc[e]);
          }
        }
      }
    }

    if (pre.ml != nullptr) {  // keys an earlier kernel accumulated for this (token, head): one more part
      const size_t idx = static_cast<size_t>(row) * p.num_q_heads + h;
      const float ms = pre.ml[2 * idx], ls = pre.ml[2 * idx + 1];
      const float M = fmaxf(m, ms);
      const float w0 = m == -INFINITY ? 0.f : expf(m - M), w1 = ms == -INFINITY ? 0.f : expf(ms - M);
#pragma unroll
      for (int e = 0; e < kMaxElemsPerLane; ++e) {
        const int d = lane + e * kWave;
        if (d < D) acc[e] = w0 * acc[e] + w1 * pre.o[idx * D + d];
      }
      l = w0 * l + w1 * ls;
      m = M;
    }
    float num_scale = 1.f, denom = l;
    if (p.sinks != nullptr && p.num_sinks > 0) {
      const float* __restrict__ sk = p.sinks + static_cast<size_t>(h) * p.num_sinks;
      float smax = -INFINITY;
      for (int i = 0; i < p.num_sinks; ++i) smax = fmaxf(smax, sk[i]);
      const float mt = fmaxf(m, smax);
      float ssum = 0.f;
      for (int i = 0; i < p.num_sinks; ++i) ssum += expf(sk[i] - mt);
      num_scale = (m == -INFINITY) ? 0.f : expf(m - mt);
      denom = num_scale * l + ssum;
    }
    denom = fmaxf(denom, 1e-6f);
#pragma unroll
    for (int e = 0; e < kMaxElemsPerLane; ++e) {
      const int d = lane + e * kWave;
      if (d < D) Elem<T>::store(out + (static_cast<size_t>(row) * p.num_q_heads + h) * D + d, num_scale * o_scale * acc[e] / denom);
    }
  }
}

int launch_generic(const RpaParams& p, const KvLayout& kv, hipStream_t stream, const PreState& pre) {
  if (p.head_dim > kMaxElemsPerLane * kWave) return RPA_ERR_UNSUPPORTED;
  if (p.total_tokens == 0) return RPA_OK;
  dim3 grid(p.total_tokens, p.num_kv_heads), block(kWave);
  const size_t lds = static_cast<size_t>(p.head_dim) * sizeof(float);
  const bool bf16c = p.compute == RPA_COMPUTE_BF16;
  if (p.dtype == RPA_DTYPE_BF16) {
    if (bf16c) hipLaunchKernelGGL((rpa_generic_kernel<bf16_t, true>), grid, block, lds, stream, p, kv, pre);
    else hipLaunchKernelGGL((rpa_generic_kernel<bf16_t, false>), grid, block, lds, stream, p, kv, pre);
  } else {
    if (bf16c) hipLaunchKernelGGL((rpa_generic_kernel<float, true>), grid, block, lds, stream, p, kv, pre);
    else hipLaunchKernelGGL((rpa_generic_kernel<float, false>), grid, block, lds, stream, p, kv, pre);
  }
  return hipGetLastError() == hipSuccess ? RPA_OK : RPA_ERR_LAUNCH;
}

}  // namespace rpa
