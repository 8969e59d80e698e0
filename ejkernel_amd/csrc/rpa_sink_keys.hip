// Sink keys of ragged_decode_attention: a short pre-pass in front of the attention kernels.
//
// The reference program (ejkernel/kernels/_xla/ragged_decode_attention/_xla_impl_fwd.py) defines attention sinks
// through the keys themselves: with softmax_aux of num_sinks entries, the keys at positions
// [sequence_start, sequence_start + num_sinks) are visible whatever sequence_end and the sliding window say
// (create_attention_mask, :71-75), and a key at absolute position t < num_sinks has softmax_aux[row][t] added to its
// logit after the soft cap (apply_attention_sinks_block, :98-134).  Every visible key with a bias lies in that
// range (a visible key is at or above sequence_start), so the range is taken out of what the attention kernels
// walk -- they start at sequence_start + num_sinks -- and is accumulated here, one wavefront per (sequence, query
// head), into an attention state (maximum, sum, unnormalised output), which the attention kernels merge
// into their own before normalising.  The logit arithmetic is that of the scalar kernel in rpa_generic.hip.
#include "rpa_device.h"
#include "rpa_host.h"

namespace rpa {

constexpr int kSinkWgWaves = 4;                     // (sequence, head) pairs per workgroup, one per wavefront
constexpr int kSinkGroups = 4;                      // keys in flight per wavefront: one per group of 16 lanes
constexpr int kSinkLanes = kWave / kSinkGroups;     // lanes that share one key's dot product
constexpr int kSinkMaxElemsPerLane = 512 / kSinkLanes;  // head_dim <= 512

// One wavefront per (sequence, query head).  Each group of 16 lanes walks every fourth sink key with its own
// attention state (the K and V rows of different keys are independent loads, so four are in flight at a time);
// the four states are merged at the end.
template <typename T, bool kBf16Compute>
__global__ __launch_bounds__(kSinkWgWaves * kWave) void sink_keys_kernel(RpaParams p, KvLayout kvl, SinkKeyArgs sk) {
  // workgroups of several wavefronts: launching one workgroup per (sequence, head) costs more than the work itself
  const int s = blockIdx.x, h = blockIdx.y * kSinkWgWaves + threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (h >= p.num_q_heads) return;
  const int grp = lane / kSinkLanes, l16 = lane % kSinkLanes;
  const int D = p.head_dim;
  const int G = p.num_q_heads / p.num_kv_heads;
  const int j = h / G, g = h - j * G;
  const T* __restrict__ q = static_cast<const T*>(p.queries);
  const bool t_is_bf16 = sizeof(T) == 2;
  const float scale = t_is_bf16 ? round_bf16(p.softmax_scale) : p.softmax_scale;
  const float cap = kBf16Compute ? round_bf16(p.logits_soft_cap) : p.logits_soft_cap;  // weakly typed scalar: the logits' dtype first
  const int start = kv_start_of(p, s);
  if (h == 0 && lane == 0) sk.main_start[s] = start + sk.num_sinks;
  const int n_keys = max(0, min(sk.num_sinks, sk.seq_len - start));
  const char* seq_k = kvl.k_base + static_cast<size_t>(s) * kvl.page_b + static_cast<size_t>(j) * kvl.head_b;
  const char* seq_v = kvl.v_base + static_cast<size_t>(s) * kvl.page_b + static_cast<size_t>(j) * kvl.head_b;
  const size_t idx = static_cast<size_t>(s) * p.num_q_heads + h;
  const float* __restrict__ bias = sk.aux + static_cast<size_t>(sk.aux_rows == 1 ? 0 : g) * sk.num_sinks;

  // this lane's elements of the scaled query row and of the output: d = l16 + 16 e
  float qv[kSinkMaxElemsPerLane], acc[kSinkMaxElemsPerLane];
#pragma unroll
  for (int e = 0; e < kSinkMaxElemsPerLane; ++e) {
    const int d = l16 + kSinkLanes * e;
    float v = d < D ? Elem<T>::load(q + idx * D + d) * scale : 0.f;
    if (t_is_bf16 || kBf16Compute) v = round_bf16(v);
    qv[e] = v;
    acc[e] = 0.f;
  }
  float m = -INFINITY, l = 0.f;
  for (int k0 = 0; k0 < n_keys; k0 += kSinkGroups) {
    const int k = k0 + grp;
    const bool live = k < n_keys;
    const int t = start + (live ? k : n_keys - 1);
    const T* __restrict__ kp = reinterpret_cast<const T*>(seq_k + static_cast<size_t>(t) * kvl.stride_b);
    const T* __restrict__ vp = reinterpret_cast<const T*>(seq_v + static_cast<size_t>(t) * kvl.stride_b);
    float part = 0.f;
#pragma unroll
    for (int e = 0; e < kSinkMaxElemsPerLane; ++e) {
      const int d = l16 + kSinkLanes * e;
      if (d < D) {
        float kvv = Elem<T>::load(kp + d);
        if (kBf16Compute && !t_is_bf16) kvv = round_bf16(kvv);
        part = fmaf(qv[e], kvv, part);
      }
    }
#pragma unroll
    for (int o = kSinkLanes / 2; o > 0; o >>= 1) part += __shfl_xor(part, o, kWave);  // sum over the group's lanes
    float sc = part;
    if (kBf16Compute) sc = round_bf16(sc);
    if (cap != 0.f) {
      if (kBf16Compute) sc = round_bf16(round_bf16(tanhf(round_bf16(sc / cap))) * cap);
      else sc = cap * tanhf(sc / cap);
    }
    if (t < sk.num_sinks) sc += bias[t];
    if (!live) sc = -INFINITY;
    const float m_new = fmaxf(m, sc);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a bias of -inf takes its key out
    const float alpha = expf(m - m_use);  // m == -inf before the first key -> 0
    float pr = expf(sc - m_use);
    if (kBf16Compute) pr = round_bf16(pr);
    l = l * alpha + pr;
    m = m_new;
#pragma unroll
    for (int e = 0; e < kSinkMaxElemsPerLane; ++e) {
      const int d = l16 + kSinkLanes * e;
      if (d < D) {
        float vv = Elem<T>::load(vp + d);
        if (kBf16Compute && !t_is_bf16) vv = round_bf16(vv);
        acc[e] = fmaf(pr, vv, acc[e] * alpha);
      }
    }
  }
  // merge the groups' states: lanes l16, l16 + 16, l16 + 32, l16 + 48 hold the same elements
#pragma unroll
  for (int o = kSinkLanes; o < kWave; o <<= 1) {
    const float m_o = __shfl_xor(m, o, kWave), l_o = __shfl_xor(l, o, kWave);
    const float M = fmaxf(m, m_o);
    const float M_use = M == -INFINITY ? 0.f : M;
    const float w0 = expf(m - M_use), w1 = expf(m_o - M_use);
#pragma unroll
    for (int e = 0; e < kSinkMaxElemsPerLane; ++e) acc[e] = w0 * acc[e] + w1 * __shfl_xor(acc[e], o, kWave);
    l = w0 * l + w1 * l_o;
    m = M;
  }
  if (grp == 0) {
#pragma unroll
    for (int e = 0; e < kSinkMaxElemsPerLane; ++e) {
      const int d = l16 + kSinkLanes * e;
      if (d < D) sk.pre_o[idx * D + d] = acc[e];
    }
    if (l16 == 0) {
      sk.pre_ml[2 * idx] = m;
      sk.pre_ml[2 * idx + 1] = l;
    }
  }
}

int launch_sink_keys(const RpaParams& p, const KvLayout& kv, const SinkKeyArgs& sk, hipStream_t stream) {
  if (p.head_dim > kSinkMaxElemsPerLane * kSinkLanes) return RPA_ERR_UNSUPPORTED;
  if (p.total_tokens == 0) return RPA_OK;
  dim3 grid(p.total_tokens, (p.num_q_heads + kSinkWgWaves - 1) / kSinkWgWaves), block(kSinkWgWaves * kWave);
  const size_t lds = 0;
  const bool bf16c = p.compute == RPA_COMPUTE_BF16;
  if (p.dtype == RPA_DTYPE_BF16) {
    if (bf16c) hipLaunchKernelGGL((sink_keys_kernel<bf16_t, true>), grid, block, lds, stream, p, kv, sk);
    else hipLaunchKernelGGL((sink_keys_kernel<bf16_t, false>), grid, block, lds, stream, p, kv, sk);
  } else {
    if (bf16c) hipLaunchKernelGGL((sink_keys_kernel<float, true>), grid, block, lds, stream, p, kv, sk);
    else hipLaunchKernelGGL((sink_keys_kernel<float, false>), grid, block, lds, stream, p, kv, sk);
  }
  return hipGetLastError() == hipSuccess ? RPA_OK : RPA_ERR_LAUNCH;
}

}  // namespace rpa
