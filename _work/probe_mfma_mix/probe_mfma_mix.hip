// Measurement aid, not part of the op: a register-resident loop with the instruction mix of a prefill tile's key loop
// -- 32 v_mfma_f32_32x32x16_bf16 per block, a chosen number of softmax-like vector elements (scale, exp2, maximum,
// sum, packed conversion) and a chosen number of 16-byte LDS operand reads between them -- with nothing to wait for.
// Launched back to back it shows what the board sustains for that mix under its power limit, which is the ceiling a
// prefill tile with the same mix can reach; with no vector work and no LDS reads it is the ceiling of the matrix pipes
// themselves.  One workgroup of four wavefronts per compute unit, one wavefront per SIMD, as the pipelined tile runs.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

namespace {

constexpr int kLdsPieces = 2048;  // 16-byte pieces staged in LDS (32 KiB)
constexpr int kSrcPieces = kLdsPieces + 256 * 8;

// E: vector elements per block of 32 MFMAs (an element costs a multiply-add, an exp2, a maximum, an add and half a
// packed conversion); L: LDS operand reads per block.
template <int E, int L>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void mfma_mix_kernel(const uint4* __restrict__ src, float* __restrict__ dst, unsigned long long* __restrict__ clocks, int iters) {
  __shared__ uint4 lds[kLdsPieces];
  const int tid = threadIdx.x;
  // shader-clock counter and constant 100 MHz counter around the loop: their ratio is the clock the loop ran at
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int k = tid; k < kLdsPieces; k += 256) lds[k] = src[k];
  __syncthreads();
  bf16x8_t a[4], b[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    a[k] = __builtin_bit_cast(bf16x8_t, src[kLdsPieces + tid * 8 + k]);
    b[k] = __builtin_bit_cast(bf16x8_t, src[kLdsPieces + tid * 8 + 4 + k]);
  }
  f32x16_t acc[8];
#pragma unroll
  for (int k = 0; k < 8; ++k)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[k][r] = 0.f;
  float x[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) x[k] = 1e-3f * static_cast<float>((tid * 8 + k) & 1023);
  float mx = -1e30f, sum = 0.f, prev = 0.f;
  uint32_t packed = 0;
  int at = tid;
  for (int it = 0; it < iters; ++it) {
    const float bias = 1e-4f * static_cast<float>(it & 255);
#pragma unroll
    for (int m = 0; m < 32; ++m) {
      acc[m & 7] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[m & 3], b[(m >> 2) & 3], acc[m & 7], 0, 0, 0);
#pragma unroll
      for (int e = m * E / 32; e < (m + 1) * E / 32; ++e) {
        const float v = __builtin_fmaf(x[e & 7], 0.97f, bias);
        const float pr = __builtin_amdgcn_exp2f(v - 1.f);
        mx = __builtin_fmaxf(mx, v);
        sum += pr;
        if (e & 1) {
          const bf16x2_t pk = __builtin_convertvector(f32x2_t{prev, pr}, bf16x2_t);
          packed ^= __builtin_bit_cast(uint32_t, pk);
        }
        prev = pr;
        x[e & 7] = v;
      }
      if constexpr (L > 0) {
        if (m % (32 / L) == 0) {
          a[(m / (32 / L)) & 3] = __builtin_bit_cast(bf16x8_t, lds[at & (kLdsPieces - 1)]);
          at += 67;
        }
      }
    }
  }
  float total = mx + sum + __uint_as_float(packed & 0x3f800000u);
#pragma unroll
  for (int k = 0; k < 8; ++k)
#pragma unroll
    for (int r = 0; r < 16; ++r) total += acc[k][r];
  dst[blockIdx.x * 256 + tid] = total;
  if (tid == 0) {
    clocks[2 * blockIdx.x] = __builtin_readcyclecounter() - c0;
    clocks[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
}

// The same matrix work as 64 v_mfma_f32_16x16x32_bf16 per block (the shape the plain prefill tile and the decode loop
// use) and nothing else: what the smaller shape costs against the larger one.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void mfma_16x16_kernel(const uint4* __restrict__ src, float* __restrict__ dst, unsigned long long* __restrict__ clocks, int iters) {
  typedef __attribute__((ext_vector_type(4))) float f32x4_t;
  const int tid = threadIdx.x;
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  bf16x8_t a[4], b[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    a[k] = __builtin_bit_cast(bf16x8_t, src[kLdsPieces + tid * 8 + k]);
    b[k] = __builtin_bit_cast(bf16x8_t, src[kLdsPieces + tid * 8 + 4 + k]);
  }
  f32x4_t acc[16];
#pragma unroll
  for (int k = 0; k < 16; ++k) acc[k] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < 64; ++m)
      acc[m & 15] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[m & 3], b[(m >> 2) & 3], acc[m & 15], 0, 0, 0);
  }
  float total = 0.f;
#pragma unroll
  for (int k = 0; k < 16; ++k)
#pragma unroll
    for (int r = 0; r < 4; ++r) total += acc[k][r];
  dst[blockIdx.x * 256 + tid] = total;
  if (tid == 0) {
    clocks[2 * blockIdx.x] = __builtin_readcyclecounter() - c0;
    clocks[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
}

template <int E, int L>
int launch(int grid, const void* src, void* dst, void* clocks, int iters, hipStream_t stream) {
  hipLaunchKernelGGL((mfma_mix_kernel<E, L>), dim3(grid), dim3(256), 0, stream, static_cast<const uint4*>(src),
                     static_cast<float*>(dst), static_cast<unsigned long long*>(clocks), iters);
  return hipGetLastError() == hipSuccess ? 0 : -4;
}

}  // namespace

extern "C" {

// Bytes `src` must hold (any bf16 data; random normal values toggle the multipliers as real operands do).
uint64_t mfma_mix_probe_src_bytes(void) { return static_cast<uint64_t>(kSrcPieces) * 16; }

// One launch on `grid` workgroups (dst: grid * 256 floats; clocks: per workgroup the shader-clock cycles and the
// 100 MHz ticks its loop took).  vector_elements = -16 selects 64 MFMAs of the 16x16x32 shape per block, alone.  Returns the floating-point operations of the launch's MFMAs, or 0 for a mix that is
// not instantiated.
double mfma_mix_probe_launch(int vector_elements, int lds_reads, int grid, int iters, const void* src, void* dst, void* clocks,
                             void* stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  int rc = -1;
  if (vector_elements == 0 && lds_reads == 0) rc = launch<0, 0>(grid, src, dst, clocks, iters, s);
  else if (vector_elements == 0 && lds_reads == 16) rc = launch<0, 16>(grid, src, dst, clocks, iters, s);
  else if (vector_elements == 24 && lds_reads == 0) rc = launch<24, 0>(grid, src, dst, clocks, iters, s);
  else if (vector_elements == 48 && lds_reads == 0) rc = launch<48, 0>(grid, src, dst, clocks, iters, s);
  else if (vector_elements == 24 && lds_reads == 16) rc = launch<24, 16>(grid, src, dst, clocks, iters, s);
  else if (vector_elements == 48 && lds_reads == 16) rc = launch<48, 16>(grid, src, dst, clocks, iters, s);
  else if (vector_elements == 64 && lds_reads == 16) rc = launch<64, 16>(grid, src, dst, clocks, iters, s);
  else if (vector_elements == -16 && lds_reads == 0) {  // the 16x16x32 shape, MFMAs alone
    hipLaunchKernelGGL(mfma_16x16_kernel, dim3(grid), dim3(256), 0, s, static_cast<const uint4*>(src), static_cast<float*>(dst),
                       static_cast<unsigned long long*>(clocks), iters);
    rc = hipGetLastError() == hipSuccess ? 0 : -4;
  }
  if (rc != 0) return 0.0;
  return static_cast<double>(grid) * 4.0 * iters * 32.0 * (2.0 * 32 * 32 * 16);
}

}  // extern "C"
