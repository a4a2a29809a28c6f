// Measurement aid: what the matrix cores of this device sustain when nothing else runs.
//
// The forward kernel's roofline is quoted against the rated dense MFMA peak; the clock a
// launch actually gets depends on the power the whole instruction mix draws, so the bench
// also reports what a loop of nothing but v_mfma_f32_32x32x16_{bf16,f16} reaches on the same
// device, with two waves per SIMD (the forward kernel's occupancy) and operands that never
// leave registers.  No counterpart in the reference.
#include "../../include/omni_attn_gfx950.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace omni_attn {
// Keeps the hipError_t behind an OMNI_ATTN_ERR_LAUNCH for omni_attn_last_hip_error() (defined
// beside that function).
void record_hip_error(int hip_error);
}  // namespace omni_attn

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

constexpr int kChains = 8;          // independent accumulators per wave
constexpr int kThreads = 256;       // 4 waves: one per SIMD; two workgroups per CU
constexpr int kWorkgroupsPerCu = 2;

// 16-bit operand values with varied mantissas and signs, magnitude about 1 (a fixed
// pseudo-random pattern per lane and register: the power a matrix instruction draws
// depends on how many operand bits toggle).
__device__ __forceinline__ uint32_t operand_word(uint32_t lane, uint32_t i, bool bf16) {
  uint32_t x = (lane * 2654435761u) ^ (i * 0x9e3779b9u) ^ 0x85ebca6bu;
  x ^= x >> 15; x *= 0x2c1b3c6du; x ^= x >> 12; x *= 0x297a2d39u; x ^= x >> 15;
  // per half: sign, exponent of 0.5 .. 2, random mantissa
  const uint32_t expo = bf16 ? 0x3f00u : 0x3800u;
  const uint32_t mant_mask = bf16 ? 0x00ffu : 0x07ffu;  // mantissa + lowest exponent bit
  const uint32_t lo = (x & 0x8000u) | (expo + (x & mant_mask));
  const uint32_t hi = ((x >> 16) & 0x8000u) | (expo + ((x >> 17) & mant_mask));
  return lo | (hi << 16);
}

template <bool BF16>
__global__ void __launch_bounds__(kThreads, 2) mfma_peak_kernel(int iters, float* sink) {
  const uint32_t lane = threadIdx.x;
  u32x4_t a[2], b[2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      a[i][j] = operand_word(lane, 8 * i + j, BF16);
      b[i][j] = operand_word(lane + 977u * blockIdx.x, 8 * i + 4 + j, BF16);
    }
  f32x16_t acc[kChains];
#pragma unroll
  for (int c = 0; c < kChains; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int c = 0; c < kChains; ++c) {
      if constexpr (BF16) {
        acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[c & 1]),
                                                         __builtin_bit_cast(bf16x8_t, b[(c >> 1) & 1]),
                                                         acc[c], 0, 0, 0);
      } else {
        acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a[c & 1]),
                                                        __builtin_bit_cast(f16x8_t, b[(c >> 1) & 1]),
                                                        acc[c], 0, 0, 0);
      }
    }
  }
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < kChains; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[c][r];
  if (s == 12345.678f) sink[0] = s;  // keeps the accumulators alive; practically never true
}


}  // namespace

extern "C" int omni_attn_mfma_peak_probe_gfx950(int dtype, int iters, float* sink, double* flops_out,
                                                void* stream) {
  if (!sink || !flops_out) return OMNI_ATTN_ERR_NULL_POINTER;
  if (dtype != OMNI_ATTN_DTYPE_F16 && dtype != OMNI_ATTN_DTYPE_BF16) return OMNI_ATTN_ERR_UNSUPPORTED_DTYPE;
  if (iters <= 0 || iters > (1 << 24)) return OMNI_ATTN_ERR_BAD_SHAPE;
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e == hipSuccess && cus <= 0) e = hipErrorInvalidDevice;
  if (e != hipSuccess) {
    omni_attn::record_hip_error(int(e));
    return OMNI_ATTN_ERR_LAUNCH;
  }
  const unsigned grid = unsigned(cus) * kWorkgroupsPerCu;
  const void* kern = dtype == OMNI_ATTN_DTYPE_BF16 ? reinterpret_cast<const void*>(mfma_peak_kernel<true>)
                                                   : reinterpret_cast<const void*>(mfma_peak_kernel<false>);
  void* args[] = {&iters, &sink};
  e = hipLaunchKernel(kern, dim3(grid), dim3(kThreads), args, 0, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) {
    omni_attn::record_hip_error(int(e));
    return OMNI_ATTN_ERR_LAUNCH;
  }
  // waves x iterations x chains x (2 * 32 * 32 * 16) flop
  *flops_out = double(grid) * (kThreads / 64) * double(iters) * kChains * 32768.0;
  return OMNI_ATTN_OK;
}

