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


// ---- the same loop with the forward kernel's other work beside the matrix instructions -----
//
// The device lowers its clock until the power fits, and how far depends on everything the loop
// does, operand values included.  This variant rotates eight operand sets, can take the A
// operand of every MFMA from LDS (16 bytes per lane: 1 KiB per wave and MFMA, the forward
// kernel's rate, fetched one round ahead) and can run the vector work of a softmax beside it
// (per MFMA one fma, one exp2 and one add on a value an earlier MFMA produced; per two MFMAs a
// max3 and a 16-bit pack), scheduled by the compiler.  No barriers, tile loads or bookkeeping:
// rate and clock of such a loop show what each kind of work costs beside the matrix
// instructions.  One wave also reports the shader clock it saw: s_memtime ticks (shader cycles)
// per s_memrealtime tick (100 MHz).
constexpr int kMixLds = 1;
constexpr int kMixSoftmax = 2;
constexpr int kMixSets = 8;

template <int MIX>
__global__ void __launch_bounds__(kThreads, 2) mfma_mix_kernel(int iters, float* sink, unsigned long long* ticks) {
  __shared__ u32x4_t tile[2048];  // 32 KiB: 8 KiB per wave, 8 fragments of 1 KiB
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  for (uint32_t i = tid; i < 2048u; i += kThreads)
#pragma unroll
    for (int j = 0; j < 4; ++j) tile[i][j] = operand_word(i + 2048u * blockIdx.x, uint32_t(j), true);
  __syncthreads();
  u32x4_t a[kMixSets], b[kMixSets];
#pragma unroll
  for (int i = 0; i < kMixSets; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      a[i][j] = operand_word(lane, uint32_t(8 * i + j), true);
      b[i][j] = operand_word(lane + 977u * blockIdx.x, uint32_t(8 * i + 4 + j), true);
    }
  f32x16_t acc[kMixSets];
#pragma unroll
  for (int c = 0; c < kMixSets; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
  const u32x4_t* frag = tile + wave * 512u + lane;
  float sum = 0.f, mx = -INFINITY, e_prev = 0.f, t_prev = 0.f;
  uint32_t packed = 0u;
  const unsigned long long t0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
    if constexpr ((MIX & kMixLds) != 0) {
      // the fragments the next round multiplies; the asm statement keeps the reads in the loop
      asm volatile("" ::: "memory");
#pragma unroll
      for (int c = 0; c < kMixSets; ++c) a[c] = frag[((it + c) & 7) * 64];
    }
#pragma unroll
    for (int c = 0; c < kMixSets; ++c) {
      acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[c]),
                                                       __builtin_bit_cast(bf16x8_t, b[c]), acc[c], 0, 0, 0);
      if constexpr ((MIX & kMixSoftmax) != 0) {
        const float t = __builtin_fmaf(acc[(c + 4) % kMixSets][c], 9.765625e-4f, -0.25f);
        const float e = __builtin_amdgcn_exp2f(t);
        sum += e;
        if (c & 1) {
          mx = __builtin_fmaxf(__builtin_fmaxf(mx, t), t_prev);
          asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(packed) : "v"(e), "v"(e_prev));
        }
        e_prev = e;
        t_prev = t;
        asm volatile("" : "+v"(sum), "+v"(mx));
      }
    }
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  float s = sum + mx + __builtin_bit_cast(float, packed);
#pragma unroll
  for (int c = 0; c < kMixSets; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[c][r];
  if (s == 12345.678f) sink[0] = s;
  if (tid == 0 && blockIdx.x == gridDim.x / 2 && ticks != nullptr) {
    ticks[0] = t1 - t0;
    ticks[1] = r1 - r0;
  }
}

// ---- what the vector pipe can do beside the matrix instructions of one SIMD --------------------
//
// One workgroup on one compute unit, 1 or 2 waves per SIMD.  Every wave runs a loop of groups:
// one MFMA (four accumulators in turn, so no instruction waits for another), then NP plain
// vector instructions (v_fma_f32) and NE transcendental ones (v_exp_f32) on registers the
// matrix instructions do not touch.  Cycles per group and SIMD, over NP and NE, show how much
// softmax work fits under a matrix instruction before the vector pipe becomes the longer one.
template <int NP, int NE>
__global__ void __launch_bounds__(512) issue_probe_kernel(int iters, unsigned long long* ticks, float seed) {
  f32x16_t acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[i][j] = seed * float(j);
  u32x4_t a, b;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    a[j] = operand_word(threadIdx.x, uint32_t(j), true);
    b[j] = operand_word(threadIdx.x + 977u, uint32_t(4 + j), true);
  }
  float v[8], e[2];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = seed + float(threadIdx.x) * 1e-3f + float(j);
  e[0] = seed;
  e[1] = -seed;
  __syncthreads();
  const unsigned long long t0 = __builtin_amdgcn_s_memtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                       __builtin_bit_cast(bf16x8_t, b), acc[m], 0, 0, 0);
#pragma unroll
      for (int j = 0; j < NP; ++j) asm volatile("v_fma_f32 %0, %0, %0, %0" : "+v"(v[j]));
#pragma unroll
      for (int j = 0; j < NE; ++j) asm volatile("v_exp_f32 %0, %0" : "+v"(e[j]));
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memtime();
  if ((threadIdx.x & 63u) == 0u) {
    ticks[2 * (threadIdx.x >> 6)] = t0;
    ticks[2 * (threadIdx.x >> 6) + 1] = t1;
  }
  float s = e[0] + e[1];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) s += acc[i][j];
#pragma unroll
  for (int j = 0; j < 8; ++j) s += v[j];
  if (s == 12345.678f) ticks[16] = 1;  // keeps the results alive; practically never true
}

template <int NP>
const void* issue_probe_for(int n_exp) {
  switch (n_exp) {
    case 0: return reinterpret_cast<const void*>(issue_probe_kernel<NP, 0>);
    case 1: return reinterpret_cast<const void*>(issue_probe_kernel<NP, 1>);
    case 2: return reinterpret_cast<const void*>(issue_probe_kernel<NP, 2>);
    default: return nullptr;
  }
}

}  // namespace

extern "C" int omni_attn_mfma_peak_probe_gfx950(int dtype, int iters, float* sink, double* flops_out,
                                                void* stream) {
  if (!sink || !flops_out) return OMNI_ATTN_ERR_NULL_POINTER;
  if (dtype != OMNI_ATTN_DTYPE_F16 && dtype != OMNI_ATTN_DTYPE_BF16) return OMNI_ATTN_ERR_UNSUPPORTED_DTYPE;
  if (iters <= 0 || iters > (1 << 24)) return OMNI_ATTN_ERR_BAD_SHAPE;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return OMNI_ATTN_ERR_LAUNCH;
  const unsigned grid = unsigned(cus) * kWorkgroupsPerCu;
  const void* kern = dtype == OMNI_ATTN_DTYPE_BF16 ? reinterpret_cast<const void*>(mfma_peak_kernel<true>)
                                                   : reinterpret_cast<const void*>(mfma_peak_kernel<false>);
  void* args[] = {&iters, &sink};
  if (hipLaunchKernel(kern, dim3(grid), dim3(kThreads), args, 0, static_cast<hipStream_t>(stream)) != hipSuccess)
    return OMNI_ATTN_ERR_LAUNCH;
  // waves x iterations x chains x (2 * 32 * 32 * 16) flop
  *flops_out = double(grid) * (kThreads / 64) * double(iters) * kChains * 32768.0;
  return OMNI_ATTN_OK;
}


extern "C" int omni_attn_mfma_mix_probe_gfx950(int mix, int iters, float* sink, unsigned long long* ticks,
                                               double* flops_out, void* stream) {
  if (!sink || !flops_out) return OMNI_ATTN_ERR_NULL_POINTER;
  if (mix < 0 || mix > 3 || iters <= 0 || iters > (1 << 24)) return OMNI_ATTN_ERR_BAD_SHAPE;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return OMNI_ATTN_ERR_LAUNCH;
  const unsigned grid = unsigned(cus) * kWorkgroupsPerCu;
  const void* kerns[4] = {reinterpret_cast<const void*>(mfma_mix_kernel<0>), reinterpret_cast<const void*>(mfma_mix_kernel<1>),
                          reinterpret_cast<const void*>(mfma_mix_kernel<2>), reinterpret_cast<const void*>(mfma_mix_kernel<3>)};
  void* args[] = {&iters, &sink, &ticks};
  if (hipLaunchKernel(kerns[mix], dim3(grid), dim3(kThreads), args, 0, static_cast<hipStream_t>(stream)) != hipSuccess)
    return OMNI_ATTN_ERR_LAUNCH;
  *flops_out = double(grid) * (kThreads / 64) * double(iters) * kMixSets * 32768.0;
  return OMNI_ATTN_OK;
}


extern "C" int omni_attn_issue_probe_gfx950(int n_plain, int n_exp, int waves_per_simd, int iters,
                                            unsigned long long* ticks, void* stream) {
  if (!ticks) return OMNI_ATTN_ERR_NULL_POINTER;
  if (n_plain < 0 || n_plain > 8 || (n_plain & 1) || n_exp < 0 || n_exp > 2 || waves_per_simd < 1 ||
      waves_per_simd > 2 || iters <= 0 || iters > (1 << 20))
    return OMNI_ATTN_ERR_BAD_SHAPE;
  const void* kern = nullptr;
  switch (n_plain) {
    case 0: kern = issue_probe_for<0>(n_exp); break;
    case 2: kern = issue_probe_for<2>(n_exp); break;
    case 4: kern = issue_probe_for<4>(n_exp); break;
    case 6: kern = issue_probe_for<6>(n_exp); break;
    default: kern = issue_probe_for<8>(n_exp); break;
  }
  float seed = 1e-3f;
  void* args[] = {&iters, &ticks, &seed};
  if (hipLaunchKernel(kern, dim3(1), dim3(256u * unsigned(waves_per_simd)), args, 0,
                      static_cast<hipStream_t>(stream)) != hipSuccess)
    return OMNI_ATTN_ERR_LAUNCH;
  return OMNI_ATTN_OK;
}
