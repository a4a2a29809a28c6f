// Pre-pass: PARTIAL tiles from one byte per element to one bit per element.
//
// The reference's build_partial_block_data (omni-attn-mma/omni_attn_torch.py:148-205)
// hands the kernels bool tiles [P, QB, KB], one byte per (query, key) pair, and its
// kernels read them byte by byte (omni-attn-mma/mma/attn_naive.cu:143-154).  The forward
// here wants one 32-bit word per row and 32 keys.  It packs byte tiles on the fly; a
// caller that reuses a mask over many launches (every layer of a model, every step of a
// sampler) packs once with this kernel and passes the words instead: an eighth of the
// mask bytes per launch and no packing work inside the attention kernel.
//
// HBM-bound byte work: a thread reads 32 consecutive bytes (two 16-byte loads, neighbouring
// threads read neighbouring 32-byte runs) and writes one word; bit j of word i is byte
// 32 i + j, any non-zero byte counting as set (attn_naive.cu:151).  Rows are KB bytes and
// KB is a multiple of 32, so a word never straddles two rows and the word array is
// [P, QB, KB / 32] in the same row-major order.
#include "../../include/omni_attn_gfx950.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace omni_attn {
// Keeps the hipError_t behind an OMNI_ATTN_ERR_LAUNCH for omni_attn_last_hip_error() (defined
// beside that function).
void record_hip_error(int hip_error);
}  // namespace omni_attn

namespace {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

__device__ __forceinline__ uint32_t pack4(uint32_t bytes) {
  bytes |= bytes >> 4;  // fold every byte onto its lowest bit
  bytes |= bytes >> 2;
  bytes |= bytes >> 1;
  return ((bytes & 0x01010101u) * 0x01020408u) >> 24;  // bits 0..3 = bytes 0..3
}

__global__ void __launch_bounds__(256) pack_mask_kernel(const u32x4_t* __restrict__ bytes,
                                                        uint32_t* __restrict__ words, size_t n_words) {
  const size_t stride = size_t(gridDim.x) * blockDim.x;
  for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n_words; i += stride) {
    const u32x4_t lo = bytes[2 * i];
    const u32x4_t hi = bytes[2 * i + 1];
    uint32_t word = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      word |= pack4(lo[j]) << (4 * j);
      word |= pack4(hi[j]) << (16 + 4 * j);
    }
    words[i] = word;
  }
}

}  // namespace

extern "C" int omni_attn_pack_partial_masks_gfx950(const uint8_t* partial_masks, uint32_t* partial_bits,
                                                   int num_partial, int QB, int KB, void* stream) {
  if (num_partial < 0) return OMNI_ATTN_ERR_BAD_SHAPE;
  if (num_partial == 0) return OMNI_ATTN_OK;
  if (!partial_masks || !partial_bits) return OMNI_ATTN_ERR_NULL_POINTER;
  if ((QB != 64 && QB != 128) || (KB != 64 && KB != 128)) return OMNI_ATTN_ERR_UNSUPPORTED_BLOCK;
  if ((reinterpret_cast<uintptr_t>(partial_masks) & 15) != 0 || (reinterpret_cast<uintptr_t>(partial_bits) & 3) != 0)
    return OMNI_ATTN_ERR_MISALIGNED;
  const size_t n_words = size_t(num_partial) * QB * (KB / 32);
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e == hipSuccess && cus <= 0) e = hipErrorInvalidDevice;
  if (e != hipSuccess) {
    omni_attn::record_hip_error(int(e));
    return OMNI_ATTN_ERR_LAUNCH;
  }
  const size_t want = (n_words + 255) / 256;
  const size_t cap = size_t(cus) * 16;  // grid-stride beyond a few workgroups per compute unit
  const unsigned grid = unsigned(want < cap ? want : cap);
  const u32x4_t* src = reinterpret_cast<const u32x4_t*>(partial_masks);
  size_t n = n_words;
  void* args[] = {&src, &partial_bits, &n};
  e = hipLaunchKernel(reinterpret_cast<const void*>(pack_mask_kernel), dim3(grid), dim3(256), args, 0,
                      static_cast<hipStream_t>(stream));
  if (e != hipSuccess) {
    omni_attn::record_hip_error(int(e));
    return OMNI_ATTN_ERR_LAUNCH;
  }
  return OMNI_ATTN_OK;
}
