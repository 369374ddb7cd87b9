// bitsandbytes NF4 dequantisation (UL/utils.py:86-141 of the reference calls the library's
// cdequantize_blockwise_fp32 for the double-quantised absmax and cdequantize_blockwise_*_nf4 for the
// weight): both steps in one HBM-bound pass, one thread per 8 packed bytes (16 weights, 32 B out).
//   absmax[b] = code2[absmax_q[b]] * absmax2[b / blocksize2] + offset      (fp32 mul, fp32 add)
//   W[i]      = code[nibble(i)] * absmax[i / blocksize]                     (fp32 mul, one RNE to out)
// with the even element of a byte in its high nibble.
#include "common.h"

namespace {

template <typename OutT, bool kF32>
__global__ __launch_bounds__(256) void nf4_dequant_kernel(const uint8_t* __restrict__ packed,
                                                          const uint8_t* __restrict__ absmax_q,
                                                          const float* __restrict__ absmax2,
                                                          const float* __restrict__ code2,
                                                          const float* __restrict__ code, float offset,
                                                          int64_t n_elements, int blocksize, int blocksize2,
                                                          void* __restrict__ out) {
  __shared__ float lut[16];
  if (threadIdx.x < 16) lut[threadIdx.x] = code[threadIdx.x];
  __syncthreads();
  const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;  // 16 weights each: 2^36 weights addressable
  const int64_t i0 = (int64_t)t * 16;
  if (i0 >= n_elements) return;
  const uint32_t b = t / (uint32_t)(blocksize >> 4);  // blocksize % 16 == 0
  // two roundings (the reference adds the offset to an already-rounded product): no fma contraction
  float absmax;
  {
#pragma clang fp contract(off)
    const float prod = code2[absmax_q[b]] * absmax2[b / blocksize2];
    absmax = prod + offset;
  }
  const u32x2 pk = *reinterpret_cast<const u32x2*>(packed + (i0 >> 1));
  float v[16];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const uint32_t byte = (pk[j >> 2] >> (8 * (j & 3))) & 0xffu;
    v[2 * j] = lut[byte >> 4] * absmax;
    v[2 * j + 1] = lut[byte & 0xF] * absmax;
  }
  if constexpr (kF32) {
    f32x4* op = reinterpret_cast<f32x4*>(reinterpret_cast<float*>(out) + i0);
#pragma unroll
    for (int j = 0; j < 4; ++j) op[j] = f32x4{v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]};
  } else {
    u32x4 o[2];
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j >> 2][j & 3] = pack2<OutT>(v[2 * j], v[2 * j + 1]);
    u32x4* op = reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(out) + i0);
    op[0] = o[0];
    op[1] = o[1];
  }
}

// Re-layout for the fused GEMM kernels.  One thread per output word: (k8, n) takes the four bytes
// of row n that hold elements 8*k8 .. 8*k8+7 (even element in the high nibble) and writes them
// with element j in bits 4j .. 4j+3; threads of a workgroup share k8 and walk n, so the stores are
// coalesced (the 4-byte reads are strided by K/2 bytes: a one-time cost on a frozen weight).
__global__ __launch_bounds__(256) void nf4_words_kernel(const uint8_t* __restrict__ packed, int N, int K,
                                                        int32_t* __restrict__ qweight_out) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  const int k8 = blockIdx.y;
  if (n >= N) return;
  const uint32_t bytes = *reinterpret_cast<const uint32_t*>(packed + ((size_t)n * K + 8 * (size_t)k8) / 2);
  uint32_t word = 0;
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const uint32_t byte = (bytes >> (8 * b)) & 0xffu;
    word |= (byte >> 4) << (8 * b);           // element 2b
    word |= (byte & 0xFu) << (8 * b + 4);     // element 2b + 1
  }
  qweight_out[(size_t)k8 * N + n] = (int32_t)word;
}

// block_scale[kb, n] = absmax of block (n, kb), i.e. of flat block n * (K / blocksize) + kb
__global__ __launch_bounds__(256) void nf4_block_scale_kernel(const uint8_t* __restrict__ absmax_q,
                                                              const float* __restrict__ absmax2,
                                                              const float* __restrict__ code2, float offset, int N,
                                                              int blocks_per_row, int blocksize2,
                                                              float* __restrict__ out) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  const int kb = blockIdx.y;
  if (n >= N) return;
  const uint32_t b = (uint32_t)n * (uint32_t)blocks_per_row + (uint32_t)kb;
  float absmax;
  {
#pragma clang fp contract(off)
    const float prod = code2[absmax_q[b]] * absmax2[b / blocksize2];
    absmax = prod + offset;
  }
  out[(size_t)kb * N + n] = absmax;
}

}  // namespace

int launch_nf4_prepare(const fmsa_nf4_weight* w, int32_t* qweight_out, float* block_scale_out, hipStream_t st) {
  dim3 block(256);
  hipLaunchKernelGGL(nf4_words_kernel, dim3((w->N + 255) / 256, w->K / 8), block, 0, st, w->packed, w->N, w->K, qweight_out);
  hipLaunchKernelGGL(nf4_block_scale_kernel, dim3((w->N + 255) / 256, w->K / w->blocksize), block, 0, st, w->absmax_q, w->absmax2,
                     w->code2, w->offset, w->N, w->K / w->blocksize, w->blocksize2, block_scale_out);
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}

int launch_nf4_dequant(const fmsa_nf4_weight* w, int out_dtype, void* out, hipStream_t st) {
  const int64_t n = (int64_t)w->N * w->K;
  dim3 block(256), grid((unsigned)((n / 16 + 255) / 256));
#define ARGS w->packed, w->absmax_q, w->absmax2, w->code2, w->code, w->offset, n, w->blocksize, w->blocksize2, out
  if (out_dtype == FMSA_F16)
    hipLaunchKernelGGL((nf4_dequant_kernel<f16_t, false>), grid, block, 0, st, ARGS);
  else if (out_dtype == FMSA_BF16)
    hipLaunchKernelGGL((nf4_dequant_kernel<bf16_t, false>), grid, block, 0, st, ARGS);
  else
    hipLaunchKernelGGL((nf4_dequant_kernel<float, true>), grid, block, 0, st, ARGS);
#undef ARGS
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}
