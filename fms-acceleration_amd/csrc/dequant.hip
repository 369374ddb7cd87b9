// Standalone GPTQ dequantisation and the integer repack / column-permute helpers.
// All three are HBM-bound byte movers: one thread owns 8 adjacent output columns so every
// global access is a 16-byte (or 32-byte for fp32 output) vector and a wave writes 1 KB rows.
#include "common.h"

// W[k, n] for k = 8*k8 .. 8*k8+7, n = 8*n8 .. 8*n8+7 per thread.
// CODEBOOK: W = code[q] * block_scale[k / group_size, n] (scales, qzeros, g_idx unused).
template <typename OutT, bool kF32, bool CODEBOOK>
__global__ __launch_bounds__(256) void gptq_dequant_kernel(const int32_t* __restrict__ qweight,
                                                           const uint16_t* __restrict__ scales,
                                                           const int32_t* __restrict__ qzeros,
                                                           const int32_t* __restrict__ g_idx, int K, int N,
                                                           int group_size, int n_groups, int zero_offset,
                                                           const float* __restrict__ code,
                                                           const float* __restrict__ block_scale,
                                                           void* __restrict__ out) {
  const int n8 = blockIdx.x * blockDim.x + threadIdx.x;
  const int k8 = blockIdx.y;
  if (n8 * 8 >= N) return;
  const int n0 = n8 * 8;
  const u32x4* qp = reinterpret_cast<const u32x4*>(qweight + (size_t)k8 * N + n0);
  const u32x4 qa = qp[0], qb = qp[1];
  const uint32_t qw[8] = {qa[0], qa[1], qa[2], qa[3], qb[0], qb[1], qb[2], qb[3]};
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int k = k8 * 8 + j;
    float v[8];
    if constexpr (CODEBOOK) {
      const float* bs = block_scale + (size_t)(k / group_size) * N + n0;
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = code[(qw[i] >> (4 * j)) & 0xF] * bs[i];
    } else {
      int g = g_idx ? g_idx[k] : k / group_size;
      if (g < 0) g += n_groups;  // UL/gptq/triton/kernels.py:88-91
      const u32x4 sc = *reinterpret_cast<const u32x4*>(scales + (size_t)g * N + n0);
      const uint32_t zw = (uint32_t)qzeros[(size_t)g * (N / 8) + n8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t sbits = (i & 1) ? (sc[i >> 1] >> 16) : (sc[i >> 1] & 0xffffu);
        const float sf = fp16_bits_to_f32((uint16_t)sbits);
        const int q = (int)((qw[i] >> (4 * j)) & 0xF);
        const int z = (int)((zw >> (4 * i)) & 0xF) + zero_offset;
        v[i] = sf * (float)(q - z);  // exact in fp32
      }
    }
    if constexpr (kF32) {
      f32x4* op = reinterpret_cast<f32x4*>(reinterpret_cast<float*>(out) + (size_t)k * N + n0);
      op[0] = f32x4{v[0], v[1], v[2], v[3]};
      op[1] = f32x4{v[4], v[5], v[6], v[7]};
    } else {
      u32x4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = pack2<OutT>(v[2 * i], v[2 * i + 1]);
      *reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(out) + (size_t)k * N + n0) = o;
    }
  }
}

int launch_gptq_dequant(const fmsa_gptq_weight* w, int out_dtype, void* out, hipStream_t st) {
  const int n_groups = (w->K + w->group_size - 1) / w->group_size;
  dim3 block(64);
  dim3 grid((w->N / 8 + 63) / 64, w->K / 8);
#define ARGS w->qweight, w->scales, w->qzeros, w->g_idx, w->K, w->N, w->group_size, n_groups, w->zero_offset, w->code, w->block_scale, out
#define LAUNCH(CB)                                                                           \
  do {                                                                                       \
    if (out_dtype == FMSA_F16)                                                               \
      hipLaunchKernelGGL((gptq_dequant_kernel<f16_t, false, CB>), grid, block, 0, st, ARGS);  \
    else if (out_dtype == FMSA_BF16)                                                         \
      hipLaunchKernelGGL((gptq_dequant_kernel<bf16_t, false, CB>), grid, block, 0, st, ARGS); \
    else                                                                                     \
      hipLaunchKernelGGL((gptq_dequant_kernel<float, true, CB>), grid, block, 0, st, ARGS);   \
  } while (0)
  if (w->format == FMSA_WEIGHT_CODEBOOK)
    LAUNCH(true);
  else
    LAUNCH(false);
#undef LAUNCH
#undef ARGS
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}

// q_out[k', n] = q[perm[k'], n]: unpack one nibble per source row, repack 8 destination rows.
__global__ __launch_bounds__(256) void gptq_permute_rows_kernel(const int32_t* __restrict__ qweight,
                                                                const int32_t* __restrict__ perm, int K, int N,
                                                                int32_t* __restrict__ out) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  const int k8 = blockIdx.y;
  if (n >= N) return;
  uint32_t acc = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int src = perm[k8 * 8 + j];
    const uint32_t wsrc = (uint32_t)qweight[(size_t)(src >> 3) * N + n];
    acc |= ((wsrc >> (4 * (src & 7))) & 0xFu) << (4 * j);
  }
  out[(size_t)k8 * N + n] = (int32_t)acc;
}

int launch_gptq_permute_rows(const int32_t* qweight, const int32_t* perm, int K, int N, int32_t* out,
                             hipStream_t st) {
  dim3 block(256);
  dim3 grid((N + 255) / 256, K / 8);
  hipLaunchKernelGGL(gptq_permute_rows_kernel, grid, block, 0, st, qweight, perm, K, N, out);
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}

// 16-bit column gather / scatter of a row-major activation matrix.
// Rows go through LDS: a random permutation read (or written) straight from global memory touches one 2-byte
// element per 64-byte sector and wave, so every workgroup pulls whole rows through its L1 to use 1/32 of them
// (67 MB gathered in 100 us, scattered in 260 us).  Here a workgroup loads ROWS whole rows with 16-byte accesses,
// permutes inside LDS (gather: read at perm[c]; scatter: write at perm[c]) and stores whole rows again.
template <bool GATHER>
__global__ __launch_bounds__(256) void permute_cols_lds_kernel(const uint16_t* __restrict__ in, int64_t ld_in,
                                                               const int32_t* __restrict__ perm, int M, int C, int rows,
                                                               uint16_t* __restrict__ out, int64_t ld_out) {
  extern __shared__ __attribute__((aligned(16))) uint16_t tile[];  // [rows][C]
  const int tid = threadIdx.x;
  const int m0 = blockIdx.x * rows;
  const int nr = min(rows, M - m0);
  const int chunks = C / 8;  // C % 8 == 0
  if (GATHER) {
    for (int i = tid; i < nr * chunks; i += 256) {
      const int rr = i / chunks, ch = i % chunks;
      *reinterpret_cast<u32x4*>(tile + (size_t)rr * C + 8 * ch) = *reinterpret_cast<const u32x4*>(in + (size_t)(m0 + rr) * ld_in + 8 * ch);
    }
    __syncthreads();
    for (int ch = tid; ch < chunks; ch += 256) {
      int p[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) p[k] = perm[8 * ch + k];
      for (int rr = 0; rr < nr; ++rr) {
        const uint16_t* row = tile + (size_t)rr * C;
        u32x4 v;
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = (uint32_t)row[p[2 * k]] | ((uint32_t)row[p[2 * k + 1]] << 16);
        *reinterpret_cast<u32x4*>(out + (size_t)(m0 + rr) * ld_out + 8 * ch) = v;
      }
    }
  } else {
    for (int ch = tid; ch < chunks; ch += 256) {
      int p[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) p[k] = perm[8 * ch + k];
      for (int rr = 0; rr < nr; ++rr) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(in + (size_t)(m0 + rr) * ld_in + 8 * ch);
        uint16_t* row = tile + (size_t)rr * C;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          row[p[2 * k]] = (uint16_t)(v[k] & 0xffffu);
          row[p[2 * k + 1]] = (uint16_t)(v[k] >> 16);
        }
      }
    }
    __syncthreads();
    for (int i = tid; i < nr * chunks; i += 256) {
      const int rr = i / chunks, ch = i % chunks;
      *reinterpret_cast<u32x4*>(out + (size_t)(m0 + rr) * ld_out + 8 * ch) = *reinterpret_cast<const u32x4*>(tile + (size_t)rr * C + 8 * ch);
    }
  }
}

// fallback for rows that do not fit into LDS or are not 16-byte aligned
__global__ __launch_bounds__(256) void permute_cols_kernel(const uint16_t* __restrict__ in, int64_t ld_in,
                                                           const int32_t* __restrict__ perm, int M, int C,
                                                           int gather, uint16_t* __restrict__ out,
                                                           int64_t ld_out) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int p = perm[c];
  const int m0 = blockIdx.y * 16;
#pragma unroll 4
  for (int i = 0; i < 16; ++i) {
    const int m = m0 + i;
    if (m >= M) break;
    if (gather)
      out[(size_t)m * ld_out + c] = in[(size_t)m * ld_in + p];
    else
      out[(size_t)m * ld_out + p] = in[(size_t)m * ld_in + c];
  }
}

int launch_permute_cols(const void* in, int64_t ld_in, const int32_t* perm, int M, int C, int gather,
                        void* out, int64_t ld_out, hipStream_t st) {
  dim3 block(256);
  const bool vec_ok = C % 8 == 0 && ld_in % 8 == 0 && ld_out % 8 == 0 && (reinterpret_cast<uintptr_t>(in) & 15u) == 0 &&
                      (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
  if (vec_ok && (size_t)C * 2 <= 64 * 1024) {
    // as many rows per workgroup as fit into 64 KB, but no fewer workgroups than about four per CU
    int rows = (int)(64 * 1024 / ((size_t)C * 2));
    while (rows > 1 && (M + rows - 1) / rows < 1024) rows >>= 1;
    if (rows > 8) rows = 8;
    const size_t lds = (size_t)rows * C * 2;
    dim3 grid((M + rows - 1) / rows);
    if (gather)
      hipLaunchKernelGGL(permute_cols_lds_kernel<true>, grid, block, lds, st, (const uint16_t*)in, ld_in, perm, M, C, rows,
                         (uint16_t*)out, ld_out);
    else
      hipLaunchKernelGGL(permute_cols_lds_kernel<false>, grid, block, lds, st, (const uint16_t*)in, ld_in, perm, M, C, rows,
                         (uint16_t*)out, ld_out);
    FMSA_CHECK_LAUNCH();
    return FMSA_OK;
  }
  dim3 grid((C + 255) / 256, (M + 15) / 16);
  hipLaunchKernelGGL(permute_cols_kernel, grid, block, 0, st, (const uint16_t*)in, ld_in, perm, M, C, gather,
                     (uint16_t*)out, ld_out);
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}
