// The rank-r LoRA GEMMs.  Both stream one [M, C] activation matrix exactly once and are bound
// by HBM bandwidth, not by arithmetic:
//   lora_down  out[M, r]  = X[M, C] * Wd[r, C]^T          (U = Xd A^T,  T = dY B)
//   lora_grad  out[r, C]  = scale * L[M, r]^T * R[M, C]    (dA, dB: a reduction over tokens)
#include "common.h"

namespace {

// ---- lora_down ----------------------------------------------------------------------------------
// One workgroup = 16 tokens; its 4 waves split C into 4 contiguous quarters and each runs
// MFMA 16x16x32 over its quarter (X fragment straight from global: 16 rows x 64 B per load), then
// the four partial [16 x r] tiles are summed through LDS in a fixed order.
template <typename T, int RT>
__global__ __launch_bounds__(256) void lora_down_kernel(const uint16_t* __restrict__ X, int64_t ldx,
                                                        const uint16_t* __restrict__ Wd, int M, int C, int r,
                                                        uint16_t* __restrict__ out) {
  __shared__ float red[4][RT][64][4];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int l16 = lane & 15, q = lane >> 4;
  const int m = blockIdx.x * 16 + l16;
  const bool m_ok = m < M;
  // quarter boundaries in units of 32 columns
  const int n32 = (C + 31) / 32;
  const int per = (n32 + 3) / 4;
  const int c_begin = wave * per * 32;
  const int c_end = min(C, (wave + 1) * per * 32);

  f32x4 acc[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  const uint16_t* xrow = X + (size_t)(m_ok ? m : 0) * ldx + 8 * q;
#pragma unroll 2
  for (int c0 = c_begin; c0 < c_end; c0 += 32) {
    const bool c_ok = (c0 + 8 * q) < c_end;
    u32x4 xf = {0u, 0u, 0u, 0u};
    if (m_ok && c_ok) xf = *reinterpret_cast<const u32x4*>(xrow + c0);
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const int j = 16 * t + l16;
      u32x4 wf = {0u, 0u, 0u, 0u};
      if (j < r && c_ok) wf = *reinterpret_cast<const u32x4*>(Wd + (size_t)j * C + c0 + 8 * q);
      acc[t] = mfma16<T>(xf, wf, acc[t]);  // D[i = token][j = rank]
    }
  }
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][t][lane][i] = acc[t][i];
  __syncthreads();
  // lane l of the tile holds D[4*(l>>4) + i][l & 15]; 256 threads sum RT*256 outputs
  for (int o = tid; o < RT * 256; o += 256) {
    const int t = o >> 8, ln = (o >> 2) & 63, i = o & 3;
    const float v = (red[0][t][ln][i] + red[1][t][ln][i]) + (red[2][t][ln][i] + red[3][t][ln][i]);
    const int row = blockIdx.x * 16 + 4 * (ln >> 4) + i;
    const int j = 16 * t + (ln & 15);
    if (row < M && j < r) out[(size_t)row * r + j] = pack1<T>(v);
  }
}

// ---- lora_grad ----------------------------------------------------------------------------------
// Pass 1: a wave owns 128 adjacent columns of R (one bf16x2 per lane: 256 B rows) and a fixed
// range of tokens; the token's r coefficients L[m, :] are wave-uniform (scalar loads) and each
// R element is used for 16 FMAs.  Partial sums are written to partial[split][r][C] (fp32).
// Pass 2 adds the splits in index order, so the result does not depend on scheduling.
template <typename T>
__global__ __launch_bounds__(256) void lora_grad_partial_kernel(const uint16_t* __restrict__ L,
                                                                const uint16_t* __restrict__ R, int64_t ldr, int M,
                                                                int C, int r, int rows_per_split,
                                                                float* __restrict__ partial) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int split = blockIdx.y * 4 + wave;
  const int c = blockIdx.x * 128 + 2 * lane;
  const bool c_ok = c < C;
  const int m_begin = split * rows_per_split;
  const int m_end = min(M, m_begin + rows_per_split);
  const uint16_t* rp = R + (c_ok ? c : 0);

  for (int j0 = 0; j0 < r; j0 += 16) {
    float acc0[16], acc1[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) acc0[j] = acc1[j] = 0.f;
    int m = m_begin;
    for (; m + 4 <= m_end; m += 4) {
      uint32_t rv[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) rv[u] = *reinterpret_cast<const uint32_t*>(rp + (size_t)(m + u) * ldr);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float r0 = unpack_lo<T>(rv[u]), r1 = unpack_hi<T>(rv[u]);
        const uint16_t* lrow = L + (size_t)(m + u) * r + j0;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const float lj = (j0 + j < r) ? unpack1<T>(lrow[j]) : 0.f;
          acc0[j] = __builtin_fmaf(lj, r0, acc0[j]);
          acc1[j] = __builtin_fmaf(lj, r1, acc1[j]);
        }
      }
    }
    for (; m < m_end; ++m) {
      const uint32_t rv = *reinterpret_cast<const uint32_t*>(rp + (size_t)m * ldr);
      const float r0 = unpack_lo<T>(rv), r1 = unpack_hi<T>(rv);
      const uint16_t* lrow = L + (size_t)m * r + j0;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float lj = (j0 + j < r) ? unpack1<T>(lrow[j]) : 0.f;
        acc0[j] = __builtin_fmaf(lj, r0, acc0[j]);
        acc1[j] = __builtin_fmaf(lj, r1, acc1[j]);
      }
    }
    if (c_ok) {
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        if (j0 + j < r) {
          float2 v = make_float2(acc0[j], acc1[j]);
          *reinterpret_cast<float2*>(partial + ((size_t)split * r + j0 + j) * C + c) = v;
        }
      }
    }
  }
}

template <typename OutT, bool kF32>
__global__ __launch_bounds__(256) void lora_grad_reduce_kernel(const float* __restrict__ partial, int splits, int r,
                                                               int C, float scale, int transpose_out,
                                                               void* __restrict__ out) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;  // over r*C, c fastest
  if (idx >= r * C) return;
  const int j = idx / C, c = idx % C;
  float v = 0.f;
  for (int s = 0; s < splits; ++s) v += partial[((size_t)s * r + j) * C + c];
  v *= scale;
  const size_t o = transpose_out ? ((size_t)c * r + j) : (size_t)idx;
  if constexpr (kF32)
    reinterpret_cast<float*>(out)[o] = v;
  else
    reinterpret_cast<uint16_t*>(out)[o] = pack1<OutT>(v);
}

}  // namespace

int lora_grad_splits(int M, int C) {
  const int ncb = (C + 127) / 128;
  int splits = 1536 / ncb;
  const int max_splits = (M + 31) / 32;
  if (splits > max_splits) splits = max_splits;
  splits = (splits / 4) * 4;
  if (splits < 4) splits = 4;
  return splits;
}

int launch_lora_down(const void* X, int64_t ldx, const void* Wd, int M, int C, int r, int act_dtype, void* out,
                     hipStream_t st) {
  dim3 grid((M + 15) / 16), block(256);
  const int rt = (r + 15) / 16;
#define LAUNCH(TT, RT)                                                                                           \
  hipLaunchKernelGGL((lora_down_kernel<TT, RT>), grid, block, 0, st, (const uint16_t*)X, ldx, (const uint16_t*)Wd, \
                     M, C, r, (uint16_t*)out)
#define DISPATCH(TT)            \
  switch (rt) {                 \
    case 1: LAUNCH(TT, 1); break; \
    case 2: LAUNCH(TT, 2); break; \
    case 3: case 4: LAUNCH(TT, 4); break; \
    default: LAUNCH(TT, 8); break; \
  }
  if (act_dtype == FMSA_BF16) {
    DISPATCH(bf16_t)
  } else {
    DISPATCH(f16_t)
  }
#undef DISPATCH
#undef LAUNCH
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}

int launch_lora_grad(const void* L, const void* R, int64_t ldr, int M, int C, int r, float scale, int transpose_out,
                     int act_dtype, int out_dtype, void* out, void* workspace, hipStream_t st) {
  const int splits = lora_grad_splits(M, C);
  const int rows_per_split = (M + splits - 1) / splits;
  dim3 grid1((C + 127) / 128, splits / 4), block(256);
  if (act_dtype == FMSA_BF16)
    hipLaunchKernelGGL(lora_grad_partial_kernel<bf16_t>, grid1, block, 0, st, (const uint16_t*)L, (const uint16_t*)R,
                       ldr, M, C, r, rows_per_split, (float*)workspace);
  else
    hipLaunchKernelGGL(lora_grad_partial_kernel<f16_t>, grid1, block, 0, st, (const uint16_t*)L, (const uint16_t*)R,
                       ldr, M, C, r, rows_per_split, (float*)workspace);
  FMSA_CHECK_LAUNCH();
  dim3 grid2((r * C + 255) / 256);
  if (out_dtype == FMSA_F32)
    hipLaunchKernelGGL((lora_grad_reduce_kernel<float, true>), grid2, block, 0, st, (const float*)workspace, splits, r,
                       C, scale, transpose_out, out);
  else if (out_dtype == FMSA_BF16)
    hipLaunchKernelGGL((lora_grad_reduce_kernel<bf16_t, false>), grid2, block, 0, st, (const float*)workspace, splits,
                       r, C, scale, transpose_out, out);
  else
    hipLaunchKernelGGL((lora_grad_reduce_kernel<f16_t, false>), grid2, block, 0, st, (const float*)workspace, splits, r,
                       C, scale, transpose_out, out);
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}
