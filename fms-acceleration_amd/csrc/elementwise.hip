// Standalone SwiGLU forward / backward (UL/swiglu.py:20-98).  The fused GEMM epilogues apply the
// same arithmetic; these kernels serve the paths that cannot fuse it (act-order weights, whose
// gate/up/down projections each walk K in their own order) and the unfused baseline.
// HBM-bound: 16-byte vectors, one pass.
#include "common.h"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const uint16_t* __restrict__ e, const uint16_t* __restrict__ g,
                                                         uint16_t* __restrict__ h, int M, int I, int64_t ld) {
  const int64_t vec = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // over M * I / 8
  const int per_row = I / 8;
  if (vec >= (int64_t)M * per_row) return;
  const int64_t off = (vec / per_row) * ld + (vec % per_row) * 8;
  const u32x4 ev = *reinterpret_cast<const u32x4*>(e + off);
  const u32x4 gv = *reinterpret_cast<const u32x4*>(g + off);
  u32x4 hv;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float e0 = unpack_lo<T>(ev[i]), e1 = unpack_hi<T>(ev[i]);
    const uint32_t f = pack2<T>(e0 * sigmoidf_(e0), e1 * sigmoidf_(e1));
    hv[i] = pack2<T>(unpack_lo<T>(f) * unpack_lo<T>(gv[i]), unpack_hi<T>(f) * unpack_hi<T>(gv[i]));
  }
  *reinterpret_cast<u32x4*>(h + off) = hv;
}

// in place: h_out <- f*g, e <- d_g = dh*f, g <- d_e
template <typename T>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const uint16_t* __restrict__ dh, int64_t lddh,
                                                         uint16_t* __restrict__ e, uint16_t* __restrict__ g,
                                                         uint16_t* __restrict__ h, int M, int I, int64_t ld) {
  const int64_t vec = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int per_row = I / 8;
  if (vec >= (int64_t)M * per_row) return;
  const int64_t row = vec / per_row, col = (vec % per_row) * 8;
  const int64_t off = row * ld + col;
  const u32x4 dv = *reinterpret_cast<const u32x4*>(dh + row * lddh + col);
  const u32x4 ev = *reinterpret_cast<const u32x4*>(e + off);
  const u32x4 gv = *reinterpret_cast<const u32x4*>(g + off);
  u32x4 hv, dgv, dev;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float hh[2], dg[2], de[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const float e32 = j ? unpack_hi<T>(ev[i]) : unpack_lo<T>(ev[i]);
      const float g32 = j ? unpack_hi<T>(gv[i]) : unpack_lo<T>(gv[i]);
      const float DW = j ? unpack_hi<T>(dv[i]) : unpack_lo<T>(dv[i]);
      const float se = sigmoidf_(e32);
      const float f = unpack1<T>(pack1<T>(se * e32));
      hh[j] = f * g32;
      dg[j] = DW * f;
      const float dgt = unpack1<T>(pack1<T>(DW * g32));
      de[j] = dgt * se * (1.0f + e32 * (1.0f - se));
    }
    hv[i] = pack2<T>(hh[0], hh[1]);
    dgv[i] = pack2<T>(dg[0], dg[1]);
    dev[i] = pack2<T>(de[0], de[1]);
  }
  *reinterpret_cast<u32x4*>(h + off) = hv;
  *reinterpret_cast<u32x4*>(e + off) = dgv;
  *reinterpret_cast<u32x4*>(g + off) = dev;
}

}  // namespace

int launch_swiglu_fwd(const void* e, const void* g, void* h, int M, int I, int64_t ld, int act_dtype, hipStream_t st) {
  const int64_t nvec = (int64_t)M * (I / 8);
  dim3 grid((unsigned)((nvec + 255) / 256)), block(256);
  if (act_dtype == FMSA_BF16)
    hipLaunchKernelGGL(swiglu_fwd_kernel<bf16_t>, grid, block, 0, st, (const uint16_t*)e, (const uint16_t*)g,
                       (uint16_t*)h, M, I, ld);
  else
    hipLaunchKernelGGL(swiglu_fwd_kernel<f16_t>, grid, block, 0, st, (const uint16_t*)e, (const uint16_t*)g,
                       (uint16_t*)h, M, I, ld);
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}

int launch_swiglu_bwd(const void* dh, int64_t lddh, void* e, void* g, void* h, int M, int I, int64_t ld, int act_dtype,
                      hipStream_t st) {
  const int64_t nvec = (int64_t)M * (I / 8);
  dim3 grid((unsigned)((nvec + 255) / 256)), block(256);
  if (act_dtype == FMSA_BF16)
    hipLaunchKernelGGL(swiglu_bwd_kernel<bf16_t>, grid, block, 0, st, (const uint16_t*)dh, lddh, (uint16_t*)e,
                       (uint16_t*)g, (uint16_t*)h, M, I, ld);
  else
    hipLaunchKernelGGL(swiglu_bwd_kernel<f16_t>, grid, block, 0, st, (const uint16_t*)dh, lddh, (uint16_t*)e,
                       (uint16_t*)g, (uint16_t*)h, M, I, ld);
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}
