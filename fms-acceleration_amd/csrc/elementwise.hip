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

// ---- adapter pack ------------------------------------------------------------------------------
// One launch turns the two LoRA parameters (any float type) into the four activation-type copies
// the GEMM kernels read: A [r, K], A^T [K, r], B [N, r], B^T [r, N].  Each conversion is one RNE
// rounding of the parameter value (the `.to(dtype)` of UL/gptq/fast_lora.py:167).
template <typename TIN> FMSA_DEVI float load_param(const void* p, int64_t i);
template <> FMSA_DEVI float load_param<float>(const void* p, int64_t i) { return reinterpret_cast<const float*>(p)[i]; }
template <> FMSA_DEVI float load_param<bf16_t>(const void* p, int64_t i) { return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]); }
template <> FMSA_DEVI float load_param<f16_t>(const void* p, int64_t i) { return fp16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]); }

// The adapters of one fused operator go out together (one launch instead of one per projection); workgroup ids
// are laid end to end over the jobs.
struct LoraPackArgs {
  fmsa_lora_pack_job j[FMSA_LORA_PACK_MAX_JOBS];
  int block_start[FMSA_LORA_PACK_MAX_JOBS];
  int n_jobs;
};
FMSA_DEVI float load_param_rt(const void* p, int64_t i, int dtype) {
  if (dtype == FMSA_F32) return load_param<float>(p, i);
  return dtype == FMSA_BF16 ? load_param<bf16_t>(p, i) : load_param<f16_t>(p, i);
}

template <typename T>
__global__ __launch_bounds__(256) void lora_pack_kernel(const LoraPackArgs a) {
  // the job that owns this workgroup, copied field by field (no runtime index into the argument struct)
  fmsa_lora_pack_job J = a.j[0];
  int start = 0;
#pragma unroll
  for (int q = 1; q < FMSA_LORA_PACK_MAX_JOBS; ++q)
    if (q < a.n_jobs && (int)blockIdx.x >= a.block_start[q]) {
      J = a.j[q];
      start = a.block_start[q];
    }
  const int r = J.r, K = J.K, N = J.N;
  uint16_t* A16 = reinterpret_cast<uint16_t*>(J.A16);
  uint16_t* At16 = reinterpret_cast<uint16_t*>(J.At16);
  uint16_t* B16 = reinterpret_cast<uint16_t*>(J.B16);
  uint16_t* Bt16 = reinterpret_cast<uint16_t*>(J.Bt16);
  const int64_t idx = (int64_t)(blockIdx.x - start) * blockDim.x + threadIdx.x;
  if (idx < (int64_t)r * K) {
    const int j = (int)(idx / K), k = (int)(idx % K);
    const uint16_t v = pack1<T>(load_param_rt(J.A, idx, J.param_dtype));
    if (A16) A16[idx] = v;
    if (At16) At16[(int64_t)k * r + j] = v;
  }
  if (idx < (int64_t)N * r) {
    const int n = (int)(idx / r), j = (int)(idx % r);
    const uint16_t v = pack1<T>(load_param_rt(J.B, idx, J.param_dtype));
    if (B16) B16[idx] = v;
    if (Bt16) Bt16[(int64_t)j * N + n] = v;
  }
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

int launch_lora_pack_batch(const fmsa_lora_pack_job* jobs, int n_jobs, int act_dtype, hipStream_t st) {
  LoraPackArgs a{};
  a.n_jobs = n_jobs;
  int64_t blocks = 0;
  for (int q = 0; q < n_jobs; ++q) {
    a.j[q] = jobs[q];
    a.block_start[q] = (int)blocks;
    const int64_t n = (int64_t)jobs[q].r * (jobs[q].K > jobs[q].N ? jobs[q].K : jobs[q].N);
    blocks += (n + 255) / 256;
  }
  dim3 grid((unsigned)blocks), block(256);
  if (act_dtype == FMSA_BF16)
    hipLaunchKernelGGL(lora_pack_kernel<bf16_t>, grid, block, 0, st, a);
  else
    hipLaunchKernelGGL(lora_pack_kernel<f16_t>, grid, block, 0, st, a);
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}
