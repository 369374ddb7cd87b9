// Measurement support, not part of the hot path: a register-only MFMA loop that shows what the matrix pipe of
// the machine at hand sustains (all-zero operands: clock-bound; random bf16 operands: what the power limit leaves),
// and the same loop with the GEMM kernels' ratio of direct-to-LDS loads (one 1 KB load per wave and 8 MFMAs),
// which shows what those loads cost a wave that has nobody to hide behind; and, on top of that, the kernels' ratio of
// fragment reads from LDS (one 1 KB read per wave and 2 MFMAs, as the 256 x 64 wave tile needs) with one workgroup
// barrier per 64 MFMAs: the whole operand traffic of a main loop without any unpacking.
#include "common.h"

namespace {

FMSA_DEVI uint32_t probe_hash(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}

// MODE 0: zero operands; 1: random bf16 in +-[1, 2); 2: as 1, plus one buffer_load_dwordx4 ... lds per 8 MFMAs;
// 3: as 2, and the A operands of every 16 MFMAs come out of LDS (8 ds_read_b128, read one iteration ahead; from a second 32 KB array
// filled once), with an s_barrier every fourth iteration
template <int MODE>
__global__ __launch_bounds__(256) void probe_mfma_kernel(float* out, const uint32_t* src, int iters) {
  __shared__ __attribute__((aligned(1024))) uint32_t lds[8 * 1024];  // 32 KB: one 1 KB slot per (wave, load)
  // the fragments are read from an array of their own (filled once): reads of the array the direct loads write to would
  // make the compiler wait for all loads in flight before every read
  __shared__ __attribute__((aligned(1024))) uint32_t lds_f[MODE == 3 ? 8 * 1024 : 4];
  f32x16 acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
  u32x4 a[8], b[8];
#pragma unroll
  for (int f = 0; f < 8; ++f)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t ha = probe_hash(threadIdx.x * 64 + f * 8 + j + blockIdx.x * 7919), hb = probe_hash(ha + 12345);
      if (MODE == 0) ha = hb = 0;
      else {
        ha = (ha & 0x807f807fu) | 0x3f803f80u;
        hb = (hb & 0x807f807fu) | 0x3f803f80u;
      }
      a[f][j] = ha;
      b[f][j] = hb;
    }
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: the loads' LDS address and scalar offset derive from it
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(src, 1u << 20);
  u32x4 a2[8];  // MODE 3: the second of two fragment sets; the MFMAs of one iteration run on one set while the reads fill the other
  if (MODE == 3) {
    for (int i = lane; i < 2048; i += 64) lds_f[wave * 2048 + i] = (probe_hash(blockIdx.x * 8192 + wave * 2048 + i) & 0x807f807fu) | 0x3f803f80u;
    __syncthreads();
#pragma unroll
    for (int f = 0; f < 8; ++f) a2[f] = a[f];
  }
  // one iteration: 16 MFMAs on fragment set `cur`; every second MFMA is followed by a fragment read into set `nxt` (MODE 3),
  // MFMAs 0 and 8 by a direct load (MODE >= 2)
  auto iteration = [&](int it, u32x4(&cur)[8], u32x4(&nxt)[8]) {
    if (MODE == 3 && (it & 3) == 0) __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      acc[i] = mfma32<bf16_t>(cur[i & 7], b[(i >> 1) & 7], acc[i]);
      if (MODE == 3 && (i & 1) == 0)
        nxt[i >> 1] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(lds_f) + ((((it + 1) & 3) * 8 + (i >> 1)) * 1024 + lane * 16));
      if (MODE >= 2 && (i & 7) == 0)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)(reinterpret_cast<char*>(lds) + (2 * wave + (i >> 3)) * 1024),
                                                 16, lane * 16, (uint32_t)((it & 63) * 16384 + (2 * wave + (i >> 3)) * 1024), 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  for (int it = 0; it < iters; it += 2) {  // (iters is even)
    iteration(it, a, a2);
    iteration(it + 1, a2, a);
  }
  if (MODE >= 2) __builtin_amdgcn_s_waitcnt(0x0F70);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) s += acc[i][j];
  out[blockIdx.x * 256 + threadIdx.x] = s + (MODE >= 2 ? (float)lds[threadIdx.x] : 0.f);
}

}  // namespace

// The library's one entry point (bench.py --yardsticks binds it with ctypes).  iters even; `out`: n_workgroups * 256
// floats; `src`: >= 1 MiB of bf16 operands for modes 2 and 3.  Returns 0, or a negative FMSA_ERR_* code for bad arguments
// before any HIP call.  FLOP of a launch = n_workgroups * 4 * iters * 16 * 32768.
extern "C" int fmsa_probe_mfma(int mode, int iters, int n_workgroups, void* out, const void* src, void* stream) {
  if (!out || (mode >= 2 && !src)) return FMSA_ERR_NULL;
  if (mode < 0 || mode > 3 || iters <= 0 || (iters & 1) || n_workgroups <= 0 || n_workgroups > 65536) return FMSA_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  float* o = (float*)out;
  dim3 grid(n_workgroups), block(256);
  if (mode == 0) hipLaunchKernelGGL(probe_mfma_kernel<0>, grid, block, 0, st, o, (const uint32_t*)src, iters);
  else if (mode == 1) hipLaunchKernelGGL(probe_mfma_kernel<1>, grid, block, 0, st, o, (const uint32_t*)src, iters);
  else if (mode == 2) hipLaunchKernelGGL(probe_mfma_kernel<2>, grid, block, 0, st, o, (const uint32_t*)src, iters);
  else hipLaunchKernelGGL(probe_mfma_kernel<3>, grid, block, 0, st, o, (const uint32_t*)src, iters);
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}
