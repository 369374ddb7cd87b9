// RMS layer norm (forward / backward) and rotary embedding, the two bandwidth-bound operators on
// either side of the q/k/v projections (reference: fms_acceleration_foak/kernels/unsloth/
// rms_layernorm.py:21-102 and rope_embedding.py:22-65).  One wave handles one row; a row is read
// twice (statistics, then output), the second time out of cache.
#include "common.h"

namespace {

// eight consecutive elements of a row as fp32, for the three storage types (tag = fmsa_dtype)
template <int D> struct Vec8;
template <> struct Vec8<FMSA_BF16> {
  static FMSA_DEVI void load(const void* p, int64_t i, float (&v)[8]) {
    const u32x4 w = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p) + i);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[2 * k] = unpack_lo<bf16_t>(w[k]);
      v[2 * k + 1] = unpack_hi<bf16_t>(w[k]);
    }
  }
  static FMSA_DEVI void store(void* p, int64_t i, const float (&v)[8]) {
    u32x4 w;
#pragma unroll
    for (int k = 0; k < 4; ++k) w[k] = pack2<bf16_t>(v[2 * k], v[2 * k + 1]);
    *reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(p) + i) = w;
  }
  static FMSA_DEVI float round(float x) { return unpack1<bf16_t>(pack1<bf16_t>(x)); }
};
template <> struct Vec8<FMSA_F16> {
  static FMSA_DEVI void load(const void* p, int64_t i, float (&v)[8]) {
    const u32x4 w = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p) + i);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[2 * k] = unpack_lo<f16_t>(w[k]);
      v[2 * k + 1] = unpack_hi<f16_t>(w[k]);
    }
  }
  static FMSA_DEVI void store(void* p, int64_t i, const float (&v)[8]) {
    u32x4 w;
#pragma unroll
    for (int k = 0; k < 4; ++k) w[k] = pack2<f16_t>(v[2 * k], v[2 * k + 1]);
    *reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(p) + i) = w;
  }
  static FMSA_DEVI float round(float x) { return unpack1<f16_t>(pack1<f16_t>(x)); }
};
template <> struct Vec8<FMSA_F32> {
  static FMSA_DEVI void load(const void* p, int64_t i, float (&v)[8]) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p) + i);
    const f32x4 b = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p) + i + 4);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[k] = a[k];
      v[4 + k] = b[k];
    }
  }
  static FMSA_DEVI void store(void* p, int64_t i, const float (&v)[8]) {
    *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p) + i) = f32x4{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p) + i + 4) = f32x4{v[4], v[5], v[6], v[7]};
  }
  static FMSA_DEVI float round(float x) { return x; }
};

FMSA_DEVI float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Y = round_W(x * inv_rms) * W, stored in X's type; r[row] = inv_rms = rsqrt(mean(x^2) + eps)
// (rms_layernorm.py:36-47).  GEMMA: everything in fp32, 1/sqrt, weight W + 1 (:99-109).
template <int XD, int WD, bool GEMMA>
__global__ __launch_bounds__(256) void rms_fwd_kernel(const void* __restrict__ X, int64_t ldx, const void* __restrict__ W, int M,
                                                      int C, float eps, void* __restrict__ Y, int64_t ldy, float* __restrict__ r) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= M) return;
  const int64_t xo = (int64_t)row * ldx, yo = (int64_t)row * ldy;
  float ss = 0.f;
  for (int c = 8 * lane; c < C; c += 512) {
    float x[8];
    Vec8<XD>::load(X, xo + c, x);
#pragma unroll
    for (int k = 0; k < 8; ++k) ss += x[k] * x[k];
  }
  ss = wave_sum(ss);
  const float var = ss / (float)C + eps;
  const float inv = GEMMA ? 1.0f / __builtin_sqrtf(var) : __builtin_amdgcn_rsqf(var);
  if (lane == 0) r[row] = inv;
  for (int c = 8 * lane; c < C; c += 512) {
    float x[8], w[8], y[8];
    Vec8<XD>::load(X, xo + c, x);
    Vec8<WD>::load(W, c, w);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      if (GEMMA)
        y[k] = x[k] * inv * (w[k] + 1.0f);
      else
        y[k] = Vec8<WD>::round(Vec8<WD>::round(x[k] * inv) * w[k]);
    }
    Vec8<XD>::store(Y, yo + c, y);
  }
}

// dX = inv/n * (n * dY_W - normed * sum(dY_W * normed)), dY_W = dY * W (GEMMA: W + 1), written over
// dY (rms_layernorm.py:71-86); all in fp32.
template <int XD, int WD, bool GEMMA>
__global__ __launch_bounds__(256) void rms_bwd_kernel(void* __restrict__ dY, int64_t lddy, const void* __restrict__ X, int64_t ldx,
                                                      const void* __restrict__ W, const float* __restrict__ r, int M, int C) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= M) return;
  const int64_t xo = (int64_t)row * ldx, go = (int64_t)row * lddy;
  const float inv = r[row];
  float dot = 0.f;
  for (int c = 8 * lane; c < C; c += 512) {
    float x[8], w[8], g[8];
    Vec8<XD>::load(X, xo + c, x);
    Vec8<WD>::load(W, c, w);
    Vec8<XD>::load(dY, go + c, g);
#pragma unroll
    for (int k = 0; k < 8; ++k) dot += g[k] * (GEMMA ? w[k] + 1.0f : w[k]) * (x[k] * inv);
  }
  dot = wave_sum(dot);
  const float n = (float)C;
  for (int c = 8 * lane; c < C; c += 512) {
    float x[8], w[8], g[8], o[8];
    Vec8<XD>::load(X, xo + c, x);
    Vec8<WD>::load(W, c, w);
    Vec8<XD>::load(dY, go + c, g);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float gw = g[k] * (GEMMA ? w[k] + 1.0f : w[k]);
      o[k] = inv / n * (n * gw - x[k] * inv * dot);
    }
    Vec8<XD>::store(dY, go + c, o);
  }
}

// Register-resident variants for 16-bit rows of at most 512 * NCH columns: every 16-byte chunk of
// the row is loaded once (all loads in flight together) and kept packed until the second phase.
template <int XD> FMSA_DEVI void unpack8(const u32x4& w, float (&v)[8]) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if (XD == FMSA_BF16) {
      v[2 * k] = unpack_lo<bf16_t>(w[k]);
      v[2 * k + 1] = unpack_hi<bf16_t>(w[k]);
    } else {
      v[2 * k] = unpack_lo<f16_t>(w[k]);
      v[2 * k + 1] = unpack_hi<f16_t>(w[k]);
    }
  }
}

template <int XD, int WD, bool GEMMA, int NCH>
__global__ __launch_bounds__(256) void rms_fwd_reg_kernel(const void* __restrict__ X, int64_t ldx, const void* __restrict__ W, int M,
                                                          int C, float eps, void* __restrict__ Y, int64_t ldy,
                                                          float* __restrict__ r) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= M) return;
  const uint16_t* xp = reinterpret_cast<const uint16_t*>(X) + (int64_t)row * ldx;
  u32x4 raw[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = 8 * lane + 512 * i;
    raw[i] = u32x4{0u, 0u, 0u, 0u};
    if (c < C) raw[i] = *reinterpret_cast<const u32x4*>(xp + c);
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    float x[8];
    unpack8<XD>(raw[i], x);
#pragma unroll
    for (int k = 0; k < 8; ++k) ss += x[k] * x[k];
  }
  ss = wave_sum(ss);
  const float var = ss / (float)C + eps;
  const float inv = GEMMA ? 1.0f / __builtin_sqrtf(var) : __builtin_amdgcn_rsqf(var);
  if (lane == 0) r[row] = inv;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = 8 * lane + 512 * i;
    if (c < C) {
      float x[8], w[8], y[8];
      unpack8<XD>(raw[i], x);
      Vec8<WD>::load(W, c, w);
#pragma unroll
      for (int k = 0; k < 8; ++k) y[k] = GEMMA ? x[k] * inv * (w[k] + 1.0f) : Vec8<WD>::round(Vec8<WD>::round(x[k] * inv) * w[k]);
      Vec8<XD>::store(Y, (int64_t)row * ldy + c, y);
    }
  }
}

template <int XD, int WD, bool GEMMA, int NCH>
__global__ __launch_bounds__(256) void rms_bwd_reg_kernel(void* __restrict__ dY, int64_t lddy, const void* __restrict__ X, int64_t ldx,
                                                          const void* __restrict__ W, const float* __restrict__ r, int M, int C) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= M) return;
  const uint16_t* xp = reinterpret_cast<const uint16_t*>(X) + (int64_t)row * ldx;
  const uint16_t* gp = reinterpret_cast<const uint16_t*>(dY) + (int64_t)row * lddy;
  u32x4 xr[NCH], gr[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = 8 * lane + 512 * i;
    xr[i] = gr[i] = u32x4{0u, 0u, 0u, 0u};
    if (c < C) {
      xr[i] = *reinterpret_cast<const u32x4*>(xp + c);
      gr[i] = *reinterpret_cast<const u32x4*>(gp + c);
    }
  }
  const float inv = r[row];
  float dot = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = 8 * lane + 512 * i;
    if (c < C) {
      float x[8], g[8], w[8];
      unpack8<XD>(xr[i], x);
      unpack8<XD>(gr[i], g);
      Vec8<WD>::load(W, c, w);
#pragma unroll
      for (int k = 0; k < 8; ++k) dot += g[k] * (GEMMA ? w[k] + 1.0f : w[k]) * (x[k] * inv);
    }
  }
  dot = wave_sum(dot);
  const float n = (float)C;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = 8 * lane + 512 * i;
    if (c < C) {
      float x[8], g[8], w[8], o[8];
      unpack8<XD>(xr[i], x);
      unpack8<XD>(gr[i], g);
      Vec8<WD>::load(W, c, w);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const float gw = g[k] * (GEMMA ? w[k] + 1.0f : w[k]);
        o[k] = inv / n * (n * gw - x[k] * inv * dot);
      }
      Vec8<XD>::store(dY, (int64_t)row * lddy + c, o);
    }
  }
}

// In place: (q1, q2) <- (q1 cos - q2 sin, q2 cos + q1 sin) on the two halves of every head, sin
// negated for the backward pass (rope_embedding.py:36-65).  One thread = 8 + 8 elements; the
// position of row m is m % cs_rows.  fp32 arithmetic, one rounding to Q's type.
template <int QD, int CD>
__global__ __launch_bounds__(256) void rope_kernel(void* __restrict__ Q, int64_t ldq, const void* __restrict__ cosp,
                                                   const void* __restrict__ sinp, int64_t ldcs, int M, int n_heads, int head_dim,
                                                   int cs_rows, float sin_sign) {
  const int chunks = head_dim / 16;  // 8-element chunks in half a head
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t per_row = (int64_t)n_heads * chunks;
  if (idx >= (int64_t)M * per_row) return;
  const int row = (int)(idx / per_row);
  const int rem = (int)(idx % per_row);
  const int head = rem / chunks, ch = rem % chunks;
  const int64_t cso = (int64_t)(row % cs_rows) * ldcs + 8 * ch;
  const int64_t q1o = (int64_t)row * ldq + (int64_t)head * head_dim + 8 * ch;
  const int64_t q2o = q1o + head_dim / 2;
  float c[8], s[8], q1[8], q2[8], o1[8], o2[8];
  Vec8<CD>::load(cosp, cso, c);
  Vec8<CD>::load(sinp, cso, s);
  Vec8<QD>::load(Q, q1o, q1);
  Vec8<QD>::load(Q, q2o, q2);
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const float sk = sin_sign * s[k];
    o1[k] = q1[k] * c[k] - q2[k] * sk;
    o2[k] = q2[k] * c[k] + q1[k] * sk;
  }
  Vec8<QD>::store(Q, q1o, o1);
  Vec8<QD>::store(Q, q2o, o2);
}

}  // namespace

#define FMSA_DISPATCH_DTYPE(D, NAME, ...)                        \
  switch (D) {                                                   \
    case FMSA_F16: { constexpr int NAME = FMSA_F16; __VA_ARGS__; } break;   \
    case FMSA_BF16: { constexpr int NAME = FMSA_BF16; __VA_ARGS__; } break; \
    default: { constexpr int NAME = FMSA_F32; __VA_ARGS__; } break;         \
  }

int launch_rms_fwd(const void* X, int64_t ldx, const void* W, int M, int C, float eps, int gemma, int x_dtype, int w_dtype, void* Y,
                   int64_t ldy, float* r, hipStream_t st) {
  dim3 grid((M + 3) / 4), block(256);
  FMSA_DISPATCH_DTYPE(x_dtype, XD, FMSA_DISPATCH_DTYPE(w_dtype, WD, {
    if constexpr (XD != FMSA_F32) {
      if (C <= 4096 && !gemma) {
        hipLaunchKernelGGL((rms_fwd_reg_kernel<XD, WD, false, 8>), grid, block, 0, st, X, ldx, W, M, C, eps, Y, ldy, r);
        FMSA_CHECK_LAUNCH();
        return FMSA_OK;
      }
      if (C <= 8192 && !gemma) {
        hipLaunchKernelGGL((rms_fwd_reg_kernel<XD, WD, false, 16>), grid, block, 0, st, X, ldx, W, M, C, eps, Y, ldy, r);
        FMSA_CHECK_LAUNCH();
        return FMSA_OK;
      }
    }
    if (gemma)
      hipLaunchKernelGGL((rms_fwd_kernel<XD, WD, true>), grid, block, 0, st, X, ldx, W, M, C, eps, Y, ldy, r);
    else
      hipLaunchKernelGGL((rms_fwd_kernel<XD, WD, false>), grid, block, 0, st, X, ldx, W, M, C, eps, Y, ldy, r);
  }))
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}

int launch_rms_bwd(void* dY, int64_t lddy, const void* X, int64_t ldx, const void* W, const float* r, int M, int C, int gemma,
                   int x_dtype, int w_dtype, hipStream_t st) {
  dim3 grid((M + 3) / 4), block(256);
  FMSA_DISPATCH_DTYPE(x_dtype, XD, FMSA_DISPATCH_DTYPE(w_dtype, WD, {
    if constexpr (XD != FMSA_F32) {
      if (C <= 4096 && !gemma) {
        hipLaunchKernelGGL((rms_bwd_reg_kernel<XD, WD, false, 8>), grid, block, 0, st, dY, lddy, X, ldx, W, r, M, C);
        FMSA_CHECK_LAUNCH();
        return FMSA_OK;
      }
      if (C <= 8192 && !gemma) {
        hipLaunchKernelGGL((rms_bwd_reg_kernel<XD, WD, false, 16>), grid, block, 0, st, dY, lddy, X, ldx, W, r, M, C);
        FMSA_CHECK_LAUNCH();
        return FMSA_OK;
      }
    }
    if (gemma)
      hipLaunchKernelGGL((rms_bwd_kernel<XD, WD, true>), grid, block, 0, st, dY, lddy, X, ldx, W, r, M, C);
    else
      hipLaunchKernelGGL((rms_bwd_kernel<XD, WD, false>), grid, block, 0, st, dY, lddy, X, ldx, W, r, M, C);
  }))
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}

int launch_rope(void* Q, int64_t ldq, const void* cosp, const void* sinp, int64_t ldcs, int M, int n_heads, int head_dim, int cs_rows,
                int backward, int q_dtype, int cs_dtype, hipStream_t st) {
  const int64_t n = (int64_t)M * n_heads * (head_dim / 16);
  dim3 grid((unsigned)((n + 255) / 256)), block(256);
  const float sign = backward ? -1.0f : 1.0f;
  FMSA_DISPATCH_DTYPE(q_dtype, QD, FMSA_DISPATCH_DTYPE(cs_dtype, CD, {
    hipLaunchKernelGGL((rope_kernel<QD, CD>), grid, block, 0, st, Q, ldq, cosp, sinp, ldcs, M, n_heads, head_dim, cs_rows, sign);
  }))
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}

// ---- cross entropy over the vocabulary (reference: kernels/unsloth/cross_entropy_loss.py:22-190) --------
// forward: one workgroup per row streams the logits once with an online (max, sum exp) pair per
// thread, combines the 256 pairs through LDS, and writes logsumexp and loss = logsumexp - x[label]
// (0 for label == -100).  backward, in place: logits <- dloss * (exp(x - logsumexp) - [col == label]).
namespace {

template <int D> FMSA_DEVI float load1(const void* p, int64_t i);
template <> FMSA_DEVI float load1<FMSA_F32>(const void* p, int64_t i) { return reinterpret_cast<const float*>(p)[i]; }
template <> FMSA_DEVI float load1<FMSA_BF16>(const void* p, int64_t i) { return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]); }
template <> FMSA_DEVI float load1<FMSA_F16>(const void* p, int64_t i) { return fp16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]); }
template <int D> FMSA_DEVI void store1(void* p, int64_t i, float v);
template <> FMSA_DEVI void store1<FMSA_F32>(void* p, int64_t i, float v) { reinterpret_cast<float*>(p)[i] = v; }
template <> FMSA_DEVI void store1<FMSA_BF16>(void* p, int64_t i, float v) { reinterpret_cast<uint16_t*>(p)[i] = pack1<bf16_t>(v); }
template <> FMSA_DEVI void store1<FMSA_F16>(void* p, int64_t i, float v) { reinterpret_cast<uint16_t*>(p)[i] = pack1<f16_t>(v); }

constexpr float kLog2e = 1.44269504088896341f;
constexpr float kLn2 = 0.69314718055994531f;

// (m, s) <- (m, s) (+) (x): running maximum and sum of exp(. - m)
// While everything seen so far is -inf (a masked vocabulary span) the pair stays (-inf, 0): the update
// would form (-inf) - (-inf) = NaN, which no later finite logit could remove from s.
FMSA_DEVI void online_add(float& m, float& s, float x) {
  const float mn = fmaxf(m, x);
  if (mn != -INFINITY) s = s * __builtin_amdgcn_exp2f((m - mn) * kLog2e) + __builtin_amdgcn_exp2f((x - mn) * kLog2e);
  m = mn;
}

template <int D, bool VEC>
__global__ __launch_bounds__(256) void ce_fwd_kernel(const void* __restrict__ logits, int64_t ld, const int64_t* __restrict__ labels,
                                                     int V, float* __restrict__ losses, float* __restrict__ lse_out) {
  __shared__ float red_m[256], red_s[256];
  const int row = blockIdx.x, tid = threadIdx.x;
  const int64_t base = (int64_t)row * ld;
  float m = -INFINITY, s = 0.f;
  if (VEC) {
    for (int c = 8 * tid; c < V; c += 2048) {  // V % 8 == 0
      float x[8];
      Vec8<D>::load(logits, base + c, x);
      float mx = x[0];
#pragma unroll
      for (int k = 1; k < 8; ++k) mx = fmaxf(mx, x[k]);
      const float mn = fmaxf(m, mx);
      if (mn == -INFINITY) continue;  // nothing finite yet: (m, s) stays (-inf, 0), see online_add
      float acc = 0.f;
#pragma unroll
      for (int k = 0; k < 8; ++k) acc += __builtin_amdgcn_exp2f((x[k] - mn) * kLog2e);
      s = s * __builtin_amdgcn_exp2f((m - mn) * kLog2e) + acc;
      m = mn;
    }
  } else {
    for (int c = tid; c < V; c += 256) online_add(m, s, load1<D>(logits, base + c));
  }
  red_m[tid] = m;
  red_s[tid] = s;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (tid < o) {
      const float m2 = red_m[tid + o], s2 = red_s[tid + o];
      const float mn = fmaxf(red_m[tid], m2);
      // a thread that saw no element holds (-inf, 0): its term must not turn into NaN
      const float a = red_m[tid] == -INFINITY ? 0.f : red_s[tid] * __builtin_amdgcn_exp2f((red_m[tid] - mn) * kLog2e);
      const float b = m2 == -INFINITY ? 0.f : s2 * __builtin_amdgcn_exp2f((m2 - mn) * kLog2e);
      red_m[tid] = mn;
      red_s[tid] = a + b;
    }
    __syncthreads();
  }
  if (tid == 0) {
    const float lse = red_m[0] + __builtin_amdgcn_logf(red_s[0]) * kLn2;
    const int64_t label = labels[row];
    lse_out[row] = lse;
    // a label outside [0, V) that is not -100 is a caller error: it is treated as ignored rather than read out of bounds
    losses[row] = (label < 0 || label >= V) ? 0.f : lse - load1<D>(logits, base + label);
  }
}

template <int D, bool VEC>
__global__ __launch_bounds__(256) void ce_bwd_kernel(void* __restrict__ logits, int64_t ld, const float* __restrict__ dloss,
                                                     int64_t dloss_stride, const float* __restrict__ lse,
                                                     const int64_t* __restrict__ labels, int V) {
  const int row = blockIdx.x;
  const int64_t base = (int64_t)row * ld;
  const int64_t label = labels[row];
  // -100 and any other label outside [0, V) are ignored rows, as in the forward kernel: loss 0, gradient 0
  const float dl = (label < 0 || label >= V) ? 0.f : dloss[(int64_t)row * dloss_stride];
  const float l = lse[row];
  if (VEC) {
    const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
    if (c >= V) return;
    float x[8], y[8];
    Vec8<D>::load(logits, base + c, x);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      float p = __builtin_amdgcn_exp2f((x[k] - l) * kLog2e);
      if (c + k == label) p -= 1.0f;
      y[k] = dl * p;
    }
    Vec8<D>::store(logits, base + c, y);
  } else {
    for (int c = blockIdx.y * 2048 + threadIdx.x; c < min(V, (int)(blockIdx.y + 1) * 2048); c += 256) {
      float p = __builtin_amdgcn_exp2f((load1<D>(logits, base + c) - l) * kLog2e);
      if (c == label) p -= 1.0f;
      store1<D>(logits, base + c, dl * p);
    }
  }
}


// Loss and logits gradient in one launch (reference: fused_ops/liger_ce/cross_entropy.py:33-186): the
// loss head calls this on each freshly computed chunk of logits, so nothing is saved for a backward
// pass.  One workgroup per row: pass 1 streams the row (online max / sum exp, and sum x for label
// smoothing), pass 2 re-reads it (the row was just fetched, so mostly from cache) and overwrites it
// with  scale * (softmax - eps - [col == label] (1 - smoothing)),  eps = smoothing / V.
// loss = scale * ((1 - smoothing) (lse - x[label]) + smoothing * lse - eps * sum x).  Rows whose label
// equals ignore_index get loss 0 and an all-zero gradient.  `scale` is read from device memory so the
// caller never has to wait for the count of valid labels.
template <int D, bool VEC>
__global__ __launch_bounds__(256) void ce_fused_kernel(void* __restrict__ logits, int64_t ld, const int64_t* __restrict__ labels,
                                                       int V, int64_t ignore_index, const float* __restrict__ scale_ptr,
                                                       float smoothing, float* __restrict__ losses) {
  __shared__ float red_m[256], red_s[256], red_x[256];
  const int row = blockIdx.x, tid = threadIdx.x;
  const int64_t base = (int64_t)row * ld;
  const int64_t label = labels[row];
  if (label == ignore_index || label < 0 || label >= V) {  // uniform over the workgroup; out-of-range labels count as ignored
    if (VEC) {
      float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      for (int c = 8 * tid; c < V; c += 2048) Vec8<D>::store(logits, base + c, z);
    } else {
      for (int c = tid; c < V; c += 256) store1<D>(logits, base + c, 0.f);
    }
    if (tid == 0) losses[row] = 0.f;
    return;
  }
  const float scale = scale_ptr ? scale_ptr[0] : 1.0f;
  const float x_label = load1<D>(logits, base + label);  // read by every thread before any store of pass 2
  float m = -INFINITY, s = 0.f, sx = 0.f;
  if (VEC) {
    for (int c = 8 * tid; c < V; c += 2048) {
      float x[8];
      Vec8<D>::load(logits, base + c, x);
      float mx = x[0];
#pragma unroll
      for (int k = 1; k < 8; ++k) mx = fmaxf(mx, x[k]);
      const float mn = fmaxf(m, mx);
#pragma unroll
      for (int k = 0; k < 8; ++k) sx += x[k];
      if (mn == -INFINITY) continue;  // nothing finite yet: (m, s) stays (-inf, 0), see online_add
      float acc = 0.f;
#pragma unroll
      for (int k = 0; k < 8; ++k) acc += __builtin_amdgcn_exp2f((x[k] - mn) * kLog2e);
      s = s * __builtin_amdgcn_exp2f((m - mn) * kLog2e) + acc;
      m = mn;
    }
  } else {
    for (int c = tid; c < V; c += 256) {
      const float x = load1<D>(logits, base + c);
      online_add(m, s, x);
      sx += x;
    }
  }
  red_m[tid] = m;
  red_s[tid] = s;
  red_x[tid] = sx;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (tid < o) {
      const float m2 = red_m[tid + o], s2 = red_s[tid + o];
      const float mn = fmaxf(red_m[tid], m2);
      const float a = red_m[tid] == -INFINITY ? 0.f : red_s[tid] * __builtin_amdgcn_exp2f((red_m[tid] - mn) * kLog2e);
      const float b = m2 == -INFINITY ? 0.f : s2 * __builtin_amdgcn_exp2f((m2 - mn) * kLog2e);
      red_m[tid] = mn;
      red_s[tid] = a + b;
      red_x[tid] += red_x[tid + o];
    }
    __syncthreads();
  }
  const float lse = red_m[0] + __builtin_amdgcn_logf(red_s[0]) * kLn2;
  const float eps = smoothing / (float)V;
  // without smoothing the sum of the logits is not used (it is -inf for a row with masked logits, and 0 * inf is NaN)
  const float smooth_term = smoothing != 0.f ? smoothing * lse - eps * red_x[0] : 0.f;
  if (tid == 0) losses[row] = scale * ((1.0f - smoothing) * (lse - x_label) + smooth_term);
  const float hit = 1.0f - smoothing;
  if (VEC) {
    for (int c = 8 * tid; c < V; c += 2048) {
      float x[8], y[8];
      Vec8<D>::load(logits, base + c, x);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        float p = __builtin_amdgcn_exp2f((x[k] - lse) * kLog2e) - eps;
        if (c + k == label) p -= hit;
        y[k] = scale * p;
      }
      Vec8<D>::store(logits, base + c, y);
    }
  } else {
    for (int c = tid; c < V; c += 256) {
      float p = __builtin_amdgcn_exp2f((load1<D>(logits, base + c) - lse) * kLog2e) - eps;
      if (c == label) p -= hit;
      store1<D>(logits, base + c, scale * p);
    }
  }
}

}  // namespace

int launch_ce_fwd(const void* logits, int64_t ld, const int64_t* labels, int M, int V, int dtype, int vec, float* losses, float* lse,
                  hipStream_t st) {
  dim3 grid(M), block(256);
  FMSA_DISPATCH_DTYPE(dtype, D, {
    if (vec)
      hipLaunchKernelGGL((ce_fwd_kernel<D, true>), grid, block, 0, st, logits, ld, labels, V, losses, lse);
    else
      hipLaunchKernelGGL((ce_fwd_kernel<D, false>), grid, block, 0, st, logits, ld, labels, V, losses, lse);
  })
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}

int launch_ce_bwd(void* logits, int64_t ld, const float* dloss, int64_t dloss_stride, const float* lse, const int64_t* labels, int M,
                  int V, int dtype, int vec, hipStream_t st) {
  dim3 grid(M, (V + 2047) / 2048), block(256);
  FMSA_DISPATCH_DTYPE(dtype, D, {
    if (vec)
      hipLaunchKernelGGL((ce_bwd_kernel<D, true>), grid, block, 0, st, logits, ld, dloss, dloss_stride, lse, labels, V);
    else
      hipLaunchKernelGGL((ce_bwd_kernel<D, false>), grid, block, 0, st, logits, ld, dloss, dloss_stride, lse, labels, V);
  })
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}

int launch_ce_fused(void* logits, int64_t ld, const int64_t* labels, int M, int V, int dtype, int vec, int64_t ignore_index,
                    const float* scale, float smoothing, float* losses, hipStream_t st) {
  dim3 grid(M), block(256);
  FMSA_DISPATCH_DTYPE(dtype, D, {
    if (vec)
      hipLaunchKernelGGL((ce_fused_kernel<D, true>), grid, block, 0, st, logits, ld, labels, V, ignore_index, scale, smoothing, losses);
    else
      hipLaunchKernelGGL((ce_fused_kernel<D, false>), grid, block, 0, st, logits, ld, labels, V, ignore_index, scale, smoothing, losses);
  })
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}
