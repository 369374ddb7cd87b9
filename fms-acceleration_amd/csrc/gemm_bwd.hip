// Fused input gradient:  dX = sum_p dY_p * deq(W_p)^T + mask_p (.) (T_p * (s_p A_p)), optional
// SwiGLU backward over the result (the down-projection half of the MLP backward).
//
// The contraction now runs over the weight's N axis while qweight packs 8 nibbles along K, so a
// lane that loads 8 adjacent words of one qweight row,  qweight[k8, n .. n+7],  holds an 8(k) x 8(n)
// block: nibble t of those 8 words is the 8-element MFMA fragment (contraction n .. n+7) of
// output column k = 8*k8 + t.  No transpose through LDS is needed; the only price is that output
// columns of one MFMA tile are 8 apart.
//
// Tiling (one workgroup = 4 waves, one workgroup per CU):
//   workgroup tile  256 tokens x 256 output columns (32 qweight rows x 8 nibbles)
//   wave w          nibbles 2w, 2w+1 of every word -> 256 tokens x 2 column tiles, 256 accumulators
//                   (all four waves read the same words -- 4-bit data, served by L1/L2 -- but every
//                   weight is unpacked by exactly one wave)
//   dY operand      global -> registers -> LDS, double buffered, stages of 64 along N
// Scale/zero for a lane's block are 8 fp16 scales and one qzeros word (8 columns, one group).
#include "common.h"

namespace {

constexpr int BM = 256;
constexpr int BK = 64;
constexpr int LDS_STRIDE = BK + 8;
constexpr int MT = 8;
constexpr int NT = 2;

struct BwdProjDev {
  const int32_t* qweight;
  const uint16_t* scales;
  const int32_t* qzeros;
  const uint16_t* dY;
  int64_t lddy;
  const uint16_t* T;
  const uint16_t* At;  // [K, r]
  const uint16_t* mask_src;
  int64_t ldmask;
  int N, group_size, zero_offset, r;
  float s;
};

struct BwdArgs {
  BwdProjDev p[3];
  int n_proj, M, K, mode, nbm, nbk;
  uint16_t* dX;
  int64_t lddx;
  uint16_t* e;
  uint16_t* g;
  uint16_t* h;
  int64_t ldeg;
};

// byte `sel` (0..3) of four words -> one word
FMSA_DEVI uint32_t gather_byte(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3, int shift) {
  return ((w0 >> shift) & 0xffu) | (((w1 >> shift) & 0xffu) << 8) | (((w2 >> shift) & 0xffu) << 16) |
         (((w3 >> shift) & 0xffu) << 24);
}

// a.p[p] for a runtime (wave-uniform) p without dynamic indexing of the kernel-argument struct,
// which would force a copy of it into scratch memory.
FMSA_DEVI BwdProjDev select_proj(const BwdArgs& a, int p) { return p == 0 ? a.p[0] : (p == 1 ? a.p[1] : a.p[2]); }

template <typename T>
__global__ __launch_bounds__(256) void gptq_lora_bwd_dx_kernel(const BwdArgs a) {
  __shared__ __attribute__((aligned(16))) uint16_t lds[2][BM * LDS_STRIDE];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int half = lane >> 5;

  int pid = xcd_remap(blockIdx.x, a.nbm * a.nbk);
  constexpr int GROUP_M = 8;
  const int width = GROUP_M * a.nbk;
  const int first_m = (pid / width) * GROUP_M;
  const int gsz = min(a.nbm - first_m, GROUP_M);
  const int bm = first_m + (pid % width) % gsz;
  const int bk = (pid % width) / gsz;
  const int m0 = bm * BM;
  const int k8base = bk * 32;

  const int K = a.K;
  const bool row_ok = (k8base + l32) < (K >> 3);
  const int k8 = row_ok ? (k8base + l32) : 0;
  const int byte_shift = 8 * wave;

  f32x16 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;

  u32x4 a_st[8];
  u32x4 qn[4][2];       // in flight: 8 words per k16 step
  u32x4 scn[4];         // in flight: 8 fp16 scales per k16 step
  uint32_t zwn[4];      // in flight: zeros word per k16 step
  uint32_t qc[4][2];    // current: this wave's byte of the 8 words
  u32x4 scc[4];
  uint32_t zwc[4];

  // flattened (projection, n0) stage iterator
  int n_stages = 0;
  {
    n_stages = (a.p[0].N + BK - 1) / BK;
    if (a.n_proj > 1) n_stages += (a.p[1].N + BK - 1) / BK;
    if (a.n_proj > 2) n_stages += (a.p[2].N + BK - 1) / BK;
  }

  auto load_stage = [&](int p, int n0) {
    const BwdProjDev P = select_proj(a, p);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int c = tid + 256 * i;
      const int row = c >> 3, oct = c & 7;
      const int gm = m0 + row, gn = n0 + 8 * oct;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (gm < a.M && gn < P.N) v = *reinterpret_cast<const u32x4*>(P.dY + (size_t)gm * P.lddy + gn);
      a_st[i] = v;
    }
    const int g = (8 * k8) / P.group_size;
    const int32_t* qrow = P.qweight + (size_t)k8 * P.N;
    const uint16_t* srow = P.scales + (size_t)g * P.N;
    const int32_t* zrow = P.qzeros + (size_t)g * (P.N >> 3);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int n = n0 + 16 * t + 8 * half;
      if (n < P.N) {
        qn[t][0] = *reinterpret_cast<const u32x4*>(qrow + n);
        qn[t][1] = *reinterpret_cast<const u32x4*>(qrow + n + 4);
        scn[t] = *reinterpret_cast<const u32x4*>(srow + n);
        zwn[t] = (uint32_t)zrow[n >> 3];
      } else {
        qn[t][0] = qn[t][1] = scn[t] = u32x4{0u, 0u, 0u, 0u};
        zwn[t] = 0u;
      }
    }
  };
  auto commit_stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int c = tid + 256 * i;
      const int row = c >> 3, oct = c & 7;
      *reinterpret_cast<u32x4*>(&lds[buf][row * LDS_STRIDE + oct * 8]) = a_st[i];
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      qc[t][0] = gather_byte(qn[t][0][0], qn[t][0][1], qn[t][0][2], qn[t][0][3], byte_shift);
      qc[t][1] = gather_byte(qn[t][1][0], qn[t][1][1], qn[t][1][2], qn[t][1][3], byte_shift);
      scc[t] = scn[t];
      zwc[t] = zwn[t];
    }
  };

  int p_ld = 0, n_ld = 0;  // next stage to load
  auto advance = [&]() {
    n_ld += BK;
    if (n_ld >= (p_ld == 0 ? a.p[0].N : (p_ld == 1 ? a.p[1].N : a.p[2].N))) {
      n_ld = 0;
      ++p_ld;
    }
  };
  int zoff_cur = a.p[0].zero_offset, zoff_nxt = zoff_cur;

  load_stage(p_ld, n_ld);
  zoff_nxt = (p_ld == 0 ? a.p[0].zero_offset : (p_ld == 1 ? a.p[1].zero_offset : a.p[2].zero_offset));
  advance();
  commit_stage(0);
  zoff_cur = zoff_nxt;
  __syncthreads();

  for (int s = 0; s < n_stages; ++s) {
    const int buf = s & 1;
    if (s + 1 < n_stages) {
      load_stage(p_ld, n_ld);
      zoff_nxt = (p_ld == 0 ? a.p[0].zero_offset : (p_ld == 1 ? a.p[1].zero_offset : a.p[2].zero_offset));
      advance();
    }
    const uint16_t* lb = lds[buf];
    const float zo = (float)zoff_cur;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      // per-column scale and -scale*zero for the lane's 8 columns
      float sfv[8], nszv[8];
      const uint32_t zlo = opaque(zwc[t] & 0x0F0F0F0Fu), zhi = opaque((zwc[t] >> 4) & 0x0F0F0F0Fu);
      const float zf[8] = {ubyte0(zlo), ubyte0(zhi), ubyte1(zlo), ubyte1(zhi),
                           ubyte2(zlo), ubyte2(zhi), ubyte3(zlo), ubyte3(zhi)};
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t sb = (i & 1) ? (scc[t][i >> 1] >> 16) : (scc[t][i >> 1] & 0xffffu);
        sfv[i] = fp16_bits_to_f32((uint16_t)sb);
        nszv[i] = -sfv[i] * (zf[i] + zo);
      }
      u32x4 wf[NT];
      {
        const uint32_t lo0 = opaque(qc[t][0] & 0x0F0F0F0Fu), hi0 = opaque((qc[t][0] >> 4) & 0x0F0F0F0Fu);
        const uint32_t lo1 = opaque(qc[t][1] & 0x0F0F0F0Fu), hi1 = opaque((qc[t][1] >> 4) & 0x0F0F0F0Fu);
        // tile 0 = low nibble (k = 8*k8 + 2*wave), tile 1 = high nibble (k + 1); element i <-> column n+i
        wf[0][0] = pack2<T>(__builtin_fmaf(sfv[0], ubyte0(lo0), nszv[0]), __builtin_fmaf(sfv[1], ubyte1(lo0), nszv[1]));
        wf[0][1] = pack2<T>(__builtin_fmaf(sfv[2], ubyte2(lo0), nszv[2]), __builtin_fmaf(sfv[3], ubyte3(lo0), nszv[3]));
        wf[0][2] = pack2<T>(__builtin_fmaf(sfv[4], ubyte0(lo1), nszv[4]), __builtin_fmaf(sfv[5], ubyte1(lo1), nszv[5]));
        wf[0][3] = pack2<T>(__builtin_fmaf(sfv[6], ubyte2(lo1), nszv[6]), __builtin_fmaf(sfv[7], ubyte3(lo1), nszv[7]));
        wf[1][0] = pack2<T>(__builtin_fmaf(sfv[0], ubyte0(hi0), nszv[0]), __builtin_fmaf(sfv[1], ubyte1(hi0), nszv[1]));
        wf[1][1] = pack2<T>(__builtin_fmaf(sfv[2], ubyte2(hi0), nszv[2]), __builtin_fmaf(sfv[3], ubyte3(hi0), nszv[3]));
        wf[1][2] = pack2<T>(__builtin_fmaf(sfv[4], ubyte0(hi1), nszv[4]), __builtin_fmaf(sfv[5], ubyte1(hi1), nszv[5]));
        wf[1][3] = pack2<T>(__builtin_fmaf(sfv[6], ubyte2(hi1), nszv[6]), __builtin_fmaf(sfv[7], ubyte3(hi1), nszv[7]));
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const u32x4 xf =
            *reinterpret_cast<const u32x4*>(&lb[(32 * mt + l32) * LDS_STRIDE + 16 * t + 8 * half]);
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[mt][j] = mfma32<T>(wf[j], xf, acc[mt][j]);
      }
    }
    if (s + 1 < n_stages) {
      commit_stage(buf ^ 1);
      zoff_cur = zoff_nxt;
    }
    __syncthreads();
  }

  // ---- epilogue ---------------------------------------------------------------------------
  // register 4*i0+i1 of acc[mt][j] is dX[m0 + 32*mt + l32][8*(k8base + 8*i0 + 4*half + i1) + 2*wave + j]
  const int kcol_lane = 8 * (k8base + l32) + 2 * wave;  // column whose A^T rows this lane supplies to the LoRA MFMA
  static_for<0, MT>([&](auto mt_c) {
    constexpr int mt = decltype(mt_c)::value;
    const int m = m0 + 32 * mt + l32;
    const bool m_ok = m < a.M;
    f32x16 lora[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) lora[j][i] = 0.f;
    bool any_lora = false;
    for (int p = 0; p < a.n_proj; ++p) {
      const BwdProjDev P = select_proj(a, p);
      if (P.r <= 0) continue;
      any_lora = true;
      f32x16 tmp[NT];
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) tmp[j][i] = 0.f;
      for (int j0 = 0; j0 < P.r; j0 += 16) {
        const int ko = j0 + 8 * half;
        u32x4 tf = {0u, 0u, 0u, 0u}, af[NT] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
        if (ko < P.r) {
          if (m_ok) tf = *reinterpret_cast<const u32x4*>(P.T + (size_t)m * P.r + ko);
          if (row_ok) {
#pragma unroll
            for (int j = 0; j < NT; ++j)
              af[j] = *reinterpret_cast<const u32x4*>(P.At + (size_t)(kcol_lane + j) * P.r + ko);
          }
        }
#pragma unroll
        for (int j = 0; j < NT; ++j) tmp[j] = mfma32<T>(af[j], tf, tmp[j]);
      }
      // mask_p = (mask_src_p != 0), element-wise at the output position
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int cp = 8 * (i >> 2) + 4 * half + (i & 3);
        const int k = 8 * (k8base + cp) + 2 * wave;
        float m0f = 1.f, m1f = 1.f;
        if (P.mask_src && m_ok && k < K) {
          const uint32_t mv = *reinterpret_cast<const uint32_t*>(P.mask_src + (size_t)m * P.ldmask + k);
          m0f = (mv & 0x7fffu) ? 1.f : 0.f;          // +-0 count as zero
          m1f = ((mv >> 16) & 0x7fffu) ? 1.f : 0.f;
        }
        lora[0][i] += P.s * m0f * tmp[0][i];
        lora[1][i] += P.s * m1f * tmp[1][i];
      }
    }
    if (!m_ok) return;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int cp = 8 * (i >> 2) + 4 * half + (i & 3);
      const int k = 8 * (k8base + cp) + 2 * wave;
      if (k >= K) continue;
      if (a.mode == FMSA_BWD_SWIGLU) {
        const size_t off = (size_t)m * a.ldeg + k;
        const uint32_t ev = *reinterpret_cast<const uint32_t*>(a.e + off);
        const uint32_t gv = *reinterpret_cast<const uint32_t*>(a.g + off);
        float hh[2], dg[2], de[2];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          const float e32 = j ? unpack_hi<T>(ev) : unpack_lo<T>(ev);
          const float g32 = j ? unpack_hi<T>(gv) : unpack_lo<T>(gv);
          const float se = sigmoidf_(e32);
          const float f = unpack1<T>(pack1<T>(se * e32));
          const float h = unpack1<T>(pack1<T>(f * g32));
          // the LoRA term of dh is masked by (h != 0)            [h is the down-projection input]
          float dh = acc[mt][j][i];
          if (any_lora && h != 0.f) dh += lora[j][i];
          const float DW = unpack1<T>(pack1<T>(dh));
          hh[j] = h;
          dg[j] = DW * f;                                          // d_g  ("df" in UL/swiglu.py:77)
          const float dgt = unpack1<T>(pack1<T>(DW * g32));        // dg = DW * g in storage dtype (:79)
          de[j] = dgt * se * (1.0f + e32 * (1.0f - se));           // d_e (:81-83)
        }
        *reinterpret_cast<uint32_t*>(a.h + off) = pack2<T>(hh[0], hh[1]);
        *reinterpret_cast<uint32_t*>(a.e + off) = pack2<T>(dg[0], dg[1]);
        *reinterpret_cast<uint32_t*>(a.g + off) = pack2<T>(de[0], de[1]);
      } else {
        const float v0 = acc[mt][0][i] + lora[0][i];
        const float v1 = acc[mt][1][i] + lora[1][i];
        *reinterpret_cast<uint32_t*>(a.dX + (size_t)m * a.lddx + k) = pack2<T>(v0, v1);
      }
    }
  });
}

}  // namespace

int launch_gptq_lora_bwd_dx(const fmsa_bwd_proj* projs, int n_proj, int M, int mode, void* dX, int64_t lddx,
                            void* e, void* g, void* h_out, int64_t ldeg, int act_dtype, hipStream_t st) {
  BwdArgs a{};
  a.n_proj = n_proj;
  a.M = M;
  a.K = projs[0].w.K;
  a.mode = mode;
  a.dX = (uint16_t*)dX;
  a.lddx = lddx;
  a.e = (uint16_t*)e;
  a.g = (uint16_t*)g;
  a.h = (uint16_t*)h_out;
  a.ldeg = ldeg;
  for (int p = 0; p < n_proj; ++p) {
    const fmsa_bwd_proj& s = projs[p];
    BwdProjDev& d = a.p[p];
    d.qweight = s.w.qweight;
    d.scales = s.w.scales;
    d.qzeros = s.w.qzeros;
    d.dY = (const uint16_t*)s.dY;
    d.lddy = s.lddy;
    d.T = (const uint16_t*)s.T;
    d.At = (const uint16_t*)s.At;
    d.mask_src = (const uint16_t*)s.mask_src;
    d.ldmask = s.ldmask;
    d.N = s.w.N;
    d.group_size = s.w.group_size;
    d.zero_offset = s.w.zero_offset;
    d.r = s.r;
    d.s = s.s;
  }
  a.nbm = (M + BM - 1) / BM;
  a.nbk = (a.K + 255) / 256;
  dim3 grid(a.nbm * a.nbk), block(256);
  if (act_dtype == FMSA_BF16)
    hipLaunchKernelGGL(gptq_lora_bwd_dx_kernel<bf16_t>, grid, block, 0, st, a);
  else
    hipLaunchKernelGGL(gptq_lora_bwd_dx_kernel<f16_t>, grid, block, 0, st, a);
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}
