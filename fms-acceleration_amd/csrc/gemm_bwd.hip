// Fused input gradient:  dX = sum_p dY_p * deq(W_p)^T + mask (.) sum_p s_p T_p A_p, optional
// SwiGLU backward over the result (the down-projection half of the MLP backward).
//
// The contraction now runs over the weight's N axis while qweight packs 8 nibbles along K, so a
// lane that loads 8 adjacent words of one qweight row,  qweight[k8, n .. n+7],  holds an 8(k) x 8(n)
// block: nibble t of those 8 words is the 8-element MFMA fragment (contraction n .. n+7) of
// output column k = 8*k8 + t.  No transpose through LDS is needed; the only price is that output
// columns of one MFMA tile are 8 apart, which the epilogue undoes through LDS.
//
// Tiling (one workgroup = 4 waves, one workgroup per CU):
//   workgroup tile  256 tokens x 256 output columns (32 qweight rows x 8 nibbles)
//   wave w          nibbles 2w, 2w+1 of every word -> 256 tokens x 2 column tiles, 256 accumulators
//                   (all four waves read the same words -- 4-bit data, served by L1/L2 -- but every
//                   weight is unpacked by exactly one wave)
//   dY operand      global -> registers -> LDS, double buffered, stages of 64 along N
//   W operand       per 16-wide step and lane: 8 words, 8 fp16 scales and 8 fp32 (-scale*zero)
//                   values of its row's group, fetched two steps ahead with buffer loads
// Main loop: software pipeline at the granularity of one MFMA K step, as in the forward kernel
// (LDS fragments and unpacked weights of step t+1 are produced while the 16 MFMAs of step t run,
// and all other instructions are interleaved between those MFMAs).
// Epilogue: 64 tokens at a time the accumulators (and, separately, the LoRA term) are rounded to
// the storage type, transposed through LDS and written as 16-byte row segments; mask and SwiGLU
// backward are applied on that coalesced form.
#include "common.h"

namespace {

constexpr int BM = 256;
constexpr int BK = 64;
constexpr int LDS_STRIDE = BK + 8;
constexpr int MT = 8;
constexpr int NT = 2;
constexpr int EP_ROWS = 64;     // tokens per epilogue pass
constexpr int EP_STRIDE = 264;  // elements per staged row (256 + 8)

struct BwdProjDev {
  const int32_t* qweight;
  const uint16_t* scales;
  const float* nsz;  // [G, N] = -scale * (zero + zero_offset)
  const uint16_t* dY;
  int64_t lddy;
  const uint16_t* T;
  const uint16_t* At;  // [K, r]
  int N, group_size, r;
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
  const uint16_t* mask_src;
  int64_t ldmask;
};

FMSA_DEVI BwdProjDev select_proj(const BwdArgs& a, int p) { return p == 0 ? a.p[0] : (p == 1 ? a.p[1] : a.p[2]); }

// per-step weight operands of one lane: 8 words, 8 fp16 scales, 8 fp32 (-scale*zero)
struct BSet {
  u32x4 q0, q1, sc, nz0, nz1;
};

template <typename T, bool NTAIL>
__global__ __launch_bounds__(256) void gptq_lora_bwd_dx_kernel(const BwdArgs a) {
  __shared__ __attribute__((aligned(16))) uint16_t lds[2][BM * LDS_STRIDE];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int half = lane >> 5;
  const int oct = tid & 7;

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
  const int rows_valid = min(BM, a.M - m0);
  // byte `wave` of two words -> bytes 0,1 of the result (v_perm_b32 selector; 0x0c gives 0x00)
  const uint32_t sel_pair = 0x0c0c0000u | (uint32_t)wave | ((uint32_t)(4 + wave) << 8);

  f32x16 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;

  const uint32_t lds_w_off = (uint32_t)(((tid >> 3) * LDS_STRIDE + oct * 8) * 2);
  const uint32_t lds_r_off = (uint32_t)((l32 * LDS_STRIDE + 8 * half) * 2);
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;

  for (int p = 0; p < a.n_proj; ++p) {
    const BwdProjDev P = select_proj(a, p);
    const int N = __builtin_amdgcn_readfirstlane(P.N);
    const int gs = __builtin_amdgcn_readfirstlane(P.group_size);
    const int n_stages = (N + BK - 1) / BK;
    const int n_groups = (K + gs - 1) / gs;

    // ---- operand addressing: buffer resources + 32-bit lane offsets + scalar offsets ----------
    const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(P.dY + (size_t)m0 * P.lddy, (size_t)rows_valid * P.lddy * 2);
    const uint32_t a_off = (uint32_t)(((tid >> 3) * P.lddy + 8 * oct) * 2);    // lane part
    const uint32_t a_blk = __builtin_amdgcn_readfirstlane((uint32_t)(32 * P.lddy * 2));  // 32 rows further
    const __amdgpu_buffer_rsrc_t q_rsrc = make_rsrc(P.qweight, (size_t)(K >> 3) * N * 4);
    const __amdgpu_buffer_rsrc_t sc_rsrc = make_rsrc(P.scales, (size_t)n_groups * N * 2);
    const __amdgpu_buffer_rsrc_t nz_rsrc = make_rsrc(P.nsz, (size_t)n_groups * N * 4);
    const int grp = (8 * k8) / gs;
    const uint32_t dead = row_ok ? 0u : 0x80000000u;  // rows past K: out of range, read as zeros
    const uint32_t q_voff = (uint32_t)((k8 * N + 8 * half) * 4) | dead;
    const uint32_t sc_voff = (uint32_t)((grp * N + 8 * half) * 2) | dead;
    const uint32_t nz_voff = (uint32_t)((grp * N + 8 * half) * 4) | dead;

    u32x4 a_st[4];  // the dY tile is staged in two halves of 128 rows
    BSet bs[2];
    u32x4 xf[2][MT], wf[2][NT];

    // global loads of one half (128 rows) of the dY tile of stage `st` (clamped: the surplus loads
    // of the last iteration re-read the final stage and are never used)
    auto load_A = [&](int st, int hf) {
      const int stc = min(st, n_stages - 1);
      const uint32_t soff = (uint32_t)stc * (BK * 2) + (uint32_t)(4 * hf) * a_blk;
      uint32_t poison = 0;
      if constexpr (NTAIL) poison = ((stc * BK + 8 * oct) < N) ? 0u : 0x80000000u;  // N % 64 == 32
#pragma unroll
      for (int i = 0; i < 4; ++i) a_st[i] = __builtin_amdgcn_raw_buffer_load_b128(dy_rsrc, a_off | poison, soff + i * a_blk, 0);
    };
    auto commit_A = [&](int buf, int hf) {
      char* lw = reinterpret_cast<char*>(lds[buf]) + lds_w_off + hf * (4 * 32 * LDS_STRIDE * 2);
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(lw + i * 32 * LDS_STRIDE * 2) = a_st[i];
    };
    // weight operands of K step (st, t): columns n = 64*st + 16*t + 8*half .. +7 of the lane's row
    auto load_B = [&](BSet& b, int st, int t) {
      const int stc = min(st, n_stages - 1);
      const uint32_t n = (uint32_t)(stc * BK + 16 * t);
      uint32_t poison = 0;
      if constexpr (NTAIL) poison = ((int)n + 8 * half < N) ? 0u : 0x80000000u;
      b.q0 = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, q_voff | poison, n * 4, 0);
      b.q1 = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, (q_voff | poison) + 16, n * 4, 0);
      b.sc = __builtin_amdgcn_raw_buffer_load_b128(sc_rsrc, sc_voff | poison, n * 2, 0);
      b.nz0 = __builtin_amdgcn_raw_buffer_load_b128(nz_rsrc, nz_voff | poison, n * 4, 0);
      b.nz1 = __builtin_amdgcn_raw_buffer_load_b128(nz_rsrc, (nz_voff | poison) + 16, n * 4, 0);
    };
    // LDS fragments of step t and the two unpacked weight fragments, into parity `par`
    auto prefetch = [&](int buf, int t, const BSet& b, auto par_c) {
      constexpr int par = decltype(par_c)::value;
      const char* lr = reinterpret_cast<const char*>(lds[buf]) + lds_r_off + t * 32;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        xf[par][mt] = *reinterpret_cast<const u32x4*>(lr + mt * 32 * LDS_STRIDE * 2);
      // this wave's byte of the 8 words: low nibble = column tile 0 (k = 8*k8 + 2*wave), high = tile 1
      const uint32_t p01 = __builtin_amdgcn_perm(b.q0[1], b.q0[0], sel_pair);
      const uint32_t p23 = __builtin_amdgcn_perm(b.q0[3], b.q0[2], sel_pair);
      const uint32_t p45 = __builtin_amdgcn_perm(b.q1[1], b.q1[0], sel_pair);
      const uint32_t p67 = __builtin_amdgcn_perm(b.q1[3], b.q1[2], sel_pair);
      const uint32_t x0 = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
      const uint32_t x1 = __builtin_amdgcn_perm(p67, p45, 0x05040100u);
      const uint32_t lo0 = opaque(x0 & 0x0F0F0F0Fu), hi0 = opaque((x0 >> 4) & 0x0F0F0F0Fu);
      const uint32_t lo1 = opaque(x1 & 0x0F0F0F0Fu), hi1 = opaque((x1 >> 4) & 0x0F0F0F0Fu);
      float sfv[8], nzv[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        sfv[2 * i] = fp16_bits_to_f32((uint16_t)(b.sc[i] & 0xffffu));
        sfv[2 * i + 1] = fp16_bits_to_f32((uint16_t)(b.sc[i] >> 16));
        nzv[i] = __uint_as_float(b.nz0[i]);
        nzv[4 + i] = __uint_as_float(b.nz1[i]);
      }
      // element i of a fragment <-> column n + i; value = scale * nibble + (-scale * zero), exact in fp32
      wf[par][0][0] = pack2<T>(__builtin_fmaf(sfv[0], ubyte0(lo0), nzv[0]), __builtin_fmaf(sfv[1], ubyte1(lo0), nzv[1]));
      wf[par][0][1] = pack2<T>(__builtin_fmaf(sfv[2], ubyte2(lo0), nzv[2]), __builtin_fmaf(sfv[3], ubyte3(lo0), nzv[3]));
      wf[par][0][2] = pack2<T>(__builtin_fmaf(sfv[4], ubyte0(lo1), nzv[4]), __builtin_fmaf(sfv[5], ubyte1(lo1), nzv[5]));
      wf[par][0][3] = pack2<T>(__builtin_fmaf(sfv[6], ubyte2(lo1), nzv[6]), __builtin_fmaf(sfv[7], ubyte3(lo1), nzv[7]));
      wf[par][1][0] = pack2<T>(__builtin_fmaf(sfv[0], ubyte0(hi0), nzv[0]), __builtin_fmaf(sfv[1], ubyte1(hi0), nzv[1]));
      wf[par][1][1] = pack2<T>(__builtin_fmaf(sfv[2], ubyte2(hi0), nzv[2]), __builtin_fmaf(sfv[3], ubyte3(hi0), nzv[3]));
      wf[par][1][2] = pack2<T>(__builtin_fmaf(sfv[4], ubyte0(hi1), nzv[4]), __builtin_fmaf(sfv[5], ubyte1(hi1), nzv[5]));
      wf[par][1][3] = pack2<T>(__builtin_fmaf(sfv[6], ubyte2(hi1), nzv[6]), __builtin_fmaf(sfv[7], ubyte3(hi1), nzv[7]));
    };
    auto mfma_step = [&](auto par_c) {
      constexpr int par = decltype(par_c)::value;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[mt][j] = mfma32<T>(wf[par][j], xf[par][mt], acc[mt][j]);
    };
    // Everything else of a step sits between its 16 MFMAs (in-order issue, one wave per SIMD):
    // per MFMA 3 VALU, an LDS read after every second one, and the step's buffer loads.
    auto interleave = [&](auto n_vmem_c) {
      constexpr int n_vmem = decltype(n_vmem_c)::value;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
        if ((i & 1) == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if (i < n_vmem) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    using V9 = std::integral_constant<int, 9>;
    using V5 = std::integral_constant<int, 5>;

    // Pipeline: the weights of MFMA step u are loaded during step u-2 and unpacked during step u-1
    // (two register sets, by parity of u); the dY tile of the next stage is loaded in two halves
    // during steps 0 and 1 and written to the idle LDS buffer during steps 1 and 2.
    __syncthreads();  // the previous projection's last LDS reads are done
    load_A(0, 0);
    commit_A(0, 0);
    load_A(0, 1);
    commit_A(0, 1);
    load_B(bs[0], 0, 0);
    load_B(bs[1], 0, 1);
    __syncthreads();
    prefetch(0, 0, bs[0], P0{});

    for (int s = 0; s < n_stages; ++s) {
      const int buf = s & 1;
      // step 0
      load_A(s + 1, 0);
      load_B(bs[0], s, 2);
      prefetch(buf, 1, bs[1], P1{});
      mfma_step(P0{});
      interleave(V9{});
      // step 1
      commit_A(buf ^ 1, 0);
      load_A(s + 1, 1);
      load_B(bs[1], s, 3);
      prefetch(buf, 2, bs[0], P0{});
      mfma_step(P1{});
      interleave(V9{});
      // step 2, then hand the next dY tile over
      load_B(bs[0], s + 1, 0);
      prefetch(buf, 3, bs[1], P1{});
      mfma_step(P0{});
      interleave(V5{});
      commit_A(buf ^ 1, 1);
      __syncthreads();
      // step 3
      load_B(bs[1], s + 1, 1);
      prefetch(buf ^ 1, 0, bs[0], P0{});
      mfma_step(P1{});
      interleave(V5{});
    }
  }

  // ---- epilogue ---------------------------------------------------------------------------
  // register 4*i0+i1 of acc[mt][j] is dX[m0 + 32*mt + l32][8*(k8base + 8*i0 + 4*half + i1) + 2*wave + j]
  __syncthreads();
  uint16_t* base_plane = &lds[0][0];
  uint16_t* lora_plane = base_plane + EP_ROWS * EP_STRIDE;
  bool any_lora = false;
  for (int p = 0; p < a.n_proj; ++p) any_lora = any_lora || (select_proj(a, p).r > 0);
  const int kcol_lane = 8 * (k8base + l32) + 2 * wave;  // column whose A^T row this lane feeds to the LoRA MFMA
  const int k_tile0 = 8 * k8base;

  static_for<0, MT / 2>([&](auto q_c) {
    constexpr int q = decltype(q_c)::value;
    static_for<0, 2>([&](auto ml_c) {
      constexpr int ml = decltype(ml_c)::value;
      constexpr int mt = 2 * q + ml;
      const int m = m0 + 32 * mt + l32;
      const bool m_ok = m < a.M;
      f32x16 lora[NT];
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) lora[j][i] = 0.f;
      if (any_lora) {
        for (int p = 0; p < a.n_proj; ++p) {
          const BwdProjDev P = select_proj(a, p);
          if (P.r <= 0) continue;
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
#pragma unroll
          for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int i = 0; i < 16; ++i) lora[j][i] += P.s * tmp[j][i];
        }
      }
      // rounded pairs (tile 0, tile 1) = adjacent output columns -> one 4-byte LDS write
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int cp = 8 * (i >> 2) + 4 * half + (i & 3);
        const int o = (32 * ml + l32) * EP_STRIDE + 8 * cp + 2 * wave;
        *reinterpret_cast<uint32_t*>(base_plane + o) = pack2<T>(acc[mt][0][i], acc[mt][1][i]);
        if (any_lora) *reinterpret_cast<uint32_t*>(lora_plane + o) = pack2<T>(lora[0][i], lora[1][i]);
      }
    });
    __syncthreads();
    // coalesced pass: 64 rows x 32 chunks of 8 columns
#pragma unroll
    for (int it = 0; it < EP_ROWS * 32 / 256; ++it) {
      const int idx = tid + 256 * it;
      const int row = idx >> 5, chunk = idx & 31;
      const int m = m0 + EP_ROWS * q + row;
      const int k = k_tile0 + 8 * chunk;
      if (m < a.M && k < K) {
        const u32x4 bv = *reinterpret_cast<const u32x4*>(base_plane + row * EP_STRIDE + 8 * chunk);
        u32x4 lv = {0u, 0u, 0u, 0u};
        if (any_lora) lv = *reinterpret_cast<const u32x4*>(lora_plane + row * EP_STRIDE + 8 * chunk);
        if (a.mode == FMSA_BWD_SWIGLU) {
          const size_t off = (size_t)m * a.ldeg + k;
          const u32x4 ev = *reinterpret_cast<const u32x4*>(a.e + off);
          const u32x4 gv = *reinterpret_cast<const u32x4*>(a.g + off);
          u32x4 mv = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
          if (a.mask_src) mv = *reinterpret_cast<const u32x4*>(a.mask_src + (size_t)m * a.ldmask + k);
          u32x4 hv, dgv, dev;
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            float hh[2], dg[2], de[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const float e32 = j ? unpack_hi<T>(ev[w]) : unpack_lo<T>(ev[w]);
              const float g32 = j ? unpack_hi<T>(gv[w]) : unpack_lo<T>(gv[w]);
              const float b32 = j ? unpack_hi<T>(bv[w]) : unpack_lo<T>(bv[w]);
              const float l32f = j ? unpack_hi<T>(lv[w]) : unpack_lo<T>(lv[w]);
              const uint32_t mbits = (j ? (mv[w] >> 16) : mv[w]) & 0x7fffu;
              const float se = sigmoidf_(e32);
              const float f = unpack1<T>(pack1<T>(se * e32));
              const float h = unpack1<T>(pack1<T>(f * g32));
              // LoRA part of dh is masked by (dropout(h) != 0): mask_src holds dropout(h) when a
              // dropout was applied, otherwise h itself (recomputed here) decides
              const bool keep = a.mask_src ? (mbits != 0) : (h != 0.f);
              const float DW = unpack1<T>(pack1<T>(keep ? b32 + l32f : b32));
              hh[j] = h;
              dg[j] = DW * f;                                    // d_g ("df", UL/swiglu.py:77)
              const float dgt = unpack1<T>(pack1<T>(DW * g32));  // dg = DW * g in storage dtype (:79)
              de[j] = dgt * se * (1.0f + e32 * (1.0f - se));     // d_e (:81-83)
            }
            hv[w] = pack2<T>(hh[0], hh[1]);
            dgv[w] = pack2<T>(dg[0], dg[1]);
            dev[w] = pack2<T>(de[0], de[1]);
          }
          *reinterpret_cast<u32x4*>(a.h + off) = hv;
          *reinterpret_cast<u32x4*>(a.e + off) = dgv;
          *reinterpret_cast<u32x4*>(a.g + off) = dev;
        } else {
          u32x4 ov = bv;
          if (any_lora) {
            u32x4 mv = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
            if (a.mask_src) mv = *reinterpret_cast<const u32x4*>(a.mask_src + (size_t)m * a.ldmask + k);
#pragma unroll
            for (int w = 0; w < 4; ++w) {
              // +-0 in the mask source count as zero
              const float l0 = (mv[w] & 0x7fffu) ? unpack_lo<T>(lv[w]) : 0.f;
              const float l1 = ((mv[w] >> 16) & 0x7fffu) ? unpack_hi<T>(lv[w]) : 0.f;
              ov[w] = pack2<T>(unpack_lo<T>(bv[w]) + l0, unpack_hi<T>(bv[w]) + l1);
            }
          }
          *reinterpret_cast<u32x4*>(a.dX + (size_t)m * a.lddx + k) = ov;
        }
      }
    }
    __syncthreads();
  });
}

// nsz[g, n] = -fp32(scales[g, n]) * (z[g, n] + zero_offset): exact in fp32 (11-bit x 5-bit).
__global__ __launch_bounds__(256) void gptq_nsz_kernel(const uint16_t* __restrict__ scales,
                                                       const int32_t* __restrict__ qzeros, int G, int N,
                                                       int zero_offset, float* __restrict__ out) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= G * N) return;
  const int g = idx / N, n = idx % N;
  const uint32_t zw = (uint32_t)qzeros[(size_t)g * (N >> 3) + (n >> 3)];
  const float z = (float)(int)(((zw >> (4 * (n & 7))) & 0xFu) + zero_offset);
  out[idx] = -fp16_bits_to_f32(scales[idx]) * z;
}

}  // namespace

int launch_gptq_nsz(const fmsa_gptq_weight* w, float* out, hipStream_t st) {
  const int G = (w->K + w->group_size - 1) / w->group_size;
  dim3 grid((G * w->N + 255) / 256), block(256);
  hipLaunchKernelGGL(gptq_nsz_kernel, grid, block, 0, st, w->scales, w->qzeros, G, w->N, w->zero_offset, out);
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}

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
  bool ntail = false;
  for (int p = 0; p < n_proj; ++p) {
    const fmsa_bwd_proj& s = projs[p];
    BwdProjDev& d = a.p[p];
    d.qweight = s.w.qweight;
    d.scales = s.w.scales;
    d.nsz = s.nsz;
    d.dY = (const uint16_t*)s.dY;
    d.lddy = s.lddy;
    d.T = (const uint16_t*)s.T;
    d.At = (const uint16_t*)s.At;
    d.N = s.w.N;
    d.group_size = s.w.group_size;
    d.r = s.r;
    d.s = s.s;
    if (s.mask_src && s.r > 0) {
      a.mask_src = (const uint16_t*)s.mask_src;
      a.ldmask = s.ldmask;
    }
    ntail = ntail || (s.w.N % BK != 0);
  }
  a.nbm = (M + BM - 1) / BM;
  a.nbk = (a.K + 255) / 256;
  dim3 grid(a.nbm * a.nbk), block(256);
#define LAUNCH(TT)                                                                              \
  do {                                                                                          \
    if (ntail) hipLaunchKernelGGL((gptq_lora_bwd_dx_kernel<TT, true>), grid, block, 0, st, a);  \
    else hipLaunchKernelGGL((gptq_lora_bwd_dx_kernel<TT, false>), grid, block, 0, st, a);       \
  } while (0)
  if (act_dtype == FMSA_BF16)
    LAUNCH(bf16_t);
  else
    LAUNCH(f16_t);
#undef LAUNCH
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}
