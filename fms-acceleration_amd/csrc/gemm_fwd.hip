// Fused forward:  Y = X * deq(W) + s * U * B^T (+ bias), optional SwiGLU over a gate/up pair.
//
// Tiling (one workgroup = 4 waves = 256 lanes, one workgroup per CU):
//   workgroup tile  256 tokens x 256 output columns, K walked in stages of 64
//   wave tile       256 tokens x 64 columns = 8 x 2 MFMA 32x32x16 tiles, 256 fp32 accumulators
//   X operand       global -> LDS directly (buffer loads with the LDS bit: no staging registers, no
//                   ds_write), two stage buffers of 256 rows x 128 B, loaded one stage ahead.
//                   A direct load places lane p's 16 bytes at slot p of a 1 KB block, so the
//                   bank-conflict-free layout is obtained on the global side: slot c of row r holds
//                   the 8-element chunk c ^ ((r >> 1) & 7) of that row.  One barrier per stage.
//   W operand       never touches LDS: one packed int32 (8 nibbles along K at one column) is
//                   exactly the 8-element MFMA fragment of the lane that owns that column, so each
//                   lane loads its own words (a wave reads 2 x 128 B contiguous per load), unpacks
//                   them in registers and feeds the MFMA directly.  Each wave owns distinct
//                   columns, so no weight is unpacked twice inside a workgroup.
// The MFMA is issued as D^T = W^T-fragment x X-fragment: a lane then holds 4 consecutive output
// columns per accumulator quad, which turns the epilogue stores into 8-byte vectors.
// The rank-r LoRA term is one extra MFMA step per 16 ranks in the epilogue, scaled by s in fp32
// before the single rounding of the output.
#include "common.h"

namespace {

constexpr int BM = 256;
constexpr int BK = 64;
constexpr int EP_ROWS = 64;          // tokens per epilogue pass
constexpr int EP_STRIDE_L = 256 + 8;  // plane row stride (elements), linear: one plane of 256 columns
constexpr int EP_STRIDE_S = 128 + 8;  // SwiGLU: three planes (e, g, h) of 128 columns
constexpr int NBUF = 2;  // LDS stage buffers / register slots for the weight words
constexpr int MT = 8;
constexpr int NT = 2;

struct FwdProjDev {
  const int32_t* qweight;
  const uint16_t* scales;
  const int32_t* qzeros;
  const float* code;         // code-book format only
  const float* block_scale;  // code-book format only: fp32 [K / group_size, N]
  const uint16_t* U;
  int64_t ldu;
  const uint16_t* B;
  const uint16_t* bias;
  uint16_t* Y;
  int64_t ldy;
  int N, group_size, zero_offset, r;
  float s;
};

struct FwdArgs {
  FwdProjDev p[3];
  int nblk_start[4];
  const uint16_t* X;
  int64_t ldx;
  int M, K, mode, nbm, nbn;
  uint16_t* H;
  int64_t ldh;
  // rotary embedding in the epilogue (linear mode): projections whose bit is set in rope_mask leave rotated
  const void* rope_cos;
  const void* rope_sin;
  int64_t rope_ld;
  int rope_rows, rope_head_dim, rope_mask;
};

// a.p[p] for a runtime (wave-uniform) p without dynamic indexing of the kernel-argument struct,
// which would force a copy of it into scratch memory.
FMSA_DEVI FwdProjDev select_proj(const FwdArgs& a, int p) { return p == 0 ? a.p[0] : (p == 1 ? a.p[1] : a.p[2]); }

// GPS = scale groups per 64-wide K stage: 1 for group_size % 64 == 0, 2 / 4 for group sizes 32 / 16.
// CODEBOOK (1, 2): the nibbles index a 16-entry table and one fp32 scale per (group, column) multiplies the
// entry (W = code[q] * block_scale); 0: the affine GPTQ form W = scale * (q - zero).  1 gathers code[q] from the
// lanes of the wave (one ds_bpermute per weight) and multiplies; 2 (GPS == 1) multiplies the 16 entries by the lane's
// block scale once per stage and column, keeps the 16 rounded products as two byte planes in registers, and looks the
// weights up with byte permutes: the same products, no gather on the LDS pipe that the X fragments keep busy.
// ROPE (1: cos / sin tables in the activation type, 2: in fp32; 0: none): the Q / K projections of an attention block
// leave the kernel with the rotary embedding applied
// (kernels/unsloth/rope_embedding.py:36-65 of the reference: (q1, q2) <- (q1 cos - q2 sin, q2 cos + q1 sin) on the two
// halves of every head, on the projection output ROUNDED to the storage type, fp32 arithmetic, one more rounding).
// PK16 (fp16 activations, affine weights whose words hold their nibbles interleaved -- element 2p at position p, element
// 2p + 1 at position 4 + p --, one scale group per stage): a fragment register is (((w >> 4p) & 0x000F000F) | 0x64006400)
// + (-(1024 + z)) [exact] times the fp16 scale [one rounding] in packed half arithmetic: RNE_fp16(s * (q - z)) bit for bit
// in 15 instead of 22 instructions per word.
template <typename T, int GPS, bool KTAIL, int CODEBOOK, int ROPE = 0, bool PK16 = false>
__global__ __launch_bounds__(256) void gptq_lora_fwd_kernel(const FwdArgs a) {
  static_assert(!PK16 || (std::is_same<T, f16_t>::value && CODEBOOK == 0 && GPS == 1 && ROPE == 0), "packed half unpack");
  // two separate arrays (not one 2-D array): every access names its buffer statically, which is
  // what lets the compiler see that fragment reads of one buffer do not depend on the direct loads
  // in flight into the other
  __shared__ __attribute__((aligned(1024))) uint16_t lds0[BM * BK];
  __shared__ __attribute__((aligned(1024))) uint16_t lds1[BM * BK];
  __shared__ __attribute__((aligned(16))) uint16_t ep_planes[3 * EP_ROWS * EP_STRIDE_S];  // >= EP_ROWS * EP_STRIDE_L
  static_assert(3 * EP_STRIDE_S >= EP_STRIDE_L, "the linear plane must fit");
  auto lds_buf = [&](auto b_c) -> char* {
    constexpr int b = decltype(b_c)::value;
    return reinterpret_cast<char*>(b == 0 ? lds0 : lds1);
  };

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int half = lane >> 5;

  // ---- tile assignment: XCD-contiguous ranges, then grouped-M order inside the range --------
  int pid = xcd_remap(blockIdx.x, a.nbm * a.nbn);
  constexpr int GROUP_M = 4;  // token blocks per group: 4 x 8 tiles in flight per XCD share X and W tiles in its L2
  const int width = GROUP_M * a.nbn;
  const int first_m = (pid / width) * GROUP_M;
  const int gsz = min(a.nbm - first_m, GROUP_M);
  const int bm = first_m + (pid % width) % gsz;
  const int bn = (pid % width) / gsz;
  const int m0 = bm * BM;

  int pj[NT], col0[NT];
  bool active[NT];
  if (a.mode == FMSA_FWD_SWIGLU) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      pj[j] = j;
      col0[j] = bn * 128 + wave * 32;
    }
  } else {
    int p = 0;
    if (bn >= a.nblk_start[1]) p = 1;
    if (bn >= a.nblk_start[2]) p = 2;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      pj[j] = p;
      col0[j] = (bn - a.nblk_start[p]) * 256 + wave * 64 + j * 32;
    }
  }
  const char* qbase[NT];
  const char* scbase[NT];
  const char* zbase[NT];
  int Np[NT], zshift[NT], gs[NT];
  float zoff[NT], lut[NT];  // lut: this lane's entry of the projection's code book (lanes 0..15 serve as the table)
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const FwdProjDev P = select_proj(a, pj[j]);
    active[j] = col0[j] < P.N;
    if (!active[j]) col0[j] = 0;
    const int col = col0[j] + l32;
    // wave-uniform by construction; readfirstlane tells the compiler so (scalar offsets below)
    Np[j] = __builtin_amdgcn_readfirstlane(P.N);
    gs[j] = __builtin_amdgcn_readfirstlane(P.group_size);
    qbase[j] = reinterpret_cast<const char*>(P.qweight);
    scbase[j] = CODEBOOK ? reinterpret_cast<const char*>(P.block_scale) : reinterpret_cast<const char*>(P.scales);
    lut[j] = CODEBOOK == 1 ? P.code[lane & 15] : 0.f;
    zbase[j] = reinterpret_cast<const char*>(P.qzeros);
    zshift[j] = 4 * (col & 7);
    zoff[j] = (float)P.zero_offset;
  }

  // table flavour: the code book as wave-uniform values (the launcher takes this flavour only when the projections of
  // the launch share one code book), and per column tile the byte planes of the current stage's 16 rounded products:
  // byte e of tlo[set][j][d] / thi[set][j][d] = low / high byte of entry 4 d + e.  Two sets: while the stage in slot SB
  // looks its weights up in set SB, the steps of that stage build set SB ^ 1 for the next one, a quarter per step, so
  // the 80 instructions of a table pair sit between MFMAs like the rest.  That needs the block scale one stage earlier
  // than the weights: load_stage(st) fetches the scale of stage st + 1.
  float cd[16];
  uint32_t tlo[NBUF][NT][4], thi[NBUF][NT][4];
  int gshift[NT];  // log2 of the block size (the launcher takes this flavour for powers of two only)
  if constexpr (CODEBOOK == 2) {
#pragma unroll
    for (int i = 0; i < 16; ++i) cd[i] = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(a.p[0].code[i])));
#pragma unroll
    for (int j = 0; j < NT; ++j) gshift[j] = 31 - __builtin_clz(gs[j]);
  }

  const int K = a.K;
  const int n_stages = (K + BK - 1) / BK;

  f32x16 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;

  // ---- operand addressing: buffer loads (SGPR resource + 32-bit lane offset + SGPR offset) -----
  // No 64-bit address arithmetic in the loop, and lanes whose offset falls outside the resource
  // read zeros: rows past M need no predication.
  // X tile: wave w fills rows 64w .. 64w+63 of a stage buffer with 8 direct loads; load i covers
  // rows 64w+8i .. +7, lane p writes slot (p & 7) of row 64w + 8i + (p >> 3), which holds chunk
  // (p & 7) ^ ((row >> 1) & 7) of that row.
  const int uwave = __builtin_amdgcn_readfirstlane(wave);
  const int rows_valid = min(BM, a.M - m0);
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(a.X + (size_t)m0 * a.ldx, (size_t)rows_valid * a.ldx * 2);
  uint32_t x_off[8];
  const int chunk_even = (lane & 7) ^ (lane >> 4);  // chunk fetched by loads 0, 2, 4, 6; odd loads: ^ 4
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = 64 * wave + 8 * i + (lane >> 3);
    const int chunk = chunk_even ^ (4 * (i & 1));
    x_off[i] = (uint32_t)((row * a.ldx + 8 * chunk) * 2);
  }
  // fragment reads: row 32*mt + l32, chunk 2t + half -> slot (2t + half) ^ ((l32 >> 1) & 7)
  uint32_t lds_r_off[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) lds_r_off[t] = (uint32_t)(l32 * (BK * 2) + 16 * ((2 * t + half) ^ ((l32 >> 1) & 7)));
  // weights: word (k8, col) at k8*N*4 + col*4; the lane part is (half*N + col)*4
  __amdgpu_buffer_rsrc_t q_rsrc[NT], sc_rsrc[NT], z_rsrc[NT];
  uint32_t q_off[NT], sc_off[NT], z_off[NT];
  uint32_t q_stage_bytes[NT], q_step_bytes[NT], q_last[NT];
  int n_groups_j[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int n_groups = (K + gs[j] - 1) / gs[j];
    n_groups_j[j] = n_groups;
    q_rsrc[j] = make_rsrc(qbase[j], (size_t)(K >> 3) * Np[j] * 4);
    sc_rsrc[j] = make_rsrc(scbase[j], (size_t)n_groups * Np[j] * (CODEBOOK ? 4 : 2));
    z_rsrc[j] = make_rsrc(zbase[j], CODEBOOK ? 0 : (size_t)n_groups * (Np[j] >> 3) * 4);
    q_off[j] = (uint32_t)((half * Np[j] + col0[j] + l32) * 4);
    sc_off[j] = (uint32_t)((col0[j] + l32) * (CODEBOOK ? 4 : 2));
    z_off[j] = (uint32_t)(((col0[j] + l32) >> 3) * 4);
    q_step_bytes[j] = (uint32_t)Np[j] * 8;    // two packed rows per 16-wide K step
    q_stage_bytes[j] = (uint32_t)Np[j] * 32;  // eight packed rows per stage
    q_last[j] = (uint32_t)((K >> 3) - 2) * Np[j] * 4;
  }

  // Weight words, scales and zero words in two register slots (slot = stage % 2), loaded one
  // stage ahead together with X.
  uint32_t qw[NBUF][NT][4];
  uint16_t sc_raw[NBUF][NT][GPS];
  uint32_t zw_raw[NBUF][NT][GPS];  // code-book format: the fp32 block scale
  float sf[NT][GPS], sf16[NT][GPS], nsz[NT][GPS];
  uint32_t sp16[NT], nz16[NT];  // PK16: the stage's scale and -(1024 + zero) as fp16 pairs (both halves equal)
  const uint32_t pk_mask = opaque(0x000F000Fu), pk_bias = opaque(0x64006400u);  // in vector registers: the and-or takes no literal
  // group index of the stage being loaded, advanced without a division when GPS == 1
  int g_ld[NT], k_in_g[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) g_ld[j] = k_in_g[j] = 0;
  // issue the global loads of stage `st` (0 <= st < n_stages) into slot SB; nothing here may read
  // the loaded registers, or the wave would wait for the load on the spot
  auto load_stage = [&](int st, auto sb_c) {
    constexpr int SB = decltype(sb_c)::value;
    const uint32_t x_soff = (uint32_t)st * (BK * 2);
    // K % 64 == 32 (KTAIL): in the last stage the upper half of the stage lies past K.  Its X
    // columns are forced out of range (zeros); the weight rows are clamped to valid memory.
    uint32_t poison[2] = {0u, 0u};
    if constexpr (KTAIL) {
      poison[0] = ((st * BK + 8 * chunk_even) < K) ? 0u : 0x80000000u;
      poison[1] = ((st * BK + 8 * (chunk_even ^ 4)) < K) ? 0u : 0x80000000u;
    }
    char* lw = lds_buf(sb_c) + uwave * (64 * BK * 2);
#pragma unroll
    for (int i = 0; i < 8; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (__attribute__((address_space(3))) void*)(lw + i * (8 * BK * 2)),
                                               16, x_off[i] | poison[i & 1], x_soff, 0, 0);
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const uint32_t qs = (uint32_t)st * q_stage_bytes[j];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        uint32_t so = qs + t * q_step_bytes[j];
        if constexpr (KTAIL) so = min(so, q_last[j]);
        qw[SB][j][t] = __builtin_amdgcn_raw_buffer_load_b32(q_rsrc[j], q_off[j], so, 0);
      }
#pragma unroll
      for (int u = 0; u < GPS; ++u) {
        int gu;
        if constexpr (GPS == 1) {
          gu = min(g_ld[j], n_groups_j[j] - 1);
        } else {
          const int ku = st * BK + u * (BK / GPS);
          gu = (ku < K ? ku : st * BK) / gs[j];
        }
        gu = __builtin_amdgcn_readfirstlane(gu);  // uniform; keeps the scalar offsets out of vector registers
        if constexpr (CODEBOOK == 2) {
          const int g1 = __builtin_amdgcn_readfirstlane(min(((st + 1) * BK) >> gshift[j], n_groups_j[j] - 1));
          zw_raw[SB ^ 1][j][u] = __builtin_amdgcn_raw_buffer_load_b32(sc_rsrc[j], sc_off[j], (uint32_t)g1 * Np[j] * 4, 0);
        } else if constexpr (CODEBOOK == 1) {
          zw_raw[SB][j][u] = __builtin_amdgcn_raw_buffer_load_b32(sc_rsrc[j], sc_off[j], (uint32_t)gu * Np[j] * 4, 0);
        } else {
          sc_raw[SB][j][u] = __builtin_amdgcn_raw_buffer_load_b16(sc_rsrc[j], sc_off[j], (uint32_t)gu * Np[j] * 2, 0);
          zw_raw[SB][j][u] = __builtin_amdgcn_raw_buffer_load_b32(z_rsrc[j], z_off[j], (uint32_t)gu * (Np[j] >> 3) * 4, 0);
        }
      }
      if constexpr (GPS == 1) {  // uniform scalar bookkeeping, no division
        k_in_g[j] += BK;
        const bool wrap = k_in_g[j] >= gs[j];
        k_in_g[j] -= wrap ? gs[j] : 0;
        g_ld[j] += wrap ? 1 : 0;
      }
    }
  };
  // make the scales / zeros of slot SB current
  auto commit_stage = [&](auto sb_c) {
    constexpr int SB = decltype(sb_c)::value;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
#pragma unroll
      for (int u = 0; u < GPS; ++u) {
        if constexpr (CODEBOOK == 2) {
          // (the tables are built step by step in prefetch)
        } else if constexpr (CODEBOOK == 1) {
          sf[j][u] = __uint_as_float(zw_raw[SB][j][u]);
        } else if constexpr (PK16) {
          sp16[j] = (uint32_t)sc_raw[SB][j][u] * 0x00010001u;
          const float nz = -(1024.0f + (float)((zw_raw[SB][j][u] >> zshift[j]) & 0xFu) + zoff[j]);  // exact in fp16
          nz16[j] = pack2<f16_t>(nz, nz);
        } else {
          sf[j][u] = fp16_bits_to_f32(sc_raw[SB][j][u]);
          sf16[j][u] = sf[j][u] * 0.0625f;
          const float z = (float)((zw_raw[SB][j][u] >> zshift[j]) & 0xFu) + zoff[j];
          nsz[j][u] = -sf[j][u] * z;  // exact: 11-bit x 5-bit
        }
      }
    }
  };

  // Software pipeline at the granularity of one 16-wide MFMA K step: while the 16 MFMAs of step t
  // run, the 8 X fragments of step t+1 are read from LDS and its 2 weight fragments are unpacked,
  // into the other half of xf / wf.  The stage barrier sits after step 2, so step 3 can already
  // fetch step 0 of the next stage from the next LDS buffer.
  u32x4 xf[2][MT], wf[2][NT];
  // entries 4 d .. 4 d + 3 of table set SET from the block scales in raw slot SET: the products rounded to the storage
  // type in pairs, then the two byte planes
  auto build_table_part = [&](auto set_c, auto d_c) {
    constexpr int SET = decltype(set_c)::value;
    constexpr int d = decltype(d_c)::value;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const float sc = __uint_as_float(zw_raw[SET][j][0]);
      const uint32_t p0 = pack2<T>(cd[4 * d] * sc, cd[4 * d + 1] * sc), p1 = pack2<T>(cd[4 * d + 2] * sc, cd[4 * d + 3] * sc);
      tlo[SET][j][d] = __builtin_amdgcn_perm(p1, p0, 0x06040200u);
      thi[SET][j][d] = __builtin_amdgcn_perm(p1, p0, 0x07050301u);
    }
  };
  auto prefetch = [&](auto sb_c, auto t_c, auto par_c) {
    constexpr int SB = decltype(sb_c)::value;
    constexpr int t = decltype(t_c)::value;
    constexpr int par = decltype(par_c)::value;
    const char* lr = lds_buf(sb_c) + lds_r_off[t];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xf[par][mt] = *reinterpret_cast<const u32x4*>(lr + mt * 32 * BK * 2);
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      if constexpr (CODEBOOK == 2) {
        // nibble 2b / 2b + 1 of the word (weights k = 2b, 2b + 1 of the step) sit in byte b: per byte plane two
        // permutes over entries 0-7 and 8-15 with the nibble's low three bits, a third picks by its top bit
        const uint32_t w = qw[SB][j][t];
        const uint32_t se = w & 0x07070707u, so = (w >> 4) & 0x07070707u;
        const uint32_t pe = ((w >> 1) & 0x04040404u) | 0x03020100u, po = ((w >> 5) & 0x04040404u) | 0x03020100u;
        const uint32_t loe = __builtin_amdgcn_perm(__builtin_amdgcn_perm(tlo[SB][j][3], tlo[SB][j][2], se), __builtin_amdgcn_perm(tlo[SB][j][1], tlo[SB][j][0], se), pe);
        const uint32_t hie = __builtin_amdgcn_perm(__builtin_amdgcn_perm(thi[SB][j][3], thi[SB][j][2], se), __builtin_amdgcn_perm(thi[SB][j][1], thi[SB][j][0], se), pe);
        const uint32_t loo = __builtin_amdgcn_perm(__builtin_amdgcn_perm(tlo[SB][j][3], tlo[SB][j][2], so), __builtin_amdgcn_perm(tlo[SB][j][1], tlo[SB][j][0], so), po);
        const uint32_t hio = __builtin_amdgcn_perm(__builtin_amdgcn_perm(thi[SB][j][3], thi[SB][j][2], so), __builtin_amdgcn_perm(thi[SB][j][1], thi[SB][j][0], so), po);
        // 16-bit values of weights (0, 2), (4, 6) and (1, 3), (5, 7), then the pairs (k, k + 1) the fragment holds
        const uint32_t e01 = __builtin_amdgcn_perm(hie, loe, 0x05010400u), e23 = __builtin_amdgcn_perm(hie, loe, 0x07030602u);
        const uint32_t o01 = __builtin_amdgcn_perm(hio, loo, 0x05010400u), o23 = __builtin_amdgcn_perm(hio, loo, 0x07030602u);
        wf[par][j][0] = __builtin_amdgcn_perm(o01, e01, 0x05040100u);
        wf[par][j][1] = __builtin_amdgcn_perm(o01, e01, 0x07060302u);
        wf[par][j][2] = __builtin_amdgcn_perm(o23, e23, 0x05040100u);
        wf[par][j][3] = __builtin_amdgcn_perm(o23, e23, 0x07060302u);
      } else if constexpr (PK16) {
        static_for<0, 4>([&](auto r_c) {
          constexpr int r = decltype(r_c)::value;
          wf[par][j][r] = pk_sub_mul_f16(((qw[SB][j][t] >> (4 * r)) & pk_mask) | pk_bias, nz16[j], sp16[j]);
        });
      } else {
        wf[par][j] = dequant8<T>(qw[SB][j][t], sf[j][t * GPS / 4], sf16[j][t * GPS / 4], nsz[j][t * GPS / 4]);
      }
    }
    if constexpr (CODEBOOK == 2) build_table_part(std::integral_constant<int, SB ^ 1>{}, t_c);
  };
  // Code-book flavour in two phases, so that a step's first 8 MFMAs cover the table gathers and its
  // last 8 the arithmetic on what they returned.  Phase a: the 8 X fragments and the 16 gathers
  // (ds_bpermute from the lane-resident table; element 2b / 2b+1 of a word in gath[j][b] / [4 + b]).
  uint32_t gath[NT][8];
  auto prefetch_a = [&](auto sb_c, auto t_c, auto par_c) {
    constexpr int SB = decltype(sb_c)::value;
    constexpr int t = decltype(t_c)::value;
    constexpr int par = decltype(par_c)::value;
    const char* lr = lds_buf(sb_c) + lds_r_off[t];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xf[par][mt] = *reinterpret_cast<const u32x4*>(lr + mt * 32 * BK * 2);
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const uint32_t w = qw[SB][j][t];
      const uint32_t e = opaque((w << 2) & 0x3C3C3C3Cu);  // byte b: 4 * nibble 2b (a lane's byte address)
      const uint32_t o = opaque((w >> 2) & 0x3C3C3C3Cu);  // byte b: 4 * nibble 2b+1
      const int li = (int)__float_as_uint(lut[j]);
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        gath[j][b] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((e >> (8 * b)) & 0xffu), li);
        gath[j][4 + b] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((o >> (8 * b)) & 0xffu), li);
      }
    }
  };
  // phase b: code * block scale in fp32, one rounding
  auto prefetch_b = [&](auto t_c, auto par_c) {
    constexpr int t = decltype(t_c)::value;
    constexpr int par = decltype(par_c)::value;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const float sc = sf[j][t * GPS / 4];
#pragma unroll
      for (int b = 0; b < 4; ++b) wf[par][j][b] = pack2<T>(__uint_as_float(gath[j][b]) * sc, __uint_as_float(gath[j][4 + b]) * sc);
    }
  };
  auto mfma_step = [&](auto par_c) {
    constexpr int par = decltype(par_c)::value;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < NT; ++j) acc[mt][j] = mfma32<T>(wf[par][j], xf[par][mt], acc[mt][j]);
  };
  auto mfma_half = [&](auto par_c, auto h_c) {
    constexpr int par = decltype(par_c)::value;
    constexpr int h = decltype(h_c)::value;
#pragma unroll
    for (int mt = h * (MT / 2); mt < (h + 1) * (MT / 2); ++mt)
#pragma unroll
      for (int j = 0; j < NT; ++j) acc[mt][j] = mfma32<T>(wf[par][j], xf[par][mt], acc[mt][j]);
  };
  // One wave per SIMD issues strictly in order, and an MFMA that finds the matrix pipe busy stalls
  // everything behind it.  The other instructions of a step therefore have to sit BETWEEN its 16
  // MFMAs (each occupies the pipe for 8 issue slots): per MFMA 3 VALU, every second one an LDS
  // read, and in step 0 also the global loads of a later stage with their scalar offset math.
  auto interleave = [&](auto with_vmem_c) {
    constexpr bool with_vmem = decltype(with_vmem_c)::value;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, CODEBOOK == 2 ? 5 : 3, 0);
      if ((i & 1) == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      if (with_vmem) {
        if (i < 6)
          __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
        else
          __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);  // nothing from the next step (or the stage hand-over) moves up
  };
  // code-book halves: (a) 8 MFMAs with the address arithmetic (3 VALU) and 3 LDS-pipe instructions
  // each (8 fragment reads + 16 gathers); (b) 8 MFMAs with the 24 multiplies / conversions and, in the
  // last step of a stage, the global loads of a later stage
  auto interleave_a = [&]() {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
      __builtin_amdgcn_sched_group_barrier(0x080, 3, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto interleave_b = [&](auto with_vmem_c) {
    constexpr bool with_vmem = decltype(with_vmem_c)::value;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
      if (with_vmem) {
        if (i < 2)
          __builtin_amdgcn_sched_group_barrier(0x020, 3, 0);
        else
          __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  using WithVmem = std::integral_constant<bool, true>;
  using NoVmem = std::integral_constant<bool, false>;
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;

  // One 64-wide K stage out of LDS buffer / register slot SB = s % 2.  Steps 0-2 read the stage's
  // fragments; then every wave waits for its own loads of stage s + 1 (issued one stage earlier),
  // and the barrier makes all four waves' parts visible and closes the reads of buffer SB.  Step 3
  // therefore is where the loads of stage s + 2 go out, into the buffer and register slot this
  // stage has just vacated.  The last two stages re-load the final stage (no branch); that data
  // is never read.
  constexpr int WAIT_VM0 = 0x0F70;  // s_waitcnt vmcnt(0) only
  // one 16-wide K step: the MFMAs of parity `cur` while fragments and weights of (buffer nb, step nt)
  // are produced into parity `nx`
  auto step = [&](auto nb_c, auto nt_c, auto nx_c, auto cur_c, auto vmem_c) {
    if constexpr (CODEBOOK == 1) {
      prefetch_a(nb_c, nt_c, nx_c);
      mfma_half(cur_c, I0{});
      interleave_a();
      prefetch_b(nt_c, nx_c);
      mfma_half(cur_c, I1{});
      interleave_b(vmem_c);
    } else {
      prefetch(nb_c, nt_c, nx_c);
      mfma_step(cur_c);
      interleave(vmem_c);
    }
  };
  // The affine step (one scale group per stage) written slot by slot, as the input-gradient kernel on the transposed
  // twin does: the 16 MFMAs of parity `cur`, behind each one its share of the work that produces step (nb, nt) into
  // parity `nx` -- a fragment read behind the first eight, one unpacked fragment register (2 conversions, 2
  // multiply-adds, 1 packed conversion) behind every even one -- and, in the last step of a stage, the 20 loads of
  // stage `st_next` into buffer / slot `lb`.  A scheduling fence closes every slot: the order below is the schedule
  // (about 1 % faster than what the group-barrier matcher makes of the same step; the fragment reads spread over the
  // odd slots instead measured no gain).
  constexpr bool HAND = CODEBOOK == 0 && GPS == 1;
  // load number `idx` of stage `st` into slot SB (GPS == 1, affine): 0-7 the X tile (direct loads), 8-15 the weight
  // words (idx - 8 = 4 j + t), 16-17 scale and zero word of column tile 0, 18-19 of column tile 1
  auto load_piece = [&](int st, auto sb_c, auto idx_c) {
    constexpr int SB = decltype(sb_c)::value;
    constexpr int idx = decltype(idx_c)::value;
    if constexpr (idx < 8) {
      uint32_t poison = 0u;
      if constexpr (KTAIL) poison = ((st * BK + 8 * (chunk_even ^ (4 * (idx & 1)))) < K) ? 0u : 0x80000000u;
      char* lw = lds_buf(sb_c) + uwave * (64 * BK * 2);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (__attribute__((address_space(3))) void*)(lw + idx * (8 * BK * 2)), 16,
                                               x_off[idx] | poison, (uint32_t)st * (BK * 2), 0, 0);
    } else if constexpr (idx < 16) {
      constexpr int j = (idx - 8) >> 2, t = (idx - 8) & 3;
      uint32_t so = (uint32_t)st * q_stage_bytes[j] + t * q_step_bytes[j];
      if constexpr (KTAIL) so = min(so, q_last[j]);
      qw[SB][j][t] = __builtin_amdgcn_raw_buffer_load_b32(q_rsrc[j], q_off[j], so, 0);
    } else {
      constexpr int j = (idx - 16) >> 1;
      const int gu = __builtin_amdgcn_readfirstlane(min(g_ld[j], n_groups_j[j] - 1));
      if constexpr (((idx - 16) & 1) == 0) {
        sc_raw[SB][j][0] = __builtin_amdgcn_raw_buffer_load_b16(sc_rsrc[j], sc_off[j], (uint32_t)gu * Np[j] * 2, 0);
      } else {
        zw_raw[SB][j][0] = __builtin_amdgcn_raw_buffer_load_b32(z_rsrc[j], z_off[j], (uint32_t)gu * (Np[j] >> 3) * 4, 0);
        k_in_g[j] += BK;  // uniform scalar bookkeeping, no division
        const bool wrap = k_in_g[j] >= gs[j];
        k_in_g[j] -= wrap ? gs[j] : 0;
        g_ld[j] += wrap ? 1 : 0;
      }
    }
  };
  auto step_affine = [&](auto nb_c, auto nt_c, auto nx_c, auto cur_c, auto vmem_c, int st_next, auto lb_c) {
    constexpr int SB = decltype(nb_c)::value;
    constexpr int t = decltype(nt_c)::value;
    constexpr int par = decltype(nx_c)::value;
    constexpr int cur = decltype(cur_c)::value;
    constexpr bool with_vmem = decltype(vmem_c)::value;
    const char* lr = lds_buf(nb_c) + lds_r_off[t];
    auto mfma_slot = [&](int slot) { acc[slot >> 1][slot & 1] = mfma32<T>(wf[cur][slot & 1], xf[cur][slot >> 1], acc[slot >> 1][slot & 1]); };
    auto frag = [&](int mt) { xf[par][mt] = *reinterpret_cast<const u32x4*>(lr + mt * 32 * BK * 2); };
    auto fence = [&]() { __builtin_amdgcn_sched_barrier(0); };
    auto dma = [&](auto idx_c) {
      if constexpr (with_vmem) load_piece(st_next, lb_c, idx_c);
    };
    uint32_t nib[NT][2];  // [tile][0]: nibbles 0, 2, 4, 6 in bytes 0..3; [1]: 16 * nibbles 1, 3, 5, 7 (the scale is pre-divided)
    auto masks = [&](auto j_c) {
      constexpr int j = decltype(j_c)::value;
      if constexpr (!PK16) {
        nib[j][0] = opaque(qw[SB][j][t] & 0x0F0F0F0Fu);
        nib[j][1] = opaque(qw[SB][j][t] & 0xF0F0F0F0u);
      }
    };
    auto piece = [&](auto j_c, auto reg_c) {
      constexpr int j = decltype(j_c)::value;
      constexpr int reg = decltype(reg_c)::value;
      if constexpr (PK16) {
        wf[par][j][reg] = pk_sub_mul_f16(((qw[SB][j][t] >> (4 * reg)) & pk_mask) | pk_bias, nz16[j], sp16[j]);
        return;
      }
      float b0, b1;
      if constexpr (reg == 0) {
        b0 = ubyte0(nib[j][0]);
        b1 = ubyte0(nib[j][1]);
      } else if constexpr (reg == 1) {
        b0 = ubyte1(nib[j][0]);
        b1 = ubyte1(nib[j][1]);
      } else if constexpr (reg == 2) {
        b0 = ubyte2(nib[j][0]);
        b1 = ubyte2(nib[j][1]);
      } else {
        b0 = ubyte3(nib[j][0]);
        b1 = ubyte3(nib[j][1]);
      }
      wf[par][j][reg] = pack2<T>(__builtin_fmaf(sf[j][0], b0, nsz[j][0]), __builtin_fmaf(sf16[j][0], b1, nsz[j][0]));
    };
    static_for<0, 16>([&](auto u_c) {
      constexpr int u = decltype(u_c)::value;
      mfma_slot(u);
      if constexpr (u == 0) masks(std::integral_constant<int, 0>{});
      if constexpr (u == 8) masks(std::integral_constant<int, 1>{});
      if constexpr ((u & 1) == 0) piece(std::integral_constant<int, (u >> 3)>{}, std::integral_constant<int, ((u >> 1) & 3)>{});
      if constexpr (u < 8) frag(u);
      dma(std::integral_constant<int, u>{});
      if constexpr (u >= 12) dma(std::integral_constant<int, 4 + u>{});  // loads 16-19: scales and zero words
      fence();
    });
  };
  auto stage = [&](int s, auto sb_c) {
    constexpr int SB = decltype(sb_c)::value;
    using S1 = std::integral_constant<int, SB ^ 1>;
    if constexpr (HAND) {
      step_affine(sb_c, I1{}, I1{}, I0{}, NoVmem{}, 0, sb_c);
      step_affine(sb_c, I2{}, I0{}, I1{}, NoVmem{}, 0, sb_c);
      step_affine(sb_c, I3{}, I1{}, I0{}, NoVmem{}, 0, sb_c);
    } else {
      step(sb_c, I1{}, I1{}, I0{}, NoVmem{});
      step(sb_c, I2{}, I0{}, I1{}, NoVmem{});
      step(sb_c, I3{}, I1{}, I0{}, NoVmem{});
    }
    __builtin_amdgcn_s_waitcnt(WAIT_VM0);
    commit_stage(S1{});
    __syncthreads();
    if constexpr (HAND) {
      step_affine(S1{}, I0{}, I0{}, I1{}, WithVmem{}, min(s + 2, n_stages - 1), sb_c);
    } else {
      load_stage(min(s + 2, n_stages - 1), sb_c);
      step(S1{}, I0{}, I0{}, I1{}, WithVmem{});
    }
  };

  // LoRA operands of ranks 0..15 (the whole adapter up to rank 16): direct loads into the epilogue planes,
  // which are idle until the epilogue, issued here so that their latency is not exposed after the main loop.
  // KB (8u + mt): rows 32mt..32mt+31 of U of the tile's u-th projection, 16 B per (row, rank half) at slot
  // 2 * row + half.  KB (16 + NT * wave + j): the same for the wave's 32 rows of B of column tile j.
  // Ranks past r and rows past M / N arrive as zeros through the range check.
  char* const lora_lds = reinterpret_cast<char*>(ep_planes);
  static_assert(sizeof(ep_planes) >= (16 + 4 * NT) * 1024, "LoRA operands must fit into the epilogue planes");
  const bool lora_any = (a.p[0].r | a.p[1].r | a.p[2].r) != 0;
  if (lora_any) {
    const int prow = lane >> 1, phalf = lane & 1;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const FwdProjDev P = select_proj(a, pj[j]);
      const int rp = __builtin_amdgcn_readfirstlane(P.r);
      const uint32_t dead = (8 * phalf < rp) ? 0u : 0x80000000u;
      if (j == 0 || a.mode == FMSA_FWD_SWIGLU) {  // linear mode: both column tiles belong to one projection
        const __amdgpu_buffer_rsrc_t u_rs = make_rsrc(P.U + (size_t)m0 * P.ldu, rp > 0 ? (size_t)rows_valid * P.ldu * 2 : 0);
#pragma unroll
        for (int i = 0; i < 2; ++i)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(
              u_rs, (__attribute__((address_space(3))) void*)(lora_lds + (8 * j + 2 * uwave + i) * 1024), 16,
              (uint32_t)(((64 * wave + 32 * i + prow) * P.ldu + 8 * phalf) * 2) | dead, 0, 0, 0);
      }
      const __amdgpu_buffer_rsrc_t b_rs = make_rsrc(P.B, rp > 0 ? (size_t)P.N * rp * 2 : 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rs, (__attribute__((address_space(3))) void*)(lora_lds + (16 + NT * uwave + j) * 1024),
                                               16, (uint32_t)(((col0[j] + prow) * rp + 8 * phalf) * 2) | dead, 0, 0, 0);
    }
  }
  if constexpr (CODEBOOK == 2) {
#pragma unroll
    for (int j = 0; j < NT; ++j) zw_raw[0][j][0] = __builtin_amdgcn_raw_buffer_load_b32(sc_rsrc[j], sc_off[j], 0, 0);
  }
  load_stage(0, I0{});
  __builtin_amdgcn_s_waitcnt(WAIT_VM0);
  commit_stage(I0{});
  if constexpr (CODEBOOK == 2) {  // the first stage's tables, all at once
    build_table_part(I0{}, I0{});
    build_table_part(I0{}, I1{});
    build_table_part(I0{}, I2{});
    build_table_part(I0{}, I3{});
  }
  __syncthreads();
  load_stage(min(1, n_stages - 1), I1{});
  if constexpr (CODEBOOK == 1) {
    prefetch_a(I0{}, I0{}, I0{});
    prefetch_b(I0{}, I0{});
  } else {
    prefetch(I0{}, I0{}, I0{});
  }

  // whole pairs in a single-exit loop (slots 0, 1), then the odd stage
  const int n_full = n_stages & ~1;
  int s = 0;
  for (; s < n_full; s += NBUF) {
    stage(s, I0{});
    stage(s + 1, I1{});
  }
  if (s < n_stages) stage(s, I0{});

  // ---- LoRA term as extra contraction steps: acc += U[:, j0..j0+15] x (s * B[:, j0..j0+15])^T -------
  // s * B is rounded to the storage type, the rounding point of the reference's
  // `(X @ A.t()) @ (s * B.t())` (UL/gptq/fast_lora.py:167-169).  Rows past M read zeros through the
  // buffer resource.
  // One loop for both modes (no mode branch around the accumulators): tile j takes U and B of its
  // own projection -- gate / up in SwiGLU mode, twice the same projection otherwise.
  {
    const uint16_t* Uj[NT];
    const uint16_t* Bj[NT];
    int rj[NT];
    int64_t lduj[NT];
    float sj[NT];
    __amdgpu_buffer_rsrc_t u_rsrc[NT];
    int r_max = 0;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const FwdProjDev P = select_proj(a, pj[j]);
      rj[j] = __builtin_amdgcn_readfirstlane(P.r);
      sj[j] = P.s;
      Uj[j] = P.U;
      Bj[j] = P.B;
      lduj[j] = P.ldu;
      u_rsrc[j] = make_rsrc(P.U + (size_t)m0 * P.ldu, rj[j] > 0 ? (size_t)rows_valid * P.ldu * 2 : 0);
      r_max = max(r_max, rj[j]);
    }
    const uint32_t slot = (uint32_t)(2 * l32 + half) * 16;
    const int u_region = a.mode == FMSA_FWD_SWIGLU ? 8 : 0;  // KB between the U blocks of column tiles 0 and 1
    for (int j0 = 0; j0 < r_max; j0 += 16) {
      const int ko = j0 + 8 * half;
      u32x4 uf[NT][MT], bw[NT];
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        u32x4 bf = {0u, 0u, 0u, 0u};
        if (j0 == 0) {  // staged in LDS before the main loop
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) uf[j][mt] = *reinterpret_cast<const u32x4*>(lora_lds + (u_region * j + mt) * 1024 + slot);
          bf = *reinterpret_cast<const u32x4*>(lora_lds + (16 + NT * wave + j) * 1024 + slot);
        } else {
          const bool live = ko < rj[j];
          const uint32_t dead = live ? 0u : 0x80000000u;
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            uf[j][mt] = __builtin_amdgcn_raw_buffer_load_b128(u_rsrc[j], (uint32_t)(((32 * mt + l32) * lduj[j] + ko) * 2) | dead, 0, 0);
          if (live) bf = *reinterpret_cast<const u32x4*>(Bj[j] + (size_t)(col0[j] + l32) * rj[j] + ko);
        }
#pragma unroll
        for (int w = 0; w < 4; ++w) bw[j][w] = pack2<T>(sj[j] * unpack_lo<T>(bf[w]), sj[j] * unpack_hi<T>(bf[w]));
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[mt][j] = mfma32<T>(bw[j], uf[j][mt], acc[mt][j]);
    }
  }

  // ---- epilogue ---------------------------------------------------------------------------
  // accumulator register 4*i0+i1 of acc[mt][j] is Y[m0 + 32*mt + l32][col0[j] + 8*i0 + 4*half + i1].
  // 64 tokens at a time the rounded outputs go through LDS planes (8-byte writes per lane) and
  // leave as 16-byte row segments through buffer stores: rows past M and columns past N are
  // dropped by the range check, so there are no branches.
  const bool swiglu = a.mode == FMSA_FWD_SWIGLU;
  const FwdProjDev PL = select_proj(a, pj[0]);
  const int cb = swiglu ? bn * 128 : (bn - a.nblk_start[pj[0]]) * 256;  // first output column of the tile
  const int lcol = swiglu ? wave * 32 : wave * 64;                      // wave's first column inside the tile
  const int estride = swiglu ? EP_STRIDE_S : EP_STRIDE_L;              // plane row stride, elements
  uint16_t* plane0 = ep_planes;
  uint16_t* plane1 = ep_planes + EP_ROWS * EP_STRIDE_S;
  uint16_t* plane2 = ep_planes + 2 * EP_ROWS * EP_STRIDE_S;
  // coalesced side: linear 32 chunks per row (8 rows per sweep), SwiGLU 16 chunks per row (16 rows)
  const int cchunk = swiglu ? (tid & 15) : (tid & 31);
  const int crow = swiglu ? (tid >> 4) : (tid >> 5);
  const int crows_per_it = swiglu ? 16 : 8;
  const int n_out = swiglu ? a.p[0].N : PL.N;
  const uint32_t col_dead = (cb + 8 * cchunk) < n_out ? 0u : 0x80000000u;
  const int64_t ld0 = swiglu ? a.p[0].ldy : PL.ldy;
  const __amdgpu_buffer_rsrc_t y0_rsrc = make_rsrc((swiglu ? a.p[0].Y : PL.Y) + (size_t)m0 * ld0, (size_t)rows_valid * ld0 * 2);
  const __amdgpu_buffer_rsrc_t y1_rsrc = make_rsrc(a.p[1].Y + (size_t)m0 * a.p[1].ldy, swiglu ? (size_t)rows_valid * a.p[1].ldy * 2 : 0);
  const __amdgpu_buffer_rsrc_t h_rsrc = make_rsrc(a.H + (size_t)m0 * a.ldh, swiglu ? (size_t)rows_valid * a.ldh * 2 : 0);
  const uint32_t y0_voff = (uint32_t)((crow * ld0 + cb + 8 * cchunk) * 2) | col_dead;
  const uint32_t y1_voff = (uint32_t)((crow * a.p[1].ldy + cb + 8 * cchunk) * 2) | col_dead;
  const uint32_t h_voff = (uint32_t)((crow * a.ldh + cb + 8 * cchunk) * 2) | col_dead;
  const uint32_t y0_row = __builtin_amdgcn_readfirstlane((uint32_t)(ld0 * 2));
  const uint32_t y1_row = __builtin_amdgcn_readfirstlane((uint32_t)(a.p[1].ldy * 2));
  const uint32_t h_row = __builtin_amdgcn_readfirstlane((uint32_t)(a.ldh * 2));
  // bias of the lane's 4 x 4 columns per tile
  float bias_v[NT][16];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const FwdProjDev P = select_proj(a, pj[j]);
#pragma unroll
    for (int i = 0; i < 16; ++i) bias_v[j][i] = 0.f;
    if (P.bias) {
#pragma unroll
      for (int i0 = 0; i0 < 4; ++i0) {
        const u32x2 bv = *reinterpret_cast<const u32x2*>(P.bias + col0[j] + 8 * i0 + 4 * half);
        bias_v[j][4 * i0 + 0] = unpack_lo<T>(bv[0]);
        bias_v[j][4 * i0 + 1] = unpack_hi<T>(bv[0]);
        bias_v[j][4 * i0 + 2] = unpack_lo<T>(bv[1]);
        bias_v[j][4 * i0 + 3] = unpack_hi<T>(bv[1]);
      }
    }
  }
  // rotary embedding (ROPE flavour, tiles of a projection named by rope_mask): the thread's pair of half-head chunks
  bool rope_on = false;
  int rp_row = 0, rp_c1 = 0, rp_c2 = 0, rp_cw = 0, rp_pos0 = 0;
  uint32_t rp_voff = 0;
  u32x4 rp_c[EP_ROWS / 16][2], rp_s[EP_ROWS / 16][2];  // cos / sin of the pair's 8 columns per sweep of the pass, as loaded:
                                                       // one 16-byte word of 16-bit values or two of fp32
  if constexpr (ROPE != 0) {
    rope_on = ((a.rope_mask >> pj[0]) & 1) != 0;
    const int hd = a.rope_head_dim, hpc = hd >> 4;  // 8-column chunks per half head (a power of two)
    const int pi = tid & 15;
    const int head = pi >> (31 - __builtin_clz(hpc)), within = pi & (hpc - 1);
    rp_row = tid >> 4;
    rp_c1 = head * (hd >> 3) + within;
    rp_c2 = rp_c1 + hpc;
    rp_cw = 8 * within;
    rp_pos0 = (m0 + rp_row) % a.rope_rows;
    rp_voff = (uint32_t)((rp_row * ld0 + cb + 8 * rp_c1) * 2) | ((cb + 8 * rp_c1) < n_out ? 0u : 0x80000000u);
  }
  __syncthreads();  // (the stage buffers are not reused, but all waves are past the main loop)

  static_for<0, MT / 2>([&](auto q_c) {
    constexpr int q = decltype(q_c)::value;
    if constexpr (ROPE != 0) {
      // cos / sin of this pass's rows, asked for before the accumulators are packed so that they arrive behind that work
      if (rope_on) {
        static_for<0, EP_ROWS / 16>([&](auto it_c) {
          constexpr int it = decltype(it_c)::value;
          int pos = rp_pos0 + EP_ROWS * q + 16 * it;  // token row m0 + ... takes table row (token row) % rope_rows
          if (pos >= a.rope_rows) pos %= a.rope_rows;
          const int64_t cso = (int64_t)pos * a.rope_ld + rp_cw;
          // kept as loaded and unpacked where they are used: an ALU operation here would make the wave wait for the load
          // before it goes on to pack its accumulators
          if constexpr (ROPE == 2) {
            const u32x4* cp = reinterpret_cast<const u32x4*>(reinterpret_cast<const float*>(a.rope_cos) + cso);
            const u32x4* sp = reinterpret_cast<const u32x4*>(reinterpret_cast<const float*>(a.rope_sin) + cso);
            rp_c[it][0] = cp[0];
            rp_c[it][1] = cp[1];
            rp_s[it][0] = sp[0];
            rp_s[it][1] = sp[1];
          } else {
            rp_c[it][0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(a.rope_cos) + cso);
            rp_s[it][0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(a.rope_sin) + cso);
          }
        });
      }
    }
    static_for<0, 2>([&](auto ml_c) {
      constexpr int ml = decltype(ml_c)::value;
      constexpr int mt = 2 * q + ml;
      const int prow = 32 * ml + l32;
      if (swiglu) {
#pragma unroll
        for (int i0 = 0; i0 < 4; ++i0) {
          u32x2 ev, gv, hv;
          float hf[4];
#pragma unroll
          for (int w = 0; w < 2; ++w) {
            ev[w] = pack2<T>(acc[mt][0][4 * i0 + 2 * w] + bias_v[0][4 * i0 + 2 * w],
                             acc[mt][0][4 * i0 + 2 * w + 1] + bias_v[0][4 * i0 + 2 * w + 1]);
            gv[w] = pack2<T>(acc[mt][1][4 * i0 + 2 * w] + bias_v[1][4 * i0 + 2 * w],
                             acc[mt][1][4 * i0 + 2 * w + 1] + bias_v[1][4 * i0 + 2 * w + 1]);
            // f = RNE(e32 * sigmoid(e32)) on the rounded e; h = RNE(f * g) on the rounded g
            const float e0 = unpack_lo<T>(ev[w]), e1 = unpack_hi<T>(ev[w]);
            const uint32_t fv = pack2<T>(e0 * sigmoidf_(e0), e1 * sigmoidf_(e1));
            hf[2 * w] = unpack_lo<T>(fv) * unpack_lo<T>(gv[w]);
            hf[2 * w + 1] = unpack_hi<T>(fv) * unpack_hi<T>(gv[w]);
          }
          hv[0] = pack2<T>(hf[0], hf[1]);
          hv[1] = pack2<T>(hf[2], hf[3]);
          const int o = prow * EP_STRIDE_S + lcol + 8 * i0 + 4 * half;
          *reinterpret_cast<u32x2*>(plane0 + o) = ev;
          *reinterpret_cast<u32x2*>(plane1 + o) = gv;
          *reinterpret_cast<u32x2*>(plane2 + o) = hv;
        }
      } else {
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int i0 = 0; i0 < 4; ++i0) {
            u32x2 yv;
            yv[0] = pack2<T>(acc[mt][j][4 * i0 + 0] + bias_v[j][4 * i0 + 0], acc[mt][j][4 * i0 + 1] + bias_v[j][4 * i0 + 1]);
            yv[1] = pack2<T>(acc[mt][j][4 * i0 + 2] + bias_v[j][4 * i0 + 2], acc[mt][j][4 * i0 + 3] + bias_v[j][4 * i0 + 3]);
            *reinterpret_cast<u32x2*>(plane0 + prow * EP_STRIDE_L + lcol + 32 * j + 8 * i0 + 4 * half) = yv;
          }
      }
    });
    __syncthreads();
    if (swiglu) {
#pragma unroll
      for (int it = 0; it < EP_ROWS / 16; ++it) {
        const int row = crow + 16 * it;
        const uint32_t srow = (uint32_t)(EP_ROWS * q + 16 * it);
        const int o = row * EP_STRIDE_S + 8 * cchunk;
        __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4*>(plane0 + o), y0_rsrc, y0_voff, srow * y0_row, STORE_NT);
        __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4*>(plane1 + o), y1_rsrc, y1_voff, srow * y1_row, STORE_NT);
        __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4*>(plane2 + o), h_rsrc, h_voff, srow * h_row, STORE_NT);
      }
    } else {
      if (ROPE != 0 && rope_on) {
        // Two half-head chunks per thread: 8 columns of the first half of a head and the 8 columns half a head
        // further (heads do not straddle the 256-column tile), so every cos / sin value is loaded and unpacked once
        // for the two outputs it makes.  16 pairs per row, 16 rows per sweep.
        static_for<0, EP_ROWS / 16>([&](auto it_c) {
          constexpr int it = decltype(it_c)::value;
          const int row = rp_row + 16 * it;
          const uint32_t srow = (uint32_t)(EP_ROWS * q + 16 * it);
          u32x4 v1 = *reinterpret_cast<const u32x4*>(plane0 + row * EP_STRIDE_L + 8 * rp_c1);
          u32x4 v2 = *reinterpret_cast<const u32x4*>(plane0 + row * EP_STRIDE_L + 8 * rp_c2);
          static_for<0, 4>([&](auto w_c) {
            constexpr int w = decltype(w_c)::value;  // values 2w and 2w + 1 of the 8 columns
            float c0, c1, s0, s1;
            if constexpr (ROPE == 2) {
              c0 = __uint_as_float(rp_c[it][w >> 1][2 * (w & 1)]);
              c1 = __uint_as_float(rp_c[it][w >> 1][2 * (w & 1) + 1]);
              s0 = __uint_as_float(rp_s[it][w >> 1][2 * (w & 1)]);
              s1 = __uint_as_float(rp_s[it][w >> 1][2 * (w & 1) + 1]);
            } else {
              c0 = unpack_lo<T>(rp_c[it][0][w]);
              c1 = unpack_hi<T>(rp_c[it][0][w]);
              s0 = unpack_lo<T>(rp_s[it][0][w]);
              s1 = unpack_hi<T>(rp_s[it][0][w]);
            }
            const float a0 = unpack_lo<T>(v1[w]), a1 = unpack_hi<T>(v1[w]);  // first half of the head
            const float b0 = unpack_lo<T>(v2[w]), b1 = unpack_hi<T>(v2[w]);  // second half
            v1[w] = pack2<T>(a0 * c0 - b0 * s0, a1 * c1 - b1 * s1);
            v2[w] = pack2<T>(b0 * c0 + a0 * s0, b1 * c1 + a1 * s1);
          });
          __builtin_amdgcn_raw_buffer_store_b128(v1, y0_rsrc, rp_voff, srow * y0_row, STORE_NT);
          __builtin_amdgcn_raw_buffer_store_b128(v2, y0_rsrc, rp_voff + (uint32_t)(a.rope_head_dim), srow * y0_row, STORE_NT);
        });
      } else {
#pragma unroll
        for (int it = 0; it < EP_ROWS / 8; ++it) {
          const int row = crow + 8 * it;
          const uint32_t srow = (uint32_t)(EP_ROWS * q + 8 * it);
          __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4*>(plane0 + row * EP_STRIDE_L + 8 * cchunk), y0_rsrc,
                                                 y0_voff, srow * y0_row, STORE_NT);
        }
      }
    }
    __syncthreads();
  });
  (void)estride;
  (void)crows_per_it;
  (void)active;
}

}  // namespace

int launch_gptq_lora_fwd(const fmsa_fwd_proj* projs, int n_proj, const void* X, int64_t ldx, int M, int mode,
                         void* H, int64_t ldh, const fmsa_rope* rope, int act_dtype, hipStream_t st) {
  FwdArgs a{};
  if (rope) {
    a.rope_cos = rope->cos;
    a.rope_sin = rope->sin;
    a.rope_ld = rope->ld;
    a.rope_rows = rope->rows;
    a.rope_head_dim = rope->head_dim;
    a.rope_mask = rope->proj_mask;
  }
  a.X = (const uint16_t*)X;
  a.ldx = ldx;
  a.M = M;
  a.K = projs[0].w.K;
  a.mode = mode;
  a.H = (uint16_t*)H;
  a.ldh = ldh;
  int nb = 0;
  for (int p = 0; p < 3; ++p) {
    a.nblk_start[p] = (p < n_proj) ? nb : 0x7fffffff;
    if (p >= n_proj) continue;
    const fmsa_fwd_proj& s = projs[p];
    FwdProjDev& d = a.p[p];
    d.qweight = s.w.qweight;
    d.scales = s.w.scales;
    d.qzeros = s.w.qzeros;
    d.code = s.w.code;
    d.block_scale = s.w.block_scale;
    d.U = (const uint16_t*)s.U;
    d.ldu = s.ldu;
    d.B = (const uint16_t*)s.B;
    d.bias = (const uint16_t*)s.bias;
    d.Y = (uint16_t*)s.Y;
    d.ldy = s.ldy;
    d.N = s.w.N;
    d.group_size = s.w.group_size;
    d.zero_offset = s.w.zero_offset;
    d.r = s.r;
    d.s = s.s;
    nb += (s.w.N + 255) / 256;
  }
  a.nblk_start[3] = 0x7fffffff;
  if (mode == FMSA_FWD_SWIGLU) nb = (projs[0].w.N + 127) / 128;
  a.nbn = nb;
  a.nbm = (M + BM - 1) / BM;
  dim3 grid(a.nbm * a.nbn), block(256);
  int gps = 1;
  for (int p = 0; p < n_proj; ++p) {
    const int gsz = projs[p].w.group_size;
    if (gsz % 64 != 0) gps = (gsz % 32 == 0) ? (gps > 2 ? gps : 2) : 4;
  }
  const bool ktail = (a.K % BK) != 0;
  const bool codebook = projs[0].w.format == FMSA_WEIGHT_CODEBOOK;  // api.hip: all projections of a launch share the format
  // table flavour: one code book for the launch, one block per 64-wide stage
  // packed-half unpack: fp16 activations and interleaved words (api.hip: then every projection is affine, interleaved, with
  // group_size % 64 == 0, and there is no rotary epilogue)
  const bool pk16 = act_dtype == FMSA_F16 && !codebook && projs[0].w.nibble_order == 1;
  bool table = codebook && gps == 1;
  for (int p = 0; p < n_proj; ++p)
    table = table && projs[p].w.code == projs[0].w.code && (projs[p].w.group_size & (projs[p].w.group_size - 1)) == 0;
#define LAUNCH3(TT, KT, CB)                                                                          \
  do {                                                                                               \
    if (rope && rope->dtype == FMSA_F32) hipLaunchKernelGGL((gptq_lora_fwd_kernel<TT, 1, false, CB, 2>), grid, block, 0, st, a); \
    else if (rope) hipLaunchKernelGGL((gptq_lora_fwd_kernel<TT, 1, false, CB, 1>), grid, block, 0, st, a); /* api.hip: gps 1, no K tail */ \
    else if (gps == 1) hipLaunchKernelGGL((gptq_lora_fwd_kernel<TT, 1, KT, CB>), grid, block, 0, st, a);  \
    else if (gps == 2) hipLaunchKernelGGL((gptq_lora_fwd_kernel<TT, 2, KT, CB>), grid, block, 0, st, a); \
    else hipLaunchKernelGGL((gptq_lora_fwd_kernel<TT, 4, KT, CB>), grid, block, 0, st, a);           \
  } while (0)
#define LAUNCH2(TT, KT)          \
  do {                           \
    if (table && rope && rope->dtype == FMSA_F32) hipLaunchKernelGGL((gptq_lora_fwd_kernel<TT, 1, false, 2, 2>), grid, block, 0, st, a); \
    else if (table && rope) hipLaunchKernelGGL((gptq_lora_fwd_kernel<TT, 1, false, 2, 1>), grid, block, 0, st, a); \
    else if (table) hipLaunchKernelGGL((gptq_lora_fwd_kernel<TT, 1, KT, 2>), grid, block, 0, st, a); \
    else if (codebook) LAUNCH3(TT, KT, 1); \
    else LAUNCH3(TT, KT, 0); \
  } while (0)
#define LAUNCH(TT)            \
  do {                        \
    if (ktail) LAUNCH2(TT, true); \
    else LAUNCH2(TT, false);  \
  } while (0)
  if (pk16) {
    if (ktail) hipLaunchKernelGGL((gptq_lora_fwd_kernel<f16_t, 1, true, 0, 0, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((gptq_lora_fwd_kernel<f16_t, 1, false, 0, 0, true>), grid, block, 0, st, a);
  } else if (act_dtype == FMSA_BF16) {
    LAUNCH(bf16_t);
  } else {
    LAUNCH(f16_t);
  }
#undef LAUNCH
#undef LAUNCH2
#undef LAUNCH3
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}
