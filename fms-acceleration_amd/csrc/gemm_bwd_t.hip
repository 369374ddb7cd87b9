// Fused input gradient on the TRANSPOSED TWIN of the packed weight:
//   dX = sum_p dY_p * deq(W_p)^T + mask (.) sum_p s_p T_p A_p,  optional SwiGLU backward over the result.
//
// The checkpoint packs 8 nibbles along K into one word, which is the forward's contraction axis; the input
// gradient contracts over N.  The twin (built once per frozen weight by gptq_transpose below) packs along N:
//   qweight_t int32 [N/8, K]   word [n8, k] holds q[k, 8*n8 + e], e = 0..7, with the even elements in its low half
//                              (element 2p at nibble position p) and the odd ones in its high half (2p + 1 at 4 + p)
// so one word is again exactly the 8-element MFMA fragment of the lane that owns output column k (the interleaved
// order costs the byte-wise unpack nothing and lets (w >> 4r) & 0x000F000F pick the pair of fragment register r for
// the packed-half unpack of the fp16 flavour), and this
// kernel is the forward kernel with the roles of K and N exchanged: every lane loads its own words into
// registers and unpacks them there (no byte shuffles, no words staged through LDS), and an accumulator quad
// holds 4 ADJACENT output columns, so the epilogue's dump is the forward's (8-byte LDS writes).
// What stays different from the forward: the scale and the offset of a weight depend on (group of k, n), and n
// is the contraction index here, so the 8 weights of a word take 8 different scales / offsets.  They are the same
// for all lanes of a half wave (group_size % 64 == 0: the wave's 64 columns lie in one group), and come from a
// per-stage table in LDS (fp32 scale [groups of the tile][64], fp32 -scale*zero likewise; filled by direct loads,
// one per wave and stage) by broadcast reads: 4 reads of 16 bytes per 16-wide step.
// PK16 (fp16 activations, affine weights): the tables are the checkpoint's fp16 scales and fp16 -(1024 + zero), and a
// fragment register is (((w >> 4r) & 0x000F000F) | 0x64006400) + (-(1024 + z)) [exact] times the scale [one rounding]
// in packed half arithmetic: 15 instead of 23 instructions per word, 2 table reads per step instead of 4, same bits.
//
// Tiling as in the forward: workgroup = 4 waves = 256 tokens x 256 output columns, wave = 256 x 64 (8 x 2 MFMA
// 32x32x16 tiles), contraction walked in stages of 64 with the dY tile loaded global -> LDS directly, one stage
// ahead, two stage buffers.  Results are bit-identical to the kernel that reads the checkpoint layout
// (gemm_bwd.hip): same operand values, same MFMA operand roles and contraction order.
#include "common.h"

namespace {

constexpr int BM = 256;
constexpr int BK = 64;
constexpr int MT = 8;
constexpr int NT = 2;
constexpr int EP_ROWS = 64;     // tokens per epilogue pass
constexpr int EP_STRIDE = 264;  // elements per staged row (256 + 8)
constexpr int TB_GROUPS = 8;    // quantisation groups per 256 output columns that a stage table holds

struct BwdTProjDev {
  const int32_t* qt;   // [N/8, K]
  const float* sc;     // [G, N] fp32 scales (affine) / block scales (code book)
  const float* nsz;    // [G, N] fp32 -scale * (zero + zero_offset) (affine only)
  const uint16_t* sc16;  // PK16: [G, N] fp16 scales (the checkpoint's own)
  const uint16_t* nz16;  // PK16: [G, N] fp16 -(1024 + zero + zero_offset)
  const float* code;   // code-book format: 16 entries
  const uint16_t* dY;
  int64_t lddy;
  const uint16_t* T;
  int64_t ldt;
  const uint16_t* At;  // [K, r]
  int N, group_size, r;
  float s;
};

struct BwdTArgs {
  BwdTProjDev p[3];
  int n_proj, M, K, nbm, nbk;
  uint16_t* dX;
  int64_t lddx;
  uint16_t* e;
  uint16_t* g;
  uint16_t* h;
  int64_t ldeg;
  const uint16_t* mask_src;
  int64_t ldmask;
};

FMSA_DEVI BwdTProjDev select_proj(const BwdTArgs& a, int p) { return p == 0 ? a.p[0] : (p == 1 ? a.p[1] : a.p[2]); }

// CODEBOOK: W = code[q] * block_scale[group, n] instead of the affine scale * q + (-scale * zero).
template <typename T, bool NTAIL, int MODE, bool CODEBOOK, bool PK16 = false>
__global__ __launch_bounds__(256) void gptq_lora_bwd_dx_t_kernel(const BwdTArgs a) {
  static_assert(!PK16 || (std::is_same<T, f16_t>::value && !CODEBOOK), "packed half unpack: fp16 activations, affine weights");
  // separate arrays per stage buffer: every access names its buffer statically, so the compiler can tell fragment
  // reads of one buffer from the direct loads in flight into the other
  __shared__ __attribute__((aligned(1024))) uint16_t dy0[BM * BK];
  __shared__ __attribute__((aligned(1024))) uint16_t dy1[BM * BK];
  // per buffer 4 KB: scales [8][64] fp32 | offsets [8][64] fp32 (PK16: fp16 scales [8][64] | fp16 offsets [8][64], 2 KB used)
  __shared__ __attribute__((aligned(1024))) uint32_t tb0[1024];
  __shared__ __attribute__((aligned(1024))) uint32_t tb1[1024];
  __shared__ __attribute__((aligned(16))) uint16_t ep_planes[2 * EP_ROWS * EP_STRIDE];
  auto dy_buf = [&](auto b_c) -> char* { return reinterpret_cast<char*>(decltype(b_c)::value == 0 ? dy0 : dy1); };
  auto tb_buf = [&](auto b_c) -> char* { return reinterpret_cast<char*>(decltype(b_c)::value == 0 ? tb0 : tb1); };

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int half = lane >> 5;

  int pid = xcd_remap(blockIdx.x, a.nbm * a.nbk);
  constexpr int GROUP_M = 4;  // token blocks per group: 4 x 8 tiles in flight per XCD share dY and W tiles in its L2
  const int width = GROUP_M * a.nbk;
  const int first_m = (pid / width) * GROUP_M;
  const int gsz = min(a.nbm - first_m, GROUP_M);
  const int bm = first_m + (pid % width) % gsz;
  const int bk = (pid % width) / gsz;
  const int m0 = bm * BM;
  const int k_tile0 = bk * 256;

  const int K = a.K;
  const int rows_valid = min(BM, a.M - m0);
  // the wave's two column tiles; a tile past K (K % 32 == 0: wholly inside or wholly outside) computes on column 0
  // and is dropped by the range check of the stores
  int col0[NT];
  bool active[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    col0[j] = k_tile0 + 64 * wave + 32 * j;
    active[j] = col0[j] < K;
    if (!active[j]) col0[j] = 0;
  }

  f32x16 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;

  // dY fragment of step t: row 32*mt + l32, chunk 2t + half
  uint32_t dy_r[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) dy_r[t] = (uint32_t)(l32 * (BK * 2) + 16 * ((2 * t + half) ^ ((l32 >> 1) & 7)));
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  constexpr int WAIT_VM0 = 0x0F70;  // s_waitcnt vmcnt(0) only

  for (int p = 0; p < a.n_proj; ++p) {
    const BwdTProjDev P = select_proj(a, p);
    const int N = __builtin_amdgcn_readfirstlane(P.N);
    const int gs = __builtin_amdgcn_readfirstlane(P.group_size);
    const int n_stages = (N + BK - 1) / BK;
    const int n_groups = (K + gs - 1) / gs;

    // ---- direct-load addressing: buffer resources + 32-bit lane offsets + scalar offsets ---------
    // dY: wave w fills rows 64w .. 64w+63 with 8 loads; load i covers rows 64w+8i .. +7, lane q writes slot (q & 7) of
    // row 64w + 8i + (q >> 3), i.e. fetches chunk (q & 7) ^ ((row >> 1) & 7).
    const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(P.dY + (size_t)m0 * P.lddy, (size_t)rows_valid * P.lddy * 2);
    const int dy_chunk_even = (lane & 7) ^ (lane >> 4);  // loads 0, 2, 4, 6; odd loads: ^ 4
    uint32_t dy_off[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = 64 * wave + 8 * i + (lane >> 3);
      dy_off[i] = (uint32_t)((row * P.lddy + 8 * (dy_chunk_even ^ (4 * (i & 1)))) * 2);
    }
    // tables: waves 0, 1 load the scales of groups 0-3 / 4-7 of the tile, waves 2, 3 the offsets (lane q: group
    // q >> 4, 4-column chunk q & 15): one load per wave and stage.  The code-book format has no offsets (its
    // resource is empty: no traffic).
    // PK16: 1 KB each, wave 0 loads the scales, wave 1 the offsets (lane q: group q >> 3, 8-column chunk q & 7), waves
    // 2 and 3 issue the same instruction on an empty resource.
    const int g0 = k_tile0 / gs;
    constexpr int TB_ELEM = PK16 ? 2 : 4;  // bytes per table element
    const int tb_g = PK16 ? (lane >> 3) : 4 * (wave & 1) + (lane >> 4);
    const int tb_col = PK16 ? 8 * (lane & 7) : 4 * (lane & 15);
    const __amdgpu_buffer_rsrc_t sc_rsrc = PK16 ? make_rsrc(P.sc16, wave == 0 ? (size_t)n_groups * N * 2 : 0)
                                                : make_rsrc(P.sc, (size_t)n_groups * N * 4);
    const __amdgpu_buffer_rsrc_t nz_rsrc = PK16 ? make_rsrc(P.nz16, wave == 1 ? (size_t)n_groups * N * 2 : 0)
                                                : make_rsrc(P.nsz, CODEBOOK ? 0 : (size_t)n_groups * N * 4);
    const __amdgpu_buffer_rsrc_t tb_rsrc = PK16 ? ((wave == 0) ? sc_rsrc : nz_rsrc) : ((wave < 2) ? sc_rsrc : nz_rsrc);
    const uint32_t tb_off = (uint32_t)(((g0 + tb_g) * N + tb_col) * TB_ELEM) | ((g0 + tb_g) < n_groups ? 0u : 0x80000000u);
    constexpr int TB_ZOFF = PK16 ? 1024 : 2048;   // byte offset of the offsets inside a table buffer
    constexpr int TB_STEP = 16 * TB_ELEM;         // bytes of one group's row per 16-wide step
    // weights: word (n8, k) at (n8 * K + k) * 4; the lane part is (half * K + k) * 4
    const __amdgpu_buffer_rsrc_t q_rsrc = make_rsrc(P.qt, (size_t)(N >> 3) * K * 4);
    uint32_t q_off[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) q_off[j] = (uint32_t)((half * K + col0[j] + l32) * 4);
    // the wave's group inside the tile (its 64 columns lie in one group: group_size % 64 == 0), and the table read
    // offset (bytes): [group][16 t + 8 half ..]
    const int gl = min(max(col0[0] / gs - g0, 0), TB_GROUPS - 1);
    const uint32_t tb_r = (uint32_t)(gl * (BK * TB_ELEM) + 8 * half * TB_ELEM);
    const uint32_t q_step_bytes = (uint32_t)K * 8;    // two packed rows per 16-wide step
    const uint32_t q_stage_bytes = (uint32_t)K * 32;  // eight packed rows per stage
    const uint32_t q_last = (uint32_t)((N >> 3) - 2) * K * 4;
    const float lut = CODEBOOK ? P.code[lane & 15] : 0.f;

    uint32_t qw[2][NT][4];
    u32x4 xf[2][MT], wf[2][NT];

    // load number `idx` of stage `st` into LDS buffer / register slot SB: 0-7 the dY tile, 8 the tables (direct loads),
    // 9-16 the weight words (idx - 9 = 4 j + t).  Nothing here may read a loaded register.
    auto load_piece = [&](int st, auto sb_c, auto idx_c) {
      constexpr int SB = decltype(sb_c)::value;
      constexpr int idx = decltype(idx_c)::value;
      const uint32_t n0 = (uint32_t)st * BK;
      if constexpr (idx < 8) {
        uint32_t poison = 0u;
        if constexpr (NTAIL) poison = ((int)n0 + 8 * (dy_chunk_even ^ (4 * (idx & 1))) < N) ? 0u : 0x80000000u;
        char* ldy = dy_buf(sb_c) + wave * (64 * BK * 2);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(dy_rsrc, (__attribute__((address_space(3))) void*)(ldy + idx * (8 * BK * 2)), 16,
                                                 dy_off[idx] | poison, n0 * 2, 0, 0);
      } else if constexpr (idx == 8) {
        uint32_t poison = 0u;
        if constexpr (NTAIL) poison = ((int)n0 + tb_col < N) ? 0u : 0x80000000u;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(tb_rsrc, (__attribute__((address_space(3))) void*)(tb_buf(sb_c) + wave * 1024), 16,
                                                 tb_off | poison, n0 * TB_ELEM, 0, 0);
      } else {
        constexpr int j = (idx - 9) >> 2, t = (idx - 9) & 3;
        uint32_t so = (uint32_t)st * q_stage_bytes + t * q_step_bytes;
        if constexpr (NTAIL) so = min(so, q_last);  // N % 64 == 32: the last stage's upper rows are clamped (their dY reads zeros)
        qw[SB][j][t] = __builtin_amdgcn_raw_buffer_load_b32(q_rsrc, q_off[j], so, 0);
      }
    };
    auto load_stage = [&](int st, auto sb_c) {
      static_for<0, 17>([&](auto i_c) { load_piece(st, sb_c, i_c); });
    };

    // ---- affine: LDS -> registers for step t of buffer SB (8 dY fragments, the step's 8 scales and 8 offsets of each
    // column tile's group) and the two unpacked weight fragments, into parity `par`
    // fragment register `reg` (contraction elements 2 reg, 2 reg + 1 = columns n + 2 reg, + 1) of a word whose byte
    // planes are p0 = w & 0x0F0F0F0F (elements 0, 4, 1, 5) and p1 = (w >> 4) & 0x0F0F0F0F (elements 2, 6, 3, 7): bytes
    // reg >> 1 and (reg >> 1) + 2 of plane reg & 1; value = scale * nibble + (-scale * zero), exact in fp32, one rounding
    auto unpack_reg = [&](uint32_t p0, uint32_t p1, const u32x4 (&sv)[2], const u32x4 (&zv)[2], auto reg_c) -> uint32_t {
      constexpr int reg = decltype(reg_c)::value;
      const uint32_t pl = (reg & 1) ? p1 : p0;
      const float b0 = ubyte_n<(reg >> 1)>(pl), b1 = ubyte_n<(reg >> 1) + 2>(pl);
      const float s0 = __uint_as_float(sv[reg >> 1][2 * (reg & 1)]), s1 = __uint_as_float(sv[reg >> 1][2 * (reg & 1) + 1]);
      const float z0 = __uint_as_float(zv[reg >> 1][2 * (reg & 1)]), z1 = __uint_as_float(zv[reg >> 1][2 * (reg & 1) + 1]);
      return pack2<T>(__builtin_fmaf(s0, b0, z0), __builtin_fmaf(s1, b1, z1));
    };
    // PK16: the pair (1024 + element 2 reg, 1024 + element 2 reg + 1) in packed half precision straight out of the word
    // (mask and bias sit in vector registers: the three-operand and-or takes no literal and one scalar at most)
    const uint32_t pk_mask = opaque(0x000F000Fu), pk_bias = opaque(0x64006400u);
    auto pair16 = [&](uint32_t w, auto reg_c) -> uint32_t {
      constexpr int reg = decltype(reg_c)::value;
      return ((w >> (4 * reg)) & pk_mask) | pk_bias;
    };
    // ---- affine: LDS -> registers for step t of buffer SB (8 dY fragments, the step's 8 scales and 8 offsets of the
    // wave's group) and the two unpacked weight fragments, into parity `par` (the very first step of a projection)
    auto prefetch = [&](auto sb_c, auto t_c, auto par_c) {
      constexpr int SB = decltype(sb_c)::value;
      constexpr int t = decltype(t_c)::value;
      constexpr int par = decltype(par_c)::value;
      const char* lt = tb_buf(sb_c);
      const char* lr = dy_buf(sb_c) + dy_r[t];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) xf[par][mt] = *reinterpret_cast<const u32x4*>(lr + mt * 32 * BK * 2);
      if constexpr (PK16) {
        const u32x4 s16 = *reinterpret_cast<const u32x4*>(lt + tb_r + t * TB_STEP);
        const u32x4 z16 = *reinterpret_cast<const u32x4*>(lt + TB_ZOFF + tb_r + t * TB_STEP);
#pragma unroll
        for (int j = 0; j < NT; ++j)
          static_for<0, 4>([&](auto r_c) {
            constexpr int r = decltype(r_c)::value;
            wf[par][j][r] = pk_sub_mul_f16(pair16(qw[SB][j][t], r_c), z16[r], s16[r]);
          });
      } else {
        u32x4 sv[2], zv[2];
        sv[0] = *reinterpret_cast<const u32x4*>(lt + tb_r + t * TB_STEP);
        sv[1] = *reinterpret_cast<const u32x4*>(lt + tb_r + t * TB_STEP + 16);
        zv[0] = *reinterpret_cast<const u32x4*>(lt + TB_ZOFF + tb_r + t * TB_STEP);
        zv[1] = *reinterpret_cast<const u32x4*>(lt + TB_ZOFF + tb_r + t * TB_STEP + 16);
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          const uint32_t w = qw[SB][j][t];
          const uint32_t p0 = opaque(w & 0x0F0F0F0Fu), p1 = opaque((w >> 4) & 0x0F0F0F0Fu);
          static_for<0, 4>([&](auto r_c) { wf[par][j][decltype(r_c)::value] = unpack_reg(p0, p1, sv, zv, r_c); });
        }
      }
    };
    // ---- code book, two phases so that no gather is waited for right after its issue.  Phase a: fragment reads,
    // the block scales of the step, and the 16 gathers from the lane-resident table (ds_bpermute; the codes of
    // elements 2b / 2b+1 of a word in gath[j][b] / [4 + b]); phase b: code * block scale in fp32, one rounding.
    uint32_t gath[NT][8];
    u32x4 bsv[2];
    auto prefetch_a = [&](auto sb_c, auto t_c, auto par_c) {
      constexpr int SB = decltype(sb_c)::value;
      constexpr int t = decltype(t_c)::value;
      constexpr int par = decltype(par_c)::value;
      const char* lt = tb_buf(sb_c);
      const char* lr = dy_buf(sb_c) + dy_r[t];
      bsv[0] = *reinterpret_cast<const u32x4*>(lt + tb_r + t * TB_STEP);
      bsv[1] = *reinterpret_cast<const u32x4*>(lt + tb_r + t * TB_STEP + 16);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) xf[par][mt] = *reinterpret_cast<const u32x4*>(lr + mt * 32 * BK * 2);
      const int li = (int)__float_as_uint(lut);
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const uint32_t w = qw[SB][j][t];
        // byte planes of table addresses (4 * code): a0 = elements 0, 4, 1, 5, a1 = elements 2, 6, 3, 7; fragment
        // register b takes bytes b >> 1 and (b >> 1) + 2 of plane b & 1
        const uint32_t a0 = opaque((w << 2) & 0x3C3C3C3Cu), a1 = opaque((w >> 2) & 0x3C3C3C3Cu);
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const uint32_t pl = (b & 1) ? a1 : a0;
          gath[j][b] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((pl >> (8 * (b >> 1))) & 0xffu), li);
          gath[j][4 + b] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((pl >> (8 * ((b >> 1) + 2))) & 0xffu), li);
        }
      }
    };
    auto prefetch_b = [&](auto par_c) {
      constexpr int par = decltype(par_c)::value;
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int b = 0; b < 4; ++b)
          wf[par][j][b] = pack2<T>(__uint_as_float(gath[j][b]) * __uint_as_float(bsv[b >> 1][2 * (b & 1)]),
                                   __uint_as_float(gath[j][4 + b]) * __uint_as_float(bsv[b >> 1][2 * (b & 1) + 1]));
    };
    using WithVmem = std::integral_constant<bool, true>;
    using NoVmem = std::integral_constant<bool, false>;
    // The affine step written slot by slot: the 16 MFMAs of parity `cur`, each followed by its share of the work that
    // produces step (nb, nt) into parity `nx`.  A step's arithmetic needs the table values, so the table reads lead
    // (slots 0, 1, with the nibble masks, which need nothing), the fragment reads follow (slots 2-7), and one unpacked
    // fragment register (2 conversions, 2 multiply-adds, 1 packed conversion) goes behind each of the MFMAs 4-11, by
    // which time the tables are back; in the last step of a stage the 17 loads of stage `st_next` into buffer / slot
    // `lb` ride along.  A scheduling fence closes every slot: the order below is the schedule (the group-barrier
    // matcher picks the multiply-adds right behind their table reads and the wave then waits for LDS in every step).
    auto step_affine = [&](auto nb_c, auto nt_c, auto nx_c, auto cur_c, auto vmem_c, int st_next, auto lb_c) {
      constexpr int SB = decltype(nb_c)::value;
      constexpr int t = decltype(nt_c)::value;
      constexpr int par = decltype(nx_c)::value;
      constexpr int cur = decltype(cur_c)::value;
      constexpr bool with_vmem = decltype(vmem_c)::value;
      const char* lt = tb_buf(nb_c);
      const char* lr = dy_buf(nb_c) + dy_r[t];
      auto mfma_slot = [&](int slot) { acc[slot >> 1][slot & 1] = mfma32<T>(wf[cur][slot & 1], xf[cur][slot >> 1], acc[slot >> 1][slot & 1]); };
      auto frag = [&](int mt) { xf[par][mt] = *reinterpret_cast<const u32x4*>(lr + mt * 32 * BK * 2); };
      auto fence = [&]() { __builtin_amdgcn_sched_barrier(0); };
      auto dma = [&](auto idx_c) {
        if constexpr (with_vmem) load_piece(st_next, lb_c, idx_c);
      };
      u32x4 sv[2], zv[2];   // PK16: sv[0] / zv[0] hold the 8 fp16 scales / offsets of the step
      uint32_t nib[NT][2];  // byte planes of a word: [tile][0] elements 0, 4, 1, 5; [1] elements 2, 6, 3, 7 (unused by PK16)
      mfma_slot(0);
      sv[0] = *reinterpret_cast<const u32x4*>(lt + tb_r + t * TB_STEP);
      if constexpr (!PK16) {
        sv[1] = *reinterpret_cast<const u32x4*>(lt + tb_r + t * TB_STEP + 16);
        nib[0][0] = opaque(qw[SB][0][t] & 0x0F0F0F0Fu);
        nib[0][1] = opaque((qw[SB][0][t] >> 4) & 0x0F0F0F0Fu);
      }
      dma(std::integral_constant<int, 0>{});
      fence();
      mfma_slot(1);
      zv[0] = *reinterpret_cast<const u32x4*>(lt + TB_ZOFF + tb_r + t * TB_STEP);
      if constexpr (!PK16) {
        zv[1] = *reinterpret_cast<const u32x4*>(lt + TB_ZOFF + tb_r + t * TB_STEP + 16);
        nib[1][0] = opaque(qw[SB][1][t] & 0x0F0F0F0Fu);
        nib[1][1] = opaque((qw[SB][1][t] >> 4) & 0x0F0F0F0Fu);
      }
      dma(std::integral_constant<int, 1>{});
      fence();
      mfma_slot(2);
      frag(0);
      frag(1);
      dma(std::integral_constant<int, 2>{});
      fence();
      mfma_slot(3);
      frag(2);
      frag(3);
      dma(std::integral_constant<int, 3>{});
      fence();
      // fragment register `reg` of tile `j` (5 instructions; PK16: 4, the pair straight out of the word)
      auto piece = [&](auto j_c, auto reg_c) {
        constexpr int j = decltype(j_c)::value;
        constexpr int reg = decltype(reg_c)::value;
        if constexpr (PK16)
          wf[par][j][reg] = pk_sub_mul_f16(pair16(qw[SB][j][t], reg_c), zv[0][reg], sv[0][reg]);
        else
          wf[par][j][reg] = unpack_reg(nib[j][0], nib[j][1], sv, zv, reg_c);
      };
      static_for<0, 12>([&](auto u_c) {
        constexpr int u = decltype(u_c)::value;  // slots 4 .. 15
        mfma_slot(4 + u);
        if constexpr (u < 4) frag(4 + u);
        if constexpr (u < 8) piece(std::integral_constant<int, (u >> 2)>{}, std::integral_constant<int, (u & 3)>{});
        if constexpr (u < 8) dma(std::integral_constant<int, 9 + u>{});        // the 8 weight words
        if constexpr (u >= 8) dma(std::integral_constant<int, u - 4>{});       // slots 12-15: dY loads 4-7
        if constexpr (u == 8) dma(std::integral_constant<int, 8>{});           // the tables
        fence();
      });
    };
    // The code-book step slot by slot.  The LDS pipe carries 26 instructions per step here (8 fragment reads, 2 table
    // reads, 16 gathers) next to the other waves' share, so they are spread as evenly as the dependencies allow: the
    // gathers of a fragment register's two weights go out first, its product follows about four MFMAs later.
    auto step_codebook = [&](auto nb_c, auto nt_c, auto nx_c, auto cur_c, auto vmem_c, int st_next, auto lb_c) {
      constexpr int SB = decltype(nb_c)::value;
      constexpr int t = decltype(nt_c)::value;
      constexpr int par = decltype(nx_c)::value;
      constexpr int cur = decltype(cur_c)::value;
      constexpr bool with_vmem = decltype(vmem_c)::value;
      const char* lt = tb_buf(nb_c);
      const char* lr = dy_buf(nb_c) + dy_r[t];
      const int li = (int)__float_as_uint(lut);
      auto mfma_slot = [&](int slot) { acc[slot >> 1][slot & 1] = mfma32<T>(wf[cur][slot & 1], xf[cur][slot >> 1], acc[slot >> 1][slot & 1]); };
      auto frag = [&](int mt) { xf[par][mt] = *reinterpret_cast<const u32x4*>(lr + mt * 32 * BK * 2); };
      auto fence = [&]() { __builtin_amdgcn_sched_barrier(0); };
      auto dma = [&](auto idx_c) {
        if constexpr (with_vmem) load_piece(st_next, lb_c, idx_c);
      };
      uint32_t ad[NT][2];  // byte planes of table addresses (4 * code): [tile][0] elements 0, 4, 1, 5; [1] elements 2, 6, 3, 7
      uint32_t ga[NT][8];  // code of element 2b in [b], of element 2b + 1 in [4 + b]
      u32x4 bs[2];
      // the two gathers of fragment register `reg` of tile `j`
      auto gather2 = [&](auto j_c, auto reg_c) {
        constexpr int j = decltype(j_c)::value;
        constexpr int reg = decltype(reg_c)::value;
        ga[j][reg] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((ad[j][reg & 1] >> (8 * (reg >> 1))) & 0xffu), li);
        ga[j][4 + reg] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((ad[j][reg & 1] >> (8 * ((reg >> 1) + 2))) & 0xffu), li);
      };
      auto piece = [&](auto j_c, auto reg_c) {
        constexpr int j = decltype(j_c)::value;
        constexpr int reg = decltype(reg_c)::value;
        wf[par][j][reg] = pack2<T>(__uint_as_float(ga[j][reg]) * __uint_as_float(bs[reg >> 1][2 * (reg & 1)]),
                                   __uint_as_float(ga[j][4 + reg]) * __uint_as_float(bs[reg >> 1][2 * (reg & 1) + 1]));
      };
      using J0 = std::integral_constant<int, 0>;
      using J1 = std::integral_constant<int, 1>;
      mfma_slot(0);
      bs[0] = *reinterpret_cast<const u32x4*>(lt + tb_r + t * TB_STEP);
      bs[1] = *reinterpret_cast<const u32x4*>(lt + tb_r + t * TB_STEP + 16);
      ad[0][0] = opaque((qw[SB][0][t] << 2) & 0x3C3C3C3Cu);
      ad[0][1] = opaque((qw[SB][0][t] >> 2) & 0x3C3C3C3Cu);
      gather2(J0{}, I0{});
      dma(std::integral_constant<int, 0>{});
      fence();
      mfma_slot(1);
      ad[1][0] = opaque((qw[SB][1][t] << 2) & 0x3C3C3C3Cu);
      ad[1][1] = opaque((qw[SB][1][t] >> 2) & 0x3C3C3C3Cu);
      gather2(J1{}, I0{});
      dma(std::integral_constant<int, 1>{});
      fence();
      mfma_slot(2);
      gather2(J0{}, I1{});
      dma(std::integral_constant<int, 2>{});
      fence();
      mfma_slot(3);
      gather2(J1{}, I1{});
      dma(std::integral_constant<int, 3>{});
      fence();
      mfma_slot(4);
      frag(0);
      frag(1);
      dma(std::integral_constant<int, 4>{});
      fence();
      mfma_slot(5);
      frag(2);
      gather2(J0{}, I2{});
      piece(J0{}, I0{});
      dma(std::integral_constant<int, 5>{});
      fence();
      mfma_slot(6);
      frag(3);
      gather2(J1{}, I2{});
      piece(J1{}, I0{});
      dma(std::integral_constant<int, 6>{});
      fence();
      mfma_slot(7);
      frag(4);
      piece(J0{}, I1{});
      dma(std::integral_constant<int, 7>{});
      fence();
      mfma_slot(8);
      frag(5);
      gather2(J0{}, I3{});
      piece(J1{}, I1{});
      dma(std::integral_constant<int, 8>{});
      fence();
      mfma_slot(9);
      frag(6);
      gather2(J1{}, I3{});
      dma(std::integral_constant<int, 9>{});
      fence();
      mfma_slot(10);
      frag(7);
      piece(J0{}, I2{});
      dma(std::integral_constant<int, 10>{});
      fence();
      mfma_slot(11);
      piece(J1{}, I2{});
      dma(std::integral_constant<int, 11>{});
      fence();
      mfma_slot(12);
      dma(std::integral_constant<int, 12>{});
      dma(std::integral_constant<int, 13>{});
      fence();
      mfma_slot(13);
      dma(std::integral_constant<int, 14>{});
      dma(std::integral_constant<int, 15>{});
      fence();
      mfma_slot(14);
      piece(J0{}, I3{});
      dma(std::integral_constant<int, 16>{});
      fence();
      mfma_slot(15);
      piece(J1{}, I3{});
      fence();
    };
    auto step = [&](auto nb_c, auto nt_c, auto nx_c, auto cur_c, auto vmem_c, int st_next, auto lb_c) {
      if constexpr (CODEBOOK) {
        step_codebook(nb_c, nt_c, nx_c, cur_c, vmem_c, st_next, lb_c);
      } else {
        step_affine(nb_c, nt_c, nx_c, cur_c, vmem_c, st_next, lb_c);
      }
    };
    // One stage out of buffer / register slot SB = s % 2: steps 0-2 prepare steps 1-3 of the same buffer; then the
    // wave waits for its own loads of stage s+1 (issued one stage earlier) and the barrier makes all four waves'
    // parts visible and closes the reads of buffer SB, so the last step can issue the loads of stage s+2 into it while
    // preparing step 0 of stage s+1 from the other buffer.  The last two stages re-load the final stage (no branch);
    // that data is never used.
    auto stage = [&](int s, auto sb_c) {
      constexpr int SB = decltype(sb_c)::value;
      using S1 = std::integral_constant<int, SB ^ 1>;
      step(sb_c, I1{}, I1{}, I0{}, NoVmem{}, 0, sb_c);
      step(sb_c, I2{}, I0{}, I1{}, NoVmem{}, 0, sb_c);
      step(sb_c, I3{}, I1{}, I0{}, NoVmem{}, 0, sb_c);
      __builtin_amdgcn_s_waitcnt(WAIT_VM0);
      __syncthreads();
      const int st_next = min(s + 2, n_stages - 1);
      step(S1{}, I0{}, I0{}, I1{}, WithVmem{}, st_next, sb_c);
    };

    __syncthreads();  // the previous projection's last LDS reads are done
    load_stage(0, I0{});
    __builtin_amdgcn_s_waitcnt(WAIT_VM0);
    __syncthreads();
    load_stage(min(1, n_stages - 1), I1{});
    if constexpr (CODEBOOK) {
      prefetch_a(I0{}, I0{}, I0{});
      prefetch_b(I0{});
    } else {
      prefetch(I0{}, I0{}, I0{});
    }

    const int n_full = n_stages & ~1;
    int s = 0;
    for (; s < n_full; s += 2) {
      stage(s, I0{});
      stage(s + 1, I1{});
    }
    if (s < n_stages) stage(s, I0{});
  }

  // ---- epilogue ---------------------------------------------------------------------------
  // register 4*i0+i1 of acc[mt][j] is dX[m0 + 32*mt + l32][k_tile0 + 64*wave + 32*j + 8*i0 + 4*half + i1]
  //
  // Four passes of 64 tokens.  Each pass (a) "dump": the waves round their accumulators (and the LoRA product of the
  // pass, formed by a few more MFMAs) into two LDS planes with 8-byte writes, (b) "sweep": all 256 threads walk the
  // planes in coalesced order -- lane = (row tid/32 of each group of 8 rows, 8-column chunk tid%32) -- apply the
  // mode's arithmetic and store.  The pass loop is a real loop around ONE copy of the sweep; only the small dump,
  // which names accumulator registers, exists four times.  All global accesses go through buffer resources over the
  // tile's rows, so rows past M and columns past K need no branches.  The operands the sweep of pass q+1 reads (e and
  // g, the mask source) are requested during the sweep of pass q, each into the registers the sweep has just finished
  // with.
  __builtin_amdgcn_s_waitcnt(WAIT_VM0);  // the surplus direct loads of the last stage have landed
  __syncthreads();
  constexpr bool swiglu = MODE == FMSA_BWD_SWIGLU;
  uint16_t* base_plane = ep_planes;
  uint16_t* lora_plane = base_plane + EP_ROWS * EP_STRIDE;
  bool any_lora = false;
  for (int p = 0; p < a.n_proj; ++p) any_lora = any_lora || (select_proj(a, p).r > 0);
  const int chunk = tid & 31;
  const uint32_t col_dead = (k_tile0 + 8 * chunk) < K ? 0u : 0x80000000u;
  const uint32_t eg_row_bytes = __builtin_amdgcn_readfirstlane((uint32_t)(a.ldeg * 2));
  const uint32_t dx_row_bytes = __builtin_amdgcn_readfirstlane((uint32_t)(a.lddx * 2));
  const uint32_t mk_row_bytes = __builtin_amdgcn_readfirstlane((uint32_t)(a.ldmask * 2));
  const bool has_mask = a.mask_src != nullptr && any_lora;
  const __amdgpu_buffer_rsrc_t e_rsrc = make_rsrc(a.e + (size_t)m0 * a.ldeg, swiglu ? (size_t)rows_valid * a.ldeg * 2 : 0);
  const __amdgpu_buffer_rsrc_t g_rsrc = make_rsrc(a.g + (size_t)m0 * a.ldeg, swiglu ? (size_t)rows_valid * a.ldeg * 2 : 0);
  const __amdgpu_buffer_rsrc_t h_rsrc = make_rsrc(a.h + (size_t)m0 * a.ldeg, swiglu ? (size_t)rows_valid * a.ldeg * 2 : 0);
  const __amdgpu_buffer_rsrc_t dx_rsrc = make_rsrc(a.dX + (size_t)m0 * a.lddx, swiglu ? 0 : (size_t)rows_valid * a.lddx * 2);
  // without a mask source the resource is empty: its loads cost no traffic and return zeros
  const __amdgpu_buffer_rsrc_t mk_rsrc =
      make_rsrc(a.mask_src + (size_t)m0 * a.ldmask, has_mask ? (size_t)rows_valid * a.ldmask * 2 : 0);
  const uint32_t eg_voff = (uint32_t)(((tid >> 5) * a.ldeg + k_tile0 + 8 * chunk) * 2) | col_dead;
  const uint32_t dx_voff = (uint32_t)(((tid >> 5) * a.lddx + k_tile0 + 8 * chunk) * 2) | col_dead;
  const uint32_t mk_voff = (uint32_t)(((tid >> 5) * a.ldmask + k_tile0 + 8 * chunk) * 2) | col_dead;
  constexpr int SWEEP = EP_ROWS * 32 / 256;  // 16-byte chunks per thread and pass
  u32x4 pre_e[swiglu ? SWEEP : 1], pre_g[swiglu ? SWEEP : 1], pre_m[SWEEP];
  auto issue_loads = [&](int q, auto it_c) {  // operands of chunk `it` of pass q
    constexpr int it = decltype(it_c)::value;
    const uint32_t row = (uint32_t)(EP_ROWS * q + 8 * it);
    if constexpr (swiglu) {
      pre_e[it] = __builtin_amdgcn_raw_buffer_load_b128(e_rsrc, eg_voff, row * eg_row_bytes, 0);
      pre_g[it] = __builtin_amdgcn_raw_buffer_load_b128(g_rsrc, eg_voff, row * eg_row_bytes, 0);
    }
    pre_m[it] = __builtin_amdgcn_raw_buffer_load_b128(mk_rsrc, mk_voff, row * mk_row_bytes, 0);
  };
  // LoRA operands of the first 16 ranks of every projection: the A^T fragments of the lane's two columns are the same
  // for all token tiles (loaded once), the T fragments of the two token tiles of a pass are fetched one pass ahead.
  constexpr int NP = swiglu ? 1 : 3;  // the SwiGLU-backward launch has one projection (the entry point checks)
  u32x4 af0[NP][NT], tf0[NP][2];
  bool lora_live[NP];
  static_for<0, NP>([&](auto p_c) {
    constexpr int p = decltype(p_c)::value;
    const BwdTProjDev& P = a.p[p];
    lora_live[p] = p < a.n_proj && P.r > 0;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      af0[p][j] = u32x4{0u, 0u, 0u, 0u};
      if (lora_live[p] && active[j] && 8 * half < P.r)
        af0[p][j] = *reinterpret_cast<const u32x4*>(P.At + (size_t)(col0[j] + l32) * P.r + 8 * half);
    }
  });
  auto load_tf = [&](int q) {
    static_for<0, NP>([&](auto p_c) {
      constexpr int p = decltype(p_c)::value;
      const BwdTProjDev& P = a.p[p];
#pragma unroll
      for (int ml = 0; ml < 2; ++ml) {
        const int m = m0 + 32 * (2 * q + ml) + l32;
        tf0[p][ml] = u32x4{0u, 0u, 0u, 0u};
        if (lora_live[p] && m < a.M && 8 * half < P.r) tf0[p][ml] = *reinterpret_cast<const u32x4*>(P.T + (size_t)m * P.ldt + 8 * half);
      }
    });
  };
  // (a) of pass q: accumulators of token tiles 2q, 2q+1 (+ their LoRA products) -> planes
  auto dump = [&](auto q_c) {
    constexpr int q = decltype(q_c)::value;
    static_for<0, 2>([&](auto ml_c) {
      constexpr int ml = decltype(ml_c)::value;
      constexpr int mt = 2 * q + ml;
      const int m = m0 + 32 * mt + l32;
      const bool m_ok = m < a.M;
      const int prow = (32 * ml + l32) * EP_STRIDE + 64 * wave + 4 * half;
      if (any_lora) {
        f32x16 lora[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int i = 0; i < 16; ++i) lora[j][i] = 0.f;
        static_for<0, NP>([&](auto p_c) {
          constexpr int p = decltype(p_c)::value;
          if (lora_live[p]) {
            const BwdTProjDev& P = a.p[p];
            f32x16 tmp[NT];
#pragma unroll
            for (int j = 0; j < NT; ++j) {
#pragma unroll
              for (int i = 0; i < 16; ++i) tmp[j][i] = 0.f;
              tmp[j] = mfma32<T>(af0[p][j], tf0[p][ml], tmp[j]);
            }
            for (int j0 = 16; j0 < P.r; j0 += 16) {  // ranks beyond the prefetched 16
              const int ko = j0 + 8 * half;
              u32x4 tf = {0u, 0u, 0u, 0u}, af[NT] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
              if (ko < P.r) {
                if (m_ok) tf = *reinterpret_cast<const u32x4*>(P.T + (size_t)m * P.ldt + ko);
#pragma unroll
                for (int j = 0; j < NT; ++j)
                  if (active[j]) af[j] = *reinterpret_cast<const u32x4*>(P.At + (size_t)(col0[j] + l32) * P.r + ko);
              }
#pragma unroll
              for (int j = 0; j < NT; ++j) tmp[j] = mfma32<T>(af[j], tf, tmp[j]);
            }
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
              for (int i = 0; i < 16; ++i) lora[j][i] += P.s * tmp[j][i];
          }
        });
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int i0 = 0; i0 < 4; ++i0) {
            u32x2 v;
            v[0] = pack2<T>(lora[j][4 * i0 + 0], lora[j][4 * i0 + 1]);
            v[1] = pack2<T>(lora[j][4 * i0 + 2], lora[j][4 * i0 + 3]);
            *reinterpret_cast<u32x2*>(lora_plane + prow + 32 * j + 8 * i0) = v;
          }
      }
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int i0 = 0; i0 < 4; ++i0) {
          u32x2 v;
          v[0] = pack2<T>(acc[mt][j][4 * i0 + 0], acc[mt][j][4 * i0 + 1]);
          v[1] = pack2<T>(acc[mt][j][4 * i0 + 2], acc[mt][j][4 * i0 + 3]);
          *reinterpret_cast<u32x2*>(base_plane + prow + 32 * j + 8 * i0) = v;
        }
    });
  };

  load_tf(0);
  static_for<0, SWEEP>([&](auto it_c) { issue_loads(0, it_c); });

#pragma clang loop unroll(disable)
  for (int q = 0; q < MT / 2; ++q) {
    switch (q) {
      case 0: dump(I0{}); break;
      case 1: dump(I1{}); break;
      case 2: dump(I2{}); break;
      default: dump(I3{}); break;
    }
    __syncthreads();
    const bool more = q + 1 < MT / 2;
    if (more) load_tf(q + 1);
    // (b): iteration `it` handles row 8*it + tid/32 of the pass
    static_for<0, SWEEP>([&](auto it_c) {
      constexpr int it = decltype(it_c)::value;
      const int row = (tid >> 5) + 8 * it;
      const uint32_t soff_rows = (uint32_t)(EP_ROWS * q + 8 * it);
      const u32x4 bv = *reinterpret_cast<const u32x4*>(base_plane + row * EP_STRIDE + 8 * chunk);
      u32x4 lv = {0u, 0u, 0u, 0u};
      if (any_lora) lv = *reinterpret_cast<const u32x4*>(lora_plane + row * EP_STRIDE + 8 * chunk);
      const u32x4 mv = pre_m[it];
      if constexpr (swiglu) {
        const u32x4 ev = pre_e[it];
        const u32x4 gv = pre_g[it];
        // Two adjacent columns at a time: every rounding to the storage type is one packed conversion whose two
        // halves are read back as fp32 (UL/swiglu.py:69-88 rounds f, h, DW and DW * g to the storage type; their
        // products with fp32 factors are rounded once, on store).
        u32x4 hv, dgv, dev;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const float e0 = unpack_lo<T>(ev[w]), e1 = unpack_hi<T>(ev[w]);
          const float g0 = unpack_lo<T>(gv[w]), g1 = unpack_hi<T>(gv[w]);
          const float b0 = unpack_lo<T>(bv[w]), b1 = unpack_hi<T>(bv[w]);
          const float se0 = sigmoidf_(e0), se1 = sigmoidf_(e1);
          const uint32_t fp = pack2<T>(se0 * e0, se1 * e1);  // f = silu(e)
          const float f0 = unpack_lo<T>(fp), f1 = unpack_hi<T>(fp);
          const uint32_t hp = pack2<T>(f0 * g0, f1 * g1);  // h = f * g
          // LoRA part of dh is masked by (dropout(h) != 0): mask_src holds dropout(h) when a dropout was applied,
          // otherwise h itself (recomputed here) decides; +-0 count as zero
          const uint32_t sel = has_mask ? mv[w] : hp;
          const float s0 = b0 + unpack_lo<T>(lv[w]), s1 = b1 + unpack_hi<T>(lv[w]);
          const uint32_t dwp = pack2<T>((sel & 0x7fffu) ? s0 : b0, (sel & 0x7fff0000u) ? s1 : b1);
          const float DW0 = unpack_lo<T>(dwp), DW1 = unpack_hi<T>(dwp);
          const uint32_t tp = pack2<T>(DW0 * g0, DW1 * g1);  // dg = DW * g in storage dtype (:79)
          hv[w] = hp;
          dgv[w] = pack2<T>(DW0 * f0, DW1 * f1);  // d_g ("df", :77)
          dev[w] = pack2<T>(unpack_lo<T>(tp) * se0 * (1.0f + e0 * (1.0f - se0)),   // d_e (:81-83)
                            unpack_hi<T>(tp) * se1 * (1.0f + e1 * (1.0f - se1)));
        }
        __builtin_amdgcn_raw_buffer_store_b128(hv, h_rsrc, eg_voff, soff_rows * eg_row_bytes, STORE_NT);
        __builtin_amdgcn_raw_buffer_store_b128(dgv, e_rsrc, eg_voff, soff_rows * eg_row_bytes, STORE_NT);
        __builtin_amdgcn_raw_buffer_store_b128(dev, g_rsrc, eg_voff, soff_rows * eg_row_bytes, STORE_NT);
      } else {
        u32x4 ov = bv;
        if (any_lora) {
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            // +-0 in the mask source count as zero; without a mask source nothing is masked
            const float l0 = (!has_mask || (mv[w] & 0x7fffu)) ? unpack_lo<T>(lv[w]) : 0.f;
            const float l1 = (!has_mask || ((mv[w] >> 16) & 0x7fffu)) ? unpack_hi<T>(lv[w]) : 0.f;
            ov[w] = pack2<T>(unpack_lo<T>(bv[w]) + l0, unpack_hi<T>(bv[w]) + l1);
          }
        }
        __builtin_amdgcn_raw_buffer_store_b128(ov, dx_rsrc, dx_voff, soff_rows * dx_row_bytes, STORE_NT);
      }
      // the operands of this chunk are dead now: the request for the next pass can reuse their registers
      __builtin_amdgcn_sched_barrier(0);
      if (more) issue_loads(q + 1, it_c);
    });
    __syncthreads();
  }
}

// qweight [K/8, N] (nibble j of word [k8, n] = q[8 k8 + j, n]) -> qweight_t [N/8, K]: word [n8, k] holds q[k, 8 n8 + e]
// with element e = 2p at nibble position p and e = 2p + 1 at position 4 + p.  One thread per 8 x 8 block of nibbles:
// 8 adjacent words in, 8 adjacent words out.  Runs once per frozen weight.
__global__ __launch_bounds__(256) void gptq_transpose_kernel(const uint32_t* __restrict__ qweight, int K8, int N8,
                                                             uint32_t* __restrict__ out) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)K8 * N8) return;
  // consecutive threads walk k8 first, so that the 32-byte output segments of a warp are adjacent
  const int k8 = (int)(idx % K8), n8 = (int)(idx / K8);
  const int N = N8 * 8, K = K8 * 8;
  uint32_t in[8], o[8];
  const u32x4* src = reinterpret_cast<const u32x4*>(qweight + (size_t)k8 * N + 8 * n8);
  const u32x4 a = src[0], b = src[1];
  in[0] = a[0]; in[1] = a[1]; in[2] = a[2]; in[3] = a[3];
  in[4] = b[0]; in[5] = b[1]; in[6] = b[2]; in[7] = b[3];
#pragma unroll
  for (int i = 0; i < 8; ++i) {  // output word i: row k = 8 k8 + i; element j comes from input word j (column 8 n8 + j)
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) w |= ((in[j] >> (4 * i)) & 0xFu) << (4 * ((j >> 1) + 4 * (j & 1)));
    o[i] = w;
  }
  u32x4* dst = reinterpret_cast<u32x4*>(out + (size_t)n8 * K + 8 * k8);
  dst[0] = u32x4{o[0], o[1], o[2], o[3]};
  dst[1] = u32x4{o[4], o[5], o[6], o[7]};
}

// The same re-ordering inside the words of the checkpoint layout itself (no transpose): out word [k8, n] holds
// q[8 k8 + e, n] with element 2p at nibble position p and element 2p + 1 at position 4 + p.  Four words per thread.
__global__ __launch_bounds__(256) void gptq_interleave_kernel(const u32x4* __restrict__ in, int64_t quads, u32x4* __restrict__ out) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= quads) return;
  const u32x4 w = in[idx];
  u32x4 o;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    uint32_t v = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) v |= ((w[c] >> (4 * e)) & 0xFu) << (4 * ((e >> 1) + 4 * (e & 1)));
    o[c] = v;
  }
  out[idx] = o;
}

}  // namespace

int launch_gptq_interleave(const int32_t* qweight, int K, int N, int32_t* out, hipStream_t st) {
  const int64_t quads = (int64_t)(K / 8) * N / 4;
  dim3 grid((unsigned)((quads + 255) / 256)), block(256);
  hipLaunchKernelGGL(gptq_interleave_kernel, grid, block, 0, st, (const u32x4*)qweight, quads, (u32x4*)out);
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}

int launch_gptq_transpose(const int32_t* qweight, int K, int N, int32_t* out, hipStream_t st) {
  const int64_t total = (int64_t)(K / 8) * (N / 8);
  dim3 grid((unsigned)((total + 255) / 256)), block(256);
  hipLaunchKernelGGL(gptq_transpose_kernel, grid, block, 0, st, (const uint32_t*)qweight, K / 8, N / 8, (uint32_t*)out);
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}

// Which flavour of the twin kernel a call can take: 0 none (a projection without its twin, or a group that does not hold
// whole 64-column wave tiles), 1 the fp32 scale / offset tables, 2 the packed-half unpack (fp16 activations, affine
// weights, every projection with its fp16 offset table).
int bwd_dx_twin_flavour(const fmsa_bwd_proj* projs, int n_proj, int act_dtype) {
  bool fp32_tables = true, pk16 = act_dtype == FMSA_F16;
  for (int p = 0; p < n_proj; ++p) {
    const fmsa_bwd_proj& s = projs[p];
    if (!s.qweight_t || s.w.group_size % 64 != 0) return 0;
    const bool cb = s.w.format == FMSA_WEIGHT_CODEBOOK;
    fp32_tables = fp32_tables && (cb || (s.scale_f32 && s.nsz));
    pk16 = pk16 && !cb && s.negzp_f16 && s.w.scales;
  }
  return pk16 ? 2 : (fp32_tables ? 1 : 0);
}

int launch_gptq_lora_bwd_dx_t(const fmsa_bwd_proj* projs, int n_proj, int M, int mode, void* dX, int64_t lddx,
                              void* e, void* g, void* h_out, int64_t ldeg, int act_dtype, hipStream_t st) {
  BwdTArgs a{};
  a.n_proj = n_proj;
  a.M = M;
  a.K = projs[0].w.K;
  a.dX = (uint16_t*)dX;
  a.lddx = lddx;
  a.e = (uint16_t*)e;
  a.g = (uint16_t*)g;
  a.h = (uint16_t*)h_out;
  a.ldeg = ldeg;
  bool ntail = false;
  for (int p = 0; p < n_proj; ++p) {
    const fmsa_bwd_proj& s = projs[p];
    BwdTProjDev& d = a.p[p];
    const bool cb = s.w.format == FMSA_WEIGHT_CODEBOOK;
    d.qt = s.qweight_t;
    d.sc = cb ? s.w.block_scale : s.scale_f32;
    d.nsz = cb ? nullptr : s.nsz;
    d.sc16 = s.w.scales;
    d.nz16 = (const uint16_t*)s.negzp_f16;
    d.code = s.w.code;
    d.dY = (const uint16_t*)s.dY;
    d.lddy = s.lddy;
    d.T = (const uint16_t*)s.T;
    d.ldt = s.ldt;
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
  const bool codebook = projs[0].w.format == FMSA_WEIGHT_CODEBOOK;  // api.hip: all projections of a launch share the format
  const bool pk16 = bwd_dx_twin_flavour(projs, n_proj, act_dtype) == 2;
#define LAUNCH_PK(MD)                                                                                          \
  do {                                                                                                         \
    if (ntail) hipLaunchKernelGGL((gptq_lora_bwd_dx_t_kernel<f16_t, true, MD, false, true>), grid, block, 0, st, a);  \
    else hipLaunchKernelGGL((gptq_lora_bwd_dx_t_kernel<f16_t, false, MD, false, true>), grid, block, 0, st, a);       \
  } while (0)
#define LAUNCH_C(TT, MD, CB)                                                                             \
  do {                                                                                                   \
    if (ntail) hipLaunchKernelGGL((gptq_lora_bwd_dx_t_kernel<TT, true, MD, CB>), grid, block, 0, st, a);  \
    else hipLaunchKernelGGL((gptq_lora_bwd_dx_t_kernel<TT, false, MD, CB>), grid, block, 0, st, a);       \
  } while (0)
#define LAUNCH_M(TT, MD)                  \
  do {                                    \
    if (codebook) LAUNCH_C(TT, MD, true); \
    else LAUNCH_C(TT, MD, false);         \
  } while (0)
#define LAUNCH(TT)                                              \
  do {                                                          \
    if (mode == FMSA_BWD_SWIGLU) LAUNCH_M(TT, FMSA_BWD_SWIGLU); \
    else LAUNCH_M(TT, FMSA_BWD_LINEAR);                         \
  } while (0)
  if (pk16) {
    if (mode == FMSA_BWD_SWIGLU) LAUNCH_PK(FMSA_BWD_SWIGLU);
    else LAUNCH_PK(FMSA_BWD_LINEAR);
  } else if (act_dtype == FMSA_BF16) {
    LAUNCH(bf16_t);
  } else {
    LAUNCH(f16_t);
  }
#undef LAUNCH
#undef LAUNCH_M
#undef LAUNCH_C
#undef LAUNCH_PK
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}
