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
//                   (every weight is unpacked by exactly one wave)
//   operands        everything a stage of 64 contraction columns needs is loaded straight into LDS
//                   (buffer loads with the LDS bit), once per workgroup, double buffered:
//                     dY tile   256 rows x 128 B, slot c of row r holds chunk c ^ ((r >> 1) & 7)
//                     words     32 qweight rows x 256 B, slot c of row r holds chunk c ^ (r & 15)
//                     scales    [8 groups][64] fp16 and (-scale*zero) [8 groups][64] fp32 of the
//                               at most 8 quantisation groups the tile's 256 columns span
//                   A direct load puts lane p's 16 bytes at slot p of a 1 KB block; the swizzles are
//                   applied on the global side, and make the 16-byte fragment reads conflict-free.
// Main loop: software pipeline at the granularity of one 16-wide MFMA K step.  While the 16 MFMAs
// of step t run, the wave reads its 8 words, 8 scales and 8 offsets of step t+1 and the 8 dY
// fragments from LDS and unpacks the two weight fragments; the loads of stage s+2 are issued in
// the last step of stage s, after the barrier that closes the reads of the buffer they overwrite.
// Epilogue: 64 tokens at a time the accumulators (and, separately, the LoRA term) are rounded to
// the storage type, transposed through LDS and written as 16-byte row segments; mask and SwiGLU
// backward are applied on that coalesced form.
#include "common.h"

namespace {

constexpr int BM = 256;
constexpr int BK = 64;
constexpr int MAX_TILE_GROUPS = 8;  // quantisation groups per 256 output columns (group_size >= 32)
constexpr int MT = 8;
constexpr int NT = 2;
constexpr int EP_ROWS = 64;     // tokens per epilogue pass
constexpr int EP_STRIDE = 264;  // elements per staged row (256 + 8)

struct BwdProjDev {
  const int32_t* qweight;
  const uint16_t* scales;
  const float* nsz;  // [G, N] = -scale * (zero + zero_offset); code-book format: the block scales [G, N]
  const float* code;  // code-book format: 16 entries
  const uint16_t* dY;
  int64_t lddy;
  const uint16_t* T;
  int64_t ldt;
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

// CODEBOOK: W = code[q] * block_scale[group, n] instead of the affine scale * (q - zero).
template <typename T, bool NTAIL, int MODE, bool CODEBOOK>
__global__ __launch_bounds__(256) void gptq_lora_bwd_dx_kernel(const BwdArgs a) {
  // separate arrays per stage buffer: every access names its buffer statically, so the compiler
  // can tell fragment reads of one buffer from the direct loads in flight into the other
  __shared__ __attribute__((aligned(1024))) uint16_t dy0[BM * BK];
  __shared__ __attribute__((aligned(1024))) uint16_t dy1[BM * BK];
  __shared__ __attribute__((aligned(1024))) uint32_t wq0[32 * BK];
  __shared__ __attribute__((aligned(1024))) uint32_t wq1[32 * BK];
  // per buffer 4 KB: scales [8][64] fp16 | offsets [8][64] fp32 | 1 KB written by the idle wave
  __shared__ __attribute__((aligned(1024))) uint32_t tb0[1024];
  __shared__ __attribute__((aligned(1024))) uint32_t tb1[1024];
  __shared__ __attribute__((aligned(16))) uint16_t ep_planes[2 * EP_ROWS * EP_STRIDE];
  auto dy_buf = [&](auto b_c) -> char* { return reinterpret_cast<char*>(decltype(b_c)::value == 0 ? dy0 : dy1); };
  auto wq_buf = [&](auto b_c) -> char* { return reinterpret_cast<char*>(decltype(b_c)::value == 0 ? wq0 : wq1); };
  auto tb_buf = [&](auto b_c) -> char* { return reinterpret_cast<char*>(decltype(b_c)::value == 0 ? tb0 : tb1); };

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int half = lane >> 5;

  int pid = xcd_remap(blockIdx.x, a.nbm * a.nbk);
  constexpr int GROUP_M = 4;  // token blocks per group: 4 x 8 tiles in flight per XCD share X and W tiles in its L2
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

  // ---- LDS read offsets (bytes) ----------------------------------------------------------------
  // dY fragment of step t: row 32*mt + l32, chunk 2t + half
  uint32_t dy_r[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) dy_r[t] = (uint32_t)(l32 * (BK * 2) + 16 * ((2 * t + half) ^ ((l32 >> 1) & 7)));
  // words of step t: row l32, chunks 4t + 2*half + {0, 1}
  uint32_t wq_r[4][2];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int u = 0; u < 2; ++u) wq_r[t][u] = (uint32_t)(l32 * 256 + 16 * ((4 * t + 2 * half + u) ^ (l32 & 15)));
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  constexpr int WAIT_VM0 = 0x0F70;  // s_waitcnt vmcnt(0) only

  for (int p = 0; p < a.n_proj; ++p) {
    const BwdProjDev P = select_proj(a, p);
    const int N = __builtin_amdgcn_readfirstlane(P.N);
    const int gs = __builtin_amdgcn_readfirstlane(P.group_size);
    const int n_stages = (N + BK - 1) / BK;
    const int n_groups = (K + gs - 1) / gs;

    // ---- direct-load addressing: buffer resources + 32-bit lane offsets + scalar offsets ---------
    // dY: wave w fills rows 64w .. 64w+63 with 8 loads; load i covers rows 64w+8i .. +7, lane q
    // writes slot (q & 7) of row 64w + 8i + (q >> 3), i.e. fetches chunk (q & 7) ^ ((row >> 1) & 7).
    const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(P.dY + (size_t)m0 * P.lddy, (size_t)rows_valid * P.lddy * 2);
    const int dy_chunk_even = (lane & 7) ^ (lane >> 4);  // loads 0, 2, 4, 6; odd loads: ^ 4
    uint32_t dy_off[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = 64 * wave + 8 * i + (lane >> 3);
      dy_off[i] = (uint32_t)((row * P.lddy + 8 * (dy_chunk_even ^ (4 * (i & 1)))) * 2);
    }
    // words: wave w fills rows 8w .. 8w+7 with 2 loads of 4 rows; lane q writes slot (q & 15) of
    // row 8w + 4i + (q >> 4), i.e. fetches the 4-word chunk (q & 15) ^ (row & 15).
    const __amdgpu_buffer_rsrc_t q_rsrc = make_rsrc(P.qweight, (size_t)(K >> 3) * N * 4);
    uint32_t wq_off[2];
    int wq_chunk[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = 8 * wave + 4 * i + (lane >> 4);
      wq_chunk[i] = (lane & 15) ^ (row & 15);
      const uint32_t dead_row = (k8base + row) < (K >> 3) ? 0u : 0x80000000u;  // rows past K read as zeros
      wq_off[i] = (uint32_t)(((k8base + row) * N + 4 * wq_chunk[i]) * 4) | dead_row;
    }
    // tables: wave 0 loads the scales (lane q: group q >> 3, 8-column chunk q & 7), waves 1 and 2
    // the offsets of groups 0-3 / 4-7 (lane q: group q >> 4, 4-column chunk q & 15); wave 3 issues
    // the same instruction fully out of range, into the spare 1 KB.
    const int g0 = (8 * k8base) / gs;
    const int tb_elem = (wave == 0) ? 2 : 4;  // bytes per table element
    const int tb_g = (wave == 0) ? (lane >> 3) : (4 * (wave - 1) + (lane >> 4));
    const int tb_col = (wave == 0) ? 8 * (lane & 7) : 4 * (lane & 15);  // first column of the lane's chunk
    const __amdgpu_buffer_rsrc_t sc_rsrc = make_rsrc(P.scales, CODEBOOK ? 0 : (size_t)n_groups * N * 2);
    const __amdgpu_buffer_rsrc_t nz_rsrc = make_rsrc(P.nsz, (size_t)n_groups * N * 4);
    const __amdgpu_buffer_rsrc_t tb_rsrc = (wave == 0) ? sc_rsrc : nz_rsrc;
    const bool tb_live = (wave < 3) && (g0 + tb_g) < n_groups;
    const uint32_t tb_off = (uint32_t)(((g0 + tb_g) * N + tb_col) * tb_elem) | (tb_live ? 0u : 0x80000000u);
    // this lane's group inside the tile, and its table read offsets
    const int gl = row_ok ? ((8 * k8) / gs - g0) : 0;
    const uint32_t sc_r = (uint32_t)(gl * (BK * 2) + 8 * half * 2);
    const uint32_t nz_r = (uint32_t)(1024 + gl * (BK * 4) + 8 * half * 4);

    u32x4 xf[2][MT], wf[2][NT];

    // direct loads of stage `st` into buffer SB
    // direct load number `idx` of stage `st` into buffer SB: 0-7 dY, 8-9 words, 10 tables
    auto load_piece = [&](int st, auto sb_c, auto idx_c) {
      constexpr int idx = decltype(idx_c)::value;
      const uint32_t n0 = (uint32_t)st * BK;
      if constexpr (idx < 8) {
        uint32_t poison = 0u;
        if constexpr (NTAIL) poison = ((int)n0 + 8 * (dy_chunk_even ^ (4 * (idx & 1))) < N) ? 0u : 0x80000000u;
        char* ldy = dy_buf(sb_c) + wave * (64 * BK * 2);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(dy_rsrc, (__attribute__((address_space(3))) void*)(ldy + idx * (8 * BK * 2)), 16,
                                                 dy_off[idx] | poison, n0 * 2, 0, 0);
      } else if constexpr (idx < 10) {
        constexpr int i = idx - 8;
        uint32_t poison = 0u;
        if constexpr (NTAIL) poison = ((int)n0 + 4 * wq_chunk[i] < N) ? 0u : 0x80000000u;
        char* lwq = wq_buf(sb_c) + wave * 2048;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(q_rsrc, (__attribute__((address_space(3))) void*)(lwq + i * 1024), 16,
                                                 wq_off[i] | poison, n0 * 4, 0, 0);
      } else {
        uint32_t poison = 0u;
        if constexpr (NTAIL) poison = ((int)n0 + tb_col < N) ? 0u : 0x80000000u;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(tb_rsrc, (__attribute__((address_space(3))) void*)(tb_buf(sb_c) + wave * 1024), 16,
                                                 tb_off | poison, n0 * (uint32_t)tb_elem, 0, 0);
      }
    };
    auto load_stage = [&](int st, auto sb_c) {
      static_for<0, 11>([&](auto i_c) { load_piece(st, sb_c, i_c); });
    };
    // LDS -> registers for step t of buffer SB: the 8 dY fragments and the two unpacked weight
    // fragments, into parity `par`
    auto prep = [&](auto sb_c, auto t_c, auto par_c) {
      constexpr int t = decltype(t_c)::value;
      constexpr int par = decltype(par_c)::value;
      const char* lq = wq_buf(sb_c);
      const char* lt = tb_buf(sb_c);
      const u32x4 q0 = *reinterpret_cast<const u32x4*>(lq + wq_r[t][0]);
      const u32x4 q1 = *reinterpret_cast<const u32x4*>(lq + wq_r[t][1]);
      const u32x4 sc = *reinterpret_cast<const u32x4*>(lt + sc_r + t * 32);
      const u32x4 nz0 = *reinterpret_cast<const u32x4*>(lt + nz_r + t * 64);
      const u32x4 nz1 = *reinterpret_cast<const u32x4*>(lt + nz_r + t * 64 + 16);
      const char* lr = dy_buf(sb_c) + dy_r[t];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) xf[par][mt] = *reinterpret_cast<const u32x4*>(lr + mt * 32 * BK * 2);
      // this wave's byte of the 8 words: low nibble = column tile 0 (k = 8*k8 + 2*wave), high = tile 1
      const uint32_t p01 = __builtin_amdgcn_perm(q0[1], q0[0], sel_pair);
      const uint32_t p23 = __builtin_amdgcn_perm(q0[3], q0[2], sel_pair);
      const uint32_t p45 = __builtin_amdgcn_perm(q1[1], q1[0], sel_pair);
      const uint32_t p67 = __builtin_amdgcn_perm(q1[3], q1[2], sel_pair);
      const uint32_t x0 = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
      const uint32_t x1 = __builtin_amdgcn_perm(p67, p45, 0x05040100u);
      const uint32_t lo0 = opaque(x0 & 0x0F0F0F0Fu), hi0 = opaque((x0 >> 4) & 0x0F0F0F0Fu);
      const uint32_t lo1 = opaque(x1 & 0x0F0F0F0Fu), hi1 = opaque((x1 >> 4) & 0x0F0F0F0Fu);
      float sfv[8], nzv[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        sfv[2 * i] = fp16_bits_to_f32((uint16_t)(sc[i] & 0xffffu));
        sfv[2 * i + 1] = fp16_bits_to_f32((uint16_t)(sc[i] >> 16));
        nzv[i] = __uint_as_float(nz0[i]);
        nzv[4 + i] = __uint_as_float(nz1[i]);
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
    // Code-book flavour of prep in two phases (see the forward kernel): (a) fragment reads, byte
    // shuffles, address arithmetic and the 16 table gathers under the first 8 MFMAs of a step; (b) the
    // multiplies by the block scales of the lane's 8 columns and the conversions under the last 8.
    const float lut = CODEBOOK ? P.code[lane & 15] : 0.f;
    uint32_t gath[NT][8];
    u32x4 bs_lo, bs_hi;  // block scales of the fragment's 8 columns
    // the same work without MFMAs in between, for the very first step of a projection
    auto prep_first = [&](auto sb_c, auto t_c, auto par_c) {
      constexpr int t = decltype(t_c)::value;
      constexpr int par = decltype(par_c)::value;
      const char* lq = wq_buf(sb_c);
      const char* lt = tb_buf(sb_c);
      const u32x4 q0 = *reinterpret_cast<const u32x4*>(lq + wq_r[t][0]);
      const u32x4 q1 = *reinterpret_cast<const u32x4*>(lq + wq_r[t][1]);
      bs_lo = *reinterpret_cast<const u32x4*>(lt + nz_r + t * 64);
      bs_hi = *reinterpret_cast<const u32x4*>(lt + nz_r + t * 64 + 16);
      const char* lr = dy_buf(sb_c) + dy_r[t];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) xf[par][mt] = *reinterpret_cast<const u32x4*>(lr + mt * 32 * BK * 2);
      const uint32_t p01 = __builtin_amdgcn_perm(q0[1], q0[0], sel_pair);
      const uint32_t p23 = __builtin_amdgcn_perm(q0[3], q0[2], sel_pair);
      const uint32_t p45 = __builtin_amdgcn_perm(q1[1], q1[0], sel_pair);
      const uint32_t p67 = __builtin_amdgcn_perm(q1[3], q1[2], sel_pair);
      const uint32_t x0 = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
      const uint32_t x1 = __builtin_amdgcn_perm(p67, p45, 0x05040100u);
      const uint32_t a0[2] = {(x0 << 2) & 0x3C3C3C3Cu, (x0 >> 2) & 0x3C3C3C3Cu};
      const uint32_t a1[2] = {(x1 << 2) & 0x3C3C3C3Cu, (x1 >> 2) & 0x3C3C3C3Cu};
      const int li = (int)__float_as_uint(lut);
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          gath[j][b] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((a0[j] >> (8 * b)) & 0xffu), li);
          gath[j][4 + b] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((a1[j] >> (8 * b)) & 0xffu), li);
        }
    };
    // Phase a of step (sb, t) into parity `par`, written slot by slot under the first 8 MFMAs of the
    // running step (parity `cur`): the order below IS the schedule (a fence closes every slot), because the
    // dependency chain  word reads -> byte shuffles -> addresses -> gathers  has to be spread by hand.
    auto phase_a = [&](auto sb_c, auto t_c, auto par_c, auto cur_c) {
      constexpr int t = decltype(t_c)::value;
      constexpr int par = decltype(par_c)::value;
      constexpr int cur = decltype(cur_c)::value;
      const char* lq = wq_buf(sb_c);
      const char* lt = tb_buf(sb_c);
      const char* lr = dy_buf(sb_c) + dy_r[t];
      const int li = (int)__float_as_uint(lut);
      auto mfma_slot = [&](int slot) { acc[slot >> 1][slot & 1] = mfma32<T>(wf[cur][slot & 1], xf[cur][slot >> 1], acc[slot >> 1][slot & 1]); };
      auto frag = [&](int mt) { xf[par][mt] = *reinterpret_cast<const u32x4*>(lr + mt * 32 * BK * 2); };
      auto fence = [&]() { __builtin_amdgcn_sched_barrier(0); };
      mfma_slot(0);
      const u32x4 q0 = *reinterpret_cast<const u32x4*>(lq + wq_r[t][0]);
      const u32x4 q1 = *reinterpret_cast<const u32x4*>(lq + wq_r[t][1]);
      bs_lo = *reinterpret_cast<const u32x4*>(lt + nz_r + t * 64);
      fence();
      mfma_slot(1);
      bs_hi = *reinterpret_cast<const u32x4*>(lt + nz_r + t * 64 + 16);
      frag(0);
      frag(1);
      fence();
      mfma_slot(2);
      frag(2);
      frag(3);
      frag(4);
      const uint32_t p01 = __builtin_amdgcn_perm(q0[1], q0[0], sel_pair);
      const uint32_t p23 = __builtin_amdgcn_perm(q0[3], q0[2], sel_pair);
      const uint32_t p45 = __builtin_amdgcn_perm(q1[1], q1[0], sel_pair);
      const uint32_t p67 = __builtin_amdgcn_perm(q1[3], q1[2], sel_pair);
      fence();
      mfma_slot(3);
      frag(5);
      frag(6);
      frag(7);
      const uint32_t x0 = __builtin_amdgcn_perm(p23, p01, 0x05040100u);  // byte i: (tile 1 << 4 | tile 0) of column n + i
      const uint32_t x1 = __builtin_amdgcn_perm(p67, p45, 0x05040100u);  // columns n + 4 .. n + 7
      // [tile]: byte i = 4 * nibble = the byte address of the table's lane
      const uint32_t a0[2] = {(x0 << 2) & 0x3C3C3C3Cu, (x0 >> 2) & 0x3C3C3C3Cu};
      const uint32_t a1[2] = {(x1 << 2) & 0x3C3C3C3Cu, (x1 >> 2) & 0x3C3C3C3Cu};
      fence();
      // 4 gathers per MFMA: (tile j, columns 0-3 or 4-7)
      static_for<0, 4>([&](auto u_c) {
        constexpr int u = decltype(u_c)::value;
        constexpr int j = u >> 1;
        mfma_slot(4 + u);
        const uint32_t a = (u & 1) ? a1[j] : a0[j];
#pragma unroll
        for (int b = 0; b < 4; ++b) gath[j][4 * (u & 1) + b] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((a >> (8 * b)) & 0xffu), li);
        fence();
      });
    };
    auto prep_b = [&](auto par_c) {
      constexpr int par = decltype(par_c)::value;
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        wf[par][j][0] = pack2<T>(__uint_as_float(gath[j][0]) * __uint_as_float(bs_lo[0]), __uint_as_float(gath[j][1]) * __uint_as_float(bs_lo[1]));
        wf[par][j][1] = pack2<T>(__uint_as_float(gath[j][2]) * __uint_as_float(bs_lo[2]), __uint_as_float(gath[j][3]) * __uint_as_float(bs_lo[3]));
        wf[par][j][2] = pack2<T>(__uint_as_float(gath[j][4]) * __uint_as_float(bs_hi[0]), __uint_as_float(gath[j][5]) * __uint_as_float(bs_hi[1]));
        wf[par][j][3] = pack2<T>(__uint_as_float(gath[j][6]) * __uint_as_float(bs_hi[2]), __uint_as_float(gath[j][7]) * __uint_as_float(bs_hi[3]));
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
    // Everything else of a step sits between its 16 MFMAs (in-order issue, one wave per SIMD).  The
    // 13 LDS reads go first (one per MFMA; the 5 weight-operand reads lead, the unpack depends on
    // them), the ~60 unpack instructions follow from the fourth MFMA on, and in the last step of a
    // stage the 11 direct loads of a later stage are spread over the first MFMAs as well.
    auto interleave = [&](auto with_vmem_c) {
      constexpr bool with_vmem = decltype(with_vmem_c)::value;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (i < 13) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if (i >= 3) __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
        if (with_vmem && i < 11) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    // code-book phase b: 8 MFMAs with the 24 multiplies / conversions and, in the last step of a stage, the
    // 11 direct loads
    auto interleave_b = [&](auto with_vmem_c) {
      constexpr bool with_vmem = decltype(with_vmem_c)::value;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
        if (with_vmem) {
          if (i < 3)
            __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
          else
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    using WithVmem = std::integral_constant<bool, true>;
    using NoVmem = std::integral_constant<bool, false>;

    // One stage out of buffer SB = s % 2: steps 0-2 prepare steps 1-3 of the same buffer; then the
    // wave waits for its own direct loads of stage s+1 (issued one stage earlier) and the barrier
    // makes all four waves' parts visible and closes the reads of buffer SB, so step 3 can issue
    // the loads of stage s+2 into it while preparing step 0 of stage s+1 from the other buffer.
    // The last two stages re-load the final stage (no branch); that data is never used.
    // The affine step written slot by slot: the 16 MFMAs of parity `cur`, each followed by its share of
    // the work that produces step (nb, nt) into parity `nx` -- word / table / fragment reads first, the
    // byte shuffles once the words are back, then one unpacked fragment register (2 conversions, 2
    // multiply-adds, 1 packed conversion) per MFMA -- and, in the last step of a stage, the 11 direct loads of
    // stage `st_next` into buffer `lb`, placed where a slot has room (under the read slots, under every second
    // unpack slot and under the last four MFMAs).  A scheduling fence closes every slot: the order below is
    // the schedule.
    auto step_affine = [&](auto nb_c, auto nt_c, auto nx_c, auto cur_c, auto vmem_c, int st_next, auto lb_c) {
      constexpr int t = decltype(nt_c)::value;
      constexpr int par = decltype(nx_c)::value;
      constexpr int cur = decltype(cur_c)::value;
      constexpr bool with_vmem = decltype(vmem_c)::value;
      const char* lq = wq_buf(nb_c);
      const char* lt = tb_buf(nb_c);
      const char* lr = dy_buf(nb_c) + dy_r[t];
      auto mfma_slot = [&](int slot) { acc[slot >> 1][slot & 1] = mfma32<T>(wf[cur][slot & 1], xf[cur][slot >> 1], acc[slot >> 1][slot & 1]); };
      auto frag = [&](int mt) { xf[par][mt] = *reinterpret_cast<const u32x4*>(lr + mt * 32 * BK * 2); };
      auto fence = [&]() { __builtin_amdgcn_sched_barrier(0); };
      auto dma = [&](auto idx_c) {
        if constexpr (with_vmem) load_piece(st_next, lb_c, idx_c);
      };
      mfma_slot(0);
      const u32x4 q0 = *reinterpret_cast<const u32x4*>(lq + wq_r[t][0]);
      const u32x4 q1 = *reinterpret_cast<const u32x4*>(lq + wq_r[t][1]);
      const u32x4 sc = *reinterpret_cast<const u32x4*>(lt + sc_r + t * 32);
      dma(std::integral_constant<int, 0>{});
      fence();
      mfma_slot(1);
      const u32x4 nz0 = *reinterpret_cast<const u32x4*>(lt + nz_r + t * 64);
      const u32x4 nz1 = *reinterpret_cast<const u32x4*>(lt + nz_r + t * 64 + 16);
      frag(0);
      dma(std::integral_constant<int, 1>{});
      fence();
      mfma_slot(2);
      frag(1);
      frag(2);
      dma(std::integral_constant<int, 2>{});
      // this wave's byte of the 8 words: low nibble = column tile 0 (k = 8*k8 + 2*wave), high = tile 1
      const uint32_t p01 = __builtin_amdgcn_perm(q0[1], q0[0], sel_pair);
      const uint32_t p23 = __builtin_amdgcn_perm(q0[3], q0[2], sel_pair);
      const uint32_t p45 = __builtin_amdgcn_perm(q1[1], q1[0], sel_pair);
      const uint32_t p67 = __builtin_amdgcn_perm(q1[3], q1[2], sel_pair);
      fence();
      mfma_slot(3);
      frag(3);
      frag(4);
      dma(std::integral_constant<int, 3>{});
      const uint32_t x0 = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
      const uint32_t x1 = __builtin_amdgcn_perm(p67, p45, 0x05040100u);
      // nib[tile][half]: byte i = nibble of column n + 4*half + i
      const uint32_t nib[2][2] = {{opaque(x0 & 0x0F0F0F0Fu), opaque(x1 & 0x0F0F0F0Fu)},
                                  {opaque((x0 >> 4) & 0x0F0F0F0Fu), opaque((x1 >> 4) & 0x0F0F0F0Fu)}};
      fence();
      // fragment register `reg` of tile `j`: columns n + 2*reg, n + 2*reg + 1; value = scale * nibble + (-scale * zero)
      auto piece = [&](auto j_c, auto reg_c) {
        constexpr int j = decltype(j_c)::value;
        constexpr int reg = decltype(reg_c)::value;
        const uint32_t src = nib[j][reg >> 1];
        const uint32_t sw = sc[reg];
        const float s0 = fp16_bits_to_f32((uint16_t)(sw & 0xffffu)), s1 = fp16_bits_to_f32((uint16_t)(sw >> 16));
        const u32x4& nz = (reg < 2) ? nz0 : nz1;
        const float z0 = __uint_as_float(nz[2 * (reg & 1)]), z1 = __uint_as_float(nz[2 * (reg & 1) + 1]);
        float b0, b1;
        if constexpr ((reg & 1) == 0) {
          b0 = ubyte0(src);
          b1 = ubyte1(src);
        } else {
          b0 = ubyte2(src);
          b1 = ubyte3(src);
        }
        wf[par][j][reg] = pack2<T>(__builtin_fmaf(s0, b0, z0), __builtin_fmaf(s1, b1, z1));
      };
      static_for<0, 12>([&](auto u_c) {
        constexpr int u = decltype(u_c)::value;  // slots 4 .. 15
        mfma_slot(4 + u);
        if constexpr (u < 3) frag(5 + u);
        if constexpr (u < 8) piece(std::integral_constant<int, (u >> 2)>{}, std::integral_constant<int, (u & 3)>{});
        if constexpr (u >= 8) dma(std::integral_constant<int, u - 4>{});            // slots 12-15: loads 4-7
        if constexpr (u == 0 || u == 2 || u == 4) dma(std::integral_constant<int, 8 + u / 2>{});  // loads 8-10
        fence();
      });
    };
    auto step = [&](auto nb_c, auto nt_c, auto nx_c, auto cur_c, auto vmem_c, int st_next, auto lb_c) {
      if constexpr (CODEBOOK) {
        phase_a(nb_c, nt_c, nx_c, cur_c);
        prep_b(nx_c);
        mfma_half(cur_c, I1{});
        interleave_b(vmem_c);
      } else {
        step_affine(nb_c, nt_c, nx_c, cur_c, vmem_c, st_next, lb_c);
      }
    };
    auto stage = [&](int s, auto sb_c) {
      constexpr int SB = decltype(sb_c)::value;
      using S1 = std::integral_constant<int, SB ^ 1>;
      step(sb_c, I1{}, I1{}, I0{}, NoVmem{}, 0, sb_c);
      step(sb_c, I2{}, I0{}, I1{}, NoVmem{}, 0, sb_c);
      step(sb_c, I3{}, I1{}, I0{}, NoVmem{}, 0, sb_c);
      __builtin_amdgcn_s_waitcnt(WAIT_VM0);
      __syncthreads();
      const int st_next = min(s + 2, n_stages - 1);
      if constexpr (CODEBOOK) load_stage(st_next, sb_c);  // spread under phase b by the group barriers
      step(S1{}, I0{}, I0{}, I1{}, WithVmem{}, st_next, sb_c);
    };

    __syncthreads();  // the previous projection's last LDS reads are done
    load_stage(0, I0{});
    __builtin_amdgcn_s_waitcnt(WAIT_VM0);
    __syncthreads();
    load_stage(min(1, n_stages - 1), I1{});
    if constexpr (CODEBOOK) {
      prep_first(I0{}, I0{}, I0{});
      prep_b(I0{});
    } else {
      prep(I0{}, I0{}, I0{});
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
  // register 4*i0+i1 of acc[mt][j] is dX[m0 + 32*mt + l32][8*(k8base + 8*i0 + 4*half + i1) + 2*wave + j]
  //
  // Four passes of 64 tokens.  Each pass (a) "dump": the waves round their accumulators (and the
  // LoRA product of the pass, formed by a few more MFMAs) into two LDS planes, (b) "sweep": all
  // 256 threads walk the planes in coalesced order -- lane = (row tid/32 of each group of 8 rows,
  // 8-column chunk tid%32) -- apply the mode's arithmetic and store.  The code of an epilogue runs
  // once per tile, so its size is what it costs (instruction fetch): the mode is a template
  // parameter, the pass loop is a real loop around ONE copy of the sweep, and only the small
  // dump, which names accumulator registers, exists four times.  All global accesses go through
  // buffer resources over the tile's rows, so rows past M and columns past K need no branches
  // (loads return zero, stores are dropped).  The operands the sweep of pass q+1 reads (e and g,
  // the mask source) are requested during the sweep of pass q, each into the registers the sweep
  // has just finished with, so no load is ever waited for right after its issue and no value
  // has to be copied between registers (a copy would wait for its load) where the loop closes.
  __builtin_amdgcn_s_waitcnt(WAIT_VM0);  // the surplus direct loads of the last stage have landed
  __syncthreads();
  constexpr bool swiglu = MODE == FMSA_BWD_SWIGLU;
  uint16_t* base_plane = ep_planes;
  uint16_t* lora_plane = base_plane + EP_ROWS * EP_STRIDE;
  bool any_lora = false;
  for (int p = 0; p < a.n_proj; ++p) any_lora = any_lora || (select_proj(a, p).r > 0);
  const int kcol_lane = 8 * (k8base + l32) + 2 * wave;  // column whose A^T row this lane feeds to the LoRA MFMA
  const int k_tile0 = 8 * k8base;
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
  // LoRA operands of the first 16 ranks of every projection: the A^T fragments of the lane's two
  // columns are the same for all token tiles (loaded once), the T fragments of the two token tiles
  // of a pass are fetched one pass ahead.
  u32x4 af0[3][NT], tf0[3][2];
  bool lora_live[3];
  static_for<0, 3>([&](auto p_c) {
    constexpr int p = decltype(p_c)::value;
    const BwdProjDev& P = a.p[p];
    lora_live[p] = p < a.n_proj && P.r > 0;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      af0[p][j] = u32x4{0u, 0u, 0u, 0u};
      if (lora_live[p] && row_ok && 8 * half < P.r) af0[p][j] = *reinterpret_cast<const u32x4*>(P.At + (size_t)(kcol_lane + j) * P.r + 8 * half);
    }
  });
  auto load_tf = [&](int q) {
    static_for<0, 3>([&](auto p_c) {
      constexpr int p = decltype(p_c)::value;
      const BwdProjDev& P = a.p[p];
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
      if (any_lora) {
        f32x16 lora[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int i = 0; i < 16; ++i) lora[j][i] = 0.f;
        static_for<0, 3>([&](auto p_c) {
          constexpr int p = decltype(p_c)::value;
          if (lora_live[p]) {
            const BwdProjDev& P = a.p[p];
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
        });
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int cp = 8 * (i >> 2) + 4 * half + (i & 3);
          *reinterpret_cast<uint32_t*>(lora_plane + (32 * ml + l32) * EP_STRIDE + 8 * cp + 2 * wave) = pack2<T>(lora[0][i], lora[1][i]);
        }
      }
      // rounded pairs (tile 0, tile 1) = adjacent output columns -> one 4-byte LDS write
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int cp = 8 * (i >> 2) + 4 * half + (i & 3);
        *reinterpret_cast<uint32_t*>(base_plane + (32 * ml + l32) * EP_STRIDE + 8 * cp + 2 * wave) = pack2<T>(acc[mt][0][i], acc[mt][1][i]);
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
        // Two adjacent columns at a time: every rounding to the storage type is one packed
        // conversion whose two halves are read back as fp32 (UL/swiglu.py:69-88 rounds f, h, DW and
        // DW * g to the storage type; their products with fp32 factors are rounded once, on store).
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
          // LoRA part of dh is masked by (dropout(h) != 0): mask_src holds dropout(h) when a
          // dropout was applied, otherwise h itself (recomputed here) decides; +-0 count as zero
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
    d.nsz = s.w.format == FMSA_WEIGHT_CODEBOOK ? s.w.block_scale : s.nsz;
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
#define LAUNCH_C(TT, MD, CB)                                                                           \
  do {                                                                                                 \
    if (ntail) hipLaunchKernelGGL((gptq_lora_bwd_dx_kernel<TT, true, MD, CB>), grid, block, 0, st, a);  \
    else hipLaunchKernelGGL((gptq_lora_bwd_dx_kernel<TT, false, MD, CB>), grid, block, 0, st, a);       \
  } while (0)
#define LAUNCH_M(TT, MD)                  \
  do {                                    \
    if (codebook) LAUNCH_C(TT, MD, true); \
    else LAUNCH_C(TT, MD, false);         \
  } while (0)
#define LAUNCH(TT)                                           \
  do {                                                       \
    if (mode == FMSA_BWD_SWIGLU) LAUNCH_M(TT, FMSA_BWD_SWIGLU); \
    else LAUNCH_M(TT, FMSA_BWD_LINEAR);                      \
  } while (0)
  if (act_dtype == FMSA_BF16)
    LAUNCH(bf16_t);
  else
    LAUNCH(f16_t);
#undef LAUNCH
#undef LAUNCH_M
#undef LAUNCH_C
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}
