// The rank-r LoRA GEMMs.  Both stream one [M, C] activation matrix exactly once and are bound
// by HBM bandwidth, not by arithmetic:
//   lora_down  out[M, r]  = X[M, C] * Wd[r, C]^T          (U = Xd A^T,  T = dY B)
//   lora_grad  out[r, C]  = scale * L[M, r]^T * R[M, C]    (dA, dB: a reduction over tokens)
#include "common.h"

#include <algorithm>

namespace {

// The big operand is read exactly once: its loads carry the non-temporal hint (`nt`: direct-to-LDS loads through the
// aux operand, register loads through __builtin_nontemporal_load), so that the stream does not push the small operand
// that every workgroup re-reads (Wd, L) out of L2.  Worth 5-10 % of the launch at 235 MB and rank <= 32.
// ---- lora_down ----------------------------------------------------------------------------------
// One workgroup = 16 * MTL tokens; its NW waves split C into NW contiguous slices and each runs
// MFMA 16x16x32 over its slice (X fragments straight from global: 16 rows x 64 B per load; a Wd
// fragment is loaded once per step and used for all MTL token tiles).  The kernel lives on memory
// latency, so a workgroup is up to 16 waves: that many independent load streams per CU are what
// keeps enough bytes in flight.  The NW partial [16 * MTL x r] tiles are summed through LDS in a
// fixed order: the upper half of the waves hands its tiles to the lower half, whose sums are then
// added up by all threads.
template <typename T, int RT, int MTL, int NW>
__global__ __launch_bounds__(64 * NW) void lora_down_kernel(const uint16_t* __restrict__ X, int64_t ldx,
                                                            const uint16_t* __restrict__ Wd, int M, int C, int r,
                                                            uint16_t* __restrict__ out, int64_t ldo) {
  constexpr int NH = NW / 2;
  __shared__ float red[NH][MTL][RT][64][4];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int l16 = lane & 15, q = lane >> 4;
  const int m_base = blockIdx.x * (16 * MTL);
  // slice boundaries in units of 32 columns
  const int n32 = (C + 31) / 32;
  const int per = (n32 + NW - 1) / NW;
  const int c_begin = min(C, wave * per * 32);
  const int c_end = min(C, (wave + 1) * per * 32);

  f32x4 acc[MTL][RT];
#pragma unroll
  for (int u = 0; u < MTL; ++u)
#pragma unroll
    for (int t = 0; t < RT; ++t) acc[u][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  const uint16_t* xrow[MTL];
  bool m_ok[MTL];
#pragma unroll
  for (int u = 0; u < MTL; ++u) {
    const int m = m_base + 16 * u + l16;
    m_ok[u] = m < M;
    xrow[u] = X + (size_t)(m_ok[u] ? m : 0) * ldx + 8 * q;
  }
#pragma unroll 4
  for (int c0 = c_begin; c0 < c_end; c0 += 32) {
    const bool c_ok = (c0 + 8 * q) < c_end;
    u32x4 xf[MTL];
#pragma unroll
    for (int u = 0; u < MTL; ++u) {
      xf[u] = u32x4{0u, 0u, 0u, 0u};
      if (m_ok[u] && c_ok) xf[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xrow[u] + c0));
    }
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const int j = 16 * t + l16;
      u32x4 wf = {0u, 0u, 0u, 0u};
      if (j < r && c_ok) wf = *reinterpret_cast<const u32x4*>(Wd + (size_t)j * C + c0 + 8 * q);
#pragma unroll
      for (int u = 0; u < MTL; ++u) acc[u][t] = mfma16<T>(xf[u], wf, acc[u][t]);  // D[i = token][j = rank]
    }
  }
  if (wave >= NH) {
#pragma unroll
    for (int u = 0; u < MTL; ++u)
#pragma unroll
      for (int t = 0; t < RT; ++t) *reinterpret_cast<f32x4*>(red[wave - NH][u][t][lane]) = acc[u][t];
  }
  __syncthreads();
  if (wave < NH) {
#pragma unroll
    for (int u = 0; u < MTL; ++u)
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        const f32x4 o = *reinterpret_cast<const f32x4*>(red[wave][u][t][lane]);
        *reinterpret_cast<f32x4*>(red[wave][u][t][lane]) = acc[u][t] + o;
      }
  }
  __syncthreads();
  // lane l of a tile holds D[4*(l>>4) + i][l & 15]; all threads sum MTL*RT*256 outputs over the NH slots
  for (int o = tid; o < MTL * RT * 256; o += 64 * NW) {
    const int u = o / (RT * 256), t = (o >> 8) % RT, ln = (o >> 2) & 63, i = o & 3;
    float v = red[0][u][t][ln][i];
#pragma unroll
    for (int w = 1; w < NH; ++w) v += red[w][u][t][ln][i];
    const int row = m_base + 16 * u + 4 * (ln >> 4) + i;
    const int j = 16 * t + (ln & 15);
    if (row < M && j < r) out[(size_t)row * ldo + j] = pack1<T>(v);
  }
}

// ---- lora_down, staged ----------------------------------------------------------------------------
// The same product for the large-M case, with X going through LDS: a direct load of one wave moves a
// whole 1 KB run of one row (512 columns), where the fragment loads above fetch 64 B of each of 16
// rows per instruction.  Workgroup = 32 tokens, 8 waves; a stage = 32 rows x 512 columns (32 KB) in
// one of four LDS buffers, so up to two stages are in flight while a third is multiplied.  Slot c of
// row m holds chunk c ^ (m & 15) of the row's run (the permutation is applied on the global side: a
// direct load writes lane p's 16 bytes to slot p), which spreads the 16 rows a fragment read touches
// over all banks.  Wave w multiplies columns 64w .. 64w+63 of every stage; its Wd fragments come
// straight from global (L2) one stage ahead.  Partial sums of the 8 waves are added as above.
template <typename T, int RT, int MTL>
__global__ __launch_bounds__(512) void lora_down_staged_kernel(const uint16_t* __restrict__ X, int64_t ldx,
                                                               const uint16_t* __restrict__ Wd, int M, int C, int r,
                                                               uint16_t* __restrict__ out, int64_t ldo) {
  constexpr int NW = 8, NH = 4, ROWS = 16 * MTL, SC = 512;  // a wave moves 2 * MTL rows per stage
  static_assert(RT <= 8 && (MTL == 1 || MTL == 2), "rank tiles are reduced four at a time through one stage buffer");
  // four separate arrays: every access names its buffer statically, so the compiler's wait counts
  // can tell reads of one buffer from direct loads in flight into the others
  __shared__ __attribute__((aligned(1024))) uint16_t s0[ROWS * SC];
  __shared__ __attribute__((aligned(1024))) uint16_t s1[ROWS * SC];
  __shared__ __attribute__((aligned(1024))) uint16_t s2[ROWS * SC];
  __shared__ __attribute__((aligned(1024))) uint16_t s3[ROWS * SC];
  auto buf = [&](auto b_c) -> char* {
    constexpr int b = decltype(b_c)::value;
    return reinterpret_cast<char*>(b == 0 ? s0 : (b == 1 ? s1 : (b == 2 ? s2 : s3)));
  };
  using B0 = std::integral_constant<int, 0>;
  using B1 = std::integral_constant<int, 1>;
  using B2 = std::integral_constant<int, 2>;
  using B3 = std::integral_constant<int, 3>;
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int uwave = __builtin_amdgcn_readfirstlane(wave);
  const int l16 = lane & 15, q = lane >> 4;
  const int m_base = blockIdx.x * ROWS;
  const int rows_valid = min(ROWS, M - m_base);
  const int n_stages = (C + SC - 1) / SC;
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(X + (size_t)m_base * ldx, (size_t)rows_valid * ldx * 2);
  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(Wd, (size_t)r * C * 2);

  // direct loads: wave w moves rows RPW * w .. of a stage
  // (arrays of fixed size and the template parameter itself in the loops: a local constant that depends on MTL,
  // used inside the generic lambdas below, makes the host pass drop the kernel's stub without a diagnostic)
  uint32_t d_off[4], d_col[4];
#pragma unroll
  for (int i = 0; i < 2 * MTL; ++i) {
    const int row = 2 * MTL * wave + i;
    d_col[i] = 8 * (lane ^ (row & 15));
    d_off[i] = (uint32_t)((row * ldx + d_col[i]) * 2);
  }
  auto dma = [&](int st, auto b_c) {
#pragma unroll
    for (int i = 0; i < 2 * MTL; ++i) {
      const uint32_t dead = (st * SC + (int)d_col[i]) < C ? 0u : 0x80000000u;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (__attribute__((address_space(3))) void*)(buf(b_c) + (2 * MTL * uwave + i) * (SC * 2)),
                                               16, d_off[i] | dead, (uint32_t)st * (SC * 2), 0, 2);
    }
  };
  // Wd fragments of the wave's two 32-column steps of a stage
  uint32_t w_off[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) w_off[t] = (uint32_t)(((16 * t + l16) * (int64_t)C + 8 * q) * 2);
  auto wld = [&](int st, u32x4(&wf)[2][RT]) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int c0 = st * SC + 32 * (2 * wave + kk);
      const uint32_t dead = (c0 + 8 * q) < C ? 0u : 0x80000000u;
#pragma unroll
      for (int t = 0; t < RT; ++t) wf[kk][t] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (w_off[t] + 2 * c0) | dead, 0, 0);
    }
  };
  f32x4 acc[MTL][RT];
#pragma unroll
  for (int u = 0; u < MTL; ++u)
#pragma unroll
    for (int t = 0; t < RT; ++t) acc[u][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto mul = [&](auto b_c, const u32x4(&wf)[2][RT]) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int chunk = 4 * (2 * wave + kk) + q;
#pragma unroll
      for (int u = 0; u < MTL; ++u) {
        const u32x4 xf = *reinterpret_cast<const u32x4*>(buf(b_c) + (16 * u + l16) * (SC * 2) + ((chunk ^ l16) * 16));
#pragma unroll
        for (int t = 0; t < RT; ++t) acc[u][t] = mfma16<T>(xf, wf[kk][t], acc[u][t]);  // D[i = token][j = rank]
      }
    }
  };
  // s_waitcnt vmcnt(n) only (expcnt / lgkmcnt fields left at their maxima)
  constexpr int YOUNGER = 4 * MTL + 4 * RT;  // loads a wave issues after the direct loads of a stage and before that stage's turn
  constexpr int WAIT_STEADY = (YOUNGER & 0xF) | ((YOUNGER >> 4) << 14) | 0x0F70;
  constexpr int YOUNGER0 = 4 * MTL + 2 * RT;  // ... for stage 0 (prologue order)
  constexpr int WAIT_FIRST = (YOUNGER0 & 0xF) | ((YOUNGER0 >> 4) << 14) | 0x0F70;
  // one stage: its own direct loads have landed -> barrier (all waves' parts are there, and everybody has
  // left the buffer that is re-filled next) -> requests two and three stages ahead -> multiply
  u32x4 wa[2][RT], wb[2][RT];
  auto turn = [&](int st, auto cur_c, auto refill_c, const u32x4(&wcur)[2][RT], u32x4(&wnext)[2][RT]) {
    if (st == 0)
      __builtin_amdgcn_s_waitcnt(WAIT_FIRST);
    else
      __builtin_amdgcn_s_waitcnt(WAIT_STEADY);
    // a bare barrier: the fence of __syncthreads() would wait for ALL direct loads in flight (they
    // are stores to LDS), the two stages ahead included
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    wld(st + 1, wnext);
    dma(st + 3, refill_c);
    mul(cur_c, wcur);
  };
  dma(0, B0{});
  dma(1, B1{});
  dma(2, B2{});
  wld(0, wa);
  for (int st = 0; st < n_stages; st += 4) {
    turn(st, B0{}, B3{}, wa, wb);
    turn(st + 1, B1{}, B0{}, wb, wa);
    turn(st + 2, B2{}, B1{}, wa, wb);
    turn(st + 3, B3{}, B2{}, wb, wa);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the surplus direct loads (all lanes out of range) have landed too
  __syncthreads();

  // the waves' partial tiles are added through stage buffer 0, RC rank tiles at a time ([NH][MTL][RC] KB <= its size)
  constexpr int RC = RT < 4 ? RT : 4;
  float(*red)[MTL][RC][64][4] = reinterpret_cast<float(*)[MTL][RC][64][4]>(s0);
  static_for<0, RT / RC>([&](auto c_c) {
    constexpr int t0 = decltype(c_c)::value * RC;
    if (wave >= NH) {
#pragma unroll
      for (int u = 0; u < MTL; ++u)
#pragma unroll
        for (int t = 0; t < RC; ++t) *reinterpret_cast<f32x4*>(red[wave - NH][u][t][lane]) = acc[u][t0 + t];
    }
    __syncthreads();
    if (wave < NH) {
#pragma unroll
      for (int u = 0; u < MTL; ++u)
#pragma unroll
        for (int t = 0; t < RC; ++t) {
          const f32x4 o = *reinterpret_cast<const f32x4*>(red[wave][u][t][lane]);
          *reinterpret_cast<f32x4*>(red[wave][u][t][lane]) = acc[u][t0 + t] + o;
        }
    }
    __syncthreads();
    for (int o = tid; o < MTL * RC * 256; o += 64 * NW) {
      const int u = o / (RC * 256), t = (o >> 8) % RC, ln = (o >> 2) & 63, i = o & 3;
      float v = red[0][u][t][ln][i];
#pragma unroll
      for (int w = 1; w < NH; ++w) v += red[w][u][t][ln][i];
      const int row = m_base + 16 * u + 4 * (ln >> 4) + i;
      const int j = 16 * (t0 + t) + (ln & 15);
      if (row < M && j < r) out[(size_t)row * ldo + j] = pack1<T>(v);
    }
    if constexpr (t0 + RC < RT) __syncthreads();  // the next four rank tiles reuse the buffer
  });
}

// ---- lora_down, staged, many tokens per workgroup, columns split over workgroups ----------------------
// Every workgroup of the kernels above reads all of Wd, which at 16-32 tokens per workgroup is r / 16 .. r / 32 times
// the bytes of X it consumes: from rank 32 on the L2 traffic of Wd, not HBM, sets the pace.  Here a workgroup owns
// 32 * G tokens and one of `n_split` contiguous column ranges: the stages of a 512-column chunk are its G row groups one
// after the other, multiplied by the same Wd fragments (loaded once per chunk), so Wd is read once per 32 * G tokens;
// the column split gives the chip its workgroups back when M / (32 * G) falls short of the CUs.  With n_split > 1 the
// fp32 sums of the ranges go to partial[split][M][r] and lora_down_reduce_kernel adds them in index order (same result
// whatever the scheduling) and rounds once.  Stage buffers, swizzle and the waits are those of the kernel above.
template <typename T, int RT, int G>
__global__ __launch_bounds__(512) void lora_down_split_kernel(const uint16_t* __restrict__ X, int64_t ldx,
                                                              const uint16_t* __restrict__ Wd, int M, int C, int r,
                                                              uint16_t* __restrict__ out, int64_t ldo,
                                                              float* __restrict__ partial, int n_tb, int n_split) {
  constexpr int NW = 8, NH = 4, MTL = 2, ROWS = 32, SC = 512;
  static_assert(G == 2 || G == 4, "a chunk's row groups fill the four stage buffers a whole number of times");
  static_assert(G * MTL * RT <= 32, "accumulator registers");
  __shared__ __attribute__((aligned(1024))) uint16_t s0[ROWS * SC];
  __shared__ __attribute__((aligned(1024))) uint16_t s1[ROWS * SC];
  __shared__ __attribute__((aligned(1024))) uint16_t s2[ROWS * SC];
  __shared__ __attribute__((aligned(1024))) uint16_t s3[ROWS * SC];
  auto buf = [&](auto b_c) -> char* {
    constexpr int b = decltype(b_c)::value;
    return reinterpret_cast<char*>(b == 0 ? s0 : (b == 1 ? s1 : (b == 2 ? s2 : s3)));
  };
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int uwave = __builtin_amdgcn_readfirstlane(wave);
  const int l16 = lane & 15, q = lane >> 4;
  const int tb = blockIdx.x % n_tb, sp = blockIdx.x / n_tb;
  const int m_base = tb * (ROWS * G);
  const int rows_valid = min(ROWS * G, M - m_base);
  // this workgroup's chunks [ch_lo, ch_hi) of 512 columns
  const int n_chunks = (C + SC - 1) / SC;
  const int per = (n_chunks + n_split - 1) / n_split;
  const int ch_lo = min(n_chunks, sp * per), ch_hi = min(n_chunks, ch_lo + per);
  const int n_stages = (ch_hi - ch_lo) * G;
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(X + (size_t)m_base * ldx, (size_t)rows_valid * ldx * 2);
  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(Wd, (size_t)r * C * 2);

  // direct loads: wave w moves rows 4 w .. 4 w + 3 of a stage (row group g of the workgroup's tokens)
  uint32_t d_off[4], d_col[4];
#pragma unroll
  for (int i = 0; i < 2 * MTL; ++i) {
    const int row = 2 * MTL * wave + i;
    d_col[i] = 8 * (lane ^ (row & 15));
    d_off[i] = (uint32_t)((row * ldx + d_col[i]) * 2);
  }
  const uint32_t group_bytes = (uint32_t)(ROWS * ldx * 2);
  // stage st = chunk ch_lo + st / G, row group st % G; stages past the last one load nothing (every lane out of range)
  auto dma = [&](int st, auto b_c) {
    const int ch = ch_lo + st / G, g = st % G;
#pragma unroll
    for (int i = 0; i < 2 * MTL; ++i) {
      const uint32_t dead = (ch < ch_hi && (ch * SC + (int)d_col[i]) < C) ? 0u : 0x80000000u;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (__attribute__((address_space(3))) void*)(buf(b_c) + (2 * MTL * uwave + i) * (SC * 2)),
                                               16, (d_off[i] + (uint32_t)g * group_bytes) | dead, (uint32_t)ch * (SC * 2), 0, 2);
    }
  };
  uint32_t w_off[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) w_off[t] = (uint32_t)(((16 * t + l16) * (int64_t)C + 8 * q) * 2);
  auto wld = [&](int ch, u32x4(&wf)[2][RT]) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int c0 = ch * SC + 32 * (2 * wave + kk);
      const uint32_t dead = (ch < ch_hi && (c0 + 8 * q) < C) ? 0u : 0x80000000u;
#pragma unroll
      for (int t = 0; t < RT; ++t) wf[kk][t] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (w_off[t] + 2 * c0) | dead, 0, 0);
    }
  };
  f32x4 acc[G][MTL][RT];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int u = 0; u < MTL; ++u)
#pragma unroll
      for (int t = 0; t < RT; ++t) acc[g][u][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto mul = [&](auto b_c, auto g_c, const u32x4(&wf)[2][RT]) {
    constexpr int g = decltype(g_c)::value;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int chunk = 4 * (2 * wave + kk) + q;
#pragma unroll
      for (int u = 0; u < MTL; ++u) {
        const u32x4 xf = *reinterpret_cast<const u32x4*>(buf(b_c) + (16 * u + l16) * (SC * 2) + ((chunk ^ l16) * 16));
#pragma unroll
        for (int t = 0; t < RT; ++t) acc[g][u][t] = mfma16<T>(xf, wf[kk][t], acc[g][u][t]);
      }
    }
  };
  // Loads a wave issues after the direct loads of stage st and before that stage's turn: the direct loads of the two
  // stages after it (2 x 4), and one batch of Wd fragments when turn st - 1 or st - 2 closed a chunk (g = 0 or 1).
  // A smaller count than the true one only waits longer, so the first turns use the same figures.
  auto wait_for = [&](auto g_c) {
    constexpr int g = decltype(g_c)::value;
    constexpr int YOUNGER = 4 * MTL + ((g == 0 || g == 1) ? 2 * RT : 0);
    __builtin_amdgcn_s_waitcnt((YOUNGER & 0xF) | ((YOUNGER >> 4) << 14) | 0x0F70);
  };
  u32x4 wa[2][RT], wb[2][RT];
  // turn st: its direct loads have landed -> barrier -> (last row group of a chunk: the next chunk's Wd fragments) ->
  // the direct loads three stages ahead -> multiply
  auto turn = [&](int st, auto cur_c, auto refill_c, auto g_c, const u32x4(&wcur)[2][RT], u32x4(&wnext)[2][RT]) {
    constexpr int g = decltype(g_c)::value;
    wait_for(g_c);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (g == G - 1) wld(ch_lo + st / G + 1, wnext);
    dma(st + 3, refill_c);
    mul(cur_c, g_c, wcur);
  };
  using B0 = std::integral_constant<int, 0>;
  using B1 = std::integral_constant<int, 1>;
  using B2 = std::integral_constant<int, 2>;
  using B3 = std::integral_constant<int, 3>;
  dma(0, B0{});
  dma(1, B1{});
  dma(2, B2{});
  wld(ch_lo, wa);
  if constexpr (G == 2) {
    for (int st = 0; st < n_stages; st += 4) {  // two chunks per round
      turn(st, B0{}, B3{}, B0{}, wa, wb);
      turn(st + 1, B1{}, B0{}, B1{}, wa, wb);
      turn(st + 2, B2{}, B1{}, B0{}, wb, wa);
      turn(st + 3, B3{}, B2{}, B1{}, wb, wa);
    }
  } else {
    for (int st = 0; st < n_stages; st += 8) {
      turn(st, B0{}, B3{}, B0{}, wa, wb);
      turn(st + 1, B1{}, B0{}, B1{}, wa, wb);
      turn(st + 2, B2{}, B1{}, B2{}, wa, wb);
      turn(st + 3, B3{}, B2{}, B3{}, wa, wb);
      turn(st + 4, B0{}, B3{}, B0{}, wb, wa);
      turn(st + 5, B1{}, B0{}, B1{}, wb, wa);
      turn(st + 6, B2{}, B1{}, B2{}, wb, wa);
      turn(st + 7, B3{}, B2{}, B3{}, wb, wa);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the surplus direct loads (all lanes out of range) have landed too
  __syncthreads();

  // the waves' partial tiles are added through stage buffer 0, one row group and RC rank tiles at a time
  constexpr int RC = RT < 4 ? RT : 4;
  float(*red)[MTL][RC][64][4] = reinterpret_cast<float(*)[MTL][RC][64][4]>(s0);
  float* const pdst = partial + (size_t)sp * M * r;
  static_for<0, G>([&](auto g_c) {
    constexpr int g = decltype(g_c)::value;
    static_for<0, RT / RC>([&](auto c_c) {
      constexpr int t0 = decltype(c_c)::value * RC;
      if (wave >= NH) {
#pragma unroll
        for (int u = 0; u < MTL; ++u)
#pragma unroll
          for (int t = 0; t < RC; ++t) *reinterpret_cast<f32x4*>(red[wave - NH][u][t][lane]) = acc[g][u][t0 + t];
      }
      __syncthreads();
      if (wave < NH) {
#pragma unroll
        for (int u = 0; u < MTL; ++u)
#pragma unroll
          for (int t = 0; t < RC; ++t) {
            const f32x4 o = *reinterpret_cast<const f32x4*>(red[wave][u][t][lane]);
            *reinterpret_cast<f32x4*>(red[wave][u][t][lane]) = acc[g][u][t0 + t] + o;
          }
      }
      __syncthreads();
      for (int o = tid; o < MTL * RC * 256; o += 64 * NW) {
        const int u = o / (RC * 256), t = (o >> 8) % RC, ln = (o >> 2) & 63, i = o & 3;
        float v = red[0][u][t][ln][i];
#pragma unroll
        for (int w = 1; w < NH; ++w) v += red[w][u][t][ln][i];
        const int row = m_base + ROWS * g + 16 * u + 4 * (ln >> 4) + i;
        const int j = 16 * (t0 + t) + (ln & 15);
        if (row < M && j < r) {
          if (n_split == 1)
            out[(size_t)row * ldo + j] = pack1<T>(v);
          else
            pdst[(size_t)row * r + j] = v;
        }
      }
      __syncthreads();  // the next tiles reuse the buffer
    });
  });
}

// out[m, j] = round(sum over splits, in index order, of partial[split][m][j]); r % 8 == 0: four ranks per thread
template <typename T>
__global__ __launch_bounds__(256) void lora_down_reduce_kernel(const float* __restrict__ partial, int n_split, int M, int r,
                                                               uint16_t* __restrict__ out, int64_t ldo) {
  const int64_t q4 = (int64_t)blockIdx.x * 256 + threadIdx.x;  // quad of ranks
  const int per_row = r / 4;
  if (q4 >= (int64_t)M * per_row) return;
  const int m = (int)(q4 / per_row), j = 4 * (int)(q4 % per_row);
  const size_t plane = (size_t)M * r;
  f32x4 v = *reinterpret_cast<const f32x4*>(partial + (size_t)m * r + j);
  for (int s = 1; s < n_split; ++s) v += *reinterpret_cast<const f32x4*>(partial + s * plane + (size_t)m * r + j);
  u32x2 o;
  o[0] = pack2<T>(v[0], v[1]);
  o[1] = pack2<T>(v[2], v[3]);
  *reinterpret_cast<u32x2*>(out + (size_t)m * ldo + j) = o;
}

// ---- lora_grad ----------------------------------------------------------------------------------
// out[j, c] = sum_m L[m, j] * R[m, c]: the contraction runs over tokens, which is the row index of
// both row-major operands, so each MFMA fragment (8 consecutive contraction elements per lane) is a
// column walk.  Tiles of 32 tokens are staged through LDS (coalesced 16-byte global loads in, transposing
// 8-byte reads out: column_frag below); token e of a tile is the MFMA's contraction index e, rows are padded
// by 32 B.
// Pass 1: workgroup = 256 columns of R (eight waves) x one fixed range of tokens (split); wave w owns columns
// 32w .. 32w+31 (two 16-wide MFMA tiles) and all r ranks.  Partial sums go to partial[split][r][C]
// (fp32).  Pass 2 adds the splits in index order, so the result does not depend on scheduling.
constexpr int LG_TM = 32;               // tokens per tile
constexpr int LG_TC_T = 256;   // columns of R per workgroup (8 waves x 32)

// Several gradients over the same M tokens go out as ONE launch of each pass (the dA of stacked
// adapters and their dB's; a launch of a small gradient alone neither fills the chip nor hides its
// own start-up): workgroup ids are laid end to end over the jobs.
struct LoraGradJobDev {
  const uint16_t* L;
  const uint16_t* R;
  void* out;
  float* partial;  // [splits][r][C] of this job
  int64_t ldl, ldr;
  int C, r, splits, rows_per_split;
  int block_start;   // first workgroup of the job in pass 1
  int rblock_start;  // ... in pass 2
  int transpose_out, out_dtype;
  float scale;
  // optional second product of the same pass over R: T[M, r] = R * Wt^T (see below)
  const uint16_t* Wt;  // [r, C]
  float* tpart;        // [column blocks][M][r]
  uint16_t* T;
  int64_t ldt;
};
struct LoraGradArgs {
  LoraGradJobDev j[FMSA_LORA_GRAD_MAX_JOBS];
  int n_jobs, M, act_dtype;
};
// the job that owns workgroup `block` (wave-uniform), copied field by field: indexing the
// kernel-argument struct with a runtime value would force a copy of it into scratch memory
template <bool REDUCE>
FMSA_DEVI LoraGradJobDev select_job(const LoraGradArgs& a, int block) {
  LoraGradJobDev J = a.j[0];
#pragma unroll
  for (int q = 1; q < FMSA_LORA_GRAD_MAX_JOBS; ++q)
    if (q < a.n_jobs && block >= (REDUCE ? a.j[q].rblock_start : a.j[q].block_start)) J = a.j[q];
  return J;
}

// WITH_T: a job with Wt set also produces T = R * Wt^T (the `dY @ B` every backward needs next to
// dB = s * dY^T U: both read dY, which is the whole cost of either).  The R tile is in LDS anyway, and
// row-major, which is the natural MFMA layout for a contraction over columns: wave w multiplies the
// tile's 32 tokens by its own 32 columns (2 * rt MFMAs per tile), the four waves' partial tiles meet in
// LDS and are summed in wave order by the whole workgroup one iteration later (behind the barrier the
// loop has anyway), and leave as the column block's partial T[column block][token][rank] (fp32).  The
// reduce pass adds the column blocks in index order and rounds once: deterministic like the rest.
// Eight waves and 256 columns per workgroup: the L tile every workgroup re-reads is r / 256 of the R bytes it consumes
// (a four-wave, 128-column workgroup measured slower at every rank: 44.6 vs 41.8 us over 235 MB at rank 16).
template <typename T, int RT, bool WITH_T>
__global__ __launch_bounds__(512) void lora_grad_partial_kernel(const LoraGradArgs a) {
  constexpr int NWV = 8;  // waves
  constexpr int NTH = 64 * NWV;             // threads
  constexpr int TC = 32 * NWV;              // columns of R per workgroup
  constexpr int LG_RSTRIDE = TC + 16;       // elements: row + 32 B pad
  constexpr int LSTRIDE = (RT == 1) ? 16 : RT * 16 + 16;  // elements; row pitch = 8 banks mod 32
  __shared__ __attribute__((aligned(16))) uint16_t r_lds[2][LG_TM * LG_RSTRIDE];
  __shared__ __attribute__((aligned(16))) uint16_t l_lds[2][LG_TM * LSTRIDE];
  __shared__ __attribute__((aligned(16))) float t_lds[WITH_T ? 2 : 1][WITH_T ? NWV : 1][2][WITH_T ? RT : 1][64][WITH_T ? 4 : 1];
  const LoraGradJobDev J = select_job<false>(a, blockIdx.x);
  const uint16_t* __restrict__ L = J.L;
  const uint16_t* __restrict__ R = J.R;
  float* __restrict__ partial = J.partial;
  const int64_t ldl = J.ldl, ldr = J.ldr;
  const int M = a.M, C = J.C, r = J.r, rows_per_split = J.rows_per_split;
  const int rt = (r + 15) / 16;  // 16-rank tiles this job uses of the RT the launch is built for
  const int ncb = (C + TC - 1) / TC;
  const int local = blockIdx.x - J.block_start;
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int l16 = lane & 15, kg = lane >> 4;
  const int split = local / ncb;
  const int c0 = (local % ncb) * TC;
  const int m_begin = split * rows_per_split;
  const int m_end = min(M, m_begin + rows_per_split);
  const int n_tiles = (m_end - m_begin + LG_TM - 1) / LG_TM;

  // global -> LDS assignment: R tile = 32 rows x TC/8 chunks of 16 B -> 2 chunks per thread (16 rows per pass);
  // L tile = 32 rows x (RT*2) chunks = 64*RT chunks -> LP per thread (chunk tid + NTH*p), threads
  // past the last chunk idle
  const int r_row = tid / (TC / 8), r_chunk = tid % (TC / 8);
  const bool r_col_ok = (c0 + 8 * r_chunk) < C;  // C % 8 == 0
  constexpr int LP = (64 * RT + NTH - 1) / NTH;
  int l_row[LP], l_chunk[LP];
  bool l_thread[LP], l_col_ok[LP];
#pragma unroll
  for (int p = 0; p < LP; ++p) {
    const int ci = tid + NTH * p;
    l_row[p] = ci / (2 * RT);
    l_chunk[p] = ci % (2 * RT);
    l_thread[p] = ci < 64 * RT;
    l_col_ok[p] = 8 * l_chunk[p] < r;  // r % 8 == 0
  }

  u32x4 rst[2], lst[LP];
  auto load_tile = [&](int tile) {
    const int m0 = m_begin + tile * LG_TM;
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const int m = m0 + r_row + 16 * p;
      rst[p] = u32x4{0u, 0u, 0u, 0u};
      if (m < m_end && r_col_ok) rst[p] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(R + (size_t)m * ldr + c0 + 8 * r_chunk));
    }
#pragma unroll
    for (int p = 0; p < LP; ++p) {
      lst[p] = u32x4{0u, 0u, 0u, 0u};
      const int m = m0 + l_row[p];
      if (l_thread[p] && m < m_end && l_col_ok[p]) lst[p] = *reinterpret_cast<const u32x4*>(L + (size_t)m * ldl + 8 * l_chunk[p]);
    }
  };
  auto commit_tile = [&](int buf) {
#pragma unroll
    for (int p = 0; p < 2; ++p)
      *reinterpret_cast<u32x4*>(&r_lds[buf][(r_row + 16 * p) * LG_RSTRIDE + 8 * r_chunk]) = rst[p];
#pragma unroll
    for (int p = 0; p < LP; ++p)
      if (l_thread[p]) *reinterpret_cast<u32x4*>(&l_lds[buf][l_row[p] * LSTRIDE + 8 * l_chunk[p]]) = lst[p];
  };
  // The MFMA operand of a 16-column tile starting at column `col0`: lane 16 kg + m gets column col0 + m at the 8 tokens
  // 8 kg .. 8 kg + 7 (contraction index k = 8 kg + e <-> token 8 kg + e of the tile).  Two transposing LDS reads
  // (ds_read_b64_tr_b16) do it: in a group of 16 lanes, lane 4 a + b receives element b of the four 16-bit values that
  // lanes a, a + 4, a + 8, a + 12 address, so lane j of the group addresses token 8 kg + 4 h + j / 4, columns
  // col0 + 4 (j % 4) .. + 3 (h = 0, 1: the two reads).  Was eight 16-bit reads and their packing per operand.
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  auto column_frag = [&](const uint16_t* base, int stride, int col0) {
    const uint16_t* p = base + (8 * kg + (l16 >> 2)) * stride + col0 + 4 * (l16 & 3);
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p + 4 * stride));
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    return u32x4{l2[0], l2[1], h2[0], h2[1]};
  };

  f32x4 acc[2][RT];
#pragma unroll
  for (int g = 0; g < 2; ++g)
#pragma unroll
    for (int t = 0; t < RT; ++t) acc[g][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // T product: this lane's Wt fragments (rank 16t + l16, columns c0 + 32*wave + 8*kg ..), fixed for the workgroup
  const bool with_t = WITH_T && J.Wt != nullptr;
  u32x4 wtf[RT];
  if constexpr (WITH_T) {
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      wtf[t] = u32x4{0u, 0u, 0u, 0u};
      const int j = 16 * t + l16, c = c0 + 32 * wave + 8 * kg;
      if (with_t && j < r && c < C) wtf[t] = *reinterpret_cast<const u32x4*>(J.Wt + (size_t)j * C + c);
    }
  }
  // sums the four waves' partial T tiles of token tile `tile` (parked in t_lds[tile & 1]) and stores them
  auto flush_t = [&](int tile) {
    if constexpr (WITH_T) {
      if (!with_t) return;
      const int tb = tile & 1;
      const int m0 = m_begin + tile * LG_TM;
      float* dst = J.tpart + ((size_t)(local % ncb) * M) * r;
      for (int v = tid; v < LG_TM * 16 * RT; v += NTH) {
        const int j = v % (16 * RT), m = v / (16 * RT);
        const int u = m >> 4, ln = ((m & 15) >> 2) * 16 + (j & 15), i = m & 3, t = j >> 4;
        float sum = t_lds[tb][0][u][t][ln][i];
#pragma unroll
        for (int w = 1; w < NWV; ++w) sum += t_lds[tb][w][u][t][ln][i];
        if (m0 + m < m_end && j < r) dst[(size_t)(m0 + m) * r + j] = sum;
      }
    }
  };

  if (n_tiles > 0) {
    load_tile(0);
    commit_tile(0);
  }
  __syncthreads();
  for (int tile = 0; tile < n_tiles; ++tile) {
    const int buf = tile & 1;
    if (tile + 1 < n_tiles) load_tile(tile + 1);
    if (tile > 0) flush_t(tile - 1);
    if constexpr (WITH_T) {
      if (with_t) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const u32x4 yf = *reinterpret_cast<const u32x4*>(&r_lds[buf][(16 * u + l16) * LG_RSTRIDE + 32 * wave + 8 * kg]);
#pragma unroll
          for (int t = 0; t < RT; ++t)
            if (t < rt)
              *reinterpret_cast<f32x4*>(t_lds[buf][wave][u][t][lane]) = mfma16<T>(yf, wtf[t], f32x4{0.f, 0.f, 0.f, 0.f});  // D[token][rank]
        }
      }
    }
    u32x4 lf[RT], rf[2];
#pragma unroll
    for (int t = 0; t < RT; ++t)
      if (t < rt) lf[t] = column_frag(l_lds[buf], LSTRIDE, 16 * t);
#pragma unroll
    for (int g = 0; g < 2; ++g) rf[g] = column_frag(r_lds[buf], LG_RSTRIDE, 32 * wave + 16 * g);
#pragma unroll
    for (int t = 0; t < RT; ++t)
      if (t < rt) {
#pragma unroll
        for (int g = 0; g < 2; ++g) acc[g][t] = mfma16<T>(rf[g], lf[t], acc[g][t]);  // D[c][j]
      }
    if (tile + 1 < n_tiles) commit_tile(buf ^ 1);
    __syncthreads();
  }
  if (n_tiles > 0) flush_t(n_tiles - 1);
  // lane holds D[c = 4*kg + i][j = l16]: four consecutive columns -> one 16-byte store
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    const int c = c0 + 32 * wave + 16 * g + 4 * kg;
    if (c >= C) continue;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const int j = 16 * t + l16;
      if (j >= r) continue;
      float* dst = partial + ((size_t)split * r + j) * C + c;
      if (c + 4 <= C) {
        *reinterpret_cast<f32x4*>(dst) = acc[g][t];
      } else {
        for (int i = 0; i < 4; ++i)
          if (c + i < C) dst[i] = acc[g][t][i];
      }
    }
  }
}

__global__ __launch_bounds__(256) void lora_grad_reduce_kernel(const LoraGradArgs a) {
  const LoraGradJobDev J = select_job<true>(a, blockIdx.x);
  const int r = J.r, C = J.C;
  const int nb_grad = (r * C + 255) / 256;
  const int lb = blockIdx.x - J.rblock_start;
  if (lb >= nb_grad) {  // the job's T: column blocks added in index order, one rounding; four ranks per thread
    const int64_t ti = ((int64_t)(lb - nb_grad) * 256 + threadIdx.x) * 4;
    if (ti >= (int64_t)a.M * r) return;  // r % 8 == 0: the four stay inside one token's row
    const int m = (int)(ti / r), j = (int)(ti % r);
    const int ncb = (C + LG_TC_T - 1) / LG_TC_T;
    // eight loads in flight per thread (a plain loop waits for each load before it issues the next); the sum
    // itself stays in index order
    const float* src = J.tpart + (size_t)m * r + j;
    const size_t step = (size_t)a.M * r;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    int cb = 0;
    for (; cb + 8 <= ncb; cb += 8) {
      f32x4 p[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) p[k] = *reinterpret_cast<const f32x4*>(src + (size_t)(cb + k) * step);
#pragma unroll
      for (int k = 0; k < 8; ++k) v += p[k];
    }
    for (; cb < ncb; ++cb) v += *reinterpret_cast<const f32x4*>(src + (size_t)cb * step);
    u32x2 pk;
    pk[0] = a.act_dtype == FMSA_BF16 ? pack2<bf16_t>(v[0], v[1]) : pack2<f16_t>(v[0], v[1]);
    pk[1] = a.act_dtype == FMSA_BF16 ? pack2<bf16_t>(v[2], v[3]) : pack2<f16_t>(v[2], v[3]);
    *reinterpret_cast<u32x2*>(J.T + (size_t)m * J.ldt + j) = pk;
    return;
  }
  const int idx = lb * 256 + threadIdx.x;  // over r*C, c fastest
  if (idx >= r * C) return;
  const int j = idx / C, c = idx % C;
  const float* src = J.partial + (size_t)j * C + c;
  const size_t step = (size_t)r * C;
  float v = 0.f;
  int sp = 0;
  for (; sp + 8 <= J.splits; sp += 8) {  // eight loads in flight, summed in index order
    float p[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) p[k] = src[(size_t)(sp + k) * step];
#pragma unroll
    for (int k = 0; k < 8; ++k) v += p[k];
  }
  for (; sp < J.splits; ++sp) v += src[(size_t)sp * step];
  v *= J.scale;
  const size_t o = J.transpose_out ? ((size_t)c * r + j) : (size_t)idx;
  if (J.out_dtype == FMSA_F32)
    reinterpret_cast<float*>(J.out)[o] = v;
  else
    reinterpret_cast<uint16_t*>(J.out)[o] = J.out_dtype == FMSA_BF16 ? pack1<bf16_t>(v) : pack1<f16_t>(v);
}

}  // namespace

int lora_grad_splits(int M, int C) {
  const int ncb = (C + LG_TC_T - 1) / LG_TC_T;
  // about two 512-thread workgroups per CU (16 waves), but at least 512 tokens (16 tiles) per split: shorter
  // splits spend their time in the prologue and in writing / re-reading partial sums.  (The count equals what
  // 1024 / number of 128-column blocks gave for widths that are multiples of 256; part of the workspace contract.)
  int splits = 512 / ncb;
  const int max_splits = (M + 511) / 512;
  if (splits > max_splits) splits = max_splits;
  if (splits < 1) splits = 1;
  return splits;
}

int launch_lora_down(const void* X, int64_t ldx, const void* Wd, int M, int C, int r, int act_dtype, void* out,
                     int64_t ldo, hipStream_t st) {
  // 32 tokens per workgroup once that still leaves a workgroup per CU (halves the re-reads of Wd)
  const int mtl = (M >= 32 * 256 && r <= 64) ? 2 : 1;
  constexpr int NW = 8;  // waves per workgroup: measured best of 4 / 8 / 16 at 8192 tokens
  dim3 grid((M + 16 * mtl - 1) / (16 * mtl)), block(64 * NW);
  const int rt = (r + 15) / 16;
  // staged kernel: 32 (from 8192 tokens) or 16 (from 4096) tokens per workgroup, worth it once that gives every CU a
  // workgroup and the rows are long enough to amortise its pipeline fill (measured at 8192 tokens: 59 -> 48 us at
  // C = 14336, r = 16; 32 -> 28 us at C = 4096, r = 48; 20 -> 21 us at C = 4096, r = 16; at 4096 tokens, C = 28672,
  // r = 64: 205 us with the fragment loads above)
  const bool staged = M >= 16 * 256 && rt <= 8 && (C >= 8192 || (rt >= 2 && C >= 2048));
  if (staged) {
    const int smtl = M >= 32 * 256 ? 2 : 1;
    dim3 sgrid((M + 16 * smtl - 1) / (16 * smtl)), sblock(512);
#define SLAUNCH(TT, RT)                                                                                                           \
  do {                                                                                                                            \
    if (smtl == 2)                                                                                                                \
      hipLaunchKernelGGL((lora_down_staged_kernel<TT, RT, 2>), sgrid, sblock, 0, st, (const uint16_t*)X, ldx, (const uint16_t*)Wd, \
                         M, C, r, (uint16_t*)out, ldo);                                                                           \
    else                                                                                                                          \
      hipLaunchKernelGGL((lora_down_staged_kernel<TT, RT, 1>), sgrid, sblock, 0, st, (const uint16_t*)X, ldx, (const uint16_t*)Wd, \
                         M, C, r, (uint16_t*)out, ldo);                                                                           \
  } while (0)
#define SDISPATCH(TT)                        \
  switch (rt) {                              \
    case 1: SLAUNCH(TT, 1); break;           \
    case 2: SLAUNCH(TT, 2); break;           \
    case 3: case 4: SLAUNCH(TT, 4); break;   \
    default: SLAUNCH(TT, 8); break;          \
  }
    if (act_dtype == FMSA_BF16) {
      SDISPATCH(bf16_t)
    } else {
      SDISPATCH(f16_t)
    }
#undef SDISPATCH
#undef SLAUNCH
    FMSA_CHECK_LAUNCH();
    return FMSA_OK;
  }
#define LAUNCH(TT, RT)                                                                                                       \
  do {                                                                                                                       \
    if (mtl == 2)                                                                                                            \
      hipLaunchKernelGGL((lora_down_kernel<TT, RT, (RT > 4 ? 1 : 2), NW>), grid, block, 0, st, (const uint16_t*)X, ldx,       \
                         (const uint16_t*)Wd, M, C, r, (uint16_t*)out, ldo);                                                 \
    else                                                                                                                     \
      hipLaunchKernelGGL((lora_down_kernel<TT, RT, 1, NW>), grid, block, 0, st, (const uint16_t*)X, ldx, (const uint16_t*)Wd, \
                         M, C, r, (uint16_t*)out, ldo);                                                                      \
  } while (0)
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

namespace {
// Shape of the split launch: row groups per workgroup, column ranges, or g = 0 when the kernels without workspace do as
// well or the matrix is too small.  (At rank 16 and below Wd is a small part of the traffic; what the split kernel adds there
// is 64 tokens per workgroup with 1 KB row runs through LDS and column ranges that keep every CU busy: 21 -> 17 us on
// 8192 x 4096.)
struct DownSplit {
  int g, n_tb, n_split;
};
DownSplit lora_down_split_shape(int M, int C, int r) {
  const int rt = (std::min(r, 64) + 15) / 16;  // ranks above 64 go out 64 at a time (accumulator registers)
  if (M < 2048 || C < 2048) return {0, 0, 0};
  if (rt < 2 && M >= 16384) return {0, 0, 0};  // rank 16 and below with a workgroup per CU anyway: the 32-token kernels do as well
  const int g = rt <= 2 ? 2 : 4;  // rank 32: 64 tokens per workgroup; 48 / 64: 128
  const int n_tb = (M + 32 * g - 1) / (32 * g);
  const int n_chunks = (C + 511) / 512;
  int n_split = (256 + n_tb - 1) / n_tb;                 // a workgroup per CU at least
  n_split = std::max(1, std::min(n_split, n_chunks / 2));  // two chunks per range at least
  return {g, n_tb, n_split};
}
}  // namespace

size_t lora_down_workspace(int M, int C, int r) {
  const DownSplit d = lora_down_split_shape(M, C, r);
  return d.g && d.n_split > 1 ? (size_t)d.n_split * (size_t)M * (size_t)std::min(r, 64) * sizeof(float) : 0;
}

// The split kernel where it pays and the caller brought the partial-sum buffer (or none is needed); launch_lora_down otherwise.
int launch_lora_down_ws(const void* X, int64_t ldx, const void* Wd, int M, int C, int r, int act_dtype, void* out,
                        int64_t ldo, void* workspace, size_t workspace_bytes, hipStream_t st) {
  const DownSplit d = lora_down_split_shape(M, C, r);
  const size_t need = lora_down_workspace(M, C, r);
  const bool out_ok = ((uintptr_t)out % 8 == 0) && ldo % 4 == 0;  // the reduce pass stores four ranks at a time
  if (!d.g || (need && (!workspace || workspace_bytes < need || !out_ok)))
    return launch_lora_down(X, ldx, Wd, M, C, r, act_dtype, out, ldo, st);
  if (r > 64) {
    // 64 ranks per pass over X (launches on one stream run in order, so the passes share the workspace); cheaper than one
    // pass whose accumulators and double-buffered Wd fragments do not fit the registers
    for (int r0 = 0; r0 < r; r0 += 64) {
      const int rc = launch_lora_down_ws(X, ldx, (const uint16_t*)Wd + (size_t)r0 * C, M, C, std::min(64, r - r0), act_dtype,
                                         (uint16_t*)out + r0, ldo, workspace, workspace_bytes, st);
      if (rc != FMSA_OK) return rc;
    }
    return FMSA_OK;
  }
  const int rt = (r + 15) / 16;
  dim3 grid(d.n_tb * d.n_split), block(512);
#define SPLIT_LAUNCH(TT, RT, G)                                                                                                  \
  hipLaunchKernelGGL((lora_down_split_kernel<TT, RT, G>), grid, block, 0, st, (const uint16_t*)X, ldx, (const uint16_t*)Wd, M, \
                     C, r, (uint16_t*)out, ldo, (float*)workspace, d.n_tb, d.n_split)
#define SPLIT_DISPATCH(TT)                            \
  switch (rt) {                                       \
    case 1: SPLIT_LAUNCH(TT, 1, 2); break;            \
    case 2: SPLIT_LAUNCH(TT, 2, 2); break;            \
    default: SPLIT_LAUNCH(TT, 4, 4); break;           \
  }
  if (act_dtype == FMSA_BF16) {
    SPLIT_DISPATCH(bf16_t)
  } else {
    SPLIT_DISPATCH(f16_t)
  }
#undef SPLIT_DISPATCH
#undef SPLIT_LAUNCH
  FMSA_CHECK_LAUNCH();
  if (d.n_split > 1) {
    const int64_t quads = (int64_t)M * (r / 4);
    dim3 rgrid((unsigned)((quads + 255) / 256));
    if (act_dtype == FMSA_BF16)
      hipLaunchKernelGGL((lora_down_reduce_kernel<bf16_t>), rgrid, dim3(256), 0, st, (const float*)workspace, d.n_split, M, r,
                         (uint16_t*)out, ldo);
    else
      hipLaunchKernelGGL((lora_down_reduce_kernel<f16_t>), rgrid, dim3(256), 0, st, (const float*)workspace, d.n_split, M, r,
                         (uint16_t*)out, ldo);
    FMSA_CHECK_LAUNCH();
  }
  return FMSA_OK;
}

namespace {
size_t job_partial_bytes(const fmsa_lora_grad_job& s, int M) {
  return (size_t)lora_grad_splits(M, s.C) * (size_t)s.r * (size_t)s.C * sizeof(float);
}
size_t job_tpart_bytes(const fmsa_lora_grad_job& s, int M) {
  return s.Wt ? (size_t)((s.C + LG_TC_T - 1) / LG_TC_T) * (size_t)M * (size_t)s.r * sizeof(float) : 0;
}
}  // namespace

size_t lora_grad_batch_workspace(const fmsa_lora_grad_job* jobs, int n_jobs, int M) {
  size_t bytes = 0;
  for (int q = 0; q < n_jobs; ++q) bytes += job_partial_bytes(jobs[q], M) + job_tpart_bytes(jobs[q], M);
  return bytes;
}

int launch_lora_grad_batch(const fmsa_lora_grad_job* jobs, int n_jobs, int M, int act_dtype, void* workspace, hipStream_t st) {
  LoraGradArgs a{};
  a.n_jobs = n_jobs;
  a.M = M;
  a.act_dtype = act_dtype;
  bool any_t = false;
  for (int q = 0; q < n_jobs; ++q) any_t = any_t || jobs[q].Wt != nullptr;
  const int tc = LG_TC_T;
  int blocks = 0, rblocks = 0, r_max = 0;
  size_t ws_off = 0;
  for (int q = 0; q < n_jobs; ++q) {
    const fmsa_lora_grad_job& s = jobs[q];
    LoraGradJobDev& d = a.j[q];
    d.L = (const uint16_t*)s.L;
    d.R = (const uint16_t*)s.R;
    d.out = s.out;
    d.partial = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + ws_off);
    d.ldl = s.ldl;
    d.ldr = s.ldr;
    d.C = s.C;
    d.r = s.r;
    d.splits = lora_grad_splits(M, s.C);
    const int rows = (M + d.splits - 1) / d.splits;
    d.rows_per_split = ((rows + LG_TM - 1) / LG_TM) * LG_TM;
    d.block_start = blocks;
    d.rblock_start = rblocks;
    d.transpose_out = s.transpose_out;
    d.out_dtype = s.out_dtype;
    d.scale = s.scale;
    blocks += ((s.C + tc - 1) / tc) * d.splits;
    rblocks += (s.r * s.C + 255) / 256;
    ws_off += job_partial_bytes(s, M);
    if (s.Wt) {
      d.Wt = (const uint16_t*)s.Wt;
      d.T = (uint16_t*)s.T;
      d.ldt = s.ldt;
      d.tpart = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + ws_off);
      ws_off += job_tpart_bytes(s, M);
      rblocks += (int)(((int64_t)M * s.r / 4 + 255) / 256);
    }
    r_max = s.r > r_max ? s.r : r_max;
  }
  dim3 grid1(blocks), grid2(rblocks), block(256), block1(512);
  const int rt = (r_max + 15) / 16;
#define LAUNCH(TT, RT, WT) hipLaunchKernelGGL((lora_grad_partial_kernel<TT, RT, WT>), grid1, block1, 0, st, a)
#define DISPATCH(TT)                                                  \
  switch (rt) {                                                       \
    case 1: if (any_t) LAUNCH(TT, 1, true); else hipLaunchKernelGGL((lora_grad_partial_kernel<TT, 1, false>), grid1, block1, 0, st, a); break; \
    case 2: if (any_t) LAUNCH(TT, 2, true); else hipLaunchKernelGGL((lora_grad_partial_kernel<TT, 2, false>), grid1, block1, 0, st, a); break; \
    case 3: case 4: hipLaunchKernelGGL((lora_grad_partial_kernel<TT, 4, false>), grid1, block1, 0, st, a); break; \
    default: hipLaunchKernelGGL((lora_grad_partial_kernel<TT, 8, false>), grid1, block1, 0, st, a); break;         \
  }
  if (act_dtype == FMSA_BF16) {
    DISPATCH(bf16_t)
  } else {
    DISPATCH(f16_t)
  }
#undef DISPATCH
#undef LAUNCH
  FMSA_CHECK_LAUNCH();
  hipLaunchKernelGGL(lora_grad_reduce_kernel, grid2, block, 0, st, a);
  FMSA_CHECK_LAUNCH();
  return FMSA_OK;
}
