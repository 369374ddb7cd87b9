// Shared device helpers for the gfx950 kernels: vector types, MFMA wrappers, the GPTQ nibble
// unpack and the storage-type conversions.  Everything here is wave64 / CDNA4 specific.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/fmsa.h"

typedef __bf16 bf16_t;
typedef _Float16 f16_t;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define FMSA_DEVI __device__ __forceinline__

// Compile-time loop: the body receives std::integral_constant<int, I>, so register arrays indexed
// by the loop variable can never fall back to dynamic (scratch-memory) indexing.
template <int I, int N, typename F> FMSA_DEVI void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// ---- scalar conversions with a single round-to-nearest-even --------------------------------
FMSA_DEVI float fp16_bits_to_f32(uint16_t h) {
  union { uint16_t u; f16_t f; } c;
  c.u = h;
  return (float)c.f;
}
FMSA_DEVI float bf16_bits_to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

// Two fp32 -> packed storage type, RNE, low half = a.  Written as vector conversions so that the
// compiler selects v_cvt_pk_bf16_f32 / v_cvt_f16_f32 itself and can schedule around them.
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
template <typename T> FMSA_DEVI uint32_t pack2(float a, float b);
template <> FMSA_DEVI uint32_t pack2<bf16_t>(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){a, b}, bf16x2));
}
template <> FMSA_DEVI uint32_t pack2<f16_t>(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){a, b}, f16x2));
}
template <typename T> FMSA_DEVI uint16_t pack1(float a) { return (uint16_t)(pack2<T>(a, 0.f) & 0xffffu); }

template <typename T> FMSA_DEVI float unpack_lo(uint32_t v);
template <typename T> FMSA_DEVI float unpack_hi(uint32_t v);
template <> FMSA_DEVI float unpack_lo<bf16_t>(uint32_t v) { return __uint_as_float(v << 16); }
template <> FMSA_DEVI float unpack_hi<bf16_t>(uint32_t v) { return __uint_as_float(v & 0xffff0000u); }
template <> FMSA_DEVI float unpack_lo<f16_t>(uint32_t v) { return fp16_bits_to_f32((uint16_t)(v & 0xffffu)); }
template <> FMSA_DEVI float unpack_hi<f16_t>(uint32_t v) { return fp16_bits_to_f32((uint16_t)(v >> 16)); }
template <typename T> FMSA_DEVI float unpack1(uint16_t v) { return unpack_lo<T>((uint32_t)v); }

// byte j of x as fp32: the shift-and-mask form is what the compiler turns into v_cvt_f32_ubyte<j>
FMSA_DEVI float ubyte0(uint32_t x) { return (float)(x & 0xffu); }
FMSA_DEVI float ubyte1(uint32_t x) { return (float)((x >> 8) & 0xffu); }
FMSA_DEVI float ubyte2(uint32_t x) { return (float)((x >> 16) & 0xffu); }
FMSA_DEVI float ubyte3(uint32_t x) { return (float)(x >> 24); }
template <int B> FMSA_DEVI float ubyte_n(uint32_t x) {
  if constexpr (B == 0) return ubyte0(x);
  else if constexpr (B == 1) return ubyte1(x);
  else if constexpr (B == 2) return ubyte2(x);
  else return ubyte3(x);
}
// Stops the optimiser from narrowing the byte masks above back into nibble masks (which would
// cost a shift + and + convert per value instead of one convert).  Emits no instruction.
FMSA_DEVI uint32_t opaque(uint32_t x) {
  asm("" : "+v"(x));
  return x;
}

// ---- GPTQ: eight nibbles of one int32 -> eight storage-type values --------------------------
// value_j = RNE( sf * nib_j + nsz ) with nsz = -sf * (z + zero_offset).  sf is an fp16 scale
// widened to fp32 (11 significant bits) and nib, z are < 32, so sf*nib, nsz and their sum are
// all exact in fp32: the only rounding is the final conversion, as in
// UL/gptq/triton/kernels.py:118-122.  The odd nibbles are used in place (16 * nib in the high
// half of each byte) with the scale pre-divided by 16 -- a power of two, so still exact.
template <typename T> FMSA_DEVI u32x4 dequant8(uint32_t w, float sf, float sf16, float nsz) {
  const uint32_t lo = opaque(w & 0x0F0F0F0Fu);  // nibbles 0,2,4,6 in bytes 0..3
  const uint32_t hi = opaque(w & 0xF0F0F0F0u);  // 16 * nibbles 1,3,5,7
  u32x4 r;
  r[0] = pack2<T>(__builtin_fmaf(sf, ubyte0(lo), nsz), __builtin_fmaf(sf16, ubyte0(hi), nsz));
  r[1] = pack2<T>(__builtin_fmaf(sf, ubyte1(lo), nsz), __builtin_fmaf(sf16, ubyte1(hi), nsz));
  r[2] = pack2<T>(__builtin_fmaf(sf, ubyte2(lo), nsz), __builtin_fmaf(sf16, ubyte2(hi), nsz));
  r[3] = pack2<T>(__builtin_fmaf(sf, ubyte3(lo), nsz), __builtin_fmaf(sf16, ubyte3(hi), nsz));
  return r;
}

// ---- packed half arithmetic (fp16 only: v_pk_add_f16 / v_pk_mul_f16; fp32 packed forms stay switched off) ----------
// (1024 + q) - (1024 + z) is exact in fp16 and the product with the fp16 scale rounds once: RNE_fp16(s * (q - z)), the
// value of UL/gptq/triton/kernels.py:118-122 bit for bit, two weights per instruction.
FMSA_DEVI uint32_t pk_sub_mul_f16(uint32_t q_plus_1024, uint32_t neg_z_plus_1024, uint32_t scale) {
  const f16x2 a = __builtin_bit_cast(f16x2, q_plus_1024), b = __builtin_bit_cast(f16x2, neg_z_plus_1024);
  const f16x2 d = a + b;
  return __builtin_bit_cast(uint32_t, d * __builtin_bit_cast(f16x2, scale));
}

// ---- MFMA 32x32x16: D[i][j] += sum_k A[i][k] * B[k][j] ---------------------------------------
// Operand fragments are 8 consecutive contraction elements per lane: lane l supplies row
// (l & 31) of A / column (l & 31) of B at k = 8*(l >> 5) .. +7.  The accumulator register
// 4*i0 + i1 of lane l is D[8*i0 + 4*(l >> 5) + i1][l & 31].
template <typename T> FMSA_DEVI f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c);
template <> FMSA_DEVI f32x16 mfma32<bf16_t>(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
template <> FMSA_DEVI f32x16 mfma32<f16_t>(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}
// MFMA 16x16x32: lane l supplies row/column (l & 15) at k = 8*(l >> 4) .. +7; accumulator
// register i of lane l is D[4*(l >> 4) + i][l & 15].
template <typename T> FMSA_DEVI f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c);
template <> FMSA_DEVI f32x4 mfma16<bf16_t>(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
template <> FMSA_DEVI f32x4 mfma16<f16_t>(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// ---- buffer resources ----------------------------------------------------------------------------
// Raw buffer descriptor over [base, base + bytes): loads through it take a 32-bit per-lane offset
// plus a scalar offset, and a lane offset at or past `bytes` returns zero instead of faulting.
// The descriptor must live in scalar registers: base and size are wave-uniform by construction and
// readfirstlane states that to the compiler (otherwise every load is wrapped in a waterfall loop).
FMSA_DEVI __amdgpu_buffer_rsrc_t make_rsrc(const void* base, size_t bytes) {
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
  uint32_t n = bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : (uint32_t)bytes;
  n = __builtin_amdgcn_readfirstlane(n);
  void* ub = reinterpret_cast<void*>(((uint64_t)hi << 32) | lo);
  return __builtin_amdgcn_make_buffer_rsrc(ub, 0, (int)n, 0x00020000);
}

// Cache policy of the GEMM epilogues' output stores (the `aux` operand of the buffer-store builtins; bit 1 = nt on
// gfx94x / gfx950).  A launch writes up to 705 MB that nothing re-reads before the launch ends.  Written with the
// default policy the tail of it stays dirty in the memory-side cache, and the NEXT kernel pays for the write-back:
// every line it brings in evicts a dirty one, so a bandwidth-bound kernel right after the gate/up GEMM ran at half
// speed (86 us instead of 50 us for one pass over h).  Non-temporal stores drain to HBM while the GEMM, which is
// bound by the matrix pipe, still runs; the GEMM's own duration does not change.
constexpr int STORE_NT = 2;

// ---- workgroup-id remap: consecutive ids land on different XCDs (id % 8), each with its own
// L2.  Give every XCD a contiguous range of logical tiles so neighbours share operands in L2.
FMSA_DEVI int xcd_remap(int pid, int total) {
  const int NXCD = 8;
  if (total % NXCD != 0) return pid;
  return (pid % NXCD) * (total / NXCD) + pid / NXCD;
}

// SiLU pieces with the reference's rounding points (UL/swiglu.py:26-33, 65-83).
// 1 / (1 + 2^(-x log2 e)) with the hardware exp2 and reciprocal (1 ulp each): four instructions
// instead of the ~14 of an IEEE division; the result is rounded to the storage type right after.
FMSA_DEVI float sigmoidf_(float x) { return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504088896341f)); }

// Host-side launch helpers (api.hip)
#define FMSA_CHECK_LAUNCH()                                   \
  do {                                                        \
    if (hipGetLastError() != hipSuccess) return FMSA_ERR_LAUNCH; \
  } while (0)
