/*
 * fmsa.h -- C ABI of libfmsa_hip.so: hand-written gfx950 (MI355X) kernels for the fused
 * quantised-LoRA hot path of fms-acceleration (GPTQ 4-bit / bitsandbytes NF4 base weight,
 * LoRA adapters, SwiGLU MLP), forward and backward.
 *
 * Conventions
 *   - Every pointer that is not marked "host" is a DEVICE pointer (tensor.data_ptr()).
 *   - Every function returns FMSA_OK (0) or a negative FMSA_ERR_* code.  Nothing throws,
 *     nothing allocates, nothing synchronises: work is enqueued on `stream` (a hipStream_t
 *     passed as void*, e.g. torch.cuda.current_stream().cuda_stream; NULL = default stream).
 *   - Arguments are validated before any HIP call, so the error paths can be exercised on a
 *     machine without a GPU.
 *   - Activations / gradients are row-major 2-D with an explicit leading dimension in ELEMENTS.
 *     `act_dtype` is FMSA_BF16 or FMSA_F16 and selects both the storage type and the MFMA type.
 *
 * Each entry point cites the reference interface it replaces, relative to
 *   FOAK = plugins/fused-ops-and-kernels/src/fms_acceleration_foak
 *   UL   = FOAK/fused_ops/unsloth_lora
 *   GQ   = plugins/accelerated-peft/src/fms_acceleration_peft/gptqmodel
 */
#ifndef FMSA_H
#define FMSA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FMSA_OK 0
#define FMSA_ERR_NULL (-1)        /* a required pointer is NULL                      */
#define FMSA_ERR_SHAPE (-2)       /* a dimension is non-positive or violates a rule  */
#define FMSA_ERR_ALIGN (-3)       /* pointer / leading dimension not 16-byte aligned */
#define FMSA_ERR_DTYPE (-4)       /* unknown dtype enum                              */
#define FMSA_ERR_UNSUPPORTED (-5) /* valid input the kernels do not cover            */
#define FMSA_ERR_WORKSPACE (-6)   /* workspace missing or too small                  */
#define FMSA_ERR_LAUNCH (-7)      /* hipGetLastError() after the launch was not success */
#define FMSA_ERR_DEVICE (-8)      /* tensors on another GPU than the calling thread's current device */

enum fmsa_dtype { FMSA_F16 = 0, FMSA_BF16 = 1, FMSA_F32 = 2 };

/* Human-readable text for an error code (host pointer to a static string). */
const char* fmsa_strerror(int code);

/* ABI version; bumped on any change of a signature or struct layout (9 here).  A binding should refuse a library whose
 * version is not the one it was written for. */
int fmsa_abi_version(void);

/* ------------------------------------------------------------------------------------------
 * GPTQ 4-bit weight, laid out exactly as QuantLinear's buffers
 * (GQ/nn_modules/qlinear/qlinear_tritonv2.py:67-99; pack() :104-165):
 *   qweight int32 [K/8, N]  nibble j of word [k8, n]  = q[8*k8 + j, n]
 *   qzeros  int32 [G, N/8]  nibble j of word [g, n8]  = z[g, 8*n8 + j]
 *   scales  fp16  [G, N]
 *   g_idx   int32 [K]       group of row k; NULL means k / group_size
 * W[k, n] = fp32(scales[g, n]) * (q[k, n] - (z[g, n] + zero_offset)),  g = g_idx[k]
 * zero_offset is 1 for checkpoints in the AutoGPTQ v1 zero-point format and 0 otherwise
 * (UL/gptq/fast_lora.py:100-101, UL/gptq/triton/kernels.py:113-116).
 *
 * format FMSA_WEIGHT_CODEBOOK describes a 4-bit code-book weight in the same word layout, which is
 * what fmsa_nf4_prepare makes of a bitsandbytes NF4 tensor so that the fused kernels below can
 * read it: nibble j of qweight[k8, n] indexes `code` (16 fp32 entries) and
 *   W[k, n] = code[q[k, n]] * block_scale[k / group_size, n]      (fp32 product, one rounding)
 * with block_scale fp32 [K / group_size, N]; scales, qzeros, g_idx and zero_offset are unused.
 * ------------------------------------------------------------------------------------------ */
enum fmsa_weight_format { FMSA_WEIGHT_AFFINE = 0, FMSA_WEIGHT_CODEBOOK = 1 };

typedef struct fmsa_gptq_weight {
  const int32_t* qweight;
  const uint16_t* scales;
  const int32_t* qzeros;
  const int32_t* g_idx;
  int32_t K;          /* in-features,  K % 32 == 0  (qlinear_tritonv2.py:57-60) */
  int32_t N;          /* out-features, N % 32 == 0                               */
  int32_t group_size; /* > 0; G = ceil(K / group_size)                           */
  int32_t zero_offset;
  int32_t format;     /* enum fmsa_weight_format                                  */
  int32_t nibble_order; /* 0: the checkpoint's (nibble j = row 8*k8 + j).  1: interleaved, element 2p at nibble position
                         * p and element 2p + 1 at position 4 + p (see fmsa_gptq_interleave): accepted by fmsa_gptq_lora_fwd
                         * only, for the affine format with FMSA_F16 activations and group_size % 64 == 0 */
  const float* code;        /* CODEBOOK: 16 entries                               */
  const float* block_scale; /* CODEBOOK: [K / group_size, N]                      */
} fmsa_gptq_weight;

/* One-time re-ordering of the nibbles inside every word of qweight int32 [K/8, N] for the forward kernel's packed-half
 * unpack (FMSA_F16 activations): out word [k8, n] holds q[8*k8 + e, n] with element 2p at nibble position p and element
 * 2p + 1 at position 4 + p, so that (w >> 4p) & 0x000F000F is the pair (k, k+1) of MFMA fragment register p.  Hand the
 * result to fmsa_gptq_lora_fwd as `qweight` with nibble_order = 1; everything else of the weight is unchanged. */
int fmsa_gptq_interleave(const int32_t* qweight, int K, int N, int32_t* qweight_out, void* stream);

/* Replaces dequant248 (UL/gptq/triton/kernels.py:125-153): materialises W[K, N] row-major in
 * `out_dtype` (FMSA_F16 = the reference's output type, FMSA_BF16, FMSA_F32) with one
 * round-to-nearest-even of the exact fp32 product.  Handles any g_idx (act-order). */
int fmsa_gptq_dequant(const fmsa_gptq_weight* w /*host*/, int out_dtype, void* out, void* stream);

/* One-time repack for act-order checkpoints: rows of q are gathered so that
 * q_sorted[k', :] = q[perm[k'], :], giving a weight whose group index is k' / group_size.
 * perm int32 [K] (device) is argsort(g_idx, stable).  qweight_out int32 [K/8, N]. */
int fmsa_gptq_permute_rows(const int32_t* qweight, const int32_t* perm, int K, int N,
                           int32_t* qweight_out, void* stream);

/* out[m, j] = in[m, perm[j]] (gather == 1) or out[m, perm[j]] = in[m, j] (gather == 0);
 * used to carry activations into / out of the row order of a repacked act-order weight. */
int fmsa_permute_cols(const void* in, int64_t ld_in, const int32_t* perm, int M, int C, int gather,
                      int act_dtype, void* out, int64_t ld_out, void* stream);

/* ------------------------------------------------------------------------------------------
 * Skinny LoRA GEMMs.
 * ------------------------------------------------------------------------------------------ */

/* out[M, r] (row stride ldout >= r) = X[M, C] * Wd[r, C]^T, fp32 accumulate, one rounding to act_dtype.
 * Covers `X @ A.t()` of matmul_lora (UL/gptq/fast_lora.py:166-167) with Wd = lora_A.weight
 * [r, K], and `dY @ B` of the backward (:822) with Wd = lora_B.weight^T [r, N].
 * r % 8 == 0, r <= 128, C % 8 == 0.  Adapters that share X can be stacked: Wd = [A_q; A_k; A_v]
 * gives their U's side by side in one pass over X, and ldout lets several calls write side by side
 * into one [M, sum r] buffer. */
int fmsa_lora_down(const void* X, int64_t ldx, const void* Wd, int M, int C, int r, int act_dtype,
                   void* out, int64_t ldout, void* stream);

/* The same product with a partial-sum buffer at hand (same reference lines as fmsa_lora_down).  A workgroup takes
 * 64-128 tokens, so that Wd is re-read that much less often, and where M then leaves CUs without work
 * the columns are split over workgroups whose fp32 sums meet in `workspace` ([splits][M][r] fp32, no initialisation
 * needed, added in index order: the result does not depend on scheduling).  fmsa_lora_down_workspace gives the bytes
 * (0: the call needs none); with a buffer that is missing, too small, or an `out` that is not 8-byte aligned with
 * ldout % 4 == 0, the call runs as fmsa_lora_down does.  Calls that may overlap in time need separate workspaces. */
size_t fmsa_lora_down_workspace(int M, int C, int r);
int fmsa_lora_down_ws(const void* X, int64_t ldx, const void* Wd, int M, int C, int r, int act_dtype,
                      void* out, int64_t ldout, void* workspace, size_t workspace_bytes, void* stream);

/* out = scale * L[M, r]^T * R[M, C]   (a reduction over the M tokens; L has row stride ldl >= r), written as
 *   [r, C] when transpose_out == 0   (dA = s * (dY B)^T Xd,  UL/gptq/fast_lora.py:822,824,842)
 *   [C, r] when transpose_out == 1   (dB = s * dY^T (Xd A^T), :823,825,843)
 * Deterministic two-pass reduction: partial sums over fixed M-chunks go to `workspace`
 * (fp32, fmsa_lora_grad_workspace() bytes) and are summed in a fixed order.
 * out_dtype: FMSA_F32, FMSA_BF16 or FMSA_F16. */
size_t fmsa_lora_grad_workspace(int M, int C, int r);
int fmsa_lora_grad(const void* L, int64_t ldl, const void* R, int64_t ldr, int M, int C, int r, float scale,
                   int transpose_out, int act_dtype, int out_dtype, void* out, void* workspace,
                   size_t workspace_bytes, void* stream);

/* Several such gradients over the same M tokens in one launch of each pass: the adapter gradients
 * one backward produces (dA of the stacked adapters and every dB, :822-825 for each projection of
 * LoRA_QKV :657-674 / LoRA_MLP :351-398) are each too small to fill the chip alone.  Job q is
 * exactly fmsa_lora_grad with its fields; results are bit-identical to separate calls.  All jobs
 * share M and act_dtype; 1 <= n_jobs <= FMSA_LORA_GRAD_MAX_JOBS; `workspace` holds
 * fmsa_lora_grad_batch_workspace() bytes (the jobs' partial sums side by side). */
#define FMSA_LORA_GRAD_MAX_JOBS 8
typedef struct fmsa_lora_grad_job {
  const void* L; /* [M, r], row stride ldl */
  const void* R; /* [M, C], row stride ldr */
  void* out;     /* [r, C], or [C, r] when transpose_out */
  int64_t ldl, ldr;
  int32_t C, r;
  float scale;
  int32_t transpose_out;
  int32_t out_dtype; /* FMSA_F32, FMSA_BF16 or FMSA_F16 */
  int32_t reserved;
  /* Optional second product of the same pass over R:  T[M, r] = R * Wt^T  in act_dtype, row stride ldt
   * (what fmsa_lora_down(R, Wt) gives, up to the order of the fp32 sums).  A backward needs both
   * dB = s * dY^T U (this job: L = U, R = dY) and T = dY B (Wt = lora_B.weight^T [r, C]),
   * UL/gptq/fast_lora.py:822-823, and reading dY is the whole cost of either.  Wt == NULL: no T.
   * With Wt set every job of the call needs r <= 32; T 8-byte aligned, ldt % 4 == 0.  Worth it when the pass
   * over R it saves (2 * M * C bytes) outweighs the second launch the dependent dA then needs. */
  const void* Wt;
  void* T;
  int64_t ldt;
} fmsa_lora_grad_job;
size_t fmsa_lora_grad_batch_workspace(const fmsa_lora_grad_job* jobs, int n_jobs, int M);
int fmsa_lora_grad_batch(const fmsa_lora_grad_job* jobs, int n_jobs, int M, int act_dtype, void* workspace,
                         size_t workspace_bytes, void* stream);

/* fmsa_lora_grad for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc); it has no counterpart in the reference.  Same arguments, same two
 * kernels and bit-identical results, but the partial sums live in a buffer of FMSA_LORA_GRAD_STATIC_BYTES that
 * is part of the library's device image (each GPU the library is used on holds its own copy until the process
 * ends), and the call itself makes no hipMalloc / hipFree or any other allocating call.  Returns
 * FMSA_ERR_WORKSPACE when fmsa_lora_grad_workspace(M, C, r) exceeds that size (16 MiB covers 8192 tokens x
 * 14336 columns at rank 16, or 4096 columns at rank 64).  All calls on one GPU share the buffer: calls that
 * overlap in time on one GPU (two streams, two threads) race on it; calls on one stream are ordered.  The very
 * first call on a device looks up the buffer's address (not an allocation); make that call outside a capture.
 * The buffer used is the copy of the calling thread's CURRENT device (hipGetDevice), which must be the GPU that
 * owns L, R, out and the stream: an `out` the runtime places on another GPU returns FMSA_ERR_DEVICE. */
#define FMSA_LORA_GRAD_STATIC_BYTES (16u << 20)
int fmsa_lora_grad_static(const void* L, int64_t ldl, const void* R, int64_t ldr, int M, int C, int r, float scale,
                          int transpose_out, int act_dtype, int out_dtype, void* out, void* stream);

/* The four activation-type copies of one adapter that the kernels above and below read, in one
 * launch: A16 [r, K], At16 [K, r] from A = lora_A.weight [r, K]; B16 [N, r], Bt16 [r, N] from
 * B = lora_B.weight [N, r].  Each value is the parameter rounded once (RNE) to act_dtype -- the
 * `A.to(dtype)`, `B.to(dtype)` of matmul_lora (UL/gptq/fast_lora.py:167) plus the transposes its
 * backward takes (:822-831).  param_dtype: FMSA_F32, FMSA_BF16 or FMSA_F16.  Outputs may be NULL. */
int fmsa_lora_pack(const void* A, const void* B, int r, int K, int N, int param_dtype, int act_dtype,
                   void* A16, void* At16, void* B16, void* Bt16, void* stream);

/* The same for up to FMSA_LORA_PACK_MAX_JOBS adapters in one launch (q, k, v; gate, up, down): job q is
 * fmsa_lora_pack with its fields. */
#define FMSA_LORA_PACK_MAX_JOBS 4
typedef struct fmsa_lora_pack_job {
  const void* A; /* lora_A.weight [r, K] */
  const void* B; /* lora_B.weight [N, r] */
  void* A16;     /* [r, K]   (each output may be NULL) */
  void* At16;    /* [K, r] */
  void* B16;     /* [N, r] */
  void* Bt16;    /* [r, N] */
  int32_t r, K, N;
  int32_t param_dtype; /* FMSA_F32, FMSA_BF16 or FMSA_F16 */
} fmsa_lora_pack_job;
int fmsa_lora_pack_batch(const fmsa_lora_pack_job* jobs, int n_jobs, int act_dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Fused forward:  Y_p = X * deq(W_p) + s_p * U_p * B_p^T (+ bias_p)   for 1..3 projections
 * sharing X (LoRA_W / LoRA_QKV forward, UL/gptq/fast_lora.py:770-805, 497-589), or the
 * gate/up pair of LoRA_MLP with the SwiGLU of UL/swiglu.py:20-37 fused into the epilogue
 * (UL/gptq/fast_lora.py:252-262): mode FMSA_FWD_SWIGLU writes e = Y_0, g = Y_1 and
 * h = silu(e) * g.
 * ------------------------------------------------------------------------------------------ */
typedef struct fmsa_fwd_proj {
  fmsa_gptq_weight w;
  const void* U;    /* [M, r] act_dtype = Xd * A^T (fmsa_lora_down); NULL when r == 0 */
  int64_t ldu;      /* row stride of U, >= r, % 8 == 0                                 */
  const void* B;    /* [N, r] act_dtype = lora_B.weight                               */
  const void* bias; /* [N] act_dtype or NULL                                           */
  void* Y;          /* [M, N] act_dtype                                                */
  int64_t ldy;
  int32_t r;        /* 0 = adapters disabled (base only); else r % 8 == 0, r <= 128    */
  float s;          /* lora_alpha / r                                                  */
} fmsa_fwd_proj;

enum fmsa_fwd_mode { FMSA_FWD_LINEAR = 0, FMSA_FWD_SWIGLU = 1 };

int fmsa_gptq_lora_fwd(const fmsa_fwd_proj* projs /*host*/, int n_proj, const void* X, int64_t ldx,
                       int M, int mode, void* H, int64_t ldh, int act_dtype, void* stream);

/* The same forward (FMSA_FWD_LINEAR) with the rotary position embedding of the attention block applied in the
 * epilogue of the projections named by `proj_mask` (bit p = projection p; q and k of LoRA_QKV): replaces the
 * separate in-place pass of kernels/unsloth/rope_embedding.py:36-65, 68-103 over Q and K,
 *   (y1, y2) <- (y1 cos - y2 sin, y2 cos + y1 sin)   on the two halves of every head,
 * applied to the projection output rounded to act_dtype (what that pass reads), fp32 arithmetic, one rounding.
 * cos / sin: [rows, ld] with head_dim / 2 meaningful values per row (the first half of each row of the
 * [positions, head_dim] tables transformers passes); token row m takes table row m % rows (rope_embedding.py:60-63
 * with rows = seq_len; a [batch * seq, .] table is used row by row).  dtype: act_dtype or FMSA_F32.
 * head_dim % 16 == 0, 256 % head_dim == 0, N_p % head_dim == 0 for the rotated projections; every group_size
 * % 64 == 0 and K % 64 == 0.  The backward takes dQ, dK through fmsa_rope_embedding(backward = 1) first. */
typedef struct fmsa_rope {
  const void* cos;
  const void* sin;
  int64_t ld;        /* row stride in elements, >= head_dim / 2; % 8 == 0 (16-bit) or % 4 == 0 (fp32) */
  int32_t rows;      /* > 0 */
  int32_t head_dim;
  int32_t dtype;     /* act_dtype or FMSA_F32 */
  int32_t proj_mask; /* bit p set: projection p leaves rotated */
} fmsa_rope;
int fmsa_gptq_lora_fwd_rope(const fmsa_fwd_proj* projs /*host*/, int n_proj, const void* X, int64_t ldx, int M,
                            const fmsa_rope* rope /*host*/, int act_dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Fused input-gradient:
 *   dX = sum_p [ dY_p * deq(W_p)^T + mask_p (.) ( T_p * (s_p A_p) ) ],  T_p = dY_p * B_p
 * (one mask for the whole call) for 1..3 projections sharing the input (LoRA_W / LoRA_QKV / the gate+up half of LoRA_MLP
 * backward, UL/gptq/fast_lora.py:828-831, 657-674, 388-398).  mask_p = (mask_src_p != 0)
 * element-wise over [M, K] (the post-dropout input; NULL = no mask).
 * Mode FMSA_BWD_SWIGLU is the down-projection half of LoRA_MLP backward (:351-366): the result
 * is dh, and the epilogue applies UL/swiglu.py:50-89 in place: reads e, g; writes h -> `h_out`,
 * d_g = dh*f -> `e`, d_e -> `g`.  dX is not written in that mode.
 * ------------------------------------------------------------------------------------------ */
typedef struct fmsa_bwd_proj {
  fmsa_gptq_weight w;
  const float* nsz;  /* [G, N] fp32 = -scale * (zero + zero_offset), from fmsa_gptq_make_nsz */
  const void* dY;    /* [M, N] act_dtype */
  int64_t lddy;
  const void* T;     /* [M, r] act_dtype = dY * B; NULL when r == 0 */
  int64_t ldt;       /* row stride of T, >= r, % 8 == 0 */
  const void* At;    /* [K, r] act_dtype = lora_A.weight^T (contiguous) */
  const void* mask_src; /* [M, K] act_dtype or NULL; every non-NULL entry of one call must be the same */
  int64_t ldmask;
  int32_t r;
  float s;
  /* Optional per-weight twin for this kernel, built once (the base weight is frozen): the nibbles packed along N,
   * qweight_t int32 [N/8, K] from fmsa_gptq_transpose, and for the affine format the scales widened to fp32,
   * scale_f32 [G, N].  When every projection of a call carries them (and every group_size % 64 == 0) the kernel
   * reads the twin: a lane's word is then its MFMA fragment, as in the forward kernel, instead of an 8 x 8 block of
   * nibbles that has to be transposed with byte shuffles.  Same values, same contraction order: bit-identical
   * results.  NULL: the checkpoint layout in `w` is read.
   * negzp_f16 (affine format, FMSA_F16 activations only; optional): fp16 [G, N] = -(1024 + z + zero_offset), exact in
   * fp16.  With it the twin is unpacked in packed half arithmetic, (1024 + q) - (1024 + z) exactly and one rounding in
   * the product with the fp16 scale, i.e. RNE_fp16(scale * (q - z)) bit for bit at two thirds of the instructions;
   * scale_f32 and nsz may then be NULL. */
  const int32_t* qweight_t;
  const float* scale_f32;
  const void* negzp_f16;
} fmsa_bwd_proj;

enum fmsa_bwd_mode { FMSA_BWD_LINEAR = 0, FMSA_BWD_SWIGLU = 1 };

/* Per-weight table read by the input-gradient kernel: out[g, n] = -fp32(scales[g, n]) *
 * (z[g, n] + zero_offset), fp32 [G, N] (exact: 11-bit x 5-bit).  The base weight is frozen, so a
 * caller builds it once per weight. */
int fmsa_gptq_make_nsz(const fmsa_gptq_weight* w /*host*/, float* out, void* stream);

/* The transposed twin of a packed weight for fmsa_bwd_proj.qweight_t: out int32 [N/8, K] from qweight int32 [K/8, N]
 * (pack() of qlinear_tritonv2.py:132-147 packs along K).  Word [n8, k] holds q[k, 8*n8 + e] for e = 0..7 with the even
 * elements in its low half and the odd ones in its high half: element 2p at nibble position p, element 2p + 1 at
 * position 4 + p (a layout private to the kernel: (w >> 4p) & 0x000F000F is the pair of fragment register p).
 * For an act-order weight pass the row-repacked qweight (fmsa_gptq_permute_rows).  K % 8 == 0, N % 8 == 0. */
int fmsa_gptq_transpose(const int32_t* qweight, int K, int N, int32_t* qweight_t_out, void* stream);

int fmsa_gptq_lora_bwd_dx(const fmsa_bwd_proj* projs /*host*/, int n_proj, int M, int mode,
                          void* dX, int64_t lddx, void* e, void* g, void* h_out, int64_t ldeg,
                          int act_dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Standalone SwiGLU (UL/swiglu.py:20-47 and :50-98) for the paths whose GEMM epilogue cannot
 * fuse it.  e, g, h share the leading dimension ld; I % 8 == 0.
 *   fwd: h = RNE(silu_f32(e)) * g
 *   bwd: in place, h_out <- f*g, e <- d_g = dh*f, g <- d_e = RNE(f32(dh*g) * s(e) * (1 + e(1 - s(e))))
 * ------------------------------------------------------------------------------------------ */
int fmsa_swiglu_fwd(const void* e, const void* g, void* h, int M, int I, int64_t ld, int act_dtype,
                    void* stream);
int fmsa_swiglu_bwd(const void* dh, int64_t lddh, void* e, void* g, void* h_out, int M, int I,
                    int64_t ld, int act_dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * bitsandbytes NF4 weight with double-quantised absmax, as fast_dequantize reads it from a
 * quant_state (UL/utils.py:86-141): weight [N, K] row-major, flattened, `blocksize` weights per
 * absmax, two 4-bit codes per byte with the EVEN element in the high nibble.
 *   absmax[b] = code2[absmax_q[b]] * absmax2[b / blocksize2] + offset        (fp32)
 *   W[i]      = code[nibble(i)] * absmax[i / blocksize]                      (fp32, one RNE to out)
 * fmsa_nf4_dequant replaces cdequantize_blockwise_fp32 + cdequantize_blockwise_{fp16,bf16,fp32}_nf4
 * (:119-136) in one pass; out is [N, K] row-major (the reference returns its transpose as a view).
 * blocksize % 16 == 0, N*K % blocksize == 0.
 * ------------------------------------------------------------------------------------------ */
typedef struct fmsa_nf4_weight {
  const uint8_t* packed;   /* [N*K/2]                                  quant_state weight   */
  const uint8_t* absmax_q; /* [N*K/blocksize]                          quant_state.absmax   */
  const float* absmax2;    /* [ceil(N*K/blocksize/blocksize2)]         state2.absmax        */
  const float* code2;      /* [256]                                    state2.code          */
  const float* code;       /* [16] NF4 code book                       quant_state.code     */
  float offset;            /*                                          quant_state.offset   */
  int32_t N, K, blocksize, blocksize2;
} fmsa_nf4_weight;

int fmsa_nf4_dequant(const fmsa_nf4_weight* w /*host*/, int out_dtype, void* out, void* stream);

/* One-time re-layout of an NF4 weight for the fused kernels (the base weight is frozen): the codes
 * of W[n, k] move into the word layout of fmsa_gptq_weight (qweight_out int32 [K/8, N], nibble j of
 * word [k8, n] = code index of W[n, 8*k8 + j]) and the double-quantised absmax is expanded to
 * block_scale_out fp32 [K / blocksize, N] with the arithmetic of fmsa_nf4_dequant, so that
 * code[q] * block_scale reproduces its values bit for bit.  K % blocksize == 0, blocksize % 8 == 0,
 * K % 8 == 0.  No counterpart in the reference, which always materialises the dense weight
 * (UL/utils.py:250-283). */
int fmsa_nf4_prepare(const fmsa_nf4_weight* w /*host*/, int32_t* qweight_out, float* block_scale_out, void* stream);

/* ------------------------------------------------------------------------------------------
 * The two bandwidth-bound operators next to the q/k/v projections.  x_dtype / w_dtype / q_dtype /
 * cs_dtype: FMSA_F16, FMSA_BF16 or FMSA_F32; rows 16-byte aligned, C % 8 == 0, head_dim % 16 == 0.
 *
 * RMS layer norm (kernels/unsloth/rms_layernorm.py:21-47, 99-109 forward; :50-86 backward):
 *   fwd: r[m] = rsqrt(mean(x^2) + eps); Y = round_w(x * r) * W, in w_dtype arithmetic, stored in
 *        x_dtype.  gemma != 0: fp32 throughout, r = 1 / sqrt(.), weight W + 1.
 *   bwd: dX = r/C * (C * dY_W - (x r) * sum(dY_W * x r)), dY_W = dY * W (gemma: W + 1), fp32,
 *        written over dY (the weight is frozen: no dW, as in the reference).
 * Rotary embedding (kernels/unsloth/rope_embedding.py:22-65), in place on Q [M, n_heads*head_dim]:
 *   (q1, q2) <- (q1 cos - q2 sin, q2 cos + q1 sin) on the halves of every head; row m uses row
 *   m % cs_rows of cos / sin [cs_rows, >= head_dim/2]; backward != 0 negates sin.
 * ------------------------------------------------------------------------------------------ */
int fmsa_rms_layernorm_fwd(const void* X, int64_t ldx, const void* W, int M, int C, float eps, int gemma,
                           int x_dtype, int w_dtype, void* Y, int64_t ldy, float* r, void* stream);
int fmsa_rms_layernorm_bwd(void* dY, int64_t lddy, const void* X, int64_t ldx, const void* W, const float* r,
                           int M, int C, int gemma, int x_dtype, int w_dtype, void* stream);
int fmsa_rope_embedding(void* Q, int64_t ldq, const void* cos, const void* sin, int64_t ldcs, int M,
                        int n_heads, int head_dim, int cs_rows, int backward, int q_dtype, int cs_dtype,
                        void* stream);

/* ------------------------------------------------------------------------------------------
 * Cross entropy over the vocabulary (kernels/unsloth/cross_entropy_loss.py:22-73 forward,
 * :138-190 backward; any vocabulary size in one pass, so the reference's chunked variant :76-135 has
 * no separate counterpart).  logits [M, V] of dtype F32 / BF16 / F16, labels int64 [M], -100 = ignore.
 *   fwd: logsumexp[m] = log sum_v exp(x[m, v]);  losses[m] = logsumexp[m] - x[m, label] (0 if ignored)
 *   bwd: in place, logits[m, v] <- dloss[m] * (exp(x[m, v] - logsumexp[m]) - [v == label]);
 *        dloss is read with stride dloss_stride (0 for the expanded scalar of a mean reduction).
 * 16-byte vector accesses when V % 8 == 0 and rows are 16-byte aligned, element accesses otherwise.
 * ------------------------------------------------------------------------------------------ */
int fmsa_cross_entropy_fwd(const void* logits, int64_t ld, const int64_t* labels, int M, int V, int dtype,
                           float* losses, float* logsumexp, void* stream);
int fmsa_cross_entropy_bwd(void* logits, int64_t ld, const float* dloss, int64_t dloss_stride,
                           const float* logsumexp, const int64_t* labels, int M, int V, int dtype,
                           void* stream);

/* ------------------------------------------------------------------------------------------
 * Loss and logits gradient in one launch, for a loss head that consumes its logits chunk by chunk
 * (fused_ops/liger_ce/cross_entropy.py:33-186, called from
 * fused_ops/liger_ce/fused_linear_cross_entropy_loss.py:107-121).  In place on logits [M, V]:
 *   losses[m]   = scale * ((1 - ls) (lse - x[m, label]) + ls * lse - (ls / V) sum_v x[m, v])
 *   logits[m,v] <- scale * (softmax(x[m])[v] - ls / V - [v == label] (1 - ls))
 * with ls = label_smoothing in [0, 1]; rows whose label equals ignore_index (or lies outside [0, V))
 * get loss 0 and a zero gradient row.  `scale` points at ONE fp32 in device memory (1 / number of
 * valid labels for a mean reduction) or is NULL for 1.
 * ------------------------------------------------------------------------------------------ */
int fmsa_cross_entropy_fused(void* logits, int64_t ld, const int64_t* labels, int M, int V, int dtype,
                             int64_t ignore_index, const float* scale, float label_smoothing, float* losses,
                             void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FMSA_H */
