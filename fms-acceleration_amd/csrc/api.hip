// extern "C" entry points: argument validation (no HIP call before it passes) and dispatch to
// the launchers in the kernel translation units.
#include "common.h"

#include <atomic>

int launch_gptq_dequant(const fmsa_gptq_weight* w, int out_dtype, void* out, hipStream_t st);
int launch_gptq_permute_rows(const int32_t* qweight, const int32_t* perm, int K, int N, int32_t* out, hipStream_t st);
int launch_permute_cols(const void* in, int64_t ld_in, const int32_t* perm, int M, int C, int gather, void* out,
                        int64_t ld_out, hipStream_t st);
int launch_lora_down(const void* X, int64_t ldx, const void* Wd, int M, int C, int r, int act_dtype, void* out, int64_t ldo,
                     hipStream_t st);
int lora_grad_splits(int M, int C);
size_t lora_grad_batch_workspace(const fmsa_lora_grad_job* jobs, int n_jobs, int M);
size_t lora_down_workspace(int M, int C, int r);
int launch_lora_down_ws(const void* X, int64_t ldx, const void* Wd, int M, int C, int r, int act_dtype, void* out, int64_t ldo,
                        void* workspace, size_t workspace_bytes, hipStream_t st);
int launch_lora_grad_batch(const fmsa_lora_grad_job* jobs, int n_jobs, int M, int act_dtype, void* workspace, hipStream_t st);
int launch_gptq_lora_fwd(const fmsa_fwd_proj* projs, int n_proj, const void* X, int64_t ldx, int M, int mode, void* H,
                         int64_t ldh, const fmsa_rope* rope, int act_dtype, hipStream_t st);
int launch_gptq_lora_bwd_dx(const fmsa_bwd_proj* projs, int n_proj, int M, int mode, void* dX, int64_t lddx, void* e,
                            void* g, void* h_out, int64_t ldeg, int act_dtype, hipStream_t st);

int launch_gptq_lora_bwd_dx_t(const fmsa_bwd_proj* projs, int n_proj, int M, int mode, void* dX, int64_t lddx, void* e,
                              void* g, void* h_out, int64_t ldeg, int act_dtype, hipStream_t st);
int bwd_dx_twin_flavour(const fmsa_bwd_proj* projs, int n_proj, int act_dtype);
int launch_gptq_transpose(const int32_t* qweight, int K, int N, int32_t* out, hipStream_t st);
int launch_gptq_interleave(const int32_t* qweight, int K, int N, int32_t* out, hipStream_t st);
int launch_gptq_nsz(const fmsa_gptq_weight* w, float* out, hipStream_t st);
int launch_lora_pack_batch(const fmsa_lora_pack_job* jobs, int n_jobs, int act_dtype, hipStream_t st);
int launch_rms_fwd(const void* X, int64_t ldx, const void* W, int M, int C, float eps, int gemma, int x_dtype, int w_dtype, void* Y,
                   int64_t ldy, float* r, hipStream_t st);
int launch_rms_bwd(void* dY, int64_t lddy, const void* X, int64_t ldx, const void* W, const float* r, int M, int C, int gemma,
                   int x_dtype, int w_dtype, hipStream_t st);
int launch_rope(void* Q, int64_t ldq, const void* cosp, const void* sinp, int64_t ldcs, int M, int n_heads, int head_dim, int cs_rows,
                int backward, int q_dtype, int cs_dtype, hipStream_t st);
int launch_ce_fwd(const void* logits, int64_t ld, const int64_t* labels, int M, int V, int dtype, int vec, float* losses, float* lse,
                  hipStream_t st);
int launch_ce_bwd(void* logits, int64_t ld, const float* dloss, int64_t dloss_stride, const float* lse, const int64_t* labels, int M,
                  int V, int dtype, int vec, hipStream_t st);
int launch_ce_fused(void* logits, int64_t ld, const int64_t* labels, int M, int V, int dtype, int vec, int64_t ignore_index,
                    const float* scale, float smoothing, float* losses, hipStream_t st);
int launch_nf4_dequant(const fmsa_nf4_weight* w, int out_dtype, void* out, hipStream_t st);
int launch_nf4_prepare(const fmsa_nf4_weight* w, int32_t* qweight_out, float* block_scale_out, hipStream_t st);
int launch_swiglu_fwd(const void* e, const void* g, void* h, int M, int I, int64_t ld, int act_dtype, hipStream_t st);
int launch_swiglu_bwd(const void* dh, int64_t lddh, void* e, void* g, void* h, int M, int I, int64_t ld, int act_dtype,
                      hipStream_t st);


namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool is_act(int d) { return d == FMSA_BF16 || d == FMSA_F16; }

int check_weight(const fmsa_gptq_weight* w, int group_multiple, bool interleaved_ok = false) {
  if (w->format != FMSA_WEIGHT_AFFINE && w->format != FMSA_WEIGHT_CODEBOOK) return FMSA_ERR_SHAPE;
  if (w->nibble_order != 0 && w->nibble_order != 1) return FMSA_ERR_SHAPE;
  if (w->nibble_order == 1 && (!interleaved_ok || w->format != FMSA_WEIGHT_AFFINE || w->group_size % 64 != 0)) return FMSA_ERR_UNSUPPORTED;
  if (!w->qweight) return FMSA_ERR_NULL;
  if (w->K <= 0 || w->N <= 0 || w->group_size <= 0) return FMSA_ERR_SHAPE;
  if (w->K % 32 != 0 || w->N % 32 != 0) return FMSA_ERR_SHAPE;  // qlinear_tritonv2.py:57-60
  if (w->format == FMSA_WEIGHT_CODEBOOK) {
    if (!w->code || !w->block_scale) return FMSA_ERR_NULL;
    if (w->K % w->group_size != 0) return FMSA_ERR_SHAPE;
    if (w->g_idx) return FMSA_ERR_UNSUPPORTED;
    if (!aligned16(w->qweight) || !aligned16(w->block_scale)) return FMSA_ERR_ALIGN;
  } else {
    if (!w->scales || !w->qzeros) return FMSA_ERR_NULL;
    if (w->zero_offset != 0 && w->zero_offset != 1) return FMSA_ERR_SHAPE;
    if (!aligned16(w->qweight) || !aligned16(w->scales) || !aligned16(w->qzeros)) return FMSA_ERR_ALIGN;
  }
  if (group_multiple > 0) {
    // The fused kernels assume the group of row k is k / group_size: act-order weights must be
    // repacked with fmsa_gptq_permute_rows first.  The forward needs one group per 16-wide MFMA
    // K step (group_size % 16 == 0); the input-gradient kernel one group per packed qweight row
    // (group_size % 8 == 0).
    if (w->g_idx) return FMSA_ERR_UNSUPPORTED;
    if (w->group_size % group_multiple != 0) return FMSA_ERR_UNSUPPORTED;
  }
  return FMSA_OK;
}

int check_rank(int r) {
  if (r < 0) return FMSA_ERR_SHAPE;
  if (r % 8 != 0 || r > 128) return FMSA_ERR_UNSUPPORTED;
  return FMSA_OK;
}

// Partial sums of fmsa_lora_grad_static: device memory that belongs to the library's code object, so the
// entry point never allocates.  Every GPU the library runs on holds its own copy at its own address; the
// name below is only a host-side handle (not a device address), so the address is looked up once per device
// with that device current, and only that pointer is ever handed to a kernel.
static __device__ __align__(256) unsigned char scratch[FMSA_LORA_GRAD_STATIC_BYTES];
constexpr int kMaxDevices = 64;
std::atomic<void*> scratch_ptr[kMaxDevices];

// Address of the current device's copy of `scratch` (nullptr on failure).  Racing first calls look up the
// same address twice, which is harmless.
void* scratch_of_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void* p = scratch_ptr[dev].load(std::memory_order_acquire);
  if (p) return p;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
  scratch_ptr[dev].store(p, std::memory_order_release);
  return p;
}

}  // namespace

extern "C" {

const char* fmsa_strerror(int code) {
  switch (code) {
    case FMSA_OK: return "ok";
    case FMSA_ERR_NULL: return "a required pointer is NULL";
    case FMSA_ERR_SHAPE: return "invalid dimension";
    case FMSA_ERR_ALIGN: return "pointer or leading dimension is not 16-byte aligned";
    case FMSA_ERR_DTYPE: return "unknown dtype";
    case FMSA_ERR_UNSUPPORTED: return "configuration not covered by the gfx950 kernels";
    case FMSA_ERR_WORKSPACE: return "workspace missing or too small";
    case FMSA_ERR_LAUNCH: return "kernel launch failed";
    case FMSA_ERR_DEVICE: return "tensors live on another GPU than the calling thread's current device";
    default: return "unknown error";
  }
}

int fmsa_abi_version(void) { return 9; }

int fmsa_gptq_dequant(const fmsa_gptq_weight* w, int out_dtype, void* out, void* stream) {
  if (!w || !out) return FMSA_ERR_NULL;
  if (int rc = check_weight(w, 0)) return rc;
  if (out_dtype != FMSA_F16 && out_dtype != FMSA_BF16 && out_dtype != FMSA_F32) return FMSA_ERR_DTYPE;
  if (!aligned16(out)) return FMSA_ERR_ALIGN;
  return launch_gptq_dequant(w, out_dtype, out, (hipStream_t)stream);
}

int fmsa_gptq_permute_rows(const int32_t* qweight, const int32_t* perm, int K, int N, int32_t* qweight_out,
                           void* stream) {
  if (!qweight || !perm || !qweight_out) return FMSA_ERR_NULL;
  if (K <= 0 || N <= 0 || K % 8 != 0) return FMSA_ERR_SHAPE;
  if (qweight == qweight_out) return FMSA_ERR_UNSUPPORTED;  // not an in-place operation
  return launch_gptq_permute_rows(qweight, perm, K, N, qweight_out, (hipStream_t)stream);
}

int fmsa_permute_cols(const void* in, int64_t ld_in, const int32_t* perm, int M, int C, int gather, int act_dtype,
                      void* out, int64_t ld_out, void* stream) {
  if (!in || !perm || !out) return FMSA_ERR_NULL;
  if (M <= 0 || C <= 0 || ld_in < C || ld_out < C) return FMSA_ERR_SHAPE;
  if (!is_act(act_dtype)) return FMSA_ERR_DTYPE;
  if (in == out) return FMSA_ERR_UNSUPPORTED;
  return launch_permute_cols(in, ld_in, perm, M, C, gather, out, ld_out, (hipStream_t)stream);
}

int fmsa_lora_down(const void* X, int64_t ldx, const void* Wd, int M, int C, int r, int act_dtype, void* out,
                   int64_t ldout, void* stream) {
  if (!X || !Wd || !out) return FMSA_ERR_NULL;
  if (M <= 0 || C <= 0 || r <= 0 || ldx < C || ldout < r) return FMSA_ERR_SHAPE;
  if (int rc = check_rank(r)) return rc;
  if (C % 8 != 0) return FMSA_ERR_SHAPE;
  if (!is_act(act_dtype)) return FMSA_ERR_DTYPE;
  if (!aligned16(X) || !aligned16(Wd) || ldx % 8 != 0) return FMSA_ERR_ALIGN;
  return launch_lora_down(X, ldx, Wd, M, C, r, act_dtype, out, ldout, (hipStream_t)stream);
}

size_t fmsa_lora_down_workspace(int M, int C, int r) {
  if (M <= 0 || C <= 0 || r <= 0 || r > 128 || r % 8 != 0 || C % 8 != 0) return 0;
  return lora_down_workspace(M, C, r);
}

int fmsa_lora_down_ws(const void* X, int64_t ldx, const void* Wd, int M, int C, int r, int act_dtype, void* out,
                      int64_t ldout, void* workspace, size_t workspace_bytes, void* stream) {
  if (!X || !Wd || !out) return FMSA_ERR_NULL;
  if (M <= 0 || C <= 0 || r <= 0 || ldx < C || ldout < r) return FMSA_ERR_SHAPE;
  if (int rc = check_rank(r)) return rc;
  if (C % 8 != 0) return FMSA_ERR_SHAPE;
  if (!is_act(act_dtype)) return FMSA_ERR_DTYPE;
  if (!aligned16(X) || !aligned16(Wd) || ldx % 8 != 0) return FMSA_ERR_ALIGN;
  if (workspace && !aligned16(workspace)) return FMSA_ERR_ALIGN;
  return launch_lora_down_ws(X, ldx, Wd, M, C, r, act_dtype, out, ldout, workspace, workspace_bytes, (hipStream_t)stream);
}

size_t fmsa_lora_grad_workspace(int M, int C, int r) {
  if (M <= 0 || C <= 0 || r <= 0) return 0;
  return (size_t)lora_grad_splits(M, C) * (size_t)r * (size_t)C * sizeof(float);
}

size_t fmsa_lora_grad_batch_workspace(const fmsa_lora_grad_job* jobs, int n_jobs, int M) {
  if (!jobs || n_jobs < 1 || n_jobs > FMSA_LORA_GRAD_MAX_JOBS || M <= 0) return 0;
  for (int q = 0; q < n_jobs; ++q)
    if (jobs[q].C <= 0 || jobs[q].r <= 0) return 0;
  return lora_grad_batch_workspace(jobs, n_jobs, M);
}

int fmsa_lora_grad_batch(const fmsa_lora_grad_job* jobs, int n_jobs, int M, int act_dtype, void* workspace,
                         size_t workspace_bytes, void* stream) {
  if (!jobs) return FMSA_ERR_NULL;
  if (n_jobs < 1 || n_jobs > FMSA_LORA_GRAD_MAX_JOBS || M <= 0) return FMSA_ERR_SHAPE;
  if (!is_act(act_dtype)) return FMSA_ERR_DTYPE;
  bool any_t = false;
  int r_max = 0;
  for (int q = 0; q < n_jobs; ++q) {
    const fmsa_lora_grad_job& j = jobs[q];
    if (!j.L || !j.R || !j.out) return FMSA_ERR_NULL;
    if (j.C <= 0 || j.r <= 0 || j.ldr < j.C || j.ldl < j.r) return FMSA_ERR_SHAPE;
    if (j.C % 8 != 0 || j.ldr % 8 != 0 || j.ldl % 8 != 0 || j.r % 8 != 0 || j.r > 128) return FMSA_ERR_SHAPE;
    if (j.out_dtype != FMSA_F16 && j.out_dtype != FMSA_BF16 && j.out_dtype != FMSA_F32) return FMSA_ERR_DTYPE;
    if (!aligned16(j.R) || !aligned16(j.L)) return FMSA_ERR_ALIGN;
    if (j.Wt) {
      if (!j.T) return FMSA_ERR_NULL;
      if (j.ldt < j.r) return FMSA_ERR_SHAPE;
      if (!aligned16(j.Wt) || j.ldt % 4 != 0 || (reinterpret_cast<uintptr_t>(j.T) & 7u)) return FMSA_ERR_ALIGN;
      any_t = true;
    }
    r_max = j.r > r_max ? j.r : r_max;
  }
  if (any_t && r_max > 32) return FMSA_ERR_UNSUPPORTED;
  if (!workspace || workspace_bytes < lora_grad_batch_workspace(jobs, n_jobs, M)) return FMSA_ERR_WORKSPACE;
  if (!aligned16(workspace)) return FMSA_ERR_ALIGN;
  return launch_lora_grad_batch(jobs, n_jobs, M, act_dtype, workspace, (hipStream_t)stream);
}

int fmsa_lora_grad(const void* L, int64_t ldl, const void* R, int64_t ldr, int M, int C, int r, float scale, int transpose_out,
                   int act_dtype, int out_dtype, void* out, void* workspace, size_t workspace_bytes, void* stream) {
  const fmsa_lora_grad_job job = {L, R, out, ldl, ldr, C, r, scale, transpose_out, out_dtype, 0, nullptr, nullptr, 0};
  return fmsa_lora_grad_batch(&job, 1, M, act_dtype, workspace, workspace_bytes, stream);
}

int fmsa_lora_grad_static(const void* L, int64_t ldl, const void* R, int64_t ldr, int M, int C, int r, float scale,
                          int transpose_out, int act_dtype, int out_dtype, void* out, void* stream) {
  if (M <= 0 || C <= 0 || r <= 0) return FMSA_ERR_SHAPE;
  // the size check comes before any HIP call: a request beyond the static buffer is an argument error
  if (fmsa_lora_grad_workspace(M, C, r) > (size_t)FMSA_LORA_GRAD_STATIC_BYTES) return FMSA_ERR_WORKSPACE;
  const fmsa_lora_grad_job job = {L, R, out, ldl, ldr, C, r, scale, transpose_out, out_dtype, 0, nullptr, nullptr, 0};
  // validate with a stand-in workspace pointer (non-null, aligned) so that every argument error is reported
  // before the device is touched; the launch below gets the real address
  if (!job.L || !job.R || !job.out) return FMSA_ERR_NULL;
  if (!is_act(act_dtype)) return FMSA_ERR_DTYPE;
  if (ldr < C || ldl < r) return FMSA_ERR_SHAPE;
  if (C % 8 != 0 || ldr % 8 != 0 || ldl % 8 != 0 || r % 8 != 0 || r > 128) return FMSA_ERR_SHAPE;
  if (out_dtype != FMSA_F16 && out_dtype != FMSA_BF16 && out_dtype != FMSA_F32) return FMSA_ERR_DTYPE;
  if (!aligned16(R) || !aligned16(L)) return FMSA_ERR_ALIGN;
  // the launch goes to the calling thread's current device, so that is whose copy of the buffer is used: the
  // tensors (and the stream) must belong to it.  The query allocates nothing; a pointer the runtime does not
  // know is left to the kernel's own addressing.
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return FMSA_ERR_LAUNCH;
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, out) == hipSuccess) {
    if (attr.type == hipMemoryTypeDevice && attr.device != dev) return FMSA_ERR_DEVICE;
  } else {
    (void)hipGetLastError();
  }
  void* ws = scratch_of_current_device();
  if (!ws) return FMSA_ERR_LAUNCH;
  // both passes write every partial sum they later read, so the buffer needs no clearing between calls
  return launch_lora_grad_batch(&job, 1, M, act_dtype, ws, (hipStream_t)stream);
}

static int check_fwd(const fmsa_fwd_proj* projs, int n_proj, const void* X, int64_t ldx, int M, int mode, const void* H,
                     int64_t ldh, int act_dtype) {
  if (!projs || !X) return FMSA_ERR_NULL;
  if (n_proj < 1 || n_proj > 3 || M <= 0) return FMSA_ERR_SHAPE;
  if (mode != FMSA_FWD_LINEAR && mode != FMSA_FWD_SWIGLU) return FMSA_ERR_SHAPE;
  if (!is_act(act_dtype)) return FMSA_ERR_DTYPE;
  const int K = projs[0].w.K;
  if (ldx < K) return FMSA_ERR_SHAPE;
  if (!aligned16(X) || ldx % 8 != 0) return FMSA_ERR_ALIGN;
  for (int p = 0; p < n_proj; ++p) {
    const fmsa_fwd_proj& s = projs[p];
    // the interleaved nibble order belongs to the packed-half unpack: fp16 activations (and no rotary epilogue, which
    // fmsa_gptq_lora_fwd_rope checks)
    if (int rc = check_weight(&s.w, 16, act_dtype == FMSA_F16)) return rc;
    if (s.w.format != projs[0].w.format || s.w.nibble_order != projs[0].w.nibble_order) return FMSA_ERR_UNSUPPORTED;  // one kernel flavour per launch
    if (s.w.K != K) return FMSA_ERR_SHAPE;
    if (!s.Y) return FMSA_ERR_NULL;
    if (s.ldy < s.w.N) return FMSA_ERR_SHAPE;
    if (!aligned16(s.Y) || s.ldy % 8 != 0) return FMSA_ERR_ALIGN;
    if (int rc = check_rank(s.r)) return rc;
    if (s.r > 0) {
      if (!s.U || !s.B) return FMSA_ERR_NULL;
      if (!aligned16(s.U) || !aligned16(s.B) || s.ldu % 8 != 0) return FMSA_ERR_ALIGN;
      if (s.ldu < s.r) return FMSA_ERR_SHAPE;
    }
    if (s.bias && !aligned16(s.bias)) return FMSA_ERR_ALIGN;
  }
  if (mode == FMSA_FWD_SWIGLU) {
    if (n_proj != 2 || projs[0].w.N != projs[1].w.N) return FMSA_ERR_SHAPE;
    if (!H) return FMSA_ERR_NULL;
    if (ldh < projs[0].w.N) return FMSA_ERR_SHAPE;
    if (!aligned16(H) || ldh % 8 != 0) return FMSA_ERR_ALIGN;
  }
  return FMSA_OK;
}

int fmsa_gptq_lora_fwd(const fmsa_fwd_proj* projs, int n_proj, const void* X, int64_t ldx, int M, int mode, void* H,
                       int64_t ldh, int act_dtype, void* stream) {
  if (int rc = check_fwd(projs, n_proj, X, ldx, M, mode, H, ldh, act_dtype)) return rc;
  return launch_gptq_lora_fwd(projs, n_proj, X, ldx, M, mode, H, ldh, nullptr, act_dtype, (hipStream_t)stream);
}

int fmsa_gptq_lora_fwd_rope(const fmsa_fwd_proj* projs, int n_proj, const void* X, int64_t ldx, int M, const fmsa_rope* rope,
                            int act_dtype, void* stream) {
  if (!projs || !X || !rope) return FMSA_ERR_NULL;
  if (!rope->cos || !rope->sin) return FMSA_ERR_NULL;
  if (n_proj < 1 || n_proj > 3 || M <= 0) return FMSA_ERR_SHAPE;
  if (!is_act(act_dtype)) return FMSA_ERR_DTYPE;
  if (rope->dtype != act_dtype && rope->dtype != FMSA_F32) return FMSA_ERR_DTYPE;
  const int hd = rope->head_dim;
  if (hd <= 0 || rope->rows <= 0 || rope->ld < hd / 2) return FMSA_ERR_SHAPE;
  if (hd % 16 != 0 || 256 % hd != 0) return FMSA_ERR_UNSUPPORTED;
  if (rope->proj_mask < 0 || rope->proj_mask >= (1 << n_proj)) return FMSA_ERR_SHAPE;
  if (!aligned16(rope->cos) || !aligned16(rope->sin) || rope->ld % (rope->dtype == FMSA_F32 ? 4 : 8) != 0) return FMSA_ERR_ALIGN;
  // the checks of the plain forward (pointers, shapes, alignment), then what the rotating flavour of the kernel adds
  if (int rc = check_fwd(projs, n_proj, X, ldx, M, FMSA_FWD_LINEAR, nullptr, 0, act_dtype)) return rc;
  const int K = projs[0].w.K;
  for (int p = 0; p < n_proj; ++p) {
    if (((rope->proj_mask >> p) & 1) && projs[p].w.N % hd != 0) return FMSA_ERR_SHAPE;
    if (projs[p].w.group_size <= 0 || projs[p].w.group_size % 64 != 0) return FMSA_ERR_UNSUPPORTED;
    if (projs[p].w.nibble_order != 0) return FMSA_ERR_UNSUPPORTED;  // the rotating flavours read the checkpoint's order
  }
  if (K % 64 != 0) return FMSA_ERR_UNSUPPORTED;
  return launch_gptq_lora_fwd(projs, n_proj, X, ldx, M, FMSA_FWD_LINEAR, nullptr, 0, rope, act_dtype, (hipStream_t)stream);
}

int fmsa_gptq_lora_bwd_dx(const fmsa_bwd_proj* projs, int n_proj, int M, int mode, void* dX, int64_t lddx, void* e,
                          void* g, void* h_out, int64_t ldeg, int act_dtype, void* stream) {
  if (!projs) return FMSA_ERR_NULL;
  if (n_proj < 1 || n_proj > 3 || M <= 0) return FMSA_ERR_SHAPE;
  if (mode != FMSA_BWD_LINEAR && mode != FMSA_BWD_SWIGLU) return FMSA_ERR_SHAPE;
  if (!is_act(act_dtype)) return FMSA_ERR_DTYPE;
  const int K = projs[0].w.K;
  const void* mask = nullptr;
  int64_t ldmask = 0;
  for (int p = 0; p < n_proj; ++p) {
    const fmsa_bwd_proj& s = projs[p];
    if (int rc = check_weight(&s.w, 8)) return rc;
    if (s.w.format != projs[0].w.format) return FMSA_ERR_UNSUPPORTED;  // one kernel flavour per launch
    if (s.w.group_size < 32) return FMSA_ERR_UNSUPPORTED;  // at most 8 groups per 256 output columns
    if (s.w.K != K) return FMSA_ERR_SHAPE;
    // the offset table: fp32 -s*z, or (fp16 activations on the transposed twin) the fp16 -(1024 + z) table alone
    if (!s.dY) return FMSA_ERR_NULL;
    if (s.negzp_f16 && !aligned16(s.negzp_f16)) return FMSA_ERR_ALIGN;
    if (s.lddy < s.w.N) return FMSA_ERR_SHAPE;
    if (s.nsz && !aligned16(s.nsz)) return FMSA_ERR_ALIGN;
    if ((s.qweight_t && !aligned16(s.qweight_t)) || (s.scale_f32 && !aligned16(s.scale_f32))) return FMSA_ERR_ALIGN;
    if (!aligned16(s.dY) || s.lddy % 8 != 0) return FMSA_ERR_ALIGN;
    if (int rc = check_rank(s.r)) return rc;
    if (s.r > 0) {
      if (!s.T || !s.At) return FMSA_ERR_NULL;
      if (!aligned16(s.T) || !aligned16(s.At) || s.ldt % 8 != 0) return FMSA_ERR_ALIGN;
      if (s.ldt < s.r) return FMSA_ERR_SHAPE;
    }
    if (s.mask_src && s.r > 0) {
      if (s.ldmask < K) return FMSA_ERR_SHAPE;
      if (!aligned16(s.mask_src) || s.ldmask % 8 != 0) return FMSA_ERR_ALIGN;
      // one mask per call: the LoRA terms of all projections are summed before it is applied
      if (mask && (mask != s.mask_src || ldmask != s.ldmask)) return FMSA_ERR_UNSUPPORTED;
      mask = s.mask_src;
      ldmask = s.ldmask;
    }
  }
  if (mode == FMSA_BWD_SWIGLU) {
    if (n_proj != 1) return FMSA_ERR_SHAPE;
    if (!e || !g || !h_out) return FMSA_ERR_NULL;
    if (ldeg < K) return FMSA_ERR_SHAPE;
    if (!aligned16(e) || !aligned16(g) || !aligned16(h_out) || ldeg % 8 != 0) return FMSA_ERR_ALIGN;
  } else {
    if (!dX) return FMSA_ERR_NULL;
    if (lddx < K) return FMSA_ERR_SHAPE;
    if (!aligned16(dX) || lddx % 8 != 0) return FMSA_ERR_ALIGN;
  }
  const int twin = bwd_dx_twin_flavour(projs, n_proj, act_dtype);
  // the checkpoint-layout kernel needs every affine projection's fp32 offset table
  if (!twin)
    for (int p = 0; p < n_proj; ++p)
      if (!projs[p].nsz && projs[p].w.format != FMSA_WEIGHT_CODEBOOK) return FMSA_ERR_NULL;
  if (twin)
    return launch_gptq_lora_bwd_dx_t(projs, n_proj, M, mode, dX, lddx, e, g, h_out, ldeg, act_dtype, (hipStream_t)stream);
  return launch_gptq_lora_bwd_dx(projs, n_proj, M, mode, dX, lddx, e, g, h_out, ldeg, act_dtype, (hipStream_t)stream);
}

int fmsa_gptq_interleave(const int32_t* qweight, int K, int N, int32_t* qweight_out, void* stream) {
  if (!qweight || !qweight_out) return FMSA_ERR_NULL;
  if (K <= 0 || N <= 0 || K % 8 != 0 || N % 4 != 0) return FMSA_ERR_SHAPE;
  if (!aligned16(qweight) || !aligned16(qweight_out)) return FMSA_ERR_ALIGN;
  return launch_gptq_interleave(qweight, K, N, qweight_out, (hipStream_t)stream);
}

int fmsa_gptq_transpose(const int32_t* qweight, int K, int N, int32_t* qweight_t_out, void* stream) {
  if (!qweight || !qweight_t_out) return FMSA_ERR_NULL;
  if (K <= 0 || N <= 0 || K % 8 != 0 || N % 8 != 0) return FMSA_ERR_SHAPE;
  if (!aligned16(qweight) || !aligned16(qweight_t_out)) return FMSA_ERR_ALIGN;
  return launch_gptq_transpose(qweight, K, N, qweight_t_out, (hipStream_t)stream);
}

int fmsa_swiglu_fwd(const void* e, const void* g, void* h, int M, int I, int64_t ld, int act_dtype, void* stream) {
  if (!e || !g || !h) return FMSA_ERR_NULL;
  if (M <= 0 || I <= 0 || I % 8 != 0 || ld < I) return FMSA_ERR_SHAPE;
  if (!is_act(act_dtype)) return FMSA_ERR_DTYPE;
  if (!aligned16(e) || !aligned16(g) || !aligned16(h) || ld % 8 != 0) return FMSA_ERR_ALIGN;
  return launch_swiglu_fwd(e, g, h, M, I, ld, act_dtype, (hipStream_t)stream);
}

int fmsa_swiglu_bwd(const void* dh, int64_t lddh, void* e, void* g, void* h_out, int M, int I, int64_t ld,
                    int act_dtype, void* stream) {
  if (!dh || !e || !g || !h_out) return FMSA_ERR_NULL;
  if (M <= 0 || I <= 0 || I % 8 != 0 || ld < I || lddh < I) return FMSA_ERR_SHAPE;
  if (!is_act(act_dtype)) return FMSA_ERR_DTYPE;
  if (!aligned16(dh) || !aligned16(e) || !aligned16(g) || !aligned16(h_out) || ld % 8 != 0 || lddh % 8 != 0)
    return FMSA_ERR_ALIGN;
  return launch_swiglu_bwd(dh, lddh, e, g, h_out, M, I, ld, act_dtype, (hipStream_t)stream);
}

int fmsa_gptq_make_nsz(const fmsa_gptq_weight* w, float* out, void* stream) {
  if (!w || !out) return FMSA_ERR_NULL;
  if (int rc = check_weight(w, 0)) return rc;
  if (w->format != FMSA_WEIGHT_AFFINE) return FMSA_ERR_UNSUPPORTED;  // a code-book weight has no zero points
  if (!aligned16(out)) return FMSA_ERR_ALIGN;
  return launch_gptq_nsz(w, out, (hipStream_t)stream);
}

int fmsa_lora_pack_batch(const fmsa_lora_pack_job* jobs, int n_jobs, int act_dtype, void* stream) {
  if (!jobs) return FMSA_ERR_NULL;
  if (n_jobs < 1 || n_jobs > FMSA_LORA_PACK_MAX_JOBS) return FMSA_ERR_SHAPE;
  if (!is_act(act_dtype)) return FMSA_ERR_DTYPE;
  for (int q = 0; q < n_jobs; ++q) {
    const fmsa_lora_pack_job& j = jobs[q];
    if (!j.A || !j.B) return FMSA_ERR_NULL;
    if (j.r <= 0 || j.K <= 0 || j.N <= 0) return FMSA_ERR_SHAPE;
    if (j.param_dtype != FMSA_F32 && j.param_dtype != FMSA_BF16 && j.param_dtype != FMSA_F16) return FMSA_ERR_DTYPE;
  }
  return launch_lora_pack_batch(jobs, n_jobs, act_dtype, (hipStream_t)stream);
}

int fmsa_lora_pack(const void* A, const void* B, int r, int K, int N, int param_dtype, int act_dtype, void* A16, void* At16,
                   void* B16, void* Bt16, void* stream) {
  const fmsa_lora_pack_job job = {A, B, A16, At16, B16, Bt16, r, K, N, param_dtype};
  return fmsa_lora_pack_batch(&job, 1, act_dtype, stream);
}

int fmsa_nf4_dequant(const fmsa_nf4_weight* w, int out_dtype, void* out, void* stream) {
  if (!w || !out) return FMSA_ERR_NULL;
  if (!w->packed || !w->absmax_q || !w->absmax2 || !w->code2 || !w->code) return FMSA_ERR_NULL;
  if (w->N <= 0 || w->K <= 0 || w->blocksize <= 0 || w->blocksize2 <= 0) return FMSA_ERR_SHAPE;
  if (w->blocksize % 16 != 0 || ((int64_t)w->N * w->K) % w->blocksize != 0) return FMSA_ERR_SHAPE;
  if (out_dtype != FMSA_F16 && out_dtype != FMSA_BF16 && out_dtype != FMSA_F32) return FMSA_ERR_DTYPE;
  if (!aligned16(out) || (reinterpret_cast<uintptr_t>(w->packed) & 7u)) return FMSA_ERR_ALIGN;
  return launch_nf4_dequant(w, out_dtype, out, (hipStream_t)stream);
}

int fmsa_nf4_prepare(const fmsa_nf4_weight* w, int32_t* qweight_out, float* block_scale_out, void* stream) {
  if (!w || !qweight_out || !block_scale_out) return FMSA_ERR_NULL;
  if (!w->packed || !w->absmax_q || !w->absmax2 || !w->code2) return FMSA_ERR_NULL;
  if (w->N <= 0 || w->K <= 0 || w->blocksize <= 0 || w->blocksize2 <= 0) return FMSA_ERR_SHAPE;
  if (w->K % 8 != 0 || w->blocksize % 8 != 0 || w->K % w->blocksize != 0) return FMSA_ERR_SHAPE;
  if (w->K / 8 > 65535 || w->K / w->blocksize > 65535) return FMSA_ERR_UNSUPPORTED;  // grid.y
  if (!aligned16(qweight_out) || !aligned16(block_scale_out) || (reinterpret_cast<uintptr_t>(w->packed) & 3u)) return FMSA_ERR_ALIGN;
  return launch_nf4_prepare(w, qweight_out, block_scale_out, (hipStream_t)stream);
}

namespace {
inline bool is_float_dtype(int d) { return d == FMSA_F16 || d == FMSA_BF16 || d == FMSA_F32; }
inline bool aligned_rows(const void* p, int64_t ld, int d) {
  const int esz = d == FMSA_F32 ? 4 : 2;
  return aligned16(p) && (ld * esz) % 16 == 0;
}
}  // namespace

int fmsa_rms_layernorm_fwd(const void* X, int64_t ldx, const void* W, int M, int C, float eps, int gemma, int x_dtype,
                           int w_dtype, void* Y, int64_t ldy, float* r, void* stream) {
  if (!X || !W || !Y || !r) return FMSA_ERR_NULL;
  if (M <= 0 || C <= 0 || C % 8 != 0 || ldx < C || ldy < C) return FMSA_ERR_SHAPE;
  if (!is_float_dtype(x_dtype) || !is_float_dtype(w_dtype)) return FMSA_ERR_DTYPE;
  if (!aligned_rows(X, ldx, x_dtype) || !aligned_rows(Y, ldy, x_dtype) || !aligned16(W)) return FMSA_ERR_ALIGN;
  return launch_rms_fwd(X, ldx, W, M, C, eps, gemma, x_dtype, w_dtype, Y, ldy, r, (hipStream_t)stream);
}

int fmsa_rms_layernorm_bwd(void* dY, int64_t lddy, const void* X, int64_t ldx, const void* W, const float* r, int M, int C,
                           int gemma, int x_dtype, int w_dtype, void* stream) {
  if (!dY || !X || !W || !r) return FMSA_ERR_NULL;
  if (M <= 0 || C <= 0 || C % 8 != 0 || ldx < C || lddy < C) return FMSA_ERR_SHAPE;
  if (!is_float_dtype(x_dtype) || !is_float_dtype(w_dtype)) return FMSA_ERR_DTYPE;
  if (!aligned_rows(X, ldx, x_dtype) || !aligned_rows(dY, lddy, x_dtype) || !aligned16(W)) return FMSA_ERR_ALIGN;
  return launch_rms_bwd(dY, lddy, X, ldx, W, r, M, C, gemma, x_dtype, w_dtype, (hipStream_t)stream);
}

int fmsa_rope_embedding(void* Q, int64_t ldq, const void* cos, const void* sin, int64_t ldcs, int M, int n_heads,
                        int head_dim, int cs_rows, int backward, int q_dtype, int cs_dtype, void* stream) {
  if (!Q || !cos || !sin) return FMSA_ERR_NULL;
  if (M <= 0 || n_heads <= 0 || head_dim <= 0 || head_dim % 16 != 0 || cs_rows <= 0) return FMSA_ERR_SHAPE;
  if (ldq < (int64_t)n_heads * head_dim || ldcs < head_dim / 2) return FMSA_ERR_SHAPE;
  if (!is_float_dtype(q_dtype) || !is_float_dtype(cs_dtype)) return FMSA_ERR_DTYPE;
  if (!aligned_rows(Q, ldq, q_dtype) || !aligned_rows(cos, ldcs, cs_dtype) || !aligned_rows(sin, ldcs, cs_dtype))
    return FMSA_ERR_ALIGN;
  return launch_rope(Q, ldq, cos, sin, ldcs, M, n_heads, head_dim, cs_rows, backward, q_dtype, cs_dtype, (hipStream_t)stream);
}

int fmsa_cross_entropy_fwd(const void* logits, int64_t ld, const int64_t* labels, int M, int V, int dtype, float* losses,
                           float* logsumexp, void* stream) {
  if (!logits || !labels || !losses || !logsumexp) return FMSA_ERR_NULL;
  if (M <= 0 || V <= 0 || ld < V) return FMSA_ERR_SHAPE;
  if (!is_float_dtype(dtype)) return FMSA_ERR_DTYPE;
  const int vec = (V % 8 == 0) && aligned_rows(logits, ld, dtype);
  return launch_ce_fwd(logits, ld, labels, M, V, dtype, vec, losses, logsumexp, (hipStream_t)stream);
}

int fmsa_cross_entropy_bwd(void* logits, int64_t ld, const float* dloss, int64_t dloss_stride, const float* logsumexp,
                           const int64_t* labels, int M, int V, int dtype, void* stream) {
  if (!logits || !labels || !dloss || !logsumexp) return FMSA_ERR_NULL;
  if (M <= 0 || V <= 0 || ld < V || dloss_stride < 0) return FMSA_ERR_SHAPE;
  if (!is_float_dtype(dtype)) return FMSA_ERR_DTYPE;
  const int vec = (V % 8 == 0) && aligned_rows(logits, ld, dtype);
  return launch_ce_bwd(logits, ld, dloss, dloss_stride, logsumexp, labels, M, V, dtype, vec, (hipStream_t)stream);
}

int fmsa_cross_entropy_fused(void* logits, int64_t ld, const int64_t* labels, int M, int V, int dtype, int64_t ignore_index,
                             const float* scale, float label_smoothing, float* losses, void* stream) {
  if (!logits || !labels || !losses) return FMSA_ERR_NULL;
  if (M <= 0 || V <= 0 || ld < V) return FMSA_ERR_SHAPE;
  if (!(label_smoothing >= 0.0f && label_smoothing <= 1.0f)) return FMSA_ERR_SHAPE;
  if (!is_float_dtype(dtype)) return FMSA_ERR_DTYPE;
  const int vec = (V % 8 == 0) && aligned_rows(logits, ld, dtype);
  return launch_ce_fused(logits, ld, labels, M, V, dtype, vec, ignore_index, scale, label_smoothing, losses, (hipStream_t)stream);
}

}  // extern "C"
