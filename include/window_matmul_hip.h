/*
 * C ABI of the MI355X (gfx950) banded-matmul library, libwindow_matmul_hip.so.
 *
 * These entry points are what a binding of the reference's native module
 * `window_matmul_kernel` (reference csrc/window_matmul/window_matmul.cpp:100-106)
 * calls for tensors that live on the GPU.  They replace the reference's CUDA
 * launchers (reference csrc/window_matmul/cuda/window_matmul_cuda.h:5-10).
 *
 * Conventions
 *   - All pointers are device pointers on the current HIP device; the caller
 *     owns every buffer.  The library allocates nothing, never synchronises and
 *     keeps no mutable state, so it may be called from several host threads
 *     (the one exception, wm_window_attention_backward_static, says so below).
 *   - Work is enqueued on `stream` (a hipStream_t passed as void*; NULL is the
 *     legacy default stream) and the call returns as soon as it is enqueued.
 *   - Every operand is a rank-3 view described by a base pointer and ELEMENT
 *     strides for (batch, row, column); any strides are accepted.  The fast
 *     kernels need unit column stride and 16-byte aligned rows; other layouts
 *     (and float64 in every layout) run on a slower family of tiled kernels that
 *     reads element by element through the strides, with the same results.
 *   - Outputs need not be zeroed: every element is written, and band entries
 *     that fall outside the sequence are written as +0.0.
 *   - Band convention: column j of band row i addresses source row c = i+j-w,
 *     valid iff 0 <= c < M.  Invalid entries of an INPUT band are never read.
 *   - Accumulation is float32 for f32/f16/bf16 storage and float64 for f64.
 *   - Return value: WM_OK (0) when the work was enqueued, otherwise a wm_status
 *     code; nothing is enqueued on error.  wm_status_string() names the code.
 */
#ifndef WINDOW_MATMUL_HIP_H
#define WINDOW_MATMUL_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define WM_ABI_VERSION 4

typedef enum wm_dtype {
  WM_DTYPE_F32 = 0,
  WM_DTYPE_F16 = 1,
  WM_DTYPE_BF16 = 2,
  WM_DTYPE_F64 = 3
} wm_dtype;

typedef enum wm_status {
  WM_OK = 0,
  WM_ERR_NULL_POINTER = 1,     /* a required operand or its data pointer is NULL */
  WM_ERR_BAD_SHAPE = 2,        /* negative extent, or an extent beyond 2^31-1      */
  WM_ERR_BAD_DTYPE = 3,        /* dtype is not a wm_dtype value                     */
  WM_ERR_BAD_FLAGS = 4,        /* unknown bit set in flags                          */
  WM_ERR_LAUNCH_FAILED = 5,    /* the HIP runtime rejected a kernel launch          */
  WM_ERR_NO_DEVICE_CODE = 6,   /* the library holds no code object for this GPU     */
  WM_ERR_UNSUPPORTED = 7,      /* a fused entry point has no kernel for this shape, dtype or layout;
                                  nothing was launched: run the chain of the separate ops instead */
  WM_ERR_SCRATCH_TOO_SMALL = 8 /* wm_window_attention_backward_static: B * M > WM_STATIC_SCRATCH_ROWS */
} wm_status;

/* Kernel selection.  0 lets the library choose per (shape, dtype, layout). */
#define WM_FLAG_FORCE_STRIDED 0x1u   /* always use the one-thread-per-output kernels (A/B testing) */
#define WM_FLAG_NO_ALIGNED_BAND 0x2u /* MFMA kernels: never use the 16-byte aligned band variant */
#define WM_FLAG_NO_NARROW_BAND 0x4u  /* never use the narrow-band kernels (MFMA, w <= 63; vector ALU, w <= 14; fused attention, w <= 64) */
#define WM_FLAG_NO_LDS_DIRECT 0x8u   /* never use the kernels that load chunks straight into LDS (fused attention; band-out product at N = 128) */
#define WM_FLAG_NO_SPLIT_F32 0x10u   /* float32: never use the kernels that run on the bf16 matrix instruction through an exact three-way split */

/* Rank-3 operand: element (b, r, c) lives at data + b*stride_b + r*stride_r + c*stride_c. */
typedef struct wm_operand {
  void *data;
  int64_t stride_b;
  int64_t stride_r;
  int64_t stride_c;
} wm_operand;

/* A[b,i,j] = sum_h q[b,i,h] * k[b,h,i+j-w]  (0 <= i+j-w < M, else +0.0)
 *   q (B,M,N), k (B,N,M) -- the reference's orientation: K transposed -- , a (B,M,2w+1).
 * Replaces window_matmul_fw_cuda (reference cuda/window_matmul_cuda.cu:224-270),
 * reached from window_matmul_forward (reference window_matmul.cpp:74-78). */
int wm_window_matmul_forward(const wm_operand *q, const wm_operand *k, const wm_operand *a,
                             int64_t B, int64_t M, int64_t N, int64_t w, int dtype,
                             unsigned flags, void *stream);

/* grad_q[b,i,h] = sum_j grad_a[b,i,j] * k[b,h,i+j-w]           (B,M,N)
 * grad_k[b,h,c] = sum_r q[b,r,h] * grad_a[b,r,c-r+w]            (B,N,M), no atomics
 *   Either gradient may be skipped by passing NULL for its operand.
 * Replaces window_matmul_bw_cuda (reference cuda/window_matmul_cuda.cu:272-319),
 * reached from window_matmul_backward (reference window_matmul.cpp:80-85). */
int wm_window_matmul_backward(const wm_operand *q, const wm_operand *k, const wm_operand *grad_a,
                              const wm_operand *grad_q, const wm_operand *grad_k, int64_t B,
                              int64_t M, int64_t N, int64_t w, int dtype, unsigned flags,
                              void *stream);

/* o[b,i,h] = sum_{j valid} a[b,i,j] * v[b,i+j-w,h]
 *   a (B,M,2w+1), v (B,M,N), o (B,M,N).
 * Replaces unwindow_matmul_fw_cuda (reference cuda/window_matmul_cuda.cu:321-358),
 * reached from unwindow_matmul_forward (reference window_matmul.cpp:87-91). */
int wm_unwindow_matmul_forward(const wm_operand *a, const wm_operand *v, const wm_operand *o,
                               int64_t B, int64_t M, int64_t N, int64_t w, int dtype,
                               unsigned flags, void *stream);

/* grad_a[b,i,j] = sum_h v[b,i+j-w,h] * grad_o[b,i,h]  (+0.0 where invalid)   (B,M,2w+1)
 * grad_v[b,c,h] = sum_r a[b,r,c-r+w] * grad_o[b,r,h]                          (B,M,N), no atomics
 *   Either gradient may be skipped by passing NULL for its operand.
 * Replaces unwindow_matmul_bw_cuda (reference cuda/window_matmul_cuda.cu:360-416),
 * reached from unwindow_matmul_backward (reference window_matmul.cpp:93-98). */
int wm_unwindow_matmul_backward(const wm_operand *a, const wm_operand *v, const wm_operand *grad_o,
                                const wm_operand *grad_a, const wm_operand *grad_v, int64_t B,
                                int64_t M, int64_t N, int64_t w, int dtype, unsigned flags,
                                void *stream);

/* Name of the kernel family the library would pick for one banded product, for
 * logs and profiles: op is 1 (band-out: window forward, grad_a), 2 (band-in:
 * unwindow forward, grad_q) or 3 (transposed band-in: grad_k, grad_v);
 * fast_layout is non-zero when all operands have unit column stride and 16-byte
 * aligned rows.  Returns a static string.  No counterpart in the reference. */
const char *wm_kernel_choice(int op, int64_t B, int64_t M, int64_t N, int64_t w, int dtype,
                             int fast_layout, unsigned flags);

/* Softmax along the band dimension: p[b,i,:] = softmax(scale * a[b,i,:]) over the 2w+1
 * entries of each row of a (B, M, 2w+1) tensor.  No counterpart in the reference's native
 * module: it replaces the torch call its callers put between the two ops
 * (reference tests/test_attention.py:60-61, `att_scores / sqrt(N)` then `softmax(dim=-1)`).
 * With mask_out_of_range == 0 every entry takes part with the value it holds, as in that
 * caller (window_matmul leaves +0.0 in entries outside the sequence).  With
 * mask_out_of_range != 0 entries whose key position i+j-w is outside [0, M) count as
 * -infinity: their probability and their gradient are +0.0 whatever they hold.
 * a and p may be the same buffer.  Contiguous, 16-byte aligned tensors of float32 / float16 /
 * bfloat16 with rows up to ~64 KB get the LDS-staged kernel; anything else a strided one. */
int wm_band_softmax_forward(const wm_operand *a, const wm_operand *p, int64_t B, int64_t M, int64_t w,
                            double scale, int mask_out_of_range, int dtype, unsigned flags, void *stream);

/* Backward of the above from the saved probabilities:
 * grad_a[b,i,j] = scale * p[b,i,j] * (grad_p[b,i,j] - sum_j' p[b,i,j'] * grad_p[b,i,j']).
 * grad_a may alias grad_p or p.  Same masking rule (masked entries of grad_p are not read). */
int wm_band_softmax_backward(const wm_operand *p, const wm_operand *grad_p, const wm_operand *grad_a,
                             int64_t B, int64_t M, int64_t w, double scale, int mask_out_of_range,
                             int dtype, unsigned flags, void *stream);

/* Name of the kernel the two functions above would use ("staged_softmax" / "strided_softmax"). */
const char *wm_band_softmax_kernel_choice(int64_t w, int dtype, int contiguous, int backward, unsigned flags);

/* Fused window attention, forward:
 *   o = unwindow_matmul(softmax(scale * window_matmul(q, k^T, w), -1), v, w)
 * in one kernel; the (B, M, 2w+1) band never reaches memory.  No counterpart in the
 * reference's native module: it fuses the chain its callers write
 * (reference tests/test_attention.py:57-63) and keeps that chain's semantics.  With
 * mask_out_of_range == 0 the band entries outside the sequence take part in the softmax
 * with score 0, as they do when window_matmul's +0.0 entries go through torch.softmax, and
 * contribute no value row; with mask_out_of_range != 0 they are left out.
 * q, k, v, o are (B, M, N) operands (k holds key ROWS here, unlike the (B, N, M) view the
 * window op takes).  lse, if not NULL, receives the natural-log sum of exponentials of every
 * row as float32 (B * M values, contiguous) for use by a backward pass; the sum is taken over
 * the probabilities as rounded to the storage type, the values that multiply v.
 * Returns WM_ERR_UNSUPPORTED, having launched nothing, unless dtype is float16 / bfloat16,
 * N is a multiple of 16 up to 128, w >= 1, scale > 0 and all four operands have unit column
 * stride and 16-byte aligned rows (see wm_window_attention_supported). */
int wm_window_attention_forward(const wm_operand *q, const wm_operand *k, const wm_operand *v,
                                const wm_operand *o, float *lse, int64_t B, int64_t M, int64_t N,
                                int64_t w, double scale, int mask_out_of_range, int dtype,
                                unsigned flags, void *stream);

/* Backward of wm_window_attention_forward by recomputation: from q, k, v, the forward's o and
 * lse, and the upstream gradient grad_o, writes grad_q, grad_k, grad_v (all (B, M, N) operands,
 * k and grad_k as key rows).  delta is a caller-owned float32 workspace of 2 * B * M values (the
 * first kernel leaves sum_h grad_o * o and the rescaled log-sum-exp of every row there for the
 * second).  The masking choice of the forward is carried by lse and
 * needs no argument here.  Any of grad_q, grad_k, grad_v may be NULL to skip that gradient
 * (grad_q NULL shortens the first kernel to the delta pass, grad_k and grad_v both NULL drop the
 * second).  Up to two kernels are enqueued on the stream; no atomics, so results are
 * reproducible run to run.  With N <= 64 and w <= 48 (64 from N = 48) one kernel computes all three gradients and
 * delta is not touched (it must still be passed: which kernels run is the library's choice;
 * WM_FLAG_NO_NARROW_BAND selects the two-kernel form).  Same support rule and WM_ERR_UNSUPPORTED
 * behaviour as the forward.
 * No counterpart in the reference's native module (see the forward). */
int wm_window_attention_backward(const wm_operand *q, const wm_operand *k, const wm_operand *v,
                                 const wm_operand *o, const float *lse, const wm_operand *grad_o,
                                 const wm_operand *grad_q, const wm_operand *grad_k,
                                 const wm_operand *grad_v, float *delta, int64_t B, int64_t M,
                                 int64_t N, int64_t w, double scale, int dtype, unsigned flags,
                                 void *stream);

/* wm_window_attention_backward for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc): the same kernels and the
 * same results, with the delta workspace taken from a static device array inside the library
 * instead of from the caller.  No counterpart in the reference, whose launchers allocate their
 * outputs themselves (reference cuda/window_matmul_cuda.cu:239-242).
 *   - Limit: B * M <= WM_STATIC_SCRATCH_ROWS (two float32 per row: 16 MiB per GPU, resident from the first
 *     call on that GPU until the process ends); beyond it WM_ERR_SCRATCH_TOO_SMALL, nothing launched.
 *   - The call allocates and frees nothing.  The first call on a GPU looks the array's address
 *     up (hipGetSymbolAddress) and keeps it; make that call outside any stream capture.
 *   - All calls on one GPU share the one array: calls that may overlap on a GPU (different
 *     streams, or several host threads) race on it and must be serialised by the caller.
 *     Nothing in it has to be cleared between calls: every value read was written by the same call. */
#define WM_STATIC_SCRATCH_ROWS (1 << 21)
int wm_window_attention_backward_static(const wm_operand *q, const wm_operand *k, const wm_operand *v,
                                        const wm_operand *o, const float *lse, const wm_operand *grad_o,
                                        const wm_operand *grad_q, const wm_operand *grad_k,
                                        const wm_operand *grad_v, int64_t B, int64_t M, int64_t N, int64_t w,
                                        double scale, int dtype, unsigned flags, void *stream);

/* Keys that arrive as a (B, N, M) tensor with unit stride along M (the layout of the reference's
 * `other` argument when it is contiguous) copied into key rows, a contiguous (B, M, N) buffer
 * `rows`, which is what the kernels above consume in place as k with strides {M*N, 1, N}.  It
 * replaces the copy the reference makes on entry (`B.transpose(-1, -2).contiguous()`, reference
 * cuda/window_matmul_cuda.cu:236, 285) and runs at memory speed (one read and one write of the
 * tensor).  Callers that hold key rows already (key.transpose(-1, -2) of a row-major tensor) skip it.
 * WM_ERR_UNSUPPORTED, nothing launched, unless k has unit column stride, rows is 16-byte aligned,
 * N is a multiple of 16 bytes, the row stride of k is at least M (rows may be padded, they may not
 * overlap or run backwards), B <= 65535 and N <= 64 * 65535 (any M).  Callers fall back to their
 * own copy on that status, as the PyTorch extension does. */
int wm_key_rows(const wm_operand *k, void *rows, int64_t B, int64_t N, int64_t M, int dtype, void *stream);

/* 1 if the fused kernels exist for this shape, dtype and scale (layout aside), else 0. */
int wm_window_attention_supported(int64_t M, int64_t N, int64_t w, int dtype, double scale);

/* Human-readable name of a wm_status code (static string). */
const char *wm_status_string(int status);

/* WM_ABI_VERSION the library was built with. */
int wm_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* WINDOW_MATMUL_HIP_H */
