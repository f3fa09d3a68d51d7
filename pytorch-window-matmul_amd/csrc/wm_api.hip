// extern "C" entry points of libwindow_matmul_hip.so: argument validation and
// the mapping of the four ops onto the three banded primitives.
#include "wm_common.hpp"

#include <mutex>

// Workspace of wm_window_attention_backward_static: the two per-row values the first backward
// kernel hands to the second.  One copy per GPU the library runs on, held until the process ends.  In
// host code this name is only a handle for hipGetSymbolAddress, never a device address.
static __device__ __align__(256) float scratch[2 * WM_STATIC_SCRATCH_ROWS];

namespace wm {
namespace {

constexpr int kMaxDevices = 64;
std::mutex scratch_lock;
float *scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, looked up once per GPU

// Address of `scratch` on the current device.
int static_scratch(float **out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return WM_ERR_LAUNCH_FAILED;
  std::lock_guard<std::mutex> guard(scratch_lock);
  if (scratch_ptr[dev] == nullptr) {
    void *p = nullptr;
    const hipError_t err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess || p == nullptr) return err == hipErrorNoBinaryForGpu ? WM_ERR_NO_DEVICE_CODE : WM_ERR_LAUNCH_FAILED;
    scratch_ptr[dev] = static_cast<float *>(p);
  }
  *out = scratch_ptr[dev];
  return WM_OK;
}

int check_common(int64_t B, int64_t M, int64_t N, int64_t w, int dtype, unsigned flags) {
  if (dtype < WM_DTYPE_F32 || dtype > WM_DTYPE_F64) return WM_ERR_BAD_DTYPE;
  if (flags & ~(WM_FLAG_FORCE_STRIDED | WM_FLAG_NO_ALIGNED_BAND | WM_FLAG_NO_NARROW_BAND | WM_FLAG_NO_LDS_DIRECT | WM_FLAG_NO_SPLIT_F32)) return WM_ERR_BAD_FLAGS;
  const int64_t lim = 0x7fffffff;
  if (B < 0 || M < 0 || N < 0 || w < 0) return WM_ERR_BAD_SHAPE;
  if (B > lim || M > lim || N > lim || w > (lim - 1) / 2) return WM_ERR_BAD_SHAPE;
  return WM_OK;
}

bool missing(const wm_operand *op) { return op == nullptr || op->data == nullptr; }

int to_status(hipError_t err) {
  if (err == hipSuccess) return WM_OK;
  if (err == hipErrorNoBinaryForGpu || err == hipErrorInvalidDeviceFunction || err == hipErrorSharedObjectInitFailed)
    return WM_ERR_NO_DEVICE_CODE;
  return WM_ERR_LAUNCH_FAILED;
}

typedef bool (*mfma_fn)(const Problem &, const View &, const View &, const View &, hipError_t *);
typedef hipError_t (*strided_fn)(const Problem &, const View &, const View &, const View &);

// Kernel choice per primitive: vector-ALU kernels (the narrowest windows), else narrow-band MFMA
// family, else wide-band MFMA family (all 16-bit storage except the float32 vector kernels), else
// the float32 MFMA family, else the tile family (float64; every layout and head width), else strided.
// The tiled families launch one workgroup per (batch element, block of at least 16 rows), with the
// batch count rounded up to a multiple of 8; a grid beyond 2^31 - 1 workgroups does not exist, so
// such extents run on the strided kernels, whose grid strides over the work.
bool tiled_grid_fits(int64_t B, int64_t M) { return ((B + 7) / 8) * 8 * ((M + 15) / 16) <= 0x7fffffff; }

int run_primitive(mfma_fn narrow, mfma_fn vector, mfma_fn fast, mfma_fn f32, mfma_fn tile, strided_fn slow,
                  const Problem &p, const View &a, const View &y, const View &c) {
  hipError_t err = hipSuccess;
  if (!(p.flags & WM_FLAG_FORCE_STRIDED) && tiled_grid_fits(p.B, p.M)) {
    if (vector && !(p.flags & WM_FLAG_NO_NARROW_BAND) && vector(p, a, y, c, &err)) return to_status(err);
    if (narrow && !(p.flags & WM_FLAG_NO_NARROW_BAND) && narrow(p, a, y, c, &err)) return to_status(err);
    if (fast(p, a, y, c, &err)) return to_status(err);
    if (f32(p, a, y, c, &err)) return to_status(err);
    if (tile(p, a, y, c, &err)) return to_status(err);
  }
  return to_status(slow(p, a, y, c));
}

// The one-launch backward of the vector-ALU kernels stands aside for every flag that selects kernels by hand.
bool fused_backward_allowed(const Problem &p) {
  return !(p.flags & (WM_FLAG_FORCE_STRIDED | WM_FLAG_NO_NARROW_BAND)) && tiled_grid_fits(p.B, p.M);
}

int p1(const Problem &p, const View &x, const View &y, const View &c) {
  return run_primitive(try_launch_small_p1, try_launch_vector_p1, try_launch_mfma_p1, try_launch_f32_p1,
                       try_launch_tile_p1, launch_strided_p1, p, x, y, c);
}
int p2(const Problem &p, const View &a, const View &y, const View &c) {
  return run_primitive(try_launch_small_p2, try_launch_vector_p2, try_launch_mfma_p2, try_launch_f32_p2,
                       try_launch_tile_p2, launch_strided_p2, p, a, y, c);
}
int p3(const Problem &p, const View &a, const View &y, const View &c) {
  return run_primitive(try_launch_small_p3, try_launch_vector_p3, try_launch_mfma_p3, try_launch_f32_p3,
                       try_launch_tile_p3, launch_strided_p3, p, a, y, c);
}

}  // namespace
}  // namespace wm

using namespace wm;

extern "C" {

int wm_window_matmul_forward(const wm_operand *q, const wm_operand *k, const wm_operand *a, int64_t B,
                             int64_t M, int64_t N, int64_t w, int dtype, unsigned flags, void *stream) {
  if (int st = check_common(B, M, N, w, dtype, flags)) return st;
  if (B == 0 || M == 0) return WM_OK;  // nothing to write
  if (missing(a) || (N > 0 && (missing(q) || missing(k)))) return WM_ERR_NULL_POINTER;
  const Problem p{B, M, N, w, dtype, flags, (hipStream_t)stream};
  const wm_operand none{a->data, 0, 0, 0};  // N == 0: operands are never dereferenced
  // K arrives as (B,N,M); the primitives read it as rows c, columns h.
  return p1(p, make_view(N > 0 ? q : &none), transposed(make_view(N > 0 ? k : &none)), make_view(a));
}

int wm_window_matmul_backward(const wm_operand *q, const wm_operand *k, const wm_operand *grad_a,
                              const wm_operand *grad_q, const wm_operand *grad_k, int64_t B, int64_t M,
                              int64_t N, int64_t w, int dtype, unsigned flags, void *stream) {
  if (int st = check_common(B, M, N, w, dtype, flags)) return st;
  if (B == 0 || M == 0 || N == 0) return WM_OK;
  if (missing(q) || missing(k) || missing(grad_a)) return WM_ERR_NULL_POINTER;
  if ((grad_q && !grad_q->data) || (grad_k && !grad_k->data)) return WM_ERR_NULL_POINTER;
  const Problem p{B, M, N, w, dtype, flags, (hipStream_t)stream};
  if (grad_q && grad_k && fused_backward_allowed(p)) {  // small problems: both products in one launch
    hipError_t err = hipSuccess;
    if (try_launch_vector_window_backward(p, make_view(grad_a), transposed(make_view(k)), make_view(q), make_view(grad_q),
                                          transposed(make_view(grad_k)), &err))
      return to_status(err);
  }
  if (grad_q)
    if (int st = p2(p, make_view(grad_a), transposed(make_view(k)), make_view(grad_q))) return st;
  if (grad_k)
    if (int st = p3(p, make_view(grad_a), make_view(q), transposed(make_view(grad_k)))) return st;
  return WM_OK;
}

int wm_unwindow_matmul_forward(const wm_operand *a, const wm_operand *v, const wm_operand *o, int64_t B,
                               int64_t M, int64_t N, int64_t w, int dtype, unsigned flags, void *stream) {
  if (int st = check_common(B, M, N, w, dtype, flags)) return st;
  if (B == 0 || M == 0 || N == 0) return WM_OK;
  if (missing(a) || missing(v) || missing(o)) return WM_ERR_NULL_POINTER;
  const Problem p{B, M, N, w, dtype, flags, (hipStream_t)stream};
  return p2(p, make_view(a), make_view(v), make_view(o));
}

int wm_unwindow_matmul_backward(const wm_operand *a, const wm_operand *v, const wm_operand *grad_o,
                                const wm_operand *grad_a, const wm_operand *grad_v, int64_t B, int64_t M,
                                int64_t N, int64_t w, int dtype, unsigned flags, void *stream) {
  if (int st = check_common(B, M, N, w, dtype, flags)) return st;
  if (B == 0 || M == 0) return WM_OK;
  if ((grad_a && !grad_a->data) || (grad_v && !grad_v->data)) return WM_ERR_NULL_POINTER;
  if (N > 0 && (missing(a) || missing(v) || missing(grad_o))) return WM_ERR_NULL_POINTER;
  const Problem p{B, M, N, w, dtype, flags, (hipStream_t)stream};
  if (grad_a && grad_v && N > 0 && fused_backward_allowed(p)) {  // small problems: both products in one launch
    hipError_t err = hipSuccess;
    if (try_launch_vector_unwindow_backward(p, make_view(a), make_view(v), make_view(grad_o), make_view(grad_a),
                                            make_view(grad_v), &err))
      return to_status(err);
  }
  if (grad_a) {
    const wm_operand none{grad_a->data, 0, 0, 0};  // N == 0: grad_a is all +0.0
    if (int st = p1(p, make_view(N > 0 ? grad_o : &none), make_view(N > 0 ? v : &none), make_view(grad_a)))
      return st;
  }
  if (grad_v && N > 0)
    if (int st = p3(p, make_view(a), make_view(grad_o), make_view(grad_v))) return st;
  return WM_OK;
}

int wm_band_softmax_forward(const wm_operand *a, const wm_operand *p, int64_t B, int64_t M, int64_t w, double scale,
                            int mask_out_of_range, int dtype, unsigned flags, void *stream) {
  if (int st = check_common(B, M, 0, w, dtype, flags)) return st;
  if (!(scale == scale)) return WM_ERR_BAD_SHAPE;
  if (B == 0 || M == 0) return WM_OK;
  if (missing(a) || missing(p)) return WM_ERR_NULL_POINTER;
  const Problem prob{B, M, 0, w, dtype, flags, static_cast<hipStream_t>(stream)};
  return to_status(launch_band_softmax_forward(prob, make_view(a), make_view(p), scale, mask_out_of_range));
}

int wm_band_softmax_backward(const wm_operand *p, const wm_operand *grad_p, const wm_operand *grad_a, int64_t B,
                             int64_t M, int64_t w, double scale, int mask_out_of_range, int dtype, unsigned flags,
                             void *stream) {
  if (int st = check_common(B, M, 0, w, dtype, flags)) return st;
  if (!(scale == scale)) return WM_ERR_BAD_SHAPE;
  if (B == 0 || M == 0) return WM_OK;
  if (missing(p) || missing(grad_p) || missing(grad_a)) return WM_ERR_NULL_POINTER;
  const Problem prob{B, M, 0, w, dtype, flags, static_cast<hipStream_t>(stream)};
  return to_status(launch_band_softmax_backward(prob, make_view(p), make_view(grad_p), make_view(grad_a), scale,
                                                mask_out_of_range));
}

int wm_window_attention_forward(const wm_operand *q, const wm_operand *k, const wm_operand *v, const wm_operand *o,
                                float *lse, int64_t B, int64_t M, int64_t N, int64_t w, double scale,
                                int mask_out_of_range, int dtype, unsigned flags, void *stream) {
  if (int st = check_common(B, M, N, w, dtype, flags)) return st;
  if (!(scale == scale)) return WM_ERR_BAD_SHAPE;
  if (B == 0 || M == 0) return WM_OK;
  if (missing(q) || missing(k) || missing(v) || missing(o)) return WM_ERR_NULL_POINTER;
  const Problem prob{B, M, N, w, dtype, flags, static_cast<hipStream_t>(stream)};
  hipError_t err = hipSuccess;
  if (!try_launch_attention_forward(prob, make_view(q), make_view(k), make_view(v), make_view(o), lse, scale,
                                    mask_out_of_range, &err))
    return WM_ERR_UNSUPPORTED;
  return to_status(err);
}

int wm_window_attention_backward(const wm_operand *q, const wm_operand *k, const wm_operand *v, const wm_operand *o,
                                 const float *lse, const wm_operand *grad_o, const wm_operand *grad_q,
                                 const wm_operand *grad_k, const wm_operand *grad_v, float *delta, int64_t B,
                                 int64_t M, int64_t N, int64_t w, double scale, int dtype, unsigned flags,
                                 void *stream) {
  if (int st = check_common(B, M, N, w, dtype, flags)) return st;
  if (!(scale == scale)) return WM_ERR_BAD_SHAPE;
  if (B == 0 || M == 0) return WM_OK;
  if (missing(q) || missing(k) || missing(v) || missing(o) || missing(grad_o) || lse == nullptr || delta == nullptr)
    return WM_ERR_NULL_POINTER;
  if (grad_q == nullptr && grad_k == nullptr && grad_v == nullptr) return WM_OK;
  if ((grad_q && !grad_q->data) || (grad_k && !grad_k->data) || (grad_v && !grad_v->data)) return WM_ERR_NULL_POINTER;
  const Problem prob{B, M, N, w, dtype, flags, static_cast<hipStream_t>(stream)};
  const View none{nullptr, 0, 0, 0};
  hipError_t err = hipSuccess;
  if (!try_launch_attention_backward(prob, make_view(q), make_view(k), make_view(v), make_view(o), make_view(grad_o),
                                     lse, delta, grad_q ? make_view(grad_q) : none, grad_k ? make_view(grad_k) : none,
                                     grad_v ? make_view(grad_v) : none, scale, &err))
    return WM_ERR_UNSUPPORTED;
  return to_status(err);
}

int wm_window_attention_backward_static(const wm_operand *q, const wm_operand *k, const wm_operand *v,
                                        const wm_operand *o, const float *lse, const wm_operand *grad_o,
                                        const wm_operand *grad_q, const wm_operand *grad_k, const wm_operand *grad_v,
                                        int64_t B, int64_t M, int64_t N, int64_t w, double scale, int dtype,
                                        unsigned flags, void *stream) {
  if (int st = check_common(B, M, N, w, dtype, flags)) return st;
  if (B * M > (int64_t)WM_STATIC_SCRATCH_ROWS) return WM_ERR_SCRATCH_TOO_SMALL;
  if (B == 0 || M == 0) return WM_OK;
  // Every row of the workspace that the second kernel reads is written by the first one in the
  // same call, so nothing has to be cleared between calls.
  float *delta = nullptr;
  if (int st = static_scratch(&delta)) return st;
  return wm_window_attention_backward(q, k, v, o, lse, grad_o, grad_q, grad_k, grad_v, delta, B, M, N, w, scale, dtype,
                                      flags, stream);
}

int wm_key_rows(const wm_operand *k, void *rows, int64_t B, int64_t N, int64_t M, int dtype, void *stream) {
  if (int st = check_common(B, M, N, 0, dtype, 0)) return st;
  if (missing(k) || rows == nullptr) return WM_ERR_NULL_POINTER;
  if (k->stride_c != 1) return WM_ERR_UNSUPPORTED;
  hipError_t err = hipSuccess;
  if (!try_launch_transpose(k->data, rows, B, N, M, k->stride_b, k->stride_r, (int)dtype_size(dtype),
                            static_cast<hipStream_t>(stream), &err))
    return WM_ERR_UNSUPPORTED;
  return to_status(err);
}

int wm_window_attention_supported(int64_t M, int64_t N, int64_t w, int dtype, double scale) {
  return attention_supports(M, N, w, dtype, scale) ? 1 : 0;
}

const char *wm_band_softmax_kernel_choice(int64_t w, int dtype, int contiguous, int backward, unsigned flags) {
  if (w < 0 || dtype < WM_DTYPE_F32 || dtype > WM_DTYPE_F64) return "invalid";
  if (contiguous && !(flags & WM_FLAG_FORCE_STRIDED) && band_softmax_staged(2 * w + 1, dtype, backward != 0))
    return "staged_softmax";
  return "strided_softmax";
}

const char *wm_kernel_choice(int op, int64_t B, int64_t M, int64_t N, int64_t w, int dtype, int fast,
                             unsigned flags) {
  if (op < 1 || op > 3) return "invalid";
  if (!(flags & WM_FLAG_FORCE_STRIDED) && fast && tiled_grid_fits(B, M)) {
    if (!(flags & WM_FLAG_NO_NARROW_BAND) && vector_supports(op, M, N, w, dtype)) {
      static const char *names[] = {"vector_p1", "vector_p2", "vector_p3"};
      return names[op - 1];
    }
    if (!(flags & WM_FLAG_NO_NARROW_BAND) && small_supports(op, M, N, w, dtype, flags)) {
      static const char *names[] = {"narrow_p1", "narrow_p2", "narrow_p3"};
      return names[op - 1];
    }
    if (mfma_supports(op, B, M, N, w, dtype)) {
      static const char *names[] = {"mfma_p1", "mfma_p2", "mfma_p3"};
      return names[op - 1];
    }
    if (f32_split_supports(op, M, N, w, dtype, flags)) {
      static const char *names[] = {"f32_split_p1", "f32_split_p2", "f32_split_p3"};
      return names[op - 1];
    }
    if (f32_supports(op, M, N, w, dtype)) {
      static const char *names[] = {"f32_mfma_p1", "f32_mfma_p2", "f32_mfma_p3"};
      return names[op - 1];
    }
  }
  if (!(flags & WM_FLAG_FORCE_STRIDED) && tiled_grid_fits(B, M) && tile_supports(op, M, N, w, dtype)) {
    static const char *names[] = {"tile_p1", "tile_p2", "tile_p3"};  // takes every layout
    return names[op - 1];
  }
  static const char *names[] = {"strided_p1", "strided_p2", "strided_p3"};
  return names[op - 1];
}

const char *wm_status_string(int status) {
  switch (status) {
    case WM_OK: return "ok";
    case WM_ERR_NULL_POINTER: return "null operand or data pointer";
    case WM_ERR_BAD_SHAPE: return "negative or oversized extent";
    case WM_ERR_BAD_DTYPE: return "unknown dtype";
    case WM_ERR_BAD_FLAGS: return "unknown flag bit";
    case WM_ERR_LAUNCH_FAILED: return "kernel launch failed";
    case WM_ERR_UNSUPPORTED: return "this entry point has no kernel for the given shape, dtype or layout";
    case WM_ERR_SCRATCH_TOO_SMALL: return "B * M exceeds WM_STATIC_SCRATCH_ROWS, the rows of the library's static workspace";
    case WM_ERR_NO_DEVICE_CODE: return "no device code for this GPU (library is built for gfx950)";
    default: return "unknown status";
  }
}

int wm_abi_version(void) { return WM_ABI_VERSION; }

}  // extern "C"
