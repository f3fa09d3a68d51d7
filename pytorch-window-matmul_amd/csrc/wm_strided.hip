// Strided kernel family: any dtype (f32, f16, bf16, f64), any element strides,
// any M / N / w.  One thread owns one output element and walks its contraction,
// so every output is written exactly once (no atomics) and out-of-range band
// entries are stored as literal +0.0.  These kernels are the correctness
// backstop for layouts and dtypes the MFMA family does not take; they lean on
// the L2 for operand reuse and are not tuned beyond coalescing the inner lanes.
#include "wm_common.hpp"
#include "wm_types.hpp"

namespace wm {
namespace {

constexpr int kThreads = 256;

// P1: C[b,i,j] = sum_h X[b,i,h] * Y[b,i+j-w,h];  lanes run along j.
template <typename T>
__global__ __launch_bounds__(kThreads) void strided_p1_kernel(const T *__restrict__ X, const T *__restrict__ Y,
                                                              T *__restrict__ C, int64_t total, int M, int N,
                                                              int w, int64_t xsb, int64_t xsr, int64_t xsc,
                                                              int64_t ysb, int64_t ysr, int64_t ysc, int64_t csb,
                                                              int64_t csr, int64_t csc) {
  typedef typename Acc<T>::type acc_t;
  const int W = 2 * w + 1;
  for (int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * kThreads) {
    const int j = (int)(idx % W);
    const int64_t bi = idx / W;
    const int i = (int)(bi % M);
    const int64_t b = bi / M;
    const int c = i + j - w;
    acc_t acc = 0;
    if (c >= 0 && c < M) {
      const T *xr = X + b * xsb + (int64_t)i * xsr;
      const T *yr = Y + b * ysb + (int64_t)c * ysr;
      for (int h = 0; h < N; ++h) acc += to_acc<T>(xr[(int64_t)h * xsc]) * to_acc<T>(yr[(int64_t)h * ysc]);
    }
    C[b * csb + (int64_t)i * csr + (int64_t)j * csc] = from_acc<T>(acc);
  }
}

// P2: C[b,i,h] = sum_j A[b,i,j] * Y[b,i+j-w,h];  lanes run along h.
template <typename T>
__global__ __launch_bounds__(kThreads) void strided_p2_kernel(const T *__restrict__ A, const T *__restrict__ Y,
                                                              T *__restrict__ C, int64_t total, int M, int N,
                                                              int w, int64_t asb, int64_t asr, int64_t asc,
                                                              int64_t ysb, int64_t ysr, int64_t ysc, int64_t csb,
                                                              int64_t csr, int64_t csc) {
  typedef typename Acc<T>::type acc_t;
  for (int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * kThreads) {
    const int h = (int)(idx % N);
    const int64_t bi = idx / N;
    const int i = (int)(bi % M);
    const int64_t b = bi / M;
    const int lo = max(i - w, 0), hi = min(i + w, M - 1);
    const T *ar = A + b * asb + (int64_t)i * asr;
    const T *yb = Y + b * ysb + (int64_t)h * ysc;
    acc_t acc = 0;
    for (int c = lo; c <= hi; ++c)
      acc += to_acc<T>(ar[(int64_t)(c - i + w) * asc]) * to_acc<T>(yb[(int64_t)c * ysr]);
    C[b * csb + (int64_t)i * csr + (int64_t)h * csc] = from_acc<T>(acc);
  }
}

// P3: C[b,c,h] = sum_r A[b,r,c-r+w] * Y[b,r,h];  output-stationary gather, lanes along h.
template <typename T>
__global__ __launch_bounds__(kThreads) void strided_p3_kernel(const T *__restrict__ A, const T *__restrict__ Y,
                                                              T *__restrict__ C, int64_t total, int M, int N,
                                                              int w, int64_t asb, int64_t asr, int64_t asc,
                                                              int64_t ysb, int64_t ysr, int64_t ysc, int64_t csb,
                                                              int64_t csr, int64_t csc) {
  typedef typename Acc<T>::type acc_t;
  for (int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * kThreads) {
    const int h = (int)(idx % N);
    const int64_t bc = idx / N;
    const int c = (int)(bc % M);
    const int64_t b = bc / M;
    const int lo = max(c - w, 0), hi = min(c + w, M - 1);
    const T *ab = A + b * asb;
    const T *yb = Y + b * ysb + (int64_t)h * ysc;
    acc_t acc = 0;
    for (int r = lo; r <= hi; ++r)
      acc += to_acc<T>(ab[(int64_t)r * asr + (int64_t)(c - r + w) * asc]) * to_acc<T>(yb[(int64_t)r * ysr]);
    C[b * csb + (int64_t)c * csr + (int64_t)h * csc] = from_acc<T>(acc);
  }
}

inline unsigned grid_for(int64_t total) {
  const int64_t blocks = (total + kThreads - 1) / kThreads;
  const int64_t cap = 1 << 20;  // grid-stride beyond this many workgroups
  return (unsigned)(blocks < cap ? blocks : cap);
}

template <typename T>
hipError_t run(int which, const Problem &p, const View &a, const View &y, const View &c) {
  const int64_t W = 2 * p.w + 1;
  const int64_t total = p.B * p.M * (which == 1 ? W : p.N);
  if (total == 0) return hipSuccess;
  const dim3 grid(grid_for(total)), block(kThreads);
  const T *ap = (const T *)a.data;
  const T *yp = (const T *)y.data;
  T *cp = (T *)c.data;
  const int M = (int)p.M, N = (int)p.N, w = (int)p.w;
  if (which == 1)
    hipLaunchKernelGGL(strided_p1_kernel<T>, grid, block, 0, p.stream, ap, yp, cp, total, M, N, w, a.sb, a.sr,
                       a.sc, y.sb, y.sr, y.sc, c.sb, c.sr, c.sc);
  else if (which == 2)
    hipLaunchKernelGGL(strided_p2_kernel<T>, grid, block, 0, p.stream, ap, yp, cp, total, M, N, w, a.sb, a.sr,
                       a.sc, y.sb, y.sr, y.sc, c.sb, c.sr, c.sc);
  else
    hipLaunchKernelGGL(strided_p3_kernel<T>, grid, block, 0, p.stream, ap, yp, cp, total, M, N, w, a.sb, a.sr,
                       a.sc, y.sb, y.sr, y.sc, c.sb, c.sr, c.sc);
  return hipGetLastError();
}

hipError_t dispatch(int which, const Problem &p, const View &a, const View &y, const View &c) {
  switch (p.dtype) {
    case WM_DTYPE_F32: return run<float>(which, p, a, y, c);
    case WM_DTYPE_F16: return run<f16_t>(which, p, a, y, c);
    case WM_DTYPE_BF16: return run<bf16_t>(which, p, a, y, c);
    case WM_DTYPE_F64: return run<double>(which, p, a, y, c);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

hipError_t launch_strided_p1(const Problem &p, const View &x, const View &y, const View &c) {
  return dispatch(1, p, x, y, c);
}
hipError_t launch_strided_p2(const Problem &p, const View &a, const View &y, const View &c) {
  return dispatch(2, p, a, y, c);
}
hipError_t launch_strided_p3(const Problem &p, const View &a, const View &y, const View &c) {
  return dispatch(3, p, a, y, c);
}

}  // namespace wm
