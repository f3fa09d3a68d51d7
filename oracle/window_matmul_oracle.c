/*
 * CPU restatement of the reference's banded matmul semantics.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP path is compared
 * against (tests/, the smoke check and the benchmark's cpu_baseline leg).  It
 * is never linked into, loaded by or called from the product library.
 *
 * Every function follows the loop nest of the reference's scalar CPU kernels
 * in csrc/window_matmul/cpu/window_matmul_cpu.cpp:
 *   - same iteration order  b -> s -> w -> h                     (cpu:35-46)
 *   - same window bounds    [max(0,s-ws), min(M,s+ws+1))         (cpu:39)
 *   - same band column      w_idx = w - s + ws                   (cpu:41)
 *   - outputs start at +0 so never-visited band entries are +0.0 (cpu:22)
 *   - accumulation happens in the storage type, in place         (cpu:43)
 * Layouts are the reference's contiguous ones: src (B,M,N), other = K^T
 * (B,N,M) for the window op; src = band (B,M,2ws+1), other (B,M,N) for the
 * unwindow op.
 *
 * Pinning (see tests/test_oracle.py): bit-exact against the reference's own
 * compiled CPU path where oracle/_ref builds; against a dense masked matmul in
 * float64; closed forms (all-ones inputs, one-hot rows, sliding-window sums);
 * adjoint identities between forward and backward; brute force on tiny sizes.
 */
#include <stdint.h>
#include <string.h>

#define WM_MAX(a, b) ((a) > (b) ? (a) : (b))
#define WM_MIN(a, b) ((a) < (b) ? (a) : (b))

#define WM_DEFINE_ORACLE(T, SUFFIX)                                                     \
  /* reference: window_matmul_fw_cpu, cpu:6-50 */                                       \
  void wm_oracle_window_fw_##SUFFIX(const T *src, const T *other, T *out, int64_t B,    \
                                    int64_t M, int64_t N, int64_t ws) {                 \
    const int64_t W = 2 * ws + 1;                                                       \
    memset(out, 0, sizeof(T) * (size_t)(B * M * W));                                    \
    for (int64_t b = 0; b < B; b++) {                                                   \
      const T *q = src + b * M * N;                                                     \
      const T *kt = other + b * N * M;                                                  \
      T *o = out + b * M * W;                                                           \
      for (int64_t s = 0; s < M; s++) {                                                 \
        const int64_t lo = WM_MAX((int64_t)0, s - ws), hi = WM_MIN(M, s + ws + 1);      \
        for (int64_t w = lo; w < hi; w++) {                                             \
          const int64_t w_idx = w - s + ws;                                             \
          for (int64_t h = 0; h < N; h++) o[s * W + w_idx] += q[s * N + h] * kt[h * M + w]; \
        }                                                                               \
      }                                                                                 \
    }                                                                                   \
  }                                                                                     \
  /* reference: window_matmul_bw_cpu, cpu:52-99 (both grads in one gather loop) */      \
  void wm_oracle_window_bw_##SUFFIX(const T *src, const T *other, const T *grad_out,    \
                                    T *grad_src, T *grad_other, int64_t B, int64_t M,   \
                                    int64_t N, int64_t ws) {                            \
    const int64_t W = 2 * ws + 1;                                                       \
    memset(grad_src, 0, sizeof(T) * (size_t)(B * M * N));                               \
    memset(grad_other, 0, sizeof(T) * (size_t)(B * N * M));                             \
    for (int64_t b = 0; b < B; b++) {                                                   \
      const T *q = src + b * M * N;                                                     \
      const T *kt = other + b * N * M;                                                  \
      const T *g = grad_out + b * M * W;                                                \
      T *gq = grad_src + b * M * N;                                                     \
      T *gk = grad_other + b * N * M;                                                   \
      for (int64_t s = 0; s < M; s++) {                                                 \
        const int64_t lo = WM_MAX((int64_t)0, s - ws), hi = WM_MIN(M, s + ws + 1);      \
        for (int64_t w = lo; w < hi; w++) {                                             \
          const int64_t w_idx = w - s + ws;                                             \
          for (int64_t h = 0; h < N; h++) {                                             \
            gq[s * N + h] += kt[h * M + w] * g[s * W + w_idx];                          \
            gk[h * M + s] += q[w * N + h] * g[w * W + (2 * ws - w_idx)];                \
          }                                                                             \
        }                                                                               \
      }                                                                                 \
    }                                                                                   \
  }                                                                                     \
  /* reference: unwindow_matmul_fw_cpu, cpu:101-144 */                                  \
  void wm_oracle_unwindow_fw_##SUFFIX(const T *src, const T *other, T *out, int64_t B,  \
                                      int64_t M, int64_t N, int64_t ws) {               \
    const int64_t W = 2 * ws + 1;                                                       \
    memset(out, 0, sizeof(T) * (size_t)(B * M * N));                                    \
    for (int64_t b = 0; b < B; b++) {                                                   \
      const T *a = src + b * M * W;                                                     \
      const T *v = other + b * M * N;                                                   \
      T *o = out + b * M * N;                                                           \
      for (int64_t s = 0; s < M; s++) {                                                 \
        const int64_t lo = WM_MAX((int64_t)0, s - ws), hi = WM_MIN(M, s + ws + 1);      \
        for (int64_t w = lo; w < hi; w++) {                                             \
          const int64_t w_idx = w - s + ws;                                             \
          for (int64_t h = 0; h < N; h++) o[s * N + h] += a[s * W + w_idx] * v[w * N + h]; \
        }                                                                               \
      }                                                                                 \
    }                                                                                   \
  }                                                                                     \
  /* reference: unwindow_matmul_bw_cpu, cpu:146-193 */                                  \
  void wm_oracle_unwindow_bw_##SUFFIX(const T *src, const T *other, const T *grad_out,  \
                                      T *grad_src, T *grad_other, int64_t B, int64_t M, \
                                      int64_t N, int64_t ws) {                          \
    const int64_t W = 2 * ws + 1;                                                       \
    memset(grad_src, 0, sizeof(T) * (size_t)(B * M * W));                               \
    memset(grad_other, 0, sizeof(T) * (size_t)(B * M * N));                             \
    for (int64_t b = 0; b < B; b++) {                                                   \
      const T *a = src + b * M * W;                                                     \
      const T *v = other + b * M * N;                                                   \
      const T *g = grad_out + b * M * N;                                                \
      T *ga = grad_src + b * M * W;                                                     \
      T *gv = grad_other + b * M * N;                                                   \
      for (int64_t s = 0; s < M; s++) {                                                 \
        const int64_t lo = WM_MAX((int64_t)0, s - ws), hi = WM_MIN(M, s + ws + 1);      \
        for (int64_t w = lo; w < hi; w++) {                                             \
          const int64_t w_idx = w - s + ws;                                             \
          for (int64_t h = 0; h < N; h++) {                                             \
            ga[s * W + w_idx] += v[w * N + h] * g[s * N + h];                           \
            gv[s * N + h] += a[w * W + (2 * ws - w_idx)] * g[w * N + h];                \
          }                                                                             \
        }                                                                               \
      }                                                                                 \
    }                                                                                   \
  }

WM_DEFINE_ORACLE(float, f32)
WM_DEFINE_ORACLE(double, f64)

int wm_oracle_abi_version(void) { return 1; }
