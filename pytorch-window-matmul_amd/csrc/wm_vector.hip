// Vector-ALU kernels for very narrow bands on gfx950 (16-bit storage and float32, float32 accumulate).
//
// The narrow-band MFMA kernels multiply 32-row tiles against at least 48 dense columns and the
// float32 MFMA kernels walk 128-row tiles in chunks of 32 columns: mostly empty work when the band
// is a few entries wide.  For these windows the band-in products
//     P2  C[i,h] = sum_j A[i,j] Y[i+j-w,h]          P3  C[c,h] = sum_r A[r,c-r+w] Y[r,h]
// are 2w+1 multiply-adds per output element on operands that are streamed once: far too little
// arithmetic for the matrix pipe to matter, so each thread simply owns 16 bytes of one output row
// (8 or 4 consecutive columns) and walks the 2w+1 terms: one LDS read of the band entry (the same
// address for the threads of a row), one 16-byte LDS read of the Y row piece, 8 FMAs on the
// unpacked values (16-bit) or 4 FMAs (float32).  (Packed dot products that pair the entry with one
// value and a zero with its neighbour need no unpacking but are no faster, LDS reads sharing the
// bound, and would let an Inf in one column of Y turn the neighbouring output column into NaN.)
// The workgroup first copies what it needs into LDS with coalesced 16-byte loads (its band rows
// as one flat image, the Y rows they reach row-major, zero outside the sequence); the result
// leaves as 16-byte non-temporal stores, consecutive threads on consecutive pieces of a row.
// The band-out product  P1  band[i,j] = sum_h X[i,h] Y[i+j-w,h]  gets the same treatment (float32 up
// to w = 14 where the narrow-band MFMA kernel does not apply, i.e. N not a multiple of 16 or above
// 64; for 16-bit storage that kernel is faster at every w): X and Y rows
// in LDS, one thread per band entry, consecutive threads on consecutive entries of the flat band.  One barrier per workgroup; no atomics.
#include "wm_mfma_common.hpp"

#include <algorithm>

namespace wm {
namespace {

#ifndef WM_VECTOR_MAX_W
#define WM_VECTOR_MAX_W 3
#endif
constexpr int VECTOR_MAX_W = WM_VECTOR_MAX_W;
#ifndef WM_VECTOR_F32_MAX_W
#define WM_VECTOR_F32_MAX_W 14
#endif
constexpr int VECTOR_F32_MAX_W = WM_VECTOR_F32_MAX_W;
typedef float f32x4v __attribute__((ext_vector_type(4)));

// A 16-bit storage value, and the two values of a dword, as floats.
template <typename T>
__device__ __forceinline__ float to_float(uint16_t x);
template <>
__device__ __forceinline__ float to_float<bf16_t>(uint16_t x) {
  return __builtin_bit_cast(float, (uint32_t)x << 16);
}
template <>
__device__ __forceinline__ float to_float<f16_t>(uint16_t x) {
  return (float)__builtin_bit_cast(_Float16, x);
}
template <typename T>
__device__ __forceinline__ void unpack2(uint32_t x, float &lo, float &hi);
template <>
__device__ __forceinline__ void unpack2<bf16_t>(uint32_t x, float &lo, float &hi) {
  lo = __builtin_bit_cast(float, x << 16);
  hi = __builtin_bit_cast(float, x & 0xffff0000u);
}
template <>
__device__ __forceinline__ void unpack2<f16_t>(uint32_t x, float &lo, float &hi) {
  lo = (float)__builtin_bit_cast(_Float16, (uint16_t)x);
  hi = (float)__builtin_bit_cast(_Float16, (uint16_t)(x >> 16));
}

// Storage element of a type tag, and the float32 "tag".
struct f32_t {};
template <typename T>
struct Elem {
  typedef uint16_t type;
};
template <>
struct Elem<f32_t> {
  typedef float type;
};

// TRANSPOSED false: P2 (rows = band rows i).  TRANSPOSED true: P3 (rows = output rows c, the
// contraction runs over the band rows r = c-w .. c+w).
template <typename T, int NK, bool TRANSPOSED>  // N = 16 NK (16-bit) or 8 NK (float32): 2 NK pieces per row
__device__ __forceinline__ void vector_band_in_body(const typename Elem<T>::type *__restrict__ A,
                                                    const typename Elem<T>::type *__restrict__ Y,
                                                    typename Elem<T>::type *__restrict__ C, int B, int M, int w,
                                                    int nblk, int vrows, int64_t asb, int64_t ysb, int64_t ysr,
                                                    int64_t csb, int64_t csr) {
  typedef typename Elem<T>::type E;
  constexpr int VEC = 16 / sizeof(E);       // elements per 16-byte piece
  constexpr int NCG = 2 * NK, N = NCG * VEC;  // 16-byte column groups per row
  constexpr int SY = N + VEC;               // Y image rows 16 bytes apart mod 128
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  E *lds = reinterpret_cast<E *>(lds_raw);

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x;
  const int W = 2 * w + 1;
  const int o0 = blk * vrows;                      // first output row
  const int orows = min(vrows, M - o0);
  // rows held in LDS: Y rows [y0, y0 + yrows) (may reach outside the sequence: zeros), band rows
  // [a0, a0 + arows) (inside the sequence)
  const int y0 = o0 - w, yrows = orows + 2 * w;
  const int a0 = TRANSPOSED ? max(o0 - w, 0) : o0;
  const int a1 = TRANSPOSED ? min(o0 + orows - 1 + w, M - 1) : o0 + orows - 1;
  const int arows = a1 - a0 + 1;
  const E *Ab = A + (int64_t)b * asb + (int64_t)a0 * W;
  const E *Yb = Y + (int64_t)b * ysb;
  // flat band image in whole aligned 16-byte chunks: image element e is band element e - delta
  const int delta = (int)((reinterpret_cast<uintptr_t>(Ab) / sizeof(E)) & (VEC - 1));
  const int n_el = arows * W;
  const int chunks = (delta + n_el + VEC - 1) / VEC;
  E *aimg = lds;
  E *yimg = lds + (((vrows + 2 * w) * W + 2 * VEC + VEC - 1) & ~(VEC - 1));  // sized for the largest image
  const int ychunks = yrows * NCG;

  // loads go out in batches of 8 per thread before any of them is used
  constexpr int BATCH = 8;
  for (int base = 0; base < chunks + ychunks; base += BATCH * kThreads) {
    u32x4 reg[BATCH];
#pragma unroll
    for (int s = 0; s < BATCH; ++s) {
      const int q = base + s * kThreads + tid;
      const int qy = q - chunks, yr = qy / NCG, hg = qy - yr * NCG, c = y0 + yr;
      const E *src = q < chunks ? Ab - delta + VEC * q : Yb + (int64_t)c * ysr + VEC * hg;
      const bool ok = q < chunks || (q < chunks + ychunks && c >= 0 && c < M);
      reg[s] = *reinterpret_cast<const u32x4 *>(ok ? src : A);
    }
#pragma unroll
    for (int s = 0; s < BATCH; ++s) {
      const int q = base + s * kThreads + tid;
      const int qy = q - chunks, yr = qy / NCG, hg = qy - yr * NCG, c = y0 + yr;
      if (q < chunks)
        *reinterpret_cast<u32x4 *>(aimg + VEC * q) = reg[s];
      else if (q < chunks + ychunks)
        *reinterpret_cast<u32x4 *>(yimg + yr * SY + VEC * hg) = mask_row_chunk(reg[s], (c >= 0) & (c < M));
    }
  }
  __syncthreads();

  // A thread owns one 16-byte piece of two consecutive output rows o, o + 1: they share all but one of
  // their Y rows, so every Y piece is read (and unpacked) once for both.  Pair term u = 0 .. 2w+1 is the
  // Y row o - w + u (image row r + u); it is term u of row o (u <= 2w) and term u - 1 of row o + 1 (u >= 1).
  auto entry = [&](const E *p) -> float {
    if constexpr (sizeof(E) == 2)
      return to_float<T>(*p);
    else
      return *p;
  };
  auto add_piece = [&](float a, const u32x4 &y, float(&acc)[VEC]) {
    if constexpr (sizeof(E) == 2) {
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        float lo, hi;
        unpack2<T>(y[d], lo, hi);
        acc[2 * d] = __builtin_fmaf(a, lo, acc[2 * d]);
        acc[2 * d + 1] = __builtin_fmaf(a, hi, acc[2 * d + 1]);
      }
    } else {
      const f32x4v yf = __builtin_bit_cast(f32x4v, y);  // (a bit cast of one element y[d] reads element 0)
#pragma unroll
      for (int d = 0; d < 4; ++d) acc[d] = __builtin_fmaf(a, yf[d], acc[d]);
    }
  };
  auto store_piece = [&](const float(&acc)[VEC], int o, int hg) {
    u32x4 out;
    if constexpr (sizeof(E) == 2) {
      out = u32x4{Mma<T>::pack2(acc[0], acc[1]), Mma<T>::pack2(acc[2], acc[3]), Mma<T>::pack2(acc[4], acc[5]),
                  Mma<T>::pack2(acc[6], acc[7])};
    } else {
      out = u32x4{__builtin_bit_cast(uint32_t, acc[0]), __builtin_bit_cast(uint32_t, acc[1]),
                  __builtin_bit_cast(uint32_t, acc[2]), __builtin_bit_cast(uint32_t, acc[3])};
    }
    __builtin_nontemporal_store(out, reinterpret_cast<u32x4 *>(C + (int64_t)b * csb + (int64_t)o * csr + VEC * hg));
  };
  const int npairs = (orows + 1) >> 1;
  for (int item = tid; item < npairs * NCG; item += kThreads) {
    const int pr = item / NCG, hg = item - pr * NCG;
    const int r = 2 * pr, o = o0 + r;  // first row of the pair
    const bool has_b = r + 1 < orows;
    float acc_a[VEC], acc_b[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc_a[e] = 0.f, acc_b[e] = 0.f;
    const int u_lo = max(0, w - o), u_hi = min(2 * w + 1, M - 1 - o + w);  // Y rows inside the sequence
    // band entries of pair term u, as image indices:
    //   P2: row o: (o - a0) W + u;                 row o + 1: (o + 1 - a0) W + u - 1;   next term +1
    //   P3: row o: (o - w + u - a0) W + 2w - u;    row o + 1: the entry right of it;    next term +W - 1
    const int a_step = TRANSPOSED ? W - 1 : 1;
    const int u1 = max(u_lo, 1), u2 = min(u_hi, 2 * w);  // terms that belong to both rows
    const E *pa = aimg + delta + (TRANSPOSED ? (o - w + u1 - a0) * W + 2 * w - u1 : (o - a0) * W + u1);
    const E *pb = !has_b ? pa : TRANSPOSED ? pa + 1 : pa + W - 1;
    const E *yp = yimg + (r + u1) * SY + VEC * hg;
    if (u_lo == 0)  // Y row o - w: first term of row o only
      add_piece(entry(pa - a_step), *reinterpret_cast<const u32x4 *>(yp - SY), acc_a);
    for (int u = u1; u <= u2; ++u) {
      const u32x4 y = *reinterpret_cast<const u32x4 *>(yp);
      add_piece(entry(pa), y, acc_a);
      add_piece(entry(pb), y, acc_b);
      pa += a_step, pb += a_step, yp += SY;
    }
    if (u_hi == 2 * w + 1 && has_b)  // Y row o + 1 + w: last term of row o + 1 only
      add_piece(entry(pb), *reinterpret_cast<const u32x4 *>(yp), acc_b);
    store_piece(acc_a, o, hg);
    if (has_b) store_piece(acc_b, o + 1, hg);
  }
}

template <typename T, int NK, bool TRANSPOSED>
__global__ __launch_bounds__(kThreads) void vector_band_in_kernel(const typename Elem<T>::type *__restrict__ A,
                                                                  const typename Elem<T>::type *__restrict__ Y,
                                                                  typename Elem<T>::type *__restrict__ C, int B,
                                                                  int M, int w, int nblk, int vrows, int64_t asb,
                                                                  int64_t ysb, int64_t ysr, int64_t csb, int64_t csr) {
  vector_band_in_body<T, NK, TRANSPOSED>(A, Y, C, B, M, w, nblk, vrows, asb, ysb, ysr, csb, csr);
}

// Both products of window_matmul's backward in one launch: blockIdx.y = 0 forms grad_q = P2(grad_a, K rows),
// blockIdx.y = 1 forms grad_k = P3(grad_a, Q).  Same tiles, same LDS images, half the launches: what a small
// problem pays for is the launch, not the arithmetic.
template <typename T, int NK>
__global__ __launch_bounds__(kThreads) void vector_window_backward_kernel(
    const typename Elem<T>::type *__restrict__ GA, const typename Elem<T>::type *__restrict__ K,
    const typename Elem<T>::type *__restrict__ Q, typename Elem<T>::type *__restrict__ GQ,
    typename Elem<T>::type *__restrict__ GK, int B, int M, int w, int nblk, int vrows, int64_t asb, int64_t ksb,
    int64_t ksr, int64_t qsb, int64_t qsr, int64_t gqsb, int64_t gqsr, int64_t gksb, int64_t gksr) {
  if (blockIdx.y == 0)
    vector_band_in_body<T, NK, false>(GA, K, GQ, B, M, w, nblk, vrows, asb, ksb, ksr, gqsb, gqsr);
  else
    vector_band_in_body<T, NK, true>(GA, Q, GK, B, M, w, nblk, vrows, asb, qsb, qsr, gksb, gksr);
}

// x.lo * y.lo + x.hi * y.hi + acc on packed pairs of 16-bit values (v_dot2_f32_bf16 / v_dot2_f32_f16).
template <typename T>
__device__ __forceinline__ float dot2(uint32_t x, uint32_t y, float acc);
template <>
__device__ __forceinline__ float dot2<bf16_t>(uint32_t x, uint32_t y, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, x), __builtin_bit_cast(bf16x2, y), acc, false);
}
template <>
__device__ __forceinline__ float dot2<f16_t>(uint32_t x, uint32_t y, float acc) {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, x), __builtin_bit_cast(f16x2, y), acc, false);
}

// P1: band[b,i,j] = sum_h X[b,i,h] Y[b,i+j-w,h]  (+0.0 where i+j-w is outside the sequence).
// One thread per band entry, consecutive threads on consecutive entries of the flat band.
template <typename T, int NK>  // 2 NK 16-byte pieces per row: N = 16 NK (16-bit) or 8 NK (float32)
__device__ __forceinline__ void vector_band_out_body(const typename Elem<T>::type *__restrict__ X,
                                                     const typename Elem<T>::type *__restrict__ Y,
                                                     typename Elem<T>::type *__restrict__ C, int B, int M, int w,
                                                     int nblk, int vrows, int64_t xsb, int64_t xsr, int64_t ysb,
                                                     int64_t ysr, int64_t csb) {
  typedef typename Elem<T>::type E;
  constexpr int VEC = 16 / sizeof(E);
  constexpr int NCG = 2 * NK, N = NCG * VEC;
  constexpr int SX = N + VEC;  // rows 16 bytes apart mod 128
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  E *ximg = reinterpret_cast<E *>(lds_raw);  // rows i0 .. i0 + rows
  E *yimg = ximg + vrows * SX;               // rows i0 - w .. i0 + rows + w, zero outside the sequence

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x;
  const int W = 2 * w + 1;
  const int i0 = blk * vrows;
  const int rows = min(vrows, M - i0);
  const E *Xb = X + (int64_t)b * xsb, *Yb = Y + (int64_t)b * ysb;
  const int xchunks = rows * NCG, ychunks = (rows + 2 * w) * NCG;
  constexpr int BATCH = 8;
  for (int base = 0; base < xchunks + ychunks; base += BATCH * kThreads) {
    u32x4 reg[BATCH];
#pragma unroll
    for (int s = 0; s < BATCH; ++s) {
      const int q = base + s * kThreads + tid;
      const int qy = q - xchunks;
      const int xr = q / NCG, xg = q - xr * NCG, yr = qy / NCG, yg = qy - yr * NCG, c = i0 - w + yr;
      const E *src = q < xchunks ? Xb + (int64_t)(i0 + xr) * xsr + VEC * xg : Yb + (int64_t)c * ysr + VEC * yg;
      const bool ok = q < xchunks || (q < xchunks + ychunks && c >= 0 && c < M);
      reg[s] = *reinterpret_cast<const u32x4 *>(ok ? src : X);
    }
#pragma unroll
    for (int s = 0; s < BATCH; ++s) {
      const int q = base + s * kThreads + tid;
      const int qy = q - xchunks;
      const int xr = q / NCG, xg = q - xr * NCG, yr = qy / NCG, yg = qy - yr * NCG, c = i0 - w + yr;
      if (q < xchunks)
        *reinterpret_cast<u32x4 *>(ximg + xr * SX + VEC * xg) = reg[s];
      else if (q < xchunks + ychunks)
        *reinterpret_cast<u32x4 *>(yimg + yr * SX + VEC * yg) = mask_row_chunk(reg[s], (c >= 0) & (c < M));
    }
  }
  __syncthreads();

  E *Cb = C + (int64_t)b * csb + (int64_t)i0 * W;
  for (int item = tid; item < rows * W; item += kThreads) {
    const int r = item / W, j = item - r * W;
    const int c = i0 + r + j - w;
    const E *xp = ximg + r * SX, *yp = yimg + (r + j) * SX;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int g = 0; g < NCG; ++g) {
      const u32x4 x = *reinterpret_cast<const u32x4 *>(xp + VEC * g), y = *reinterpret_cast<const u32x4 *>(yp + VEC * g);
      if constexpr (sizeof(E) == 2) {
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = dot2<T>(x[e], y[e], acc[e]);
      } else {
        const f32x4v xf = __builtin_bit_cast(f32x4v, x), yf = __builtin_bit_cast(f32x4v, y);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = __builtin_fmaf(xf[e], yf[e], acc[e]);
      }
    }
    const float sum = (c >= 0 && c < M) ? (acc[0] + acc[1]) + (acc[2] + acc[3]) : 0.f;  // +0.0 outside the sequence
    if constexpr (sizeof(E) == 2)
      Cb[item] = (uint16_t)Mma<T>::pack2(sum, 0.f);
    else
      Cb[item] = sum;
  }
}

template <typename T, int NK>
__global__ __launch_bounds__(kThreads) void vector_band_out_kernel(const typename Elem<T>::type *__restrict__ X,
                                                                   const typename Elem<T>::type *__restrict__ Y,
                                                                   typename Elem<T>::type *__restrict__ C, int B,
                                                                   int M, int w, int nblk, int vrows, int64_t xsb,
                                                                   int64_t xsr, int64_t ysb, int64_t ysr, int64_t csb) {
  vector_band_out_body<T, NK>(X, Y, C, B, M, w, nblk, vrows, xsb, xsr, ysb, ysr, csb);
}

// Both products of unwindow_matmul's backward in one launch: blockIdx.y = 0 forms grad_a = P1(grad_o, V) on
// tiles of `orows` rows, blockIdx.y = 1 forms grad_v = P3(A, grad_o) on tiles of `irows` rows (the two
// products tile the sequence differently; a workgroup beyond its product's tiles returns at once).
template <typename T, int NK>
__global__ __launch_bounds__(kThreads) void vector_unwindow_backward_kernel(
    const typename Elem<T>::type *__restrict__ A, const typename Elem<T>::type *__restrict__ V,
    const typename Elem<T>::type *__restrict__ GO, typename Elem<T>::type *__restrict__ GA,
    typename Elem<T>::type *__restrict__ GV, int B, int M, int w, int oblk, int orows, int iblk, int irows,
    int64_t asb, int64_t vsb, int64_t vsr, int64_t gosb, int64_t gosr, int64_t gasb, int64_t gvsb, int64_t gvsr) {
  if (blockIdx.y == 0)
    vector_band_out_body<T, NK>(GO, V, GA, B, M, w, oblk, orows, gosb, gosr, vsb, vsr, gasb);
  else
    vector_band_in_body<T, NK, true>(A, GO, GV, B, M, w, iblk, irows, asb, gosb, gosr, gvsb, gvsr);
}

// Output rows per workgroup: as many as keep the LDS images of the widest supported window small.
int vector_rows(int64_t N, int dtype) { return dtype == WM_DTYPE_F32 && N > 64 ? 64 : 128; }
int vector_out_rows(int64_t N, int dtype) { return dtype == WM_DTYPE_F32 ? (N > 64 ? 32 : 64) : 128; }
size_t vector_lds(int64_t w, int64_t N, int dtype) {
  const int64_t W = 2 * w + 1, vec = dtype == WM_DTYPE_F32 ? 4 : 8, rows = vector_rows(N, dtype);
  return (size_t)((((rows + 2 * w) * W + 3 * vec - 1) & ~(vec - 1)) + (rows + 2 * w) * (N + vec)) * (16 / vec);
}
size_t vector_out_lds(int64_t w, int64_t N, int dtype) {
  const int64_t vec = dtype == WM_DTYPE_F32 ? 4 : 8;
  return (size_t)((2 * vector_out_rows(N, dtype) + 2 * w) * (N + vec)) * (16 / vec);
}

unsigned vector_grid(int64_t B, int64_t nblk) { return (unsigned)tiled_grid(B, nblk); }

template <typename T, bool TRANSPOSED>
hipError_t launch_vector(const Problem &p, const View &a, const View &y, const View &c) {
  typedef typename Elem<T>::type E;
  const int vrows = vector_rows(p.N, p.dtype);
  const int nblk = (int)((p.M + vrows - 1) / vrows);
  const dim3 grid(vector_grid(p.B, nblk)), block(kThreads);
  const size_t lds = vector_lds(p.w, p.N, p.dtype);
  const int pieces = (int)(p.N * sizeof(E) / 16);
#define WM_VEC(NK)                                                                                              \
  case NK:                                                                                                      \
    hipLaunchKernelGGL((vector_band_in_kernel<T, NK, TRANSPOSED>), grid, block, lds, p.stream, (const E *)a.data, \
                       (const E *)y.data, (E *)c.data, (int)p.B, (int)p.M, (int)p.w, nblk, vrows, a.sb, y.sb, y.sr, \
                       c.sb, c.sr);                                                                                   \
    break;
  switch (pieces / 2) {
    WM_VEC(1) WM_VEC(2) WM_VEC(3) WM_VEC(4) WM_VEC(5) WM_VEC(6) WM_VEC(7) WM_VEC(8)
    WM_VEC(9) WM_VEC(10) WM_VEC(11) WM_VEC(12) WM_VEC(13) WM_VEC(14) WM_VEC(15) WM_VEC(16)
    default: return hipErrorInvalidValue;
  }
#undef WM_VEC
  return hipGetLastError();
}

template <typename T>
hipError_t launch_vector_out(const Problem &p, const View &x, const View &y, const View &c) {
  typedef typename Elem<T>::type E;
  const int vrows = vector_out_rows(p.N, p.dtype);
  const int nblk = (int)((p.M + vrows - 1) / vrows);
  const dim3 grid(vector_grid(p.B, nblk)), block(kThreads);
  const size_t lds = vector_out_lds(p.w, p.N, p.dtype);
  const int pieces = (int)(p.N * sizeof(E) / 16);
#define WM_VOUT(NK)                                                                                             \
  case NK:                                                                                                      \
    hipLaunchKernelGGL((vector_band_out_kernel<T, NK>), grid, block, lds, p.stream, (const E *)x.data,          \
                       (const E *)y.data, (E *)c.data, (int)p.B, (int)p.M, (int)p.w, nblk, vrows, x.sb, x.sr,   \
                       y.sb, y.sr, c.sb);                                                                       \
    break;
  switch (pieces / 2) {
    WM_VOUT(1) WM_VOUT(2) WM_VOUT(3) WM_VOUT(4) WM_VOUT(5) WM_VOUT(6) WM_VOUT(7) WM_VOUT(8)
    WM_VOUT(9) WM_VOUT(10) WM_VOUT(11) WM_VOUT(12) WM_VOUT(13) WM_VOUT(14) WM_VOUT(15) WM_VOUT(16)
    default: return hipErrorInvalidValue;
  }
#undef WM_VOUT
  return hipGetLastError();
}

bool band_contiguous(const View &v, int64_t W) { return v.sc == 1 && v.sr == W && ((uintptr_t)v.data % 16) == 0; }

}  // namespace

// 16-bit: band-in products up to w = 3 (61-71 us against 73-86 us for the narrow-band MFMA kernels at
// B96 M16384 N64; those win from w = 4 on); the band-out product never (86-92 us against 80 us at w = 1, 2).
// float32: every window up to VECTOR_F32_MAX_W, all three products.
bool vector_supports(int op, int64_t M, int64_t N, int64_t w, int dtype) {
  if (op < 1 || op > 3 || M < 1 || M > (1 << 30) || w < 1) return false;
  if (dtype == WM_DTYPE_F32) {
    if (N < 8 || N > 128 || N % 8 != 0 || w > VECTOR_F32_MAX_W) return false;
    if (op == 1 && small_f32_p1_supports(M, N, w)) return false;  // the MFMA band-out kernel is faster there
    if (op != 1 && small_f32_in_supports(M, N, w)) return false;  // likewise the MFMA band-in kernels
    return (op == 1 ? vector_out_lds(w, N, dtype) : vector_lds(w, N, dtype)) <= 65536;
  }
  if (dtype != WM_DTYPE_BF16 && dtype != WM_DTYPE_F16) return false;
  if (N < 16 || N > 128 || N % 16 != 0) return false;
  if (op == 1) return false;  // 16-bit band-out: the narrow-band MFMA kernel is faster at every w
  return w <= VECTOR_MAX_W && vector_lds(w, N, dtype) <= 65536;
}

// One launch for both gradients of an op, for problems so small that the second launch is what they
// would pay for (at most kFusedTiles tiles per product: a few workgroups per CU).
constexpr int64_t kFusedTiles = 1024;
bool vector_16bit_out_ok(int64_t N, int64_t w, int dtype) {  // band-out product in 16-bit storage, fused launches only
  return (dtype == WM_DTYPE_BF16 || dtype == WM_DTYPE_F16) && N >= 16 && N <= 128 && N % 16 == 0 && w <= VECTOR_MAX_W &&
         vector_out_lds(w, N, dtype) <= 65536;
}

bool try_launch_vector_window_backward(const Problem &p, const View &ga, const View &k, const View &q, const View &gq,
                                       const View &gk, hipError_t *err) {
  if (!vector_supports(2, p.M, p.N, p.w, p.dtype) || !vector_supports(3, p.M, p.N, p.w, p.dtype)) return false;
  if (!band_contiguous(ga, 2 * p.w + 1) || !fast_layout(k, p.dtype) || !fast_layout(q, p.dtype) ||
      !fast_layout(gq, p.dtype) || !fast_layout(gk, p.dtype))
    return false;
  const int vrows = vector_rows(p.N, p.dtype);
  const int nblk = (int)((p.M + vrows - 1) / vrows);
  if (p.B * nblk > kFusedTiles) return false;
  const dim3 grid(vector_grid(p.B, nblk), 2), block(kThreads);
  const size_t lds = vector_lds(p.w, p.N, p.dtype);
  const int pieces = (int)(p.N * dtype_size(p.dtype) / 16);
#define WM_VWB(T, NK)                                                                                            \
  case NK:                                                                                                       \
    hipLaunchKernelGGL((vector_window_backward_kernel<T, NK>), grid, block, lds, p.stream,                       \
                       (const typename Elem<T>::type *)ga.data, (const typename Elem<T>::type *)k.data,          \
                       (const typename Elem<T>::type *)q.data, (typename Elem<T>::type *)gq.data,                \
                       (typename Elem<T>::type *)gk.data, (int)p.B, (int)p.M, (int)p.w, nblk, vrows, ga.sb, k.sb, \
                       k.sr, q.sb, q.sr, gq.sb, gq.sr, gk.sb, gk.sr);                                             \
    break;
#define WM_VWB_ALL(T)                                                                                  \
  switch (pieces / 2) {                                                                                \
    WM_VWB(T, 1) WM_VWB(T, 2) WM_VWB(T, 3) WM_VWB(T, 4) WM_VWB(T, 5) WM_VWB(T, 6) WM_VWB(T, 7) WM_VWB(T, 8)   \
    WM_VWB(T, 9) WM_VWB(T, 10) WM_VWB(T, 11) WM_VWB(T, 12) WM_VWB(T, 13) WM_VWB(T, 14) WM_VWB(T, 15) WM_VWB(T, 16) \
    default: return false;                                                                             \
  }
  if (p.dtype == WM_DTYPE_BF16) {
    WM_VWB_ALL(bf16_t)
  } else if (p.dtype == WM_DTYPE_F16) {
    WM_VWB_ALL(f16_t)
  } else {
    WM_VWB_ALL(f32_t)
  }
#undef WM_VWB_ALL
#undef WM_VWB
  *err = hipGetLastError();
  return true;
}

bool try_launch_vector_unwindow_backward(const Problem &p, const View &a, const View &v, const View &go, const View &ga,
                                         const View &gv, hipError_t *err) {
  const bool out_ok = p.dtype == WM_DTYPE_F32 ? vector_supports(1, p.M, p.N, p.w, p.dtype) : vector_16bit_out_ok(p.N, p.w, p.dtype);
  if (!out_ok || !vector_supports(3, p.M, p.N, p.w, p.dtype)) return false;
  if (!band_contiguous(a, 2 * p.w + 1) || !band_contiguous(ga, 2 * p.w + 1) || !fast_layout(v, p.dtype) ||
      !fast_layout(go, p.dtype) || !fast_layout(gv, p.dtype))
    return false;
  const int orows = vector_out_rows(p.N, p.dtype), irows = vector_rows(p.N, p.dtype);
  const int oblk = (int)((p.M + orows - 1) / orows), iblk = (int)((p.M + irows - 1) / irows);
  if (p.B * oblk > kFusedTiles) return false;
  const dim3 grid(std::max(vector_grid(p.B, oblk), vector_grid(p.B, iblk)), 2), block(kThreads);
  const size_t lds = std::max(vector_out_lds(p.w, p.N, p.dtype), vector_lds(p.w, p.N, p.dtype));
  const int pieces = (int)(p.N * dtype_size(p.dtype) / 16);
#define WM_VUB(T, NK)                                                                                            \
  case NK:                                                                                                       \
    hipLaunchKernelGGL((vector_unwindow_backward_kernel<T, NK>), grid, block, lds, p.stream,                     \
                       (const typename Elem<T>::type *)a.data, (const typename Elem<T>::type *)v.data,           \
                       (const typename Elem<T>::type *)go.data, (typename Elem<T>::type *)ga.data,               \
                       (typename Elem<T>::type *)gv.data, (int)p.B, (int)p.M, (int)p.w, oblk, orows, iblk, irows, \
                       a.sb, v.sb, v.sr, go.sb, go.sr, ga.sb, gv.sb, gv.sr);                                      \
    break;
#define WM_VUB_ALL(T)                                                                                  \
  switch (pieces / 2) {                                                                                \
    WM_VUB(T, 1) WM_VUB(T, 2) WM_VUB(T, 3) WM_VUB(T, 4) WM_VUB(T, 5) WM_VUB(T, 6) WM_VUB(T, 7) WM_VUB(T, 8)   \
    WM_VUB(T, 9) WM_VUB(T, 10) WM_VUB(T, 11) WM_VUB(T, 12) WM_VUB(T, 13) WM_VUB(T, 14) WM_VUB(T, 15) WM_VUB(T, 16) \
    default: return false;                                                                             \
  }
  if (p.dtype == WM_DTYPE_BF16) {
    WM_VUB_ALL(bf16_t)
  } else if (p.dtype == WM_DTYPE_F16) {
    WM_VUB_ALL(f16_t)
  } else {
    WM_VUB_ALL(f32_t)
  }
#undef WM_VUB_ALL
#undef WM_VUB
  *err = hipGetLastError();
  return true;
}

bool try_launch_vector_p1(const Problem &p, const View &x, const View &y, const View &c, hipError_t *err) {
  if (!vector_supports(1, p.M, p.N, p.w, p.dtype)) return false;
  if (!fast_layout(x, p.dtype) || !fast_layout(y, p.dtype) || c.sc != 1 || c.sr != 2 * p.w + 1) return false;
  *err = launch_vector_out<f32_t>(p, x, y, c);
  return true;
}

template <bool TRANSPOSED>
bool try_launch_vector_in(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  if (!vector_supports(TRANSPOSED ? 3 : 2, p.M, p.N, p.w, p.dtype)) return false;
  if (!band_contiguous(a, 2 * p.w + 1) || !fast_layout(y, p.dtype) || !fast_layout(c, p.dtype)) return false;
  *err = p.dtype == WM_DTYPE_BF16  ? launch_vector<bf16_t, TRANSPOSED>(p, a, y, c)
         : p.dtype == WM_DTYPE_F16 ? launch_vector<f16_t, TRANSPOSED>(p, a, y, c)
                                   : launch_vector<f32_t, TRANSPOSED>(p, a, y, c);
  return true;
}
bool try_launch_vector_p2(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  return try_launch_vector_in<false>(p, a, y, c, err);
}
bool try_launch_vector_p3(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  return try_launch_vector_in<true>(p, a, y, c, err);
}

}  // namespace wm
