// Vector-ALU band-in kernels for very narrow bands (16-bit storage, float32 accumulate) on gfx950.
//
// The narrow-band MFMA kernels read their skewed tile with 16-byte LDS reads, which needs the flat
// band image to keep 8-column groups aligned in every row, i.e. w % 4 == 0.  For the other small
// windows (w = 1, 2, 3, 5, 6, 7, ...) the band-in products
//     P2  C[i,h] = sum_j A[i,j] Y[i+j-w,h]          P3  C[c,h] = sum_r A[r,c-r+w] Y[r,h]
// are 2w+1 multiply-adds per output element on operands that are streamed once: far too little
// arithmetic for the matrix pipe to matter, so each thread simply owns 8 consecutive output
// columns of one row and walks the 2w+1 terms: one 2-byte LDS read of the band entry (the same
// address for the 8 threads of a row), one 16-byte LDS read of the Y row piece, 8 packed dot
// products that each pair the entry with one of the 8 values (and a zero with its neighbour).
// The workgroup first copies what it needs into LDS with coalesced 16-byte loads (its band rows
// as one flat image, the Y rows they reach row-major, zero outside the sequence); the result
// leaves as 16-byte non-temporal stores, 8 consecutive threads on one 128-byte row (N = 64).
// One barrier per workgroup; no atomics.
#include "wm_mfma_common.hpp"

namespace wm {
namespace {

constexpr int VROWS = 128;  // output rows per workgroup
#ifndef WM_VECTOR_MAX_W
#define WM_VECTOR_MAX_W 7
#endif
constexpr int VECTOR_MAX_W = WM_VECTOR_MAX_W;

// acc + a.lo * y.lo + a.hi * y.hi on packed pairs (v_dot2_f32_bf16 / v_dot2_f32_f16): with the band
// entry in one half of `a` and zero in the other, one instruction per multiply-add and no unpacking.
template <typename T>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t y, float acc);
template <>
__device__ __forceinline__ float dot2<bf16_t>(uint32_t a, uint32_t y, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, y), acc, false);
}
template <>
__device__ __forceinline__ float dot2<f16_t>(uint32_t a, uint32_t y, float acc) {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, y), acc, false);
}

// TRANSPOSED false: P2 (rows = band rows i).  TRANSPOSED true: P3 (rows = output rows c, the
// contraction runs over the band rows r = c-w .. c+w).
template <typename T, int NK, bool TRANSPOSED>  // N = 16 NK
__global__ __launch_bounds__(kThreads) void vector_band_in_kernel(const uint16_t *__restrict__ A,
                                                                  const uint16_t *__restrict__ Y,
                                                                  uint16_t *__restrict__ C, int B, int M, int w,
                                                                  int nblk, int64_t asb, int64_t ysb, int64_t ysr,
                                                                  int64_t csb, int64_t csr) {
  constexpr int N = 16 * NK, NCG = N / 8;  // 16-byte column groups per row
  constexpr int SY = N + 8;                // Y image rows 16 bytes apart mod 128
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x;
  const int W = 2 * w + 1;
  const int o0 = blk * VROWS;                      // first output row
  const int orows = min(VROWS, M - o0);
  // rows held in LDS: Y rows [y0, y0 + yrows) (may reach outside the sequence: zeros), band rows
  // [a0, a0 + arows) (inside the sequence)
  const int y0 = o0 - w, yrows = orows + 2 * w;
  const int a0 = TRANSPOSED ? max(o0 - w, 0) : o0;
  const int a1 = TRANSPOSED ? min(o0 + orows - 1 + w, M - 1) : o0 + orows - 1;
  const int arows = a1 - a0 + 1;
  const uint16_t *Ab = A + (int64_t)b * asb + (int64_t)a0 * W;
  const uint16_t *Yb = Y + (int64_t)b * ysb;
  // flat band image in whole aligned 16-byte chunks: image element e is band element e - delta
  const int delta = (int)((reinterpret_cast<uintptr_t>(Ab) >> 1) & 7);
  const int n_el = arows * W;
  const int chunks = (delta + n_el + 7) >> 3;
  uint16_t *aimg = lds;
  uint16_t *yimg = lds + (((VROWS + 2 * w) * W + 16 + 7) & ~7);  // sized for the largest image
  const int ychunks = yrows * NCG;

  // loads go out in batches of 8 per thread before any of them is used
  constexpr int BATCH = 8;
  for (int base = 0; base < chunks + ychunks; base += BATCH * kThreads) {
    u32x4 reg[BATCH];
#pragma unroll
    for (int s = 0; s < BATCH; ++s) {
      const int q = base + s * kThreads + tid;
      const int qy = q - chunks, yr = qy / NCG, hg = qy - yr * NCG, c = y0 + yr;
      const uint16_t *src = q < chunks ? Ab - delta + 8 * q : Yb + (int64_t)c * ysr + 8 * hg;
      const bool ok = q < chunks || (q < chunks + ychunks && c >= 0 && c < M);
      reg[s] = *reinterpret_cast<const u32x4 *>(ok ? src : A);
    }
#pragma unroll
    for (int s = 0; s < BATCH; ++s) {
      const int q = base + s * kThreads + tid;
      const int qy = q - chunks, yr = qy / NCG, hg = qy - yr * NCG, c = y0 + yr;
      if (q < chunks)
        *reinterpret_cast<u32x4 *>(aimg + 8 * q) = reg[s];
      else if (q < chunks + ychunks)
        *reinterpret_cast<u32x4 *>(yimg + yr * SY + 8 * hg) = mask_row_chunk(reg[s], (c >= 0) & (c < M));
    }
  }
  __syncthreads();

  for (int item = tid; item < orows * NCG; item += kThreads) {
    const int r = item / NCG, hg = item - r * NCG;
    const int o = o0 + r;  // output row
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    // term t = 0 .. 2w: the Y row is o - w + t (image row r + t) in both products
    const int t_lo = max(0, w - o), t_hi = min(2 * w, M - 1 - o + w);  // Y rows inside the sequence
    const uint16_t *yp = yimg + (r + t_lo) * SY + 8 * hg;
    // P2: band entry (o, t) -> image index (o - a0) W + t, next term +1.
    // P3: band entry (o - w + t, 2w - t) -> image index (o - w + t - a0) W + 2w - t, next term +W - 1.
    const uint16_t *ap = aimg + delta + (TRANSPOSED ? (o - w + t_lo - a0) * W + 2 * w - t_lo : (o - a0) * W + t_lo);
    const int a_step = TRANSPOSED ? W - 1 : 1;
    for (int t = t_lo; t <= t_hi; ++t) {
      const uint32_t a_lo = *ap, a_hi = a_lo << 16;  // (a, 0) and (0, a)
      const u32x4 y = *reinterpret_cast<const u32x4 *>(yp);
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        acc[2 * d] = dot2<T>(a_lo, y[d], acc[2 * d]);
        acc[2 * d + 1] = dot2<T>(a_hi, y[d], acc[2 * d + 1]);
      }
      ap += a_step;
      yp += SY;
    }
    const u32x4 out = {Mma<T>::pack2(acc[0], acc[1]), Mma<T>::pack2(acc[2], acc[3]), Mma<T>::pack2(acc[4], acc[5]),
                       Mma<T>::pack2(acc[6], acc[7])};
    __builtin_nontemporal_store(out, reinterpret_cast<u32x4 *>(C + (int64_t)b * csb + (int64_t)o * csr + 8 * hg));
  }
}

size_t vector_lds(int64_t w, int64_t N) {
  const int64_t W = 2 * w + 1;
  return (size_t)((((VROWS + 2 * w) * W + 16 + 7) & ~(int64_t)7) + (VROWS + 2 * w) * (N + 8)) * 2;
}

template <typename T, bool TRANSPOSED>
hipError_t launch_vector(const Problem &p, const View &a, const View &y, const View &c) {
  const int nblk = (int)((p.M + VROWS - 1) / VROWS);
  const dim3 grid((unsigned)(((p.B + 7) / 8) * 8 * nblk)), block(kThreads);
  const size_t lds = vector_lds(p.w, p.N);
#define WM_VEC(NK)                                                                                              \
  case NK:                                                                                                      \
    hipLaunchKernelGGL((vector_band_in_kernel<T, NK, TRANSPOSED>), grid, block, lds, p.stream,                  \
                       (const uint16_t *)a.data, (const uint16_t *)y.data, (uint16_t *)c.data, (int)p.B,        \
                       (int)p.M, (int)p.w, nblk, a.sb, y.sb, y.sr, c.sb, c.sr);                                 \
    break;
  switch (p.N / 16) {
    WM_VEC(1) WM_VEC(2) WM_VEC(3) WM_VEC(4) WM_VEC(5) WM_VEC(6) WM_VEC(7) WM_VEC(8)
    default: return hipErrorInvalidValue;
  }
#undef WM_VEC
  return hipGetLastError();
}

bool band_contiguous(const View &v, int64_t W) { return v.sc == 1 && v.sr == W && ((uintptr_t)v.data % 16) == 0; }

}  // namespace

// Windows the narrow-band MFMA kernels do not take (w % 4 != 0) and the wide-band kernels either do
// not take (w < 8) or serve poorly.
bool vector_supports(int op, int64_t M, int64_t N, int64_t w, int dtype) {
  if (op != 2 && op != 3) return false;
  if (dtype != WM_DTYPE_BF16 && dtype != WM_DTYPE_F16) return false;
  if (N < 16 || N > 128 || N % 16 != 0) return false;
  return M >= 1 && M <= (1 << 30) && w >= 1 && w <= VECTOR_MAX_W && w % 4 != 0 && vector_lds(w, N) <= 65536;
}

bool try_launch_vector_p2(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  if (!vector_supports(2, p.M, p.N, p.w, p.dtype)) return false;
  if (!band_contiguous(a, 2 * p.w + 1) || !fast_layout(y, p.dtype) || !fast_layout(c, p.dtype)) return false;
  *err = p.dtype == WM_DTYPE_BF16 ? launch_vector<bf16_t, false>(p, a, y, c) : launch_vector<f16_t, false>(p, a, y, c);
  return true;
}

bool try_launch_vector_p3(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  if (!vector_supports(3, p.M, p.N, p.w, p.dtype)) return false;
  if (!band_contiguous(a, 2 * p.w + 1) || !fast_layout(y, p.dtype) || !fast_layout(c, p.dtype)) return false;
  *err = p.dtype == WM_DTYPE_BF16 ? launch_vector<bf16_t, true>(p, a, y, c) : launch_vector<f16_t, true>(p, a, y, c);
  return true;
}

}  // namespace wm
