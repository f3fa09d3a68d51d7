// Shared declarations of the gfx950 banded-matmul kernels.
//
// The six products of the path (window forward, grad_q, grad_k, unwindow
// forward, grad_a, grad_v) are three primitives over row-major views:
//   P1 band-out            C[b,i,j] = sum_h X[b,i,h] * Y[b,i+j-w,h]      (+0 out of range)
//   P2 band-in             C[b,i,h] = sum_j A[b,i,j] * Y[b,i+j-w,h]
//   P3 transposed band-in  C[b,c,h] = sum_r A[b,r,c-r+w] * Y[b,r,h]
// with X, Y, C(P2,P3) of logical shape (B,M,N) and the band of shape (B,M,2w+1).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/window_matmul_hip.h"

namespace wm {

// Rank-3 view handed to kernels: element strides, 64-bit.
struct View {
  void *data;
  int64_t sb, sr, sc;
};

inline View make_view(const wm_operand *op) { return View{op->data, op->stride_b, op->stride_r, op->stride_c}; }
// Same storage seen with rows and columns swapped: (B,N,M) <-> (B,M,N).
inline View transposed(const View &v) { return View{v.data, v.sb, v.sc, v.sr}; }

struct Problem {
  int64_t B, M, N, w;
  int dtype;
  unsigned flags;
  hipStream_t stream;
};

// Workgroups of a tiled launch over B batch elements of nblk blocks each (the decode_block of the
// kernels maps them back): whole elements for every full group of 8, the rest of the tiles in eight
// equal ranges.  No surplus workgroups: the dispatcher places workgroups in order, and ones that
// return at once still shift the others onto fewer CUs.
inline int64_t tiled_grid(int64_t B, int64_t nblk) { return 8 * ((B >> 3) * nblk + ((B & 7) * nblk + 7) / 8); }

// Workgroup -> (batch, block).  Workgroups are dealt round-robin to the 8 XCDs, each with its
// own L2: XCD x runs ids x, x + 8, ...  Every full group of 8 batch elements gives one element to
// each XCD, so that neighbouring blocks of an element find the rows they share (the +-w halo) in
// that L2; the B % 8 elements left over are cut into 8 contiguous ranges of tiles, one per XCD
// (a whole element per XCD would leave one XCD idle at B = 7).  The launch uses tiled_grid():
// at most 7 workgroups at the end of the grid have no tile and return at once.
__device__ __forceinline__ bool decode_block(int nblk, int B, int *b, int *blk) {
  const int id = blockIdx.x, xcd = id & 7, slot = id >> 3;
  const int full = (B >> 3) * nblk;  // slots of the full groups
  if (slot < full) {
    *b = (slot / nblk) * 8 + xcd;
    *blk = slot % nblk;
    return true;
  }
  const int64_t tiles = (int64_t)(B & 7) * nblk, per = (tiles + 7) / 8, t = xcd * per + (slot - full);
  if (slot - full >= per || t >= tiles) return false;
  *b = (B & ~7) + (int)(t / nblk);
  *blk = (int)(t % nblk);
  return true;
}

// Launchers return hipSuccess or the launch error.  The strided family accepts
// any dtype and layout; the MFMA family reports whether it took the problem.
hipError_t launch_strided_p1(const Problem &p, const View &x, const View &y, const View &c);
hipError_t launch_strided_p2(const Problem &p, const View &a, const View &y, const View &c);
hipError_t launch_strided_p3(const Problem &p, const View &a, const View &y, const View &c);

// Returns true and sets *err when the MFMA family handles the problem.
bool try_launch_mfma_p1(const Problem &p, const View &x, const View &y, const View &c, hipError_t *err);
bool try_launch_mfma_p2(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err);
bool try_launch_mfma_p3(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err);
// Whether the band-in kernels of that family that load their tiles straight into LDS accept the
// layout of band `a` and operand `y` (the shape aside): what the narrow-band family asks before it
// leaves a window to them.
bool lds_direct_layout_ok(const Problem &p, const View &a, const View &y);
// Narrow-band family (w <= 32; P2 and P3 while their LDS images fit 64 KB; float32 at N <= 64).
bool try_launch_small_p1(const Problem &p, const View &x, const View &y, const View &c, hipError_t *err);
bool try_launch_small_p2(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err);
bool try_launch_small_p3(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err);
bool small_supports(int op, int64_t M, int64_t N, int64_t w, int dtype, unsigned flags);
bool small_f32_in_supports(int64_t M, int64_t N, int64_t w);  // float32 band-in kernels of the narrow-band family
bool small_f32_p1_supports(int64_t M, int64_t N, int64_t w);  // float32 band-out kernel of the narrow-band family
// Vector-ALU kernels for the narrowest windows: 16-bit up to w = 3 (band-in) and w = 2 (band-out),
// float32 up to w = 14 (the band-out product only where the narrow-band float32 kernel does not apply).
bool try_launch_vector_p1(const Problem &p, const View &x, const View &y, const View &c, hipError_t *err);
bool try_launch_vector_p2(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err);
bool try_launch_vector_p3(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err);
bool vector_supports(int op, int64_t M, int64_t N, int64_t w, int dtype);
// Both gradients of an op in one launch of the vector-ALU kernels, for small problems (false: not taken,
// nothing launched; the caller then launches the two products separately).
bool try_launch_vector_window_backward(const Problem &p, const View &ga, const View &k, const View &q, const View &gq,
                                       const View &gk, hipError_t *err);
bool try_launch_vector_unwindow_backward(const Problem &p, const View &a, const View &v, const View &go, const View &ga,
                                         const View &gv, hipError_t *err);
// float32 MFMA family (N multiple of 8 up to 128, w >= 4).
bool try_launch_f32_p1(const Problem &p, const View &x, const View &y, const View &c, hipError_t *err);
bool try_launch_f32_p2(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err);
bool try_launch_f32_p3(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err);
bool f32_supports(int op, int64_t M, int64_t N, int64_t w, int dtype);
// The same products on the bf16 matrix instruction through an exact three-way split of every float32
// value (wm_f32_split.hip); taken ahead of the kernels above from a window size on.
bool try_launch_f32_split_p1(const Problem &p, const View &x, const View &y, const View &c, hipError_t *err);
bool try_launch_f32_split_p2(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err);
bool try_launch_f32_split_p3(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err);
bool f32_split_supports(int op, int64_t M, int64_t N, int64_t w, int dtype, unsigned flags);
// Tile family: float64, and whatever the families above decline in 16-bit and float32 storage;
// 64 x 64 tiles on the 16x16x4 matrix instructions, any strides, any N and w.
bool try_launch_tile_p1(const Problem &p, const View &x, const View &y, const View &c, hipError_t *err);
bool try_launch_tile_p2(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err);
bool try_launch_tile_p3(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err);
bool tile_supports(int op, int64_t M, int64_t N, int64_t w, int dtype);
// Pure predicate behind the wide-band 16-bit functions above (shape/dtype only).
bool mfma_supports(int op, int64_t B, int64_t M, int64_t N, int64_t w, int dtype);

// Softmax along the band dimension (wm_softmax.hip).  `mask` non-zero treats entries outside
// the sequence as -infinity.  In-place use (out aliasing an input) is allowed.
hipError_t launch_band_softmax_forward(const Problem &p, const View &a, const View &out, double scale, int mask);
hipError_t launch_band_softmax_backward(const Problem &p, const View &probs, const View &grad_probs,
                                        const View &grad_a, double scale, int mask);
// Whether rows of length W get the LDS-staged kernel (given contiguous, 16-byte aligned tensors).
bool band_softmax_staged(int64_t W, int dtype, bool backward);

// Fused window attention forward (wm_attention.hip): q, k, v, o row-major (B,M,N) views, lse an
// optional float32 (B,M) buffer.  Returns false when the kernel does not take the problem.
bool attention_supports(int64_t M, int64_t N, int64_t w, int dtype, double scale);
bool try_launch_attention_forward(const Problem &p, const View &q, const View &k, const View &v, const View &o,
                                  float *lse, double scale, int mask, hipError_t *err);

// Backward of the fused attention (wm_attention_bwd.hip): two kernels on p.stream; `delta` is a
// float32 (B,M) workspace the first one fills and the second one reads.
bool try_launch_attention_backward(const Problem &p, const View &q, const View &k, const View &v, const View &o,
                                   const View &go, const float *lse, float *delta, const View &gq, const View &gk,
                                   const View &gv, double scale, hipError_t *err);

// Batched transpose of the last two dimensions (wm_transpose.hip): src (B,R,C) with unit column stride and
// batch / row strides ssb / ssr (elements), dst contiguous (B,C,R).  Returns false, nothing launched,
// unless dst is 16-byte aligned, R is a multiple of 16 bytes and elem_size is 2, 4 or 8.
bool try_launch_transpose(const void *src, void *dst, int64_t B, int64_t R, int64_t C, int64_t ssb, int64_t ssr,
                          int elem_size, hipStream_t stream, hipError_t *err);

inline size_t dtype_size(int dtype) {
  switch (dtype) {
    case WM_DTYPE_F32: return 4;
    case WM_DTYPE_F16: return 2;
    case WM_DTYPE_BF16: return 2;
    case WM_DTYPE_F64: return 8;
    default: return 0;
  }
}

// Unit column stride, every row start 16-byte aligned: what the vector paths need.
inline bool fast_layout(const View &v, int dtype) {
  const int64_t es = (int64_t)dtype_size(dtype);
  if (v.sc != 1) return false;
  if (((uintptr_t)v.data) % 16 != 0) return false;
  return (v.sr * es) % 16 == 0 && (v.sb * es) % 16 == 0;
}

// Band operands are only required to be contiguous per batch (rows of odd
// length 2w+1 are never 16-byte aligned); the kernels realign in LDS.
inline bool band_layout(const View &v, int64_t W) { return v.sc == 1 && v.sr == W; }

}  // namespace wm
