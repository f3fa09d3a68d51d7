// Tile family for everything the tuned families do not take: float64 (on v_mfma_f64_16x16x4_f64),
// and 16-bit or float32 storage in layouts or head widths outside the tuned kernels' reach (element
// strides in the rows, misaligned rows, N not a multiple of 8 or 16, N > 128), which are widened to
// float32 on the way into LDS and multiplied on v_mfma_f32_16x16x4_f32.
//
// A workgroup of four waves owns a 64 x 64 block of the (skewed) product, each wave a 32 x 32
// quarter as 2 x 2 matrix-instruction blocks, and walks the contraction in stages of 16 that pass
// through LDS.  The next stage's operands are fetched into registers while the current stage is
// multiplied.  A staged tile is kept k-major (pitch 80 elements) when consecutive threads fetch along
// its rows and row-major (pitch 17) when they fetch along the contraction: both the stores and the
// instruction's operand reads (lane l takes row l % 16, step l / 16) are then free of bank conflicts.
//
// Operands are addressed through their element strides, so every layout is taken; the strides only
// choose which way consecutive threads run over a staged tile (along the dimension that is closer
// in memory).  Entries of a band tile outside the band, outside the sequence or past an extent are
// never loaded (a predicate, not a multiplication by zero), and out-of-sequence entries of a band
// result are stored as literal +0.0.  Sums run in ascending order of the contraction index, four
// terms per instruction, in float32 (float64 for float64 storage) and are rounded once
// (reference loops: cpu/window_matmul_cpu.cpp:39-43, 129-141).
#include <cstdlib>
#include <type_traits>

#include "wm_common.hpp"
#include "wm_types.hpp"

namespace wm {
namespace {

constexpr int TS = 64;          // side of the product block
constexpr int KS = 16;          // contraction steps per LDS stage
constexpr int THREADS = 256;
constexpr int PER_THREAD = TS * KS / THREADS;
constexpr int K_MAJOR_PITCH = TS + 16, ROW_MAJOR_PITCH = KS + 1;
constexpr int TILE_ELEMS = KS * K_MAJOR_PITCH > TS * ROW_MAJOR_PITCH ? KS * K_MAJOR_PITCH : TS * ROW_MAJOR_PITCH;

typedef double d4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));

// The matrix instruction per compute type.  Lane l supplies A[l % 16][l / 16] and B[l / 16][l % 16];
// element v of its result is D[row(v, l / 16)][l % 16].
template <class C>
struct Mma;
template <>
struct Mma<double> {
  typedef d4 acc_t;
  __device__ static acc_t run(double a, double b, acc_t c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
  __device__ static int row(int v, int q) { return 4 * v + q; }
};
template <>
struct Mma<float> {
  typedef f4 acc_t;
  __device__ static acc_t run(float a, float b, acc_t c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
  __device__ static int row(int v, int q) { return 4 * q + v; }
};

template <class C>
struct Stage {
  C a[TILE_ELEMS];
  C b[TILE_ELEMS];
};

// Where element (m, k) of a staged tile lives; M_FAST tiles are k-major.
template <bool M_FAST>
__device__ inline int lds_index(int m, int k) {
  return M_FAST ? k * K_MAJOR_PITCH + m : m * ROW_MAJOR_PITCH + k;
}

// Element `i` of this thread's share of a staged TS x KS tile: (m, k), consecutive threads along m
// (M_FAST) or along k.
template <bool M_FAST>
__device__ inline void slot(int i, int &m, int &k) {
  const int e = threadIdx.x + THREADS * i;
  if (M_FAST) {
    m = e % TS;
    k = e / TS;
  } else {
    m = e / KS;
    k = e % KS;
  }
}

// The wave's 32 x 32 quarter: acc[bi][bj][v] is the entry (row_of<C>(bi, v), col_of(bj)) of the block.
template <class C>
__device__ inline int row_of(int bi, int v) {
  return 32 * (threadIdx.x / 128) + 16 * bi + Mma<C>::row(v, (threadIdx.x % 64) / 16);
}
__device__ inline int col_of(int bj) { return 32 * ((threadIdx.x / 64) % 2) + 16 * bj + threadIdx.x % 16; }

template <bool A_FAST, bool B_FAST, class C>
__device__ inline void multiply(const Stage<C> &t, typename Mma<C>::acc_t (&acc)[2][2]) {
  const int lane = threadIdx.x % 64, m0 = 32 * (threadIdx.x / 128) + lane % 16, n0 = 32 * ((threadIdx.x / 64) % 2) + lane % 16;
#pragma unroll
  for (int s = 0; s < KS / 4; ++s) {
    const int k = 4 * s + lane / 16;
    C a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      a[i] = t.a[lds_index<A_FAST>(m0 + 16 * i, k)];
      b[i] = t.b[lds_index<B_FAST>(n0 + 16 * i, k)];
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = Mma<C>::run(a[i], b[j], acc[i][j]);
  }
}

// acc[m][n] += sum over `stages` * KS steps of fetch_a(m, k) * fetch_b(n, k).  Every thread of the
// workgroup calls it with the same `stages`.
template <bool A_FAST, bool B_FAST, class C, class FA, class FB>
__device__ inline void accumulate(Stage<C> &t, int64_t stages, FA fetch_a, FB fetch_b,
                                  typename Mma<C>::acc_t (&acc)[2][2]) {
  C ra[PER_THREAD], rb[PER_THREAD];
  auto fetch = [&](int64_t s) {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      int m, k;
      slot<A_FAST>(i, m, k);
      ra[i] = fetch_a(m, s * KS + k);
      slot<B_FAST>(i, m, k);
      rb[i] = fetch_b(m, s * KS + k);
    }
  };
  if (stages > 0) fetch(0);
  for (int64_t s = 0; s < stages; ++s) {
    __syncthreads();  // the previous stage has been read
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      int m, k;
      slot<A_FAST>(i, m, k);
      t.a[lds_index<A_FAST>(m, k)] = ra[i];
      slot<B_FAST>(i, m, k);
      t.b[lds_index<B_FAST>(m, k)] = rb[i];
    }
    __syncthreads();
    if (s + 1 < stages) fetch(s + 1);
    multiply<A_FAST, B_FAST>(t, acc);
  }
}

template <class T>
struct Rows {  // one batch element of a view
  T *p;
  int64_t sr, sc;
  __device__ Rows(const View &v, int64_t b) : p((T *)v.data + b * v.sb), sr(v.sr), sc(v.sc) {}
  __device__ typename Acc<T>::type get(int64_t r, int64_t c) const { return to_acc<T>(p[r * sr + c * sc]); }
  __device__ void put(int64_t r, int64_t c, typename Acc<T>::type v) const { p[r * sr + c * sc] = from_acc<T>(v); }
};

// P1.  Block rows i0.., columns c0.. of X * Y^T for every 64-column chunk that meets the band.
template <class T, bool X_FAST, bool Y_FAST>
__global__ __launch_bounds__(THREADS) void tile_band_out_kernel(View xv, View yv, View cv, int B, int64_t M,
                                                                int64_t N, int64_t w, int64_t tiles) {
  typedef typename Acc<T>::type C;
  __shared__ Stage<C> t;
  int b, blk;
  if (!decode_block((int)tiles, B, &b, &blk)) return;  // neighbouring tiles of a batch element share an XCD's L2
  const int64_t i0 = (int64_t)blk * TS;
  const Rows<T> x(xv, b), y(yv, b), c(cv, b);
  const int64_t stages = (N + KS - 1) / KS;
  for (int64_t c0 = i0 - w; c0 <= i0 + TS - 1 + w; c0 += TS) {
    typename Mma<C>::acc_t acc[2][2] = {};
    const bool in_sequence = c0 + TS > 0 && c0 < M;
    accumulate<X_FAST, Y_FAST>(
        t, in_sequence ? stages : 0,
        [&](int m, int64_t h) { return i0 + m < M && h < N ? x.get(i0 + m, h) : C(0); },
        [&](int m, int64_t h) { return c0 + m >= 0 && c0 + m < M && h < N ? y.get(c0 + m, h) : C(0); }, acc);
#pragma unroll
    for (int bi = 0; bi < 2; ++bi)
#pragma unroll
      for (int v = 0; v < 4; ++v)
#pragma unroll
        for (int bj = 0; bj < 2; ++bj) {
          const int64_t r = i0 + row_of<C>(bi, v), col = c0 + col_of(bj), band = col - r + w;
          if (r < M && band >= 0 && band <= 2 * w) c.put(r, band, col >= 0 && col < M ? acc[bi][bj][v] : C(0));
        }
  }
}

// P2 (TRANSPOSED = false): output rows o0.., contraction over the columns lo..hi of the sequence
// that those rows' bands cover.  P3 (TRANSPOSED = true): output rows o0.., contraction over the
// band rows lo..hi that reach them.  In both the band entry of (row r, column col) is A[r, col - r + w].
template <class T, bool TRANSPOSED, bool A_FAST, bool Y_FAST>
__global__ __launch_bounds__(THREADS) void tile_band_in_kernel(View av, View yv, View cv, int B, int64_t M,
                                                               int64_t N, int64_t w, int64_t tiles) {
  typedef typename Acc<T>::type C;
  __shared__ Stage<C> t;
  int b, blk;
  if (!decode_block((int)tiles, B, &b, &blk)) return;
  const int64_t o0 = (int64_t)blk * TS, h0 = (int64_t)blockIdx.y * TS;
  const Rows<T> a(av, b), y(yv, b), c(cv, b);
  const int64_t lo = o0 > w ? o0 - w : 0, hi = o0 + TS - 1 + w < M - 1 ? o0 + TS - 1 + w : M - 1;
  typename Mma<C>::acc_t acc[2][2] = {};
  accumulate<A_FAST, Y_FAST>(
      t, (hi - lo + KS) / KS,
      [&](int m, int64_t s) {
        const int64_t out = o0 + m, in = lo + s;
        const int64_t r = TRANSPOSED ? in : out, col = TRANSPOSED ? out : in, band = col - r + w;
        return out < M && in <= hi && band >= 0 && band <= 2 * w ? a.get(r, band) : C(0);
      },
      [&](int m, int64_t s) { return lo + s <= hi && h0 + m < N ? y.get(lo + s, h0 + m) : C(0); }, acc);
#pragma unroll
  for (int bi = 0; bi < 2; ++bi)
#pragma unroll
    for (int v = 0; v < 4; ++v)
#pragma unroll
      for (int bj = 0; bj < 2; ++bj) {
        const int64_t r = o0 + row_of<C>(bi, v), h = h0 + col_of(bj);
        if (r < M && h < N) c.put(r, h, acc[bi][bj][v]);
      }
}

bool takes(const Problem &p) { return tile_supports(1, p.M, p.N, p.w, p.dtype) && p.B > 0; }

// Consecutive threads run along the rows of an operand whose rows are closer in memory than its columns.
bool rows_closer(const View &v) { return llabs(v.sr) < llabs(v.sc); }

// Calls launch(first, second) with the two flags as compile-time constants.
template <class F>
void with_flags(bool first, bool second, F launch) {
  if (first) {
    if (second) launch(std::true_type{}, std::true_type{});
    else launch(std::true_type{}, std::false_type{});
  } else {
    if (second) launch(std::false_type{}, std::true_type{});
    else launch(std::false_type{}, std::false_type{});
  }
}

template <class T>
void launch_band_out(const Problem &p, const View &x, const View &y, const View &c) {
  const int64_t tiles = (p.M + TS - 1) / TS;
  const dim3 grid((unsigned)tiled_grid(p.B, tiles)), block(THREADS);
  with_flags(rows_closer(x), rows_closer(y), [&](auto x_fast, auto y_fast) {
    hipLaunchKernelGGL((tile_band_out_kernel<T, decltype(x_fast)::value, decltype(y_fast)::value>), grid, block, 0,
                       p.stream, x, y, c, (int)p.B, p.M, p.N, p.w, tiles);
  });
}

template <class T, bool TRANSPOSED>
void launch_band_in(const Problem &p, const View &a, const View &y, const View &c) {
  const int64_t tiles = (p.M + TS - 1) / TS;
  const dim3 grid((unsigned)tiled_grid(p.B, tiles), (unsigned)((p.N + TS - 1) / TS)), block(THREADS);
  // Band tile: neighbouring staged elements along the output rows lie sr - sc apart in memory
  // (band-in) or sc apart (transposed band-in); along the contraction sc or sr - sc.
  const int64_t along_m = TRANSPOSED ? llabs(a.sc) : llabs(a.sr - a.sc);
  const int64_t along_k = TRANSPOSED ? llabs(a.sr - a.sc) : llabs(a.sc);
  with_flags(along_m < along_k, !rows_closer(y), [&](auto a_fast, auto y_fast) {
    hipLaunchKernelGGL((tile_band_in_kernel<T, TRANSPOSED, decltype(a_fast)::value, decltype(y_fast)::value>), grid,
                       block, 0, p.stream, a, y, c, (int)p.B, p.M, p.N, p.w, tiles);
  });
}

template <class T>
void launch(int op, const Problem &p, const View &a, const View &y, const View &c) {
  if (op == 1) launch_band_out<T>(p, a, y, c);
  else if (op == 2) launch_band_in<T, false>(p, a, y, c);
  else launch_band_in<T, true>(p, a, y, c);
}

bool try_launch(int op, const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  if (!takes(p)) return false;
  switch (p.dtype) {
    case WM_DTYPE_F32: launch<float>(op, p, a, y, c); break;
    case WM_DTYPE_F16: launch<f16_t>(op, p, a, y, c); break;
    case WM_DTYPE_BF16: launch<bf16_t>(op, p, a, y, c); break;
    default: launch<double>(op, p, a, y, c); break;
  }
  *err = hipGetLastError();
  return true;
}

}  // namespace

bool tile_supports(int op, int64_t M, int64_t N, int64_t w, int dtype) {
  (void)op;
  (void)w;
  return dtype >= WM_DTYPE_F32 && dtype <= WM_DTYPE_F64 && M > 0 && N > 0 && (N + TS - 1) / TS <= 65535;
}

bool try_launch_tile_p1(const Problem &p, const View &x, const View &y, const View &c, hipError_t *err) {
  return try_launch(1, p, x, y, c, err);
}
bool try_launch_tile_p2(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  return try_launch(2, p, a, y, c, err);
}
bool try_launch_tile_p3(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  return try_launch(3, p, a, y, c, err);
}

}  // namespace wm
