// Softmax along the band (last) dimension of a (B, M, 2w+1) tensor, forward and backward:
//   forward   P[r, :] = softmax(scale * A[r, :])
//   backward  dA[r, j] = scale * P[r, j] * (dP[r, j] - sum_j' P[r, j'] * dP[r, j'])
// This is the step callers put between window_matmul and unwindow_matmul
// (reference tests/test_attention.py:60-61).  Without masking every one of the 2w+1 entries
// of a row takes part with the value it holds, as in that caller (window_matmul writes +0.0
// into the entries that fall outside the sequence).  With masking those entries count as
// -infinity: probability +0.0, gradient +0.0.
//
// Band rows have odd length, so no row but the first starts on a 16-byte boundary.  The staged
// kernel therefore treats the rows of one workgroup as one flat, contiguous span of memory: the
// span is copied into LDS with aligned 16-byte non-temporal loads (its ragged first and last
// chunks element by element), groups of lanes then work on rows inside LDS, and the span is
// written back the same way.  HBM sees each byte once, in whole 16-byte pieces.
//
// The strided kernel (one wavefront per row, element accesses) covers float64, rows too long
// for LDS, non-contiguous tensors and misaligned base pointers.
#include "wm_common.hpp"
#include "wm_types.hpp"

#include <tuple>

namespace wm {
namespace {

constexpr int kSoftmaxThreads = 256;
constexpr int kLoadsInFlight = 4;      // 16-byte loads a thread issues before it touches LDS
constexpr int kSpanBytes = 16 * 1024;  // LDS image a workgroup aims for, per input tensor
constexpr int kLdsLimit = 64 * 1024;
constexpr float kLog2e = 1.4426950408889634f;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------------------------------------
// Reductions over groups of LANES consecutive lanes (a power of two, 4..64), result in every
// lane of the group.  Steps inside a row of 16 lanes are DPP modifiers on the arithmetic
// instruction; the two steps across rows use the gfx950 lane-swap instructions.
// ---------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
struct MaxOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return b > a ? b : a; }
  __device__ __forceinline__ double operator()(double a, double b) const { return b > a ? b : a; }
};
struct SumOp {
  template <typename A>
  __device__ __forceinline__ A operator()(A a, A b) const { return a + b; }
};
template <int LANES, typename Op>
__device__ __forceinline__ float group_reduce(float v, Op op) {
  v = op(v, dpp<0xB1>(v));                    // quad_perm [1,0,3,2]: neighbour lane
  v = op(v, dpp<0x4E>(v));                    // quad_perm [2,3,0,1]: other pair of the quad
  if (LANES >= 8) v = op(v, dpp<0x141>(v));   // row_half_mirror: other quad of the 8
  if (LANES >= 16) v = op(v, dpp<0x140>(v));  // row_mirror: other half of the 16
  if (LANES >= 32) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = op(__uint_as_float(r[0]), __uint_as_float(r[1]));
  }
  if (LANES >= 64) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = op(__uint_as_float(r[0]), __uint_as_float(r[1]));
  }
  return v;
}
// float64 rows only occur in the strided kernel: plain wave shuffles
template <int LANES, typename Op>
__device__ __forceinline__ double group_reduce(double v, Op op) {
  for (int off = LANES >> 1; off > 0; off >>= 1) v = op(v, __shfl_xor(v, off, 64));
  return v;
}

// Exponentials are taken in base 2 on pre-scaled arguments (float: one v_exp_f32 per element).
__device__ __forceinline__ float exp2_of(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ double exp2_of(double x) { return exp2(x); }

template <typename A>
__device__ __forceinline__ A minus_infinity() {
  return -__builtin_huge_val();
}

// Accumulator -> storage; bfloat16 through the hardware conversion (round to nearest even).
template <typename T>
__device__ __forceinline__ T narrow(typename Acc<T>::type v) {
  return from_acc<T>(v);
}
template <>
__device__ __forceinline__ bf16_t narrow<bf16_t>(float v) {
  const f32x2 pair = {v, 0.0f};
  bf16_t r;
  r.bits = (uint16_t)__builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
  return r;
}

// Valid band columns of sequence row i: [lo, hi) (reference tests/utils.py:79-81).
__device__ __forceinline__ void valid_columns(int i, int M, int w, int *lo, int *hi) {
  *lo = max(w - i, 0);
  *hi = (int)min((int64_t)(2 * w + 1), (int64_t)M + w - i);  // M + w may exceed 32 bits
}

// ---------------------------------------------------------------------------------------------
// Row arithmetic.  LANES lanes share one row; lane `gl` takes elements gl, gl + LANES, ...
// `c` is scale * log2(e).
// ---------------------------------------------------------------------------------------------
// Register variant for rows in LDS: SLOTS elements per lane, each read once.  The shape class
// (LANES, SLOTS, FULL) is picked on the host so that FULL * LANES < W <= SLOTS * LANES: the
// first FULL slots lie inside the row for every lane and run without any bounds logic, the
// others are bounds-checked.  Reads past the end of a row are harmless (the image has slack
// for them) and are discarded by selects, never by arithmetic.
template <typename T, bool MASK, int LANES, int SLOTS, int FULL>
__device__ __forceinline__ void softmax_row_forward_regs(const T *x, T *out, int W, int lo, int hi, int gl, float c) {
  const float ninf = minus_infinity<float>();
  float v[SLOTS];
#pragma unroll
  for (int k = 0; k < SLOTS; ++k) v[k] = to_acc<T>(x[gl + k * LANES]) * c;
  float m = ninf;
#pragma unroll
  for (int k = 0; k < SLOTS; ++k) {
    const int j = gl + k * LANES;
    if (k >= FULL) v[k] = j < W ? v[k] : ninf;
    if (MASK) v[k] = (j >= lo && j < hi) ? v[k] : ninf;
    m = v[k] > m ? v[k] : m;
  }
  m = group_reduce<LANES>(m, MaxOp());
  float sum = 0;
#pragma unroll
  for (int k = 0; k < SLOTS; ++k) {
    v[k] = exp2_of(v[k] - m);  // exactly 0 for the entries set to -infinity above
    sum += v[k];
  }
  sum = group_reduce<LANES>(sum, SumOp());
  const float inv = __builtin_amdgcn_rcpf(sum);
#pragma unroll
  for (int k = 0; k < SLOTS; ++k) {
    const int j = gl + k * LANES;
    if (k < FULL || j < W) out[j] = narrow<T>(v[k] * inv);
  }
}

template <typename T, bool MASK, int LANES, int SLOTS, int FULL>
__device__ __forceinline__ void softmax_row_backward_regs(const T *p, const T *g, T *out, int W, int lo, int hi, int gl,
                                                          float scale) {
  float pv[SLOTS], gv[SLOTS];
#pragma unroll
  for (int k = 0; k < SLOTS; ++k) {
    pv[k] = to_acc<T>(p[gl + k * LANES]);
    gv[k] = to_acc<T>(g[gl + k * LANES]);
  }
  float dot = 0;
#pragma unroll
  for (int k = 0; k < SLOTS; ++k) {
    const int j = gl + k * LANES;
    if (MASK || k >= FULL) {
      const bool valid = (k < FULL || j < W) && (!MASK || (j >= lo && j < hi));
      pv[k] = valid ? pv[k] : 0.0f;
      gv[k] = valid ? gv[k] : 0.0f;
    }
    dot += pv[k] * gv[k];
  }
  dot = group_reduce<LANES>(dot, SumOp());
#pragma unroll
  for (int k = 0; k < SLOTS; ++k) {
    const int j = gl + k * LANES;
    float r = scale * pv[k] * (gv[k] - dot);
    if (MASK) r = (j >= lo && j < hi) ? r : 0.0f;  // +0.0, not -0.0
    if (k < FULL || j < W) out[j] = narrow<T>(r);
  }
}

// Rows of any length, in LDS or in global memory, 64 lanes per row: the row is read three
// times (forward) or twice (backward).
template <typename T, typename Row, typename Out>
__device__ __forceinline__ void softmax_row_forward(Row x, Out out, int W, int lo, int hi, int gl,
                                                    typename Acc<T>::type c) {
  typedef typename Acc<T>::type A;
  A m = minus_infinity<A>();
  for (int j = lo + gl; j < hi; j += 64) {
    const A s = to_acc<T>(x(j)) * c;
    m = s > m ? s : m;
  }
  m = group_reduce<64>(m, MaxOp());
  A sum = 0;
  for (int j = lo + gl; j < hi; j += 64) sum += exp2_of(to_acc<T>(x(j)) * c - m);
  sum = group_reduce<64>(sum, SumOp());
  const A inv = A(1) / sum;
  for (int j = gl; j < W; j += 64) {
    const bool valid = j >= lo && j < hi;
    const A p = valid ? exp2_of(to_acc<T>(x(j)) * c - m) * inv : A(0);
    out(j, narrow<T>(p));
  }
}

template <typename T, typename Row, typename Out>
__device__ __forceinline__ void softmax_row_backward(Row p, Row g, Out out, int W, int lo, int hi, int gl,
                                                     typename Acc<T>::type scale) {
  typedef typename Acc<T>::type A;
  A dot = 0;
  for (int j = lo + gl; j < hi; j += 64) dot += to_acc<T>(p(j)) * to_acc<T>(g(j));
  dot = group_reduce<64>(dot, SumOp());
  for (int j = gl; j < W; j += 64) {
    const bool valid = j >= lo && j < hi;
    const A r = valid ? scale * to_acc<T>(p(j)) * (to_acc<T>(g(j)) - dot) : A(0);
    out(j, narrow<T>(r));
  }
}

// ---------------------------------------------------------------------------------------------
// Staged kernel
// ---------------------------------------------------------------------------------------------
// One workgroup owns `R` consecutive rows = elements [e0, e0 + n) of the flat tensor.  The LDS
// image mirrors global memory from the 16-byte boundary at or below e0: element e0 + t sits at
// image index hd + t, hd = e0 % (16 / sizeof(T)).
template <typename T>
struct Span {
  static constexpr int EPC = 16 / (int)sizeof(T);  // elements per 16-byte chunk
  int hd;      // image index of the first owned element
  int end;     // image index one past the last owned element
  int c_lo;    // first chunk that lies wholly inside the span
  int c_hi;    // one past the last such chunk (may be below c_lo for a tiny span)
  int head_end, tail_begin;  // [hd, head_end) and [tail_begin, end) are copied element by element
  __device__ Span(int64_t e0, int n) {
    hd = (int)(e0 % EPC);
    end = hd + n;
    c_lo = hd ? 1 : 0;
    c_hi = end / EPC;
    head_end = min(end, c_lo * EPC);
    tail_begin = max(c_hi * EPC, head_end);
  }
};

// global -> LDS image.  `src` points at the element with image index 0 (16-byte aligned).
template <typename T>
__device__ __forceinline__ void span_fetch(const Span<T> &s, const T *src, T *image, u32x4 (&hold)[kLoadsInFlight],
                                           int base) {
  // loads only: a chunk index past the end is replaced by a readable one and dropped later
#pragma unroll
  for (int u = 0; u < kLoadsInFlight; ++u) {
    const int c = base + u * kSoftmaxThreads;
    const int cs = c < s.c_hi ? c : s.c_lo;
    hold[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src) + cs);
  }
}
template <typename T>
__device__ __forceinline__ void span_stash(const Span<T> &s, T *image, const u32x4 (&hold)[kLoadsInFlight], int base) {
#pragma unroll
  for (int u = 0; u < kLoadsInFlight; ++u) {
    const int c = base + u * kSoftmaxThreads;
    if (c < s.c_hi) reinterpret_cast<u32x4 *>(image)[c] = hold[u];
  }
}
template <typename T>
__device__ __forceinline__ void span_edges_in(const Span<T> &s, const T *src, T *image) {
  const int t = threadIdx.x;
  if (s.hd + t < s.head_end) image[s.hd + t] = src[s.hd + t];
  if (s.tail_begin + t < s.end) image[s.tail_begin + t] = src[s.tail_begin + t];
}
template <typename T>
__device__ __forceinline__ void span_write(const Span<T> &s, T *dst, const T *image) {
  const int t = threadIdx.x;
  for (int c = s.c_lo + t; c < s.c_hi; c += kSoftmaxThreads)
    __builtin_nontemporal_store(reinterpret_cast<const u32x4 *>(image)[c], reinterpret_cast<u32x4 *>(dst) + c);
  if (s.hd + t < s.head_end) dst[s.hd + t] = image[s.hd + t];
  if (s.tail_begin + t < s.end) dst[s.tail_begin + t] = image[s.tail_begin + t];
}

template <typename T>
struct LdsRow {
  const T *p;
  __device__ __forceinline__ T operator()(int j) const { return p[j]; }
};
template <typename T>
struct LdsOut {
  T *p;
  __device__ __forceinline__ void operator()(int j, T v) const { p[j] = v; }
};

// Shape class of the register variant; SLOTS == 0 selects the re-reading variant (64 lanes).
template <int L, int S, int F>
struct Shape {
  static constexpr int lanes = L, slots = S, full = F;
};

template <typename T, bool BACKWARD, bool MASK, typename SHAPE>
__global__ __launch_bounds__(kSoftmaxThreads) void band_softmax_staged_kernel(
    const T *__restrict__ in0, const T *__restrict__ in1, T *__restrict__ out, int64_t rows, int M, int w, int R,
    int image_elems, float scale) {
  extern __shared__ u32x4 softmax_lds[];
  T *image0 = reinterpret_cast<T *>(softmax_lds);
  T *image1 = image0 + image_elems;  // backward only
  constexpr int LANES = SHAPE::lanes;

  const int W = 2 * w + 1;
  const int64_t r0 = (int64_t)blockIdx.x * R;
  const int nrows = (int)min((int64_t)R, rows - r0);
  const int64_t e0 = r0 * W;
  const Span<T> span(e0, nrows * W);
  const int64_t origin = e0 - span.hd;  // flat index of image element 0
  const int tid = threadIdx.x;

  for (int base = span.c_lo + tid; base < span.c_hi; base += kSoftmaxThreads * kLoadsInFlight) {
    u32x4 h0[kLoadsInFlight], h1[kLoadsInFlight];
    span_fetch<T>(span, in0 + origin, image0, h0, base);
    if (BACKWARD) span_fetch<T>(span, in1 + origin, image1, h1, base);
    span_stash<T>(span, image0, h0, base);
    if (BACKWARD) span_stash<T>(span, image1, h1, base);
  }
  span_edges_in<T>(span, in0 + origin, image0);
  if (BACKWARD) span_edges_in<T>(span, in1 + origin, image1);
  __syncthreads();

  constexpr int groups = kSoftmaxThreads / LANES;
  const int gid = tid / LANES, gl = tid % LANES;
  const uint32_t i0 = MASK ? (uint32_t)(r0 % M) : 0u;  // sequence row of the first owned row
  for (int r = gid; r < nrows; r += groups) {
    int lo = 0, hi = W;
    if (MASK) {
      uint32_t i = i0 + (uint32_t)r;
      if (i >= (uint32_t)M) i = (R <= M) ? i - (uint32_t)M : i % (uint32_t)M;
      valid_columns((int)i, M, w, &lo, &hi);
    }
    T *row0 = image0 + span.hd + r * W;
    T *row1 = image1 + span.hd + r * W;
    if constexpr (SHAPE::slots > 0) {
      if (BACKWARD)
        softmax_row_backward_regs<T, MASK, LANES, SHAPE::slots, SHAPE::full>(row0, row1, row0, W, lo, hi, gl, scale);
      else
        softmax_row_forward_regs<T, MASK, LANES, SHAPE::slots, SHAPE::full>(row0, row0, W, lo, hi, gl,
                                                                            scale * kLog2e);
    } else {
      if (BACKWARD)
        softmax_row_backward<T>(LdsRow<T>{row0}, LdsRow<T>{row1}, LdsOut<T>{row0}, W, lo, hi, gl, scale);
      else
        softmax_row_forward<T>(LdsRow<T>{row0}, LdsOut<T>{row0}, W, lo, hi, gl, scale * kLog2e);
    }
  }
  __syncthreads();
  span_write<T>(span, out + origin, image0);
}

// ---------------------------------------------------------------------------------------------
// Strided kernel: one wavefront per row, any dtype, any strides
// ---------------------------------------------------------------------------------------------
template <typename T>
struct GlobalRow {
  const T *p;
  int64_t sc;
  __device__ __forceinline__ T operator()(int j) const { return p[j * sc]; }
};
template <typename T>
struct GlobalOut {
  T *p;
  int64_t sc;
  __device__ __forceinline__ void operator()(int j, T v) const { p[j * sc] = v; }
};

template <typename T, bool BACKWARD>
__global__ __launch_bounds__(kSoftmaxThreads) void band_softmax_strided_kernel(View in0, View in1, View out,
                                                                               int64_t rows, int M, int w,
                                                                               double scale, int mask) {
  typedef typename Acc<T>::type A;
  const int64_t row = (int64_t)blockIdx.x * (kSoftmaxThreads / 64) + threadIdx.x / 64;
  if (row >= rows) return;
  const int gl = threadIdx.x % 64;
  const int64_t b = row / M;
  const int i = (int)(row % M);
  int lo, hi;
  const int W = 2 * w + 1;
  lo = 0, hi = W;
  if (mask) valid_columns(i, M, w, &lo, &hi);
  const GlobalRow<T> x{static_cast<const T *>(in0.data) + b * in0.sb + i * in0.sr, in0.sc};
  const GlobalOut<T> o{static_cast<T *>(out.data) + b * out.sb + i * out.sr, out.sc};
  if (BACKWARD) {
    const GlobalRow<T> g{static_cast<const T *>(in1.data) + b * in1.sb + i * in1.sr, in1.sc};
    softmax_row_backward<T>(x, g, o, W, lo, hi, gl, (A)scale);
  } else {
    softmax_row_forward<T>(x, o, W, lo, hi, gl, (A)(scale * 1.4426950408889634));
  }
}

// ---------------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------------
bool contiguous_band(const View &v, int64_t M, int64_t W) {
  return v.sc == 1 && v.sr == W && v.sb == M * W && ((uintptr_t)v.data) % 16 == 0;
}

// Shape classes of the register variant, then the re-reading one.  Lanes per row: 64 for rows
// longer than 128, else the power of two at or above W/4 (at least 4), which gives 3 or 4
// elements per lane (1..4 for the shortest rows); long rows get 3..20 per lane in steps that
// waste at most a quarter of the slots.
typedef std::tuple<Shape<4, 1, 0>, Shape<4, 2, 1>, Shape<4, 3, 2>, Shape<4, 4, 3>, Shape<8, 3, 2>, Shape<8, 4, 3>,
                   Shape<16, 3, 2>, Shape<16, 4, 3>, Shape<32, 3, 2>, Shape<32, 4, 3>, Shape<64, 3, 2>,
                   Shape<64, 4, 3>, Shape<64, 5, 4>, Shape<64, 6, 5>, Shape<64, 8, 6>, Shape<64, 10, 8>,
                   Shape<64, 12, 10>, Shape<64, 16, 12>, Shape<64, 20, 16>, Shape<64, 0, 0>>
    Shapes;
constexpr int kMaxSlots = 20;

struct StagedPlan {
  int lanes, slots, slots_class;  // slots_class: SLOTS of the chosen class (0: re-reading variant)
  int R, image_elems;
  size_t lds;
};

constexpr int class_slots(int lanes, int slots) {
  if (slots > kMaxSlots) return 0;
  if (lanes < 64 || slots <= 6) return slots < 3 && lanes > 4 ? 3 : slots;
  return slots <= 8 ? 8 : slots <= 10 ? 10 : slots <= 12 ? 12 : slots <= 16 ? 16 : 20;
}

bool plan_staged(int64_t W, size_t es, bool backward, StagedPlan *plan) {
  int lanes = 4;
  while (lanes < 64 && lanes * 4 < W) lanes *= 2;
  const int64_t slots = (W + lanes - 1) / lanes;
  const int cs = class_slots(lanes, (int)(slots > kMaxSlots ? kMaxSlots + 1 : slots));
  // elements a lane may read past the end of a row
  const int64_t slack = cs ? (int64_t)cs * lanes - W : 0;
  const int groups = kSoftmaxThreads / lanes;
  const int64_t row_bytes = W * (int64_t)es;
  const int images = backward ? 2 : 1;
  const int64_t cap = (kLdsLimit / images - 32 - slack * (int64_t)es) / row_bytes;  // rows that fit at all
  if (cap < 1) return false;
  int64_t R = kSpanBytes / row_bytes;
  R = (R + groups - 1) / groups * groups;  // every lane group gets the same number of rows
  if (R < groups) R = groups;
  if (R > cap) R = cap;
  plan->lanes = lanes;
  plan->slots = (int)slots;
  plan->slots_class = cs;
  plan->R = (int)R;
  // image: the span, up to one chunk of lead-in, the slack, rounded up to whole chunks
  const int64_t image_bytes = ((R * row_bytes + 16 + slack * (int64_t)es + 15) / 16) * 16;
  plan->image_elems = (int)(image_bytes / (int64_t)es);
  plan->lds = (size_t)(image_bytes * images);
  return true;
}

template <typename T, bool BACKWARD, bool MASK, size_t I = 0>
hipError_t launch_shape(const StagedPlan &plan, const T *a, const T *g, T *o, int64_t rows, int M, int w, float scale,
                        hipStream_t stream) {
  if constexpr (I == std::tuple_size<Shapes>::value) {
    return hipErrorInvalidValue;
  } else {
    typedef typename std::tuple_element<I, Shapes>::type S;
    if (S::lanes == plan.lanes && S::slots == plan.slots_class) {
      const int64_t blocks = (rows + plan.R - 1) / plan.R;
      if (blocks > 0x7fffffff) return hipErrorInvalidValue;
      hipLaunchKernelGGL((band_softmax_staged_kernel<T, BACKWARD, MASK, S>), dim3((unsigned)blocks),
                         dim3(kSoftmaxThreads), plan.lds, stream, a, g, o, rows, M, w, plan.R, plan.image_elems,
                         scale);
      return hipGetLastError();
    }
    return launch_shape<T, BACKWARD, MASK, I + 1>(plan, a, g, o, rows, M, w, scale, stream);
  }
}

template <typename T, bool BACKWARD>
hipError_t launch_staged(const StagedPlan &plan, const View &in0, const View &in1, const View &out, int64_t rows,
                         int64_t M, int64_t w, double scale, int mask, hipStream_t stream) {
  const T *a = static_cast<const T *>(in0.data), *g = static_cast<const T *>(in1.data);
  T *o = static_cast<T *>(out.data);
  if (mask) return launch_shape<T, BACKWARD, true>(plan, a, g, o, rows, (int)M, (int)w, (float)scale, stream);
  return launch_shape<T, BACKWARD, false>(plan, a, g, o, rows, (int)M, (int)w, (float)scale, stream);
}

template <typename T, bool BACKWARD>
hipError_t launch_strided(const View &in0, const View &in1, const View &out, int64_t rows, int64_t M, int64_t w,
                          double scale, int mask, hipStream_t stream) {
  const int per_block = kSoftmaxThreads / 64;
  const int64_t blocks = (rows + per_block - 1) / per_block;
  if (blocks > 0x7fffffff) return hipErrorInvalidValue;
  hipLaunchKernelGGL((band_softmax_strided_kernel<T, BACKWARD>), dim3((unsigned)blocks), dim3(kSoftmaxThreads), 0,
                     stream, in0, in1, out, rows, (int)M, (int)w, scale, mask);
  return hipGetLastError();
}

template <bool BACKWARD>
hipError_t dispatch(const Problem &p, const View &in0, const View &in1, const View &out, double scale, int mask) {
  const int64_t W = 2 * p.w + 1, rows = p.B * p.M;
  if (rows == 0) return hipSuccess;
  StagedPlan plan;
  const bool staged = !(p.flags & WM_FLAG_FORCE_STRIDED) && p.dtype != WM_DTYPE_F64 && contiguous_band(in0, p.M, W) &&
                      (!BACKWARD || contiguous_band(in1, p.M, W)) && contiguous_band(out, p.M, W) &&
                      plan_staged(W, dtype_size(p.dtype), BACKWARD, &plan);
  if (staged) {
    switch (p.dtype) {
      case WM_DTYPE_F32: return launch_staged<float, BACKWARD>(plan, in0, in1, out, rows, p.M, p.w, scale, mask, p.stream);
      case WM_DTYPE_F16: return launch_staged<f16_t, BACKWARD>(plan, in0, in1, out, rows, p.M, p.w, scale, mask, p.stream);
      default: return launch_staged<bf16_t, BACKWARD>(plan, in0, in1, out, rows, p.M, p.w, scale, mask, p.stream);
    }
  }
  switch (p.dtype) {
    case WM_DTYPE_F32: return launch_strided<float, BACKWARD>(in0, in1, out, rows, p.M, p.w, scale, mask, p.stream);
    case WM_DTYPE_F16: return launch_strided<f16_t, BACKWARD>(in0, in1, out, rows, p.M, p.w, scale, mask, p.stream);
    case WM_DTYPE_BF16: return launch_strided<bf16_t, BACKWARD>(in0, in1, out, rows, p.M, p.w, scale, mask, p.stream);
    default: return launch_strided<double, BACKWARD>(in0, in1, out, rows, p.M, p.w, scale, mask, p.stream);
  }
}

}  // namespace

hipError_t launch_band_softmax_forward(const Problem &p, const View &a, const View &out, double scale, int mask) {
  return dispatch<false>(p, a, a, out, scale, mask);
}
hipError_t launch_band_softmax_backward(const Problem &p, const View &probs, const View &grad_probs, const View &grad_a,
                                        double scale, int mask) {
  return dispatch<true>(p, probs, grad_probs, grad_a, scale, mask);
}
bool band_softmax_staged(int64_t W, int dtype, bool backward) {
  StagedPlan plan;
  return dtype != WM_DTYPE_F64 && plan_staged(W, dtype_size(dtype), backward, &plan);
}

}  // namespace wm
