// float32 MFMA kernel family (v_mfma_f32_32x32x2_f32) for gfx950.
//
// Same tiling idea as the 16-bit wide-band family -- a workgroup of four waves owns 128 rows
// and walks the contraction in chunks, the skewed tile T[r][c] = band[r, c-r+w] and the dense
// operand chunk go through LDS -- but with 4-byte elements and a matrix instruction whose
// operands are one float per lane (row = lane % 32, k = lane / 32).  float32 at these shapes is
// bound by the matrix pipe (157 TFLOP/s), not by HBM, so the memory side is kept simple:
// 16-byte band accesses at 4-byte alignment (no aligned column grid, no seam handling),
// one chunk of register prefetch, double-buffered LDS, one barrier per chunk.
//
// Contraction order.  An MFMA step contracts two k values, one per half-wave.  The kernels walk
// k in groups of 8: step (u, j), half-wave s, uses k = 8u + 4s + j.  Both operands use the same
// map, so the sum is unchanged, and an operand whose k runs along memory is fetched as one
// 16-byte LDS read per group (4 steps) instead of one 4-byte read per step.
#include "wm_common.hpp"

#include <algorithm>

namespace wm {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int TM = 128;  // rows per workgroup, 32 per wave
constexpr int KC = 32;   // chunk length

struct __attribute__((packed, aligned(4))) Chunk4 {
  f32x4 v;
};
__device__ __forceinline__ f32x4 load4(const float *p) { return reinterpret_cast<const Chunk4 *>(p)->v; }
__device__ __forceinline__ void store4(float *p, f32x4 v) { reinterpret_cast<Chunk4 *>(p)->v = v; }

// Elements [e_lo, e_hi] of a 4-element band chunk, the rest cleared (on bits: NaN-safe).
__device__ __forceinline__ f32x4 keep4(f32x4 v, int e_lo, int e_hi) {
  f32x4 r;
#pragma unroll
  for (int e = 0; e < 4; ++e) r[e] = (e >= e_lo && e <= e_hi) ? v[e] : 0.f;
  return r;
}
// Band chunk with valid elements [e_lo, e_hi]: read whole when any element is valid (the up-to-3
// elements beside a row's valid range are band entries of the same or the neighbouring row for
// w >= 3; the kernels are used for w >= 4), from `safe` otherwise; invalid elements cleared.
__device__ __forceinline__ f32x4 load_band4(const float *p, const float *safe, int e_lo, int e_hi) {
  const bool any = (e_hi >= 0) & (e_lo <= 3) & (e_lo <= e_hi);
  return keep4(load4(any ? p : safe), any ? e_lo : 4, e_hi);
}
__device__ __forceinline__ f32x4 load_row4(const float *p, const float *safe, bool valid) {
  const f32x4 v = *reinterpret_cast<const f32x4 *>(valid ? p : safe);
  f32x4 z = {0.f, 0.f, 0.f, 0.f};
  return valid ? v : z;
}
__device__ __forceinline__ bool band_any(int e_lo, int e_hi) { return (e_hi >= 0) & (e_lo <= 3) & (e_lo <= e_hi); }
// Keeps a loaded value opaque until here, so that whatever is computed from it (masks) is not
// scheduled right behind the load.
__device__ __forceinline__ f32x4 pin(f32x4 v) {
  asm volatile("" : "+v"(v));
  return v;
}
__device__ __forceinline__ void wave_sync_lds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ f32x16 mma(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}
// ------------------------------------------------------------------------------------------
// P2: C[b,i,h] = sum_c T[i][c] Y[b,c,h]          P3: C[b,c,h] = sum_r T[r][c] Y[b,r,h]
// acc(m = h, n = output row): A operand Y[k][h] (4-byte LDS reads along h), B operand T.
//
// Pipeline: chunk k+2 is requested (loads only, into one of two register sets) before chunk k is
// multiplied; chunk k+1, requested a whole slot earlier, is masked and moved to LDS after the
// multiply.  Loads and the masking of what they return are kept apart on purpose: a mask right
// behind its load would make the wave wait for the load where it is issued.
// ------------------------------------------------------------------------------------------
constexpr int kStage = 32 + 4;  // staged result row: 32 floats, rows 16 bytes apart mod 128

template <int NT, bool TRANSPOSED>
__global__ __launch_bounds__(kThreads, NT <= 2 ? 3 : 2) void f32_band_in_kernel(const float *__restrict__ A,
                                                                  const float *__restrict__ Y,
                                                                  float *__restrict__ C, int B, int M, int N, int w,
                                                                  int nblk, int64_t asb, int64_t ysb, int64_t ysr,
                                                                  int64_t csb, int64_t csr) {
  constexpr int NP = 32 * NT;
  constexpr int ST = TRANSPOSED ? TM + 4 : KC + 4;  // T tile: [KC][TM] (P3) or [TM][KC] (P2), floats
  constexpr int TROWS = TRANSPOSED ? KC : TM;
  constexpr int SY = NP + 4;
  __shared__ __attribute__((aligned(16))) float t_lds[2][TROWS * ST];
  __shared__ __attribute__((aligned(16))) float y_lds[2][KC * SY];
  static_assert(4 * 32 * kStage <= 2 * TROWS * ST, "the four staging areas must fit the band tile buffers");

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int W = 2 * w + 1;
  const int o0 = blk * TM;                 // first output row of the block (i for P2, c for P3)
  const int o1 = min(o0 + TM, M) - 1;      // last one
  const int k_lo = max(o0 - w, 0), k_hi = min(o1 + w, M - 1);  // contraction range (c for P2, r for P3)
  const int nk = (k_hi - k_lo + KC) / KC;
  const float *Ab = A + (int64_t)b * asb;
  // blockIdx.y selects which NP columns of Y and C this workgroup works on (one workgroup does all
  // of them unless the launch splits the columns to fill the chip)
  const int h0 = NP * blockIdx.y;
  const float *Yb = Y + (int64_t)b * ysb + h0;
  const int ncg = min(N - h0, NP) >> 2, ychunks = KC * ncg;
  int y_row[NT], y_col[NT];  // this thread's pieces of a Y chunk; row KC = none
#pragma unroll
  for (int s = 0; s < NT; ++s) {
    const int q = tid + kThreads * s;
    y_row[s] = q < ychunks ? q / ncg : KC;
    y_col[s] = q < ychunks ? (q % ncg) * 4 : 0;
  }

  // Band piece s of this thread: its address in chunk 0 (advanced by `t_step` elements per chunk)
  // and what decides its valid element range [e_lo, e_hi] (0..3) in a chunk.
  const float *t_ptr[4];
  int t_fix[4];  // P2: band row i of the piece; P3: first output column c4 of the piece
  const int64_t t_step = TRANSPOSED ? (int64_t)KC * (W - 1) : KC;
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int q = tid + kThreads * s;
    if (!TRANSPOSED) {  // tile row = band row i, 4 consecutive dense columns c
      const int i = o0 + (q >> 3);
      t_fix[s] = i;
      t_ptr[s] = Ab + (int64_t)i * W + (w - i) + k_lo + 4 * (q & 7);
    } else {  // tile row = band row r (the contraction index), 4 consecutive output columns c
      const int r = k_lo + (q >> 5), c4 = o0 + 4 * (q & 31);
      t_fix[s] = c4;
      t_ptr[s] = Ab + (int64_t)r * W + (w - r) + c4;
    }
  }
  auto piece_range = [&](int kb, int s, int &e_lo, int &e_hi) {
    const int q = tid + kThreads * s;
    if (!TRANSPOSED) {
      const int i = t_fix[s], c4 = kb + 4 * (q & 7);
      const int lo = max(i - w, 0), hi = i <= o1 ? min(i + w, k_hi) : -1;
      e_lo = lo - c4, e_hi = hi - c4;
    } else {
      const int r = kb + (q >> 5), c4 = t_fix[s];
      const int lo = max(r - w, o0), hi = r <= k_hi ? min(r + w, o1) : -1;
      e_lo = lo - c4, e_hi = hi - c4;
    }
  };
  // A chunk is interior when every band element of its tile and every Y row is valid: no address
  // selection, no masks (most chunks of a wide band).
  const bool block_whole = o1 == o0 + TM - 1;
  auto interior = [&](int k) {
    const int kb = k_lo + k * KC;
    return block_whole && kb + KC - 1 <= k_hi && kb + KC - 1 - w <= o0 && o1 <= kb + w &&
           (TRANSPOSED || kb >= o1 - w) && (!TRANSPOSED || kb + KC - 1 - w <= o0);
  };
  auto fetch = [&](int k, f32x4(&tr)[4], f32x4(&yr)[NT]) {  // loads only; chunks past the end read the safe address
    const int kb = k_lo + k * KC;
    if (interior(k)) {
#pragma unroll
      for (int s = 0; s < 4; ++s) tr[s] = load4(t_ptr[s] + k * t_step);
#pragma unroll
      for (int s = 0; s < NT; ++s)
        yr[s] = *reinterpret_cast<const f32x4 *>(y_row[s] < KC ? Yb + (int64_t)(kb + y_row[s]) * ysr + y_col[s] : Y);
    } else {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        int e_lo, e_hi;
        piece_range(kb, s, e_lo, e_hi);
        tr[s] = load4(band_any(e_lo, e_hi) ? t_ptr[s] + k * t_step : A);
      }
#pragma unroll
      for (int s = 0; s < NT; ++s) {
        const int kr = kb + y_row[s];
        const bool ok = (y_row[s] < KC) & (kr <= k_hi);
        yr[s] = *reinterpret_cast<const f32x4 *>(ok ? Yb + (int64_t)kr * ysr + y_col[s] : Y);
      }
    }
  };
  auto stash = [&](int k, f32x4(&tr)[4], f32x4(&yr)[NT]) {  // mask, then to LDS buffer k & 1
    const int kb = k_lo + k * KC, buf = k & 1;
    f32x4 tv[4], yv[NT];
#pragma unroll
    for (int s = 0; s < 4; ++s) tv[s] = pin(tr[s]);
#pragma unroll
    for (int s = 0; s < NT; ++s) yv[s] = pin(yr[s]);
    if (!interior(k)) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        int e_lo, e_hi;
        piece_range(kb, s, e_lo, e_hi);
        tv[s] = keep4(tv[s], band_any(e_lo, e_hi) ? e_lo : 4, e_hi);
      }
#pragma unroll
      for (int s = 0; s < NT; ++s) {
        const f32x4 z = {0.f, 0.f, 0.f, 0.f};
        yv[s] = kb + y_row[s] <= k_hi ? yv[s] : z;
      }
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int q = tid + kThreads * s;
      float *dst = TRANSPOSED ? &t_lds[buf][(q >> 5) * ST + 4 * (q & 31)] : &t_lds[buf][(q >> 3) * ST + 4 * (q & 7)];
      *reinterpret_cast<f32x4 *>(dst) = tv[s];
    }
#pragma unroll
    for (int s = 0; s < NT; ++s)
      if (y_row[s] < KC) *reinterpret_cast<f32x4 *>(&y_lds[buf][y_row[s] * SY + y_col[s]]) = yv[s];
  };

  f32x16 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;

  f32x4 t_reg[2][4], y_reg[2][NT];
  fetch(0, t_reg[0], y_reg[0]);
  fetch(1, t_reg[1], y_reg[1]);
  __builtin_amdgcn_sched_barrier(0);
  stash(0, t_reg[0], y_reg[0]);
  __syncthreads();
  const int half = lane >> 5, col = lane & 31;
  auto slot = [&](int k, f32x4(&mine_t)[4], f32x4(&mine_y)[NT], f32x4(&next_t)[4], f32x4(&next_y)[NT]) {
    const int buf = k & 1;
    fetch(k + 2, mine_t, mine_y);
    __builtin_amdgcn_sched_barrier(0);
    const float *tl = t_lds[buf];
    const float *yl = y_lds[buf];
    // the wave's 32 output rows meet the chunk's 32 contraction indices only where |row - index| <= w:
    // a chunk that lies wholly outside that range for this wave is all zeros in its part of the tile
    const int kb = k_lo + k * KC, ow = o0 + wave * 32;
    if (kb <= ow + 31 + w && kb + KC - 1 >= ow - w) {
#pragma unroll
      for (int u = 0; u < KC / 8; ++u) {
        const int kk = 8 * u + 4 * half;  // this half-wave's 4 k values of the group
        f32x4 bop;
        if (!TRANSPOSED) {
          bop = *reinterpret_cast<const f32x4 *>(tl + (wave * 32 + col) * ST + kk);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) bop[j] = tl[(kk + j) * ST + wave * 32 + col];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int t = 0; t < NT; ++t) acc[t] = mma(yl[(kk + j) * SY + 32 * t + col], bop[j], acc[t]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    stash(k + 1, next_t, next_y);
    __syncthreads();
  };
  // Slots run in pairs inside the loop, an odd last one after it: one loop exit, one back edge, so
  // the compiler's count of outstanding loads is the same on every way into a slot.
  int k = 0;
  for (; k + 1 < nk; k += 2) {
    slot(k, t_reg[0], y_reg[0], t_reg[1], y_reg[1]);
    slot(k + 1, t_reg[1], y_reg[1], t_reg[0], y_reg[0]);
  }
  if (k < nk) slot(k, t_reg[0], y_reg[0], t_reg[1], y_reg[1]);

  // acc[t][v]: h = 32 t + 8 (v / 4) + 4 (lane / 32) + v % 4, output row = wave * 32 + lane % 32.
  // Every wave is past the last barrier, so the tile buffers are free: each wave stages 32 columns
  // of its rows at a time in a private area and the rows leave as 16-byte pieces, 8 consecutive
  // lanes on one 128-byte line (non-temporal: the result is not read again here).
  float *stage = &t_lds[0][0] + wave * (32 * kStage);
  float *Cb = C + (int64_t)b * csb + h0;
  N -= h0;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    wave_sync_lds();
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const f32x4 out = {acc[t][4 * q4], acc[t][4 * q4 + 1], acc[t][4 * q4 + 2], acc[t][4 * q4 + 3]};
      *reinterpret_cast<f32x4 *>(stage + col * kStage + 8 * q4 + 4 * half) = out;
    }
    wave_sync_lds();
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int rr = (lane >> 3) + 8 * s, h = 32 * t + 4 * (lane & 7);
      const int o = o0 + wave * 32 + rr;
      if (o <= o1 && h < N)
        __builtin_nontemporal_store(*reinterpret_cast<const f32x4 *>(stage + rr * kStage + 4 * (lane & 7)),
                                    reinterpret_cast<f32x4 *>(Cb + (int64_t)o * csr + h));
    }
  }
}

// ------------------------------------------------------------------------------------------
// P1: band[b,i,c-i+w] = sum_h X[b,i,h] Y[b,c,h]   (+0.0 where c is outside the sequence)
// acc(m = c, n = i): A operand Y chunk (LDS, k = h along memory), B operand X rows (registers).
// The 32 x 32 result of a wave and chunk is staged in wave-private LDS and leaves as 16-byte
// pieces, 8 consecutive lanes on 128 consecutive bytes of one band row.
// ------------------------------------------------------------------------------------------
template <int NK8>  // N = 8 NK8
__global__ __launch_bounds__(kThreads, NK8 <= 8 ? 4 : 2) void f32_band_out_kernel(const float *__restrict__ X,
                                                                   const float *__restrict__ Y,
                                                                   float *__restrict__ C, int B, int M, int w,
                                                                   int nblk, int64_t xsb, int64_t xsr, int64_t ysb,
                                                                   int64_t ysr, int64_t csb) {
  constexpr int N = 8 * NK8;
  constexpr int SY = N + 4;
  constexpr int PIECES = KC * N / 4;
  constexpr int YS = (PIECES + kThreads - 1) / kThreads;
  __shared__ __attribute__((aligned(16))) float y_lds[2][KC * SY];
  __shared__ __attribute__((aligned(16))) float stage_lds[4][32 * kStage];

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  const int W = 2 * w + 1;
  const int i0 = blk * TM;
  const int rows = min(TM, M - i0);
  int c_lo = i0 - w;  // not clipped: entries outside the sequence are zeros
  const int c_hi = i0 + rows - 1 + w;
  int nk = (c_hi - c_lo + KC) / KC;
  {  // blockIdx.y selects this workgroup's share of the chunks (all of them unless the launch splits them)
    const int first = (int)((int64_t)nk * blockIdx.y / gridDim.y), last = (int)((int64_t)nk * (blockIdx.y + 1) / gridDim.y);
    c_lo += first * KC;
    nk = last - first;
  }
  const float *Yb = Y + (int64_t)b * ysb;
  float *Cb = C + (int64_t)b * csb;

  // this lane's row of X, the k values of its half-wave: xop[u][j] = X[i][8u + 4 half + j]
  const int i = i0 + wave * 32 + col;
  f32x4 xop[NK8];
#pragma unroll
  for (int u = 0; u < NK8; ++u)
    xop[u] = load_row4(X + (int64_t)b * xsb + (int64_t)i * xsr + 8 * u + 4 * half, X, i < M);

  int y_row[YS], y_col[YS];  // this thread's pieces of a Y chunk; row KC = none
#pragma unroll
  for (int s = 0; s < YS; ++s) {
    const int q = tid + kThreads * s;
    y_row[s] = q < PIECES ? q / (N / 4) : KC;
    y_col[s] = q < PIECES ? (q % (N / 4)) * 4 : 0;
  }
  auto fetch = [&](int k, f32x4(&yr)[YS]) {  // loads only; rows outside the sequence read the safe address
    const int cb = c_lo + k * KC;
#pragma unroll
    for (int s = 0; s < YS; ++s) {
      const int c = cb + y_row[s];
      const bool ok = (y_row[s] < KC) & (c >= 0) & (c < M);
      yr[s] = *reinterpret_cast<const f32x4 *>(ok ? Yb + (int64_t)c * ysr + y_col[s] : Y);
    }
  };
  auto stash = [&](int k, f32x4(&yr)[YS]) {
    const int cb = c_lo + k * KC, buf = k & 1;
    f32x4 yv[YS];
#pragma unroll
    for (int s = 0; s < YS; ++s) yv[s] = pin(yr[s]);
#pragma unroll
    for (int s = 0; s < YS; ++s) {
      const int c = cb + y_row[s];
      const f32x4 z = {0.f, 0.f, 0.f, 0.f};
      if (y_row[s] < KC) *reinterpret_cast<f32x4 *>(&y_lds[buf][y_row[s] * SY + y_col[s]]) = ((c >= 0) & (c < M)) ? yv[s] : z;
    }
  };

  f32x4 y_reg[2][YS];
  fetch(0, y_reg[0]);
  fetch(1, y_reg[1]);
  __builtin_amdgcn_sched_barrier(0);
  stash(0, y_reg[0]);
  __syncthreads();
  float *stage = stage_lds[wave];
  auto slot = [&](int k, f32x4(&mine)[YS], f32x4(&next)[YS]) {
    const int buf = k & 1;
    const int cb = c_lo + k * KC;
    fetch(k + 2, mine);
    __builtin_amdgcn_sched_barrier(0);
    // a wave whose 32 rows have no band entry among the chunk's 32 columns has nothing to compute or store
    const int iw = i0 + wave * 32;
    if (cb <= iw + 31 + w && cb + KC - 1 >= iw - w) {
    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.f;
    const float *yl = y_lds[buf] + col * SY + 4 * half;
    // a chunk that lies wholly outside the sequence (a quarter of them when the band covers the
    // sequence) holds zeros only: nothing to multiply, the stores below write the zeros
    if (cb + KC > 0 && cb < M) {
#pragma unroll
      for (int u = 0; u < NK8; ++u) {
        const f32x4 aop = *reinterpret_cast<const f32x4 *>(yl + 8 * u);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = mma(aop[j], xop[u][j], acc);
      }
    }
    // acc[v]: dense column c = cb + 8 (v / 4) + 4 half + v % 4, row i; band column j = c - i + w
    wave_sync_lds();  // the pieces of the previous chunk have been read
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const int c = cb + 8 * q4 + 4 * half;
      f32x4 out;
#pragma unroll
      for (int e = 0; e < 4; ++e) out[e] = (c + e >= 0 && c + e < M) ? acc[4 * q4 + e] : 0.f;  // +0.0 outside
      *reinterpret_cast<f32x4 *>(stage + col * kStage + 8 * q4 + 4 * half) = out;
    }
    wave_sync_lds();
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int rr = (lane >> 3) + 8 * s;
      const int i2 = i0 + wave * 32 + rr, c = cb + 4 * (lane & 7);
      const int e_lo = (i2 - w) - c, e_hi = (i2 + w) - c;
      if (i2 < M && e_hi >= 0 && e_lo <= 3) {
        const f32x4 out = *reinterpret_cast<const f32x4 *>(stage + rr * kStage + 4 * (lane & 7));
        float *dst = Cb + (int64_t)i2 * W + (w - i2) + c;
        if (e_lo <= 0 && e_hi >= 3) {
          store4(dst, out);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (e >= e_lo && e <= e_hi) dst[e] = out[e];
        }
      }
    }
    }
    __builtin_amdgcn_sched_barrier(0);
    stash(k + 1, next);
    __syncthreads();
  };
  int k = 0;
  for (; k + 1 < nk; k += 2) {
    slot(k, y_reg[0], y_reg[1]);
    slot(k + 1, y_reg[1], y_reg[0]);
  }
  if (k < nk) slot(k, y_reg[0], y_reg[1]);
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
bool f32_shape_ok(int64_t M, int64_t N, int64_t w, int dtype) {
  if (dtype != WM_DTYPE_F32) return false;
  if (N < 8 || N > 128 || N % 8 != 0) return false;
  return M >= 1 && M <= (1 << 30) && w >= 4 && w <= (1 << 28);
}
bool f32_band_ok(const View &v, int64_t W) { return v.sc == 1 && v.sr == W && ((uintptr_t)v.data % 4) == 0; }
unsigned f32_grid(int64_t B, int64_t nblk) { return (unsigned)tiled_grid(B, nblk); }

constexpr int64_t kCUs = 256;

template <bool TRANSPOSED>
hipError_t launch_band_in(const Problem &p, const View &a, const View &y, const View &c) {
  const int nblk = (int)((p.M + TM - 1) / TM);
  dim3 grid(f32_grid(p.B, nblk)), block(kThreads);
  // A wavefront multiplies its 32 rows by every 32-column block of Y in turn.  When the workgroups
  // do not even fill the CUs once or twice (config 5 at w = 1500: 168 of them), each block of
  // columns gets workgroups of its own: the band tile is then fetched once per block (the
  // workgroups that share it run on the same XCD at the same time), and the chip holds NB times
  // as many wavefronts with a third or half of the work each.
  const int64_t wgs = p.B * nblk, nb = (p.N + 31) / 32;
  if (nb > 1 && wgs < 2 * kCUs && (wgs * nb + kCUs - 1) / kCUs < nb * ((wgs + kCUs - 1) / kCUs)) {
    grid.y = (unsigned)nb;
    hipLaunchKernelGGL((f32_band_in_kernel<1, TRANSPOSED>), grid, block, 0, p.stream, (const float *)a.data,
                       (const float *)y.data, (float *)c.data, (int)p.B, (int)p.M, (int)p.N, (int)p.w, nblk, a.sb, y.sb,
                       y.sr, c.sb, c.sr);
    return hipGetLastError();
  }
#define WM_F32_IN(NT)                                                                                        \
  hipLaunchKernelGGL((f32_band_in_kernel<NT, TRANSPOSED>), grid, block, 0, p.stream, (const float *)a.data,  \
                     (const float *)y.data, (float *)c.data, (int)p.B, (int)p.M, (int)p.N, (int)p.w, nblk,   \
                     a.sb, y.sb, y.sr, c.sb, c.sr)
  switch ((p.N + 31) / 32) {
    case 1: WM_F32_IN(1); break;
    case 2: WM_F32_IN(2); break;
    case 3: WM_F32_IN(3); break;
    default: WM_F32_IN(4); break;
  }
#undef WM_F32_IN
  return hipGetLastError();
}

hipError_t launch_band_out(const Problem &p, const View &x, const View &y, const View &c) {
  const int nblk = (int)((p.M + TM - 1) / TM);
  dim3 grid(f32_grid(p.B, nblk)), block(kThreads);
  // too few workgroups to fill the chip: each takes a share of its tile's dense columns instead of
  // all of them (nothing is fetched or computed twice: the shares produce disjoint parts of the band)
  const int64_t wgs = p.B * nblk, chunks = (TM + 2 * p.w + KC - 1) / KC;
  if (wgs < 2 * kCUs) grid.y = (unsigned)std::max<int64_t>(1, std::min<int64_t>(2 * kCUs / wgs, chunks / 4));
#define WM_F32_OUT(NK8)                                                                                     \
  case NK8:                                                                                                 \
    hipLaunchKernelGGL((f32_band_out_kernel<NK8>), grid, block, 0, p.stream, (const float *)x.data,         \
                       (const float *)y.data, (float *)c.data, (int)p.B, (int)p.M, (int)p.w, nblk, x.sb,    \
                       x.sr, y.sb, y.sr, c.sb);                                                             \
    break;
  switch (p.N / 8) {
    WM_F32_OUT(1) WM_F32_OUT(2) WM_F32_OUT(3) WM_F32_OUT(4) WM_F32_OUT(5) WM_F32_OUT(6) WM_F32_OUT(7) WM_F32_OUT(8)
    WM_F32_OUT(9) WM_F32_OUT(10) WM_F32_OUT(11) WM_F32_OUT(12) WM_F32_OUT(13) WM_F32_OUT(14) WM_F32_OUT(15)
    WM_F32_OUT(16)
    default: return hipErrorInvalidValue;
  }
#undef WM_F32_OUT
  return hipGetLastError();
}

}  // namespace

bool f32_supports(int op, int64_t M, int64_t N, int64_t w, int dtype) {
  (void)op;
  return f32_shape_ok(M, N, w, dtype);
}

bool try_launch_f32_p1(const Problem &p, const View &x, const View &y, const View &c, hipError_t *err) {
  if (try_launch_f32_split_p1(p, x, y, c, err)) return true;
  if (!f32_shape_ok(p.M, p.N, p.w, p.dtype)) return false;
  if (!fast_layout(x, p.dtype) || !fast_layout(y, p.dtype) || !f32_band_ok(c, 2 * p.w + 1)) return false;
  *err = launch_band_out(p, x, y, c);
  return true;
}
bool try_launch_f32_p2(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  if (try_launch_f32_split_p2(p, a, y, c, err)) return true;
  if (!f32_shape_ok(p.M, p.N, p.w, p.dtype)) return false;
  if (!f32_band_ok(a, 2 * p.w + 1) || !fast_layout(y, p.dtype) || !fast_layout(c, p.dtype)) return false;
  *err = launch_band_in<false>(p, a, y, c);
  return true;
}
bool try_launch_f32_p3(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  if (try_launch_f32_split_p3(p, a, y, c, err)) return true;
  if (!f32_shape_ok(p.M, p.N, p.w, p.dtype)) return false;
  if (!f32_band_ok(a, 2 * p.w + 1) || !fast_layout(y, p.dtype) || !fast_layout(c, p.dtype)) return false;
  *err = launch_band_in<true>(p, a, y, c);
  return true;
}

}  // namespace wm
