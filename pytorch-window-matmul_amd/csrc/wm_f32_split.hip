// float32 banded products on the bf16 matrix instruction of gfx950, at float32 accuracy.
//
// v_mfma_f32_32x32x2_f32 runs at a sixteenth of the rate of v_mfma_f32_32x32x16_bf16, and the
// float32 products are bound by it wherever the band is wide (the band that covers a sequence of
// 3001 rows at N = 80: 7.6 GFLOP against 266 MB).  A float32 value is exactly the sum of three bf16
// values, its significand cut into 8 + 8 + 8 bits,
//     x = x1 + x2 + x3,   x1 = x with the low 16 bits cleared,  x2 = (x - x1) likewise,  x3 = the rest,
// so a product x y is the sum of nine bf16 products, each of which is exact in the float32
// accumulator of the matrix instruction.  The six with i + j <= 4 are kept,
//     x y ~ x1 y1 + (x1 y2 + x2 y1) + (x1 y3 + x3 y1 + x2 y2),
// which leaves out 3 * 2^-24 |x y| at most: the rounding of one float32 multiplication.  Six bf16
// instructions cover 16 values of the contraction in 192 cycles of the matrix pipe where eight
// float32 instructions take 512.
//
// The kernels are those of wm_f32.hip (same tiles, same way of fetching and masking: 128 rows per
// workgroup, chunks of 32 along the contraction, register prefetch, one barrier per chunk) with
// one change on the way into LDS: a chunk is stored as three bf16 planes per operand, split once per
// element, and the products read those planes like the 16-bit kernels read their tiles (rows as
// 16-byte pieces, columns through ds_read_b64_tr_b16).
//
// Non-finite values: Inf splits into Inf + NaN (Inf - Inf), so an Inf operand gives NaN where the
// float32 instruction gives +-Inf.  What is non-finite in the exact product stays non-finite, and
// nothing non-finite appears where the exact product is finite (|x_i| <= |x|).
#include "wm_mfma_common.hpp"

#include <algorithm>

namespace wm {
namespace {

constexpr int SKC = 32;            // chunk length along the contraction (band-in) / dense columns (band-out)
#ifndef WM_F32_SPLIT_FROM
#define WM_F32_SPLIT_FROM 16
#endif
constexpr int kSplitFromWindow = WM_F32_SPLIT_FROM;
constexpr int kStage = 32 + 4;     // staged result row: 32 floats, rows 16 bytes apart mod 128

struct __attribute__((packed, aligned(4))) Chunk4 {
  f32x4 v;
};
__device__ __forceinline__ f32x4 load4(const float *p) { return reinterpret_cast<const Chunk4 *>(p)->v; }
__device__ __forceinline__ void store4(float *p, f32x4 v) { reinterpret_cast<Chunk4 *>(p)->v = v; }
__device__ __forceinline__ f32x4 keep4(f32x4 v, int e_lo, int e_hi) {
  f32x4 r;
#pragma unroll
  for (int e = 0; e < 4; ++e) r[e] = (e >= e_lo && e <= e_hi) ? v[e] : 0.f;
  return r;
}
__device__ __forceinline__ bool band_any(int e_lo, int e_hi) { return (e_hi >= 0) & (e_lo <= 3) & (e_lo <= e_hi); }
__device__ __forceinline__ f32x4 pin4(f32x4 v) {
  asm volatile("" : "+v"(v));
  return v;
}

// The three bf16 planes of four consecutive floats, each plane as 8 bytes (element e in bits 16 e .. 16 e + 15).
struct Planes4 {
  u32x2 p[3];
};
__device__ __forceinline__ uint32_t high_halves(uint32_t hi, uint32_t lo) {
  return __builtin_amdgcn_perm(hi, lo, 0x07060302u);  // (hi & 0xffff0000) | (lo >> 16)
}
__device__ __forceinline__ Planes4 split4(f32x4 v) {
  uint32_t a[4], b[4], c[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    a[e] = __float_as_uint(v[e]);
    const float r1 = v[e] - __uint_as_float(a[e] & 0xffff0000u);  // exact: the low 16 bits of the significand
    b[e] = __float_as_uint(r1);
    c[e] = __float_as_uint(r1 - __uint_as_float(b[e] & 0xffff0000u));  // at most 8 significant bits left
  }
  Planes4 r;
  r.p[0] = u32x2{high_halves(a[1], a[0]), high_halves(a[3], a[2])};
  r.p[1] = u32x2{high_halves(b[1], b[0]), high_halves(b[3], b[2])};
  r.p[2] = u32x2{high_halves(c[1], c[0]), high_halves(c[3], c[2])};
  return r;
}

__device__ __forceinline__ f32x16 mma16(u32x4 a, u32x4 b, f32x16 c) { return Mma<bf16_t>::run(a, b, c); }
// acc += x y for the split operands xa (A side) and xb (B side), smallest terms first
__device__ __forceinline__ f32x16 mma_split(const u32x4 (&xa)[3], const u32x4 (&xb)[3], f32x16 acc) {
  acc = mma16(xa[2], xb[0], acc);
  acc = mma16(xa[0], xb[2], acc);
  acc = mma16(xa[1], xb[1], acc);
  acc = mma16(xa[1], xb[0], acc);
  acc = mma16(xa[0], xb[1], acc);
  acc = mma16(xa[0], xb[0], acc);
  return acc;
}

// ------------------------------------------------------------------------------------------
// P2: C[b,i,h] = sum_c T[i][c] Y[b,c,h]          P3: C[b,c,h] = sum_r T[r][c] Y[b,r,h]
// acc(m = h, n = output row): A operand Y planes [k][h] read transposed, B operand the band tile.
// Every element of the band tile is used by exactly one wavefront (the one that owns its output
// row), so the tile stays float32 in LDS, as wm_f32.hip lays it out, and a lane splits the eight
// values of its operand after reading them: the same arithmetic as splitting on the way in, a third
// less LDS, and the split runs in the shadow of the matrix instructions of the step before.  Y rows
// are used by all four wavefronts: they are split once, on the way into LDS.
// ------------------------------------------------------------------------------------------
template <int NT, bool TRANSPOSED>
__global__ __launch_bounds__(kThreads, 2) void f32_split_band_in_kernel(
    const float *__restrict__ A, const float *__restrict__ Y, float *__restrict__ C, int B, int M, int N, int w, int nblk,
    int64_t asb, int64_t ysb, int64_t ysr, int64_t csb, int64_t csr) {
  constexpr int NP = 32 * NT;
  constexpr int ST = TRANSPOSED ? TM + 4 : SKC + 4;  // T tile: [KC][TM] (P3) or [TM][KC] (P2), floats
  constexpr int TROWS = TRANSPOSED ? SKC : TM;
  constexpr int SY = lds_stride_tr(NP);
  constexpr int YPL = SKC * SY;  // elements per Y plane
  __shared__ __attribute__((aligned(16))) float t_lds[2][TROWS * ST];
  __shared__ __attribute__((aligned(16))) uint16_t y_lds[2][3][YPL];
  static_assert(4 * 32 * kStage <= 2 * TROWS * ST, "the four staging areas must fit the band tile buffers");

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int W = 2 * w + 1;
  const int o0 = blk * TM;                 // first output row of the block (i for P2, c for P3)
  const int o1 = min(o0 + TM, M) - 1;      // last one
  const int k_lo = max(o0 - w, 0), k_hi = min(o1 + w, M - 1);  // contraction range (c for P2, r for P3)
  const int nk = (k_hi - k_lo + SKC) / SKC;
  const float *Ab = A + (int64_t)b * asb;
  // blockIdx.y selects which NP columns of Y and C this workgroup works on (one workgroup does all
  // of them unless the launch splits the columns)
  const int h0 = NP * blockIdx.y;
  const float *Yb = Y + (int64_t)b * ysb + h0;
  const int ncg = min(N - h0, NP) >> 2, ychunks = SKC * ncg;
  int y_row[NT], y_col[NT];  // this thread's pieces of a Y chunk; row SKC = none
#pragma unroll
  for (int s = 0; s < NT; ++s) {
    const int q = tid + kThreads * s;
    y_row[s] = q < ychunks ? q / ncg : SKC;
    y_col[s] = q < ychunks ? (q % ncg) * 4 : 0;
  }
  // columns of the Y planes that no piece ever writes (N - h0 < NP) must read as zeros
  if (4 * ncg < NP) {
    for (int e = tid; e < 2 * 3 * YPL / 2; e += kThreads) reinterpret_cast<uint32_t *>(&y_lds[0][0][0])[e] = 0u;
    __syncthreads();
  }

  // Band piece s of this thread: its address in chunk 0 (advanced by `t_step` elements per chunk)
  // and what decides its valid element range [e_lo, e_hi] (0..3) in a chunk.
  const float *t_ptr[4];
  int t_fix[4];  // P2: band row i of the piece; P3: first output column c4 of the piece
  const int64_t t_step = TRANSPOSED ? (int64_t)SKC * (W - 1) : SKC;
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
    const int kb = k_lo + k * SKC;
    return block_whole && kb + SKC - 1 <= k_hi && kb + SKC - 1 - w <= o0 && o1 <= kb + w &&
           (TRANSPOSED || kb >= o1 - w) && (!TRANSPOSED || kb + SKC - 1 - w <= o0);
  };
  auto fetch = [&](int k, f32x4(&tr)[4], f32x4(&yr)[NT]) {  // loads only; chunks past the end read the safe address
    const int kb = k_lo + k * SKC;
    if (interior(k)) {
#pragma unroll
      for (int s = 0; s < 4; ++s) tr[s] = load4(t_ptr[s] + k * t_step);
#pragma unroll
      for (int s = 0; s < NT; ++s)
        yr[s] = *reinterpret_cast<const f32x4 *>(y_row[s] < SKC ? Yb + (int64_t)(kb + y_row[s]) * ysr + y_col[s] : Y);
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
        const bool ok = (y_row[s] < SKC) & (kr <= k_hi);
        yr[s] = *reinterpret_cast<const f32x4 *>(ok ? Yb + (int64_t)kr * ysr + y_col[s] : Y);
      }
    }
  };
  auto stash = [&](int k, f32x4(&tr)[4], f32x4(&yr)[NT]) {  // mask, then to LDS buffer k & 1 (Y rows split)
    const int kb = k_lo + k * SKC, buf = k & 1;
    f32x4 tv[4], yv[NT];
#pragma unroll
    for (int s = 0; s < 4; ++s) tv[s] = pin4(tr[s]);
#pragma unroll
    for (int s = 0; s < NT; ++s) yv[s] = pin4(yr[s]);
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
      if (y_row[s] < SKC) {
        const Planes4 pl = split4(yv[s]);
#pragma unroll
        for (int p = 0; p < 3; ++p) *reinterpret_cast<u32x2 *>(&y_lds[buf][p][y_row[s] * SY + y_col[s]]) = pl.p[p];
      }
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
    // the wave's 32 output rows meet the chunk's 32 contraction indices only where |row - index| <= w:
    // a chunk that lies wholly outside that range for this wave is all zeros in its part of the tile
    const int kb = k_lo + k * SKC, ow = o0 + wave * 32;
    if (kb <= ow + 31 + w && kb + SKC - 1 >= ow - w) {
      // the lane's eight values of the band tile per step of 16: row = its output row, k = 16 ks + 8 half ..
      f32x4 blo[SKC / 16], bhi[SKC / 16];
#pragma unroll
      for (int ks = 0; ks < SKC / 16; ++ks) {
        const int kk = 16 * ks + 8 * half;
        if (!TRANSPOSED) {
          blo[ks] = *reinterpret_cast<const f32x4 *>(tl + (wave * 32 + col) * ST + kk);
          bhi[ks] = *reinterpret_cast<const f32x4 *>(tl + (wave * 32 + col) * ST + kk + 4);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            blo[ks][j] = tl[(kk + j) * ST + wave * 32 + col];
            bhi[ks][j] = tl[(kk + 4 + j) * ST + wave * 32 + col];
          }
        }
      }
#pragma unroll
      for (int ks = 0; ks < SKC / 16; ++ks) {
        const Planes4 pl = split4(blo[ks]), ph = split4(bhi[ks]);
        u32x4 bop[3];
#pragma unroll
        for (int p = 0; p < 3; ++p) bop[p] = u32x4{pl.p[p][0], pl.p[p][1], ph.p[p][0], ph.p[p][1]};
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          u32x4 aop[3];
#pragma unroll
          for (int p = 0; p < 3; ++p) aop[p] = lds_read_transposed(y_lds[buf][p], SY, 16 * ks, 32 * t, lane);
          acc[t] = mma_split(aop, bop, acc[t]);
        }
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
// acc(m = c, n = i): A operand Y planes [c][h] read by rows, B operand X rows, split once, in registers.
// ------------------------------------------------------------------------------------------
template <int NKG>  // 16 NKG - 8 <= N <= 16 NKG
__global__ __launch_bounds__(kThreads, 2) void f32_split_band_out_kernel(const float *__restrict__ X,
                                                                        const float *__restrict__ Y,
                                                                        float *__restrict__ C, int B, int M, int N, int w,
                                                                        int nblk, int64_t xsb, int64_t xsr, int64_t ysb,
                                                                        int64_t ysr, int64_t csb) {
  constexpr int NP = 16 * NKG;
  constexpr int SY = NP + 8;  // plane rows an odd number of 16-byte slots apart: conflict-free 16-byte reads
  constexpr int YPL = SKC * SY;
  constexpr int YS = (SKC * NP / 4 + kThreads - 1) / kThreads;
  __shared__ __attribute__((aligned(16))) uint16_t y_lds[2][3][YPL];
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
  int nk = (c_hi - c_lo + SKC) / SKC;
  {  // blockIdx.y selects this workgroup's share of the chunks (all of them unless the launch splits them)
    const int first = (int)((int64_t)nk * blockIdx.y / gridDim.y), last = (int)((int64_t)nk * (blockIdx.y + 1) / gridDim.y);
    c_lo += first * SKC;
    nk = last - first;
  }
  const float *Yb = Y + (int64_t)b * ysb;
  float *Cb = C + (int64_t)b * csb;
  // columns N .. NP - 1 of the planes are never written by a piece and must read as zeros
  if (N < NP) {
    for (int e = tid; e < 2 * 3 * YPL / 2; e += kThreads) reinterpret_cast<uint32_t *>(&y_lds[0][0][0])[e] = 0u;
    __syncthreads();
  }

  // this lane's row of X, split: xop[g][p] holds plane p of X[i][16 g + 8 half .. + 7]
  const int i = i0 + wave * 32 + col;
  u32x4 xop[NKG][3];
  {
    const float *xr = X + (int64_t)b * xsb + (int64_t)i * xsr;
    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int g = 0; g < NKG; ++g) {
      const int h = 16 * g + 8 * half;
      const f32x4 lo = (i < M && h < N) ? *reinterpret_cast<const f32x4 *>(xr + h) : z;
      const f32x4 hi = (i < M && h + 4 < N) ? *reinterpret_cast<const f32x4 *>(xr + h + 4) : z;
      const Planes4 pl = split4(lo), ph = split4(hi);
#pragma unroll
      for (int p = 0; p < 3; ++p) xop[g][p] = u32x4{pl.p[p][0], pl.p[p][1], ph.p[p][0], ph.p[p][1]};
    }
  }

  const int ncg = N >> 2, pieces = SKC * ncg;
  int y_row[YS], y_col[YS];  // this thread's pieces of a Y chunk; row SKC = none
#pragma unroll
  for (int s = 0; s < YS; ++s) {
    const int q = tid + kThreads * s;
    y_row[s] = q < pieces ? q / ncg : SKC;
    y_col[s] = q < pieces ? (q % ncg) * 4 : 0;
  }
  auto fetch = [&](int k, f32x4(&yr)[YS]) {  // loads only; rows outside the sequence read the safe address
    const int cb = c_lo + k * SKC;
#pragma unroll
    for (int s = 0; s < YS; ++s) {
      const int c = cb + y_row[s];
      const bool ok = (y_row[s] < SKC) & (c >= 0) & (c < M);
      yr[s] = *reinterpret_cast<const f32x4 *>(ok ? Yb + (int64_t)c * ysr + y_col[s] : Y);
    }
  };
  auto stash = [&](int k, f32x4(&yr)[YS]) {
    const int cb = c_lo + k * SKC, buf = k & 1;
    f32x4 yv[YS];
#pragma unroll
    for (int s = 0; s < YS; ++s) yv[s] = pin4(yr[s]);
#pragma unroll
    for (int s = 0; s < YS; ++s) {
      const int c = cb + y_row[s];
      const f32x4 z = {0.f, 0.f, 0.f, 0.f};
      if (y_row[s] < SKC) {
        const Planes4 pl = split4(((c >= 0) & (c < M)) ? yv[s] : z);
#pragma unroll
        for (int p = 0; p < 3; ++p) *reinterpret_cast<u32x2 *>(&y_lds[buf][p][y_row[s] * SY + y_col[s]]) = pl.p[p];
      }
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
    const int cb = c_lo + k * SKC;
    fetch(k + 2, mine);
    __builtin_amdgcn_sched_barrier(0);
    // a wave whose 32 rows have no band entry among the chunk's 32 columns has nothing to compute or store
    const int iw = i0 + wave * 32;
    if (cb <= iw + 31 + w && cb + SKC - 1 >= iw - w) {
      f32x16 acc;
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[v] = 0.f;
      // a chunk that lies wholly outside the sequence (a quarter of them when the band covers the
      // sequence) holds zeros only: nothing to multiply, the stores below write the zeros
      if (cb + SKC > 0 && cb < M) {
#pragma unroll
        for (int g = 0; g < NKG; ++g) {
          u32x4 aop[3];
#pragma unroll
          for (int p = 0; p < 3; ++p)
            aop[p] = *reinterpret_cast<const u32x4 *>(&y_lds[buf][p][col * SY + 16 * g + 8 * half]);
          acc = mma_split(aop, xop[g], acc);
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
constexpr int64_t kCUs = 256;
bool split_band_ok(const View &v, int64_t W) { return v.sc == 1 && v.sr == W && ((uintptr_t)v.data % 4) == 0; }

template <bool TRANSPOSED>
hipError_t launch_split_band_in(const Problem &p, const View &a, const View &y, const View &c) {
  const int nblk = (int)((p.M + TM - 1) / TM);
  dim3 grid((unsigned)tiled_grid(p.B, nblk)), block(kThreads);
  const int64_t wgs = p.B * nblk, nb = (p.N + 31) / 32;
#define WM_F32S_IN(NT)                                                                                          \
  hipLaunchKernelGGL((f32_split_band_in_kernel<NT, TRANSPOSED>), grid, block, 0, p.stream, (const float *)a.data, \
                     (const float *)y.data, (float *)c.data, (int)p.B, (int)p.M, (int)p.N, (int)p.w, nblk, a.sb,  \
                     y.sb, y.sr, c.sb, c.sr)
  // When the workgroups do not fill the CUs once or twice, each 32-column block of Y gets workgroups
  // of its own (the rule of wm_f32.hip: the band tile is then fetched once per block, by workgroups
  // that run on the same XCD at the same time).
  if (nb > 1 && wgs < 2 * kCUs && (wgs * nb + kCUs - 1) / kCUs < nb * ((wgs + kCUs - 1) / kCUs)) {
    grid.y = (unsigned)nb;
    WM_F32S_IN(1);
    return hipGetLastError();
  }
  switch (nb) {
    case 1: WM_F32S_IN(1); break;
    case 2: WM_F32S_IN(2); break;
    case 3: WM_F32S_IN(3); break;
    default:  // four blocks: two workgroups of two (three planes of 128 columns would leave one workgroup per CU)
      grid.y = 2;
      WM_F32S_IN(2);
      break;
  }
#undef WM_F32S_IN
  return hipGetLastError();
}

hipError_t launch_split_band_out(const Problem &p, const View &x, const View &y, const View &c) {
  const int nblk = (int)((p.M + TM - 1) / TM);
  dim3 grid((unsigned)tiled_grid(p.B, nblk)), block(kThreads);
  // too few workgroups to fill the chip: each takes a share of its tile's dense columns instead of
  // all of them (nothing is fetched or computed twice: the shares produce disjoint parts of the band)
  const int64_t wgs = p.B * nblk, chunks = (TM + 2 * p.w + SKC - 1) / SKC;
  if (wgs < 2 * kCUs) grid.y = (unsigned)std::max<int64_t>(1, std::min<int64_t>(2 * kCUs / wgs, chunks / 4));
#define WM_F32S_OUT(NKG)                                                                                      \
  case NKG:                                                                                                   \
    hipLaunchKernelGGL((f32_split_band_out_kernel<NKG>), grid, block, 0, p.stream, (const float *)x.data,     \
                       (const float *)y.data, (float *)c.data, (int)p.B, (int)p.M, (int)p.N, (int)p.w, nblk,  \
                       x.sb, x.sr, y.sb, y.sr, c.sb);                                                         \
    break;
  switch ((p.N + 15) / 16) {
    WM_F32S_OUT(1) WM_F32S_OUT(2) WM_F32S_OUT(3) WM_F32S_OUT(4) WM_F32S_OUT(5) WM_F32S_OUT(6) WM_F32S_OUT(7)
    WM_F32S_OUT(8)
    default: return hipErrorInvalidValue;
  }
#undef WM_F32S_OUT
  return hipGetLastError();
}

}  // namespace

// Where the split kernels are used.  Measured against the kernels of wm_f32.hip (microseconds per
// launch, split / plain): B7 M3001 N80 w1500: band-out 88-94 / 130-135, band-in 106-121 / 119-134;
// B96 M4096 N64 w256: 301-351 / 361-414 and 260-287 / 318-349; w = 64: 133-142 / 152-162 and 122-140 /
// 145-165; w = 32: 97-99 / 111-116 and 95-103 / 111-124; B16 M32768 N128 w512: 1065-1150 / 1393-1448 and
// 1215-1230 / 1292-1315; B48 M8192 N80 w16: 94-95 / 119-123 and 102-112 / 127-132; B48 M8192 N128 w20:
// 168-179 / 200-220 and 172-188 / 190-200.  One exception: the band-in product with a single block of
// 32 columns (N <= 32), where the split of the band operand has too few matrix instructions to hide
// behind (B96 M16384 N32: 301-308 / 259-272 at w = 32, 382-394 / 338-356 at w = 64); the transposed
// product at that width still gains (242-257 / 288-291).  Below w = 16 nothing was measured and the
// plain kernels stay.
bool f32_split_supports(int op, int64_t M, int64_t N, int64_t w, int dtype, unsigned flags) {
  if (dtype != WM_DTYPE_F32 || (flags & WM_FLAG_NO_SPLIT_F32)) return false;
  if (N < 8 || N > 128 || N % 8 != 0) return false;
  if (op == 2 && N <= 32) return false;
  return M >= 1 && M <= (1 << 30) && w >= kSplitFromWindow && w <= (1 << 28);
}

bool try_launch_f32_split_p1(const Problem &p, const View &x, const View &y, const View &c, hipError_t *err) {
  if (!f32_split_supports(1, p.M, p.N, p.w, p.dtype, p.flags)) return false;
  if (!fast_layout(x, p.dtype) || !fast_layout(y, p.dtype) || !split_band_ok(c, 2 * p.w + 1)) return false;
  *err = launch_split_band_out(p, x, y, c);
  return true;
}
bool try_launch_f32_split_p2(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  if (!f32_split_supports(2, p.M, p.N, p.w, p.dtype, p.flags)) return false;
  if (!split_band_ok(a, 2 * p.w + 1) || !fast_layout(y, p.dtype) || !fast_layout(c, p.dtype)) return false;
  *err = launch_split_band_in<false>(p, a, y, c);
  return true;
}
bool try_launch_f32_split_p3(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  if (!f32_split_supports(3, p.M, p.N, p.w, p.dtype, p.flags)) return false;
  if (!split_band_ok(a, 2 * p.w + 1) || !fast_layout(y, p.dtype) || !fast_layout(c, p.dtype)) return false;
  *err = launch_split_band_in<true>(p, a, y, c);
  return true;
}

}  // namespace wm
