// Narrow-band kernels (w <= 32) for 16-bit storage on gfx950, and their float32 counterparts on
// v_mfma_f32_16x16x4_f32 for N <= 64 further down.
//
// With a narrow band the whole band of a block of rows is small (256 rows x 17 entries =
// 8.7 KB at w = 8), the op is a pure stream over Q/K (P1) or V/O (P2), and the dense tiles of
// the wide-band kernels would waste most of their work and all of their barriers.  Here a
// wave owns 64 (P1) or 32 (P2, P3) consecutive rows and everything it needs:
//
//   P1  the wave loads its rows of X and the rows [r0-w, r0+64+w) of Y straight from HBM
//       into MFMA operand registers (no LDS, no barrier), forms the 16x16 tiles that touch
//       the band, and scatters the band entries into a flat LDS image of the workgroup's
//       band rows, which then leaves as aligned 16-byte stores.
//       (Staging the operands in LDS with coalesced loads, 32 rows per wave, and replacing the
//       scatter by dense staging tiles were both measured: within 5 % either way, not kept.)
//   P2  the workgroup copies its band rows flat into LDS (aligned 16-byte loads) and the
//       rows [i0-w, i0+rows+w) of Y row-major into LDS; each wave then multiplies its rows:
//       the skewed tile is read back with ds_read_b128 (the flat image keeps 8-column groups
//       16-byte aligned when w % 4 == 0; for other windows the rows are re-pitched on their way
//       into LDS) and masked on bits, Y is read transposed with ds_read_b64_tr_b16.
//
// One workgroup barrier per kernel; results are written exactly once; out-of-sequence band
// entries are stored as +0.0.
#include "wm_mfma_common.hpp"


namespace wm {
namespace {

// Rows that the kernel reads exactly once and nobody else reads (the X rows of a band-out product):
// non-temporal, so that they stream past the rows neighbouring wavefronts share.  A plain read
// stream reaches 5.5-6.3 TB/s on this part, a non-temporal one 6.4-6.8 TB/s.
__device__ __forceinline__ u32x4 load_once(const uint16_t *p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
}

constexpr int SMALL_MAX_W = 32;

// ------------------------------------------------------------------------------------------
// P1 narrow: band[b,i,j] = sum_h X[b,i,h] * Y[b,i+j-w,h]
// ------------------------------------------------------------------------------------------
// 16x16x32 tiles: a 16-row block of the band meets 2 + w / 8 Y tiles of 16 rows, and a wave fetches
// 64 + 2w (+ up to 15) rows of Y.  (The same kernel on 32x32x16 tiles formed and scattered twice
// as many products per band entry and fetched 96 or 128 rows of Y: 98 us against 85 us at
// B96 M16384 N64 w8, 10-20 % slower at every N and w.)  When N is an odd multiple of 16 the upper
// half of the last 32-column step is fed zeros.
template <typename T, int NK, int NYT>  // N = 16 NK; NYT 16-row tiles of Y cover 64 + 2w rows
__global__ __launch_bounds__(kThreads) void small_p1_kernel(const uint16_t *__restrict__ X,
                                                              const uint16_t *__restrict__ Y,
                                                              uint16_t *__restrict__ C, int B, int M, int w, int nblk,
                                                              int64_t xsb, int64_t xsr, int64_t ysb, int64_t ysr,
                                                              int64_t csb) {
  constexpr int ROWS = 256;  // band rows per workgroup, 64 per wave
  constexpr int NK2 = (NK + 1) / 2;  // 32-column steps
  extern __shared__ __attribute__((aligned(16))) uint16_t flat[];  // 8 + ROWS * W (+ slack) elements

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int W = 2 * w + 1;
  const int i0 = blk * ROWS, iw0 = i0 + 64 * wave;
  const int nrows = min(ROWS, M - i0);
  uint16_t *Cb = C + (int64_t)b * csb + (int64_t)i0 * W;
  const int delta = (int)((reinterpret_cast<uintptr_t>(Cb) >> 1) & 7);

  if (iw0 < M) {
    const int l16 = lane & 15, kq = lane >> 4;  // row of a tile; 8-column group of a 32-column step
    auto has_columns = [&](int ks) { return 32 * ks + 8 * kq < 16 * NK; };  // false only in half a last step
    u32x4 xop[4][NK2], yop[NYT][NK2];
    const uint16_t *Xb = X + (int64_t)b * xsb, *Yb = Y + (int64_t)b * ysb;
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const int i = iw0 + 16 * rb + l16;
#pragma unroll
      for (int ks = 0; ks < NK2; ++ks) xop[rb][ks] = load_once(((i < M) & has_columns(ks)) ? Xb + (int64_t)i * xsr + 32 * ks + 8 * kq : X);
    }
#pragma unroll
    for (int t = 0; t < NYT; ++t) {
      const int c = iw0 - w + 16 * t + l16;
#pragma unroll
      for (int ks = 0; ks < NK2; ++ks)
        yop[t][ks] = fetch_row_chunk(Yb + (int64_t)c * ysr + 32 * ks + 8 * kq, Y, (c >= 0) & (c < M) & has_columns(ks));
    }
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const int i = iw0 + 16 * rb + l16;
#pragma unroll
      for (int ks = 0; ks < NK2; ++ks) xop[rb][ks] = mask_row_chunk(xop[rb][ks], (i < M) & has_columns(ks));
    }
#pragma unroll
    for (int t = 0; t < NYT; ++t) {
      const int c = iw0 - w + 16 * t + l16;
#pragma unroll
      for (int ks = 0; ks < NK2; ++ks) yop[t][ks] = mask_row_chunk(yop[t][ks], (c >= 0) & (c < M) & has_columns(ks));
    }

    uint16_t *img = flat + delta + (64 * wave) * W;  // this wave's 64 rows of the flat band image
    // image index of entry (r, j) is delta + r W + j = delta + 2w r + c_rel (mod 4 it is delta when w is
    // even, c_rel being a multiple of 4): then every quad of 4 consecutive entries is 8-byte aligned
    const bool quad_aligned = (w % 2 == 0) && (delta % 4 == 0);
    const bool pair_aligned = delta % 2 == 0;  // 2w r + c_rel is even
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
#pragma unroll
      for (int t = 0; t < NYT; ++t) {
        // tile columns c_rel in [16 t, 16 t + 16), rows r_rel in [16 rb, 16 rb + 16); j = c_rel - r_rel
        if (16 * (t - rb) + 15 < 0 || 16 * (t - rb) - 15 > 2 * w) continue;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < NK2; ++ks) acc = Mma<T>::run16(yop[t][ks], xop[rb][ks], acc);
        // acc[v]: c_rel = 16 t + 4 (lane / 16) + v, r_rel = 16 rb + lane % 16
        const int r_rel = 16 * rb + l16, c_rel = 16 * t + 4 * kq;
        uint16_t *row = img + r_rel * W;
        const int j = c_rel - r_rel;     // band column of the first of 4 consecutive entries
        const int c = iw0 - w + c_rel;   // their sequence positions c .. c + 3
        const uint32_t lo = Mma<T>::pack2(acc[0], acc[1]);
        const uint32_t hi = Mma<T>::pack2(acc[2], acc[3]);
        const bool seq_all = c >= 0 && c + 3 < M;  // entries outside the sequence are +0.0 by definition
        if (quad_aligned && j >= 0 && j + 3 <= 2 * w && seq_all) {
          u32x2 o = {lo, hi};  // whole quad inside band and sequence: one 8-byte LDS write
          *reinterpret_cast<u32x2 *>(row + j) = o;
        } else if (pair_aligned && j >= 0 && j + 3 <= 2 * w && seq_all) {
          *reinterpret_cast<uint32_t *>(row + j) = lo;  // odd w: every other row is 4 bytes off the quad grid
          *reinterpret_cast<uint32_t *>(row + j + 2) = hi;
        } else if (j + 3 >= 0 && j <= 2 * w) {
          if (j >= 0 && j <= 2 * w) row[j] = (c >= 0 && c < M) ? (uint16_t)lo : (uint16_t)0;
          if (j + 1 >= 0 && j + 1 <= 2 * w)
            row[j + 1] = (c + 1 >= 0 && c + 1 < M) ? (uint16_t)(lo >> 16) : (uint16_t)0;
          if (j + 2 >= 0 && j + 2 <= 2 * w) row[j + 2] = (c + 2 >= 0 && c + 2 < M) ? (uint16_t)hi : (uint16_t)0;
          if (j + 3 >= 0 && j + 3 <= 2 * w)
            row[j + 3] = (c + 3 >= 0 && c + 3 < M) ? (uint16_t)(hi >> 16) : (uint16_t)0;
        }
      }
    }
  }
  __syncthreads();

  // flat image -> HBM: chunk q holds image elements [8q, 8q+8), i.e. band elements [8q - delta, ...)
  const int n_el = nrows * W;
  const int chunks = (delta + n_el + 7) >> 3;
  for (int q = tid; q < chunks; q += kThreads) {
    const u32x4 v = *reinterpret_cast<const u32x4 *>(flat + 8 * q);
    const int first = 8 * q - delta;  // band element index of the chunk's element 0
    uint16_t *dst = Cb + first;
    if (first >= 0 && first + 8 <= n_el)
      store_chunk_streaming(dst, v);
    else
      store_chunk_elements(dst, v, -first, n_el - 1 - first);  // only the workgroup's first and last chunk
  }
}

// ------------------------------------------------------------------------------------------
// P1 narrow, float32: the same kernel on v_mfma_f32_16x16x4_f32.  A lane fetches 16 bytes of its row
// (columns 16 ks + 4 (lane / 16) ..+3) and element e of that piece feeds MFMA (ks, e): the contraction
// is split into groups of four columns {16 ks + 4 q + e : q = 0..3}, the same for both operands, so
// no value ever changes lanes.  The band image holds floats; quads are 16 bytes.
// ------------------------------------------------------------------------------------------
template <int NK, int NYT>  // N = 16 NK; NYT 16-row tiles of Y cover 64 + 2w rows
__global__ __launch_bounds__(kThreads) void small_p1_f32_kernel(const float *__restrict__ X,
                                                                const float *__restrict__ Y,
                                                                float *__restrict__ C, int B, int M, int w, int nblk,
                                                                int64_t xsb, int64_t xsr, int64_t ysb, int64_t ysr,
                                                                int64_t csb) {
  constexpr int ROWS = 256;  // band rows per workgroup, 64 per wave
  extern __shared__ __attribute__((aligned(16))) float flat_f32[];  // 4 + ROWS * W (+ slack) elements

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int W = 2 * w + 1;
  const int i0 = blk * ROWS, iw0 = i0 + 64 * wave;
  const int nrows = min(ROWS, M - i0);
  float *Cb = C + (int64_t)b * csb + (int64_t)i0 * W;
  const int delta = (int)((reinterpret_cast<uintptr_t>(Cb) >> 2) & 3);  // elements past a 16-byte boundary
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};

  if (iw0 < M) {
    const int l16 = lane & 15, kq = lane >> 4;
    f32x4 xop[4][NK], yop[NYT][NK];
    const float *Xb = X + (int64_t)b * xsb, *Yb = Y + (int64_t)b * ysb;
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const int i = iw0 + 16 * rb + l16;
#pragma unroll
      for (int ks = 0; ks < NK; ++ks)
        xop[rb][ks] = *reinterpret_cast<const f32x4 *>(i < M ? Xb + (int64_t)i * xsr + 16 * ks + 4 * kq : X);
    }
#pragma unroll
    for (int t = 0; t < NYT; ++t) {
      const int c = iw0 - w + 16 * t + l16;
#pragma unroll
      for (int ks = 0; ks < NK; ++ks)
        yop[t][ks] = *reinterpret_cast<const f32x4 *>((c >= 0) & (c < M) ? Yb + (int64_t)c * ysr + 16 * ks + 4 * kq : Y);
    }
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const int i = iw0 + 16 * rb + l16;
#pragma unroll
      for (int ks = 0; ks < NK; ++ks) xop[rb][ks] = i < M ? xop[rb][ks] : zero;
    }
#pragma unroll
    for (int t = 0; t < NYT; ++t) {
      const int c = iw0 - w + 16 * t + l16;
#pragma unroll
      for (int ks = 0; ks < NK; ++ks) yop[t][ks] = (c >= 0) & (c < M) ? yop[t][ks] : zero;
    }

    float *img = flat_f32 + delta + (64 * wave) * W;
    // image index of entry (r, j) is delta + 2w r + c_rel, c_rel a multiple of 4: 16-byte aligned quads
    const bool quad_aligned = (w % 2 == 0) && delta == 0;
    const bool pair_aligned = delta % 2 == 0;  // 2w r + c_rel is even
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
#pragma unroll
      for (int t = 0; t < NYT; ++t) {
        if (16 * (t - rb) + 15 < 0 || 16 * (t - rb) - 15 > 2 * w) continue;
        f32x4 acc = zero;
#pragma unroll
        for (int ks = 0; ks < NK; ++ks)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(yop[t][ks][e], xop[rb][ks][e], acc, 0, 0, 0);
        // acc[v]: c_rel = 16 t + 4 (lane / 16) + v, r_rel = 16 rb + lane % 16
        const int r_rel = 16 * rb + l16, c_rel = 16 * t + 4 * kq;
        float *row = img + r_rel * W;
        const int j = c_rel - r_rel;
        const int c = iw0 - w + c_rel;
        if (quad_aligned && j >= 0 && j + 3 <= 2 * w && c >= 0 && c + 3 < M) {
          *reinterpret_cast<f32x4 *>(row + j) = acc;
        } else if (pair_aligned && j >= 0 && j + 3 <= 2 * w && c >= 0 && c + 3 < M) {
          *reinterpret_cast<f32x2 *>(row + j) = f32x2{acc[0], acc[1]};
          *reinterpret_cast<f32x2 *>(row + j + 2) = f32x2{acc[2], acc[3]};
        } else if (j + 3 >= 0 && j <= 2 * w) {
#pragma unroll
          for (int v = 0; v < 4; ++v)  // entries outside the sequence are +0.0 by definition
            if (j + v >= 0 && j + v <= 2 * w) row[j + v] = (c + v >= 0 && c + v < M) ? acc[v] : 0.f;
        }
      }
    }
  }
  __syncthreads();

  // flat image -> HBM: chunk q holds image elements [4q, 4q+4), i.e. band elements [4q - delta, ...)
  const int n_el = nrows * W;
  const int chunks = (delta + n_el + 3) >> 2;
  for (int q = tid; q < chunks; q += kThreads) {
    const f32x4 v = *reinterpret_cast<const f32x4 *>(flat_f32 + 4 * q);
    const int first = 4 * q - delta;
    float *dst = Cb + first;
    if (first >= 0 && first + 4 <= n_el) {
      __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(dst));
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (first + e >= 0 && first + e < n_el) dst[e] = v[e];
    }
  }
}

// ------------------------------------------------------------------------------------------
// P2 / P3 narrow, float32:  C[i,h] = sum_j A[i,j] Y[i+j-w,h]   and   C[c,h] = sum_r A[r,c-r+w] Y[r,h]
// on v_mfma_f32_16x16x4_f32, one template.  A workgroup owns 64 output rows, a wave 16 of them.
// LDS holds two images, both written element by element on the way in:
//   * the band rows, re-pitched to an even window wp (row pitch 2wp + 1, entry j at j + wp - w), so
//     that the four consecutive entries a lane needs are one aligned 16-byte read.  For P3 the
//     image is that of the transposed band: entry (r, j) goes to row c = r + j - w, column 2w - j,
//     and everything after the barrier is the same code;
//   * the Y rows the block reaches, transposed (Yt[h][c]), so that four consecutive sequence
//     positions of one column are one 16-byte read as well.
// As in the band-out kernel the contraction is split into groups {16 ks + 4 q + e : q = 0..3}:
// element e of a lane's two 16-byte reads feeds MFMA (ks, e).
// ------------------------------------------------------------------------------------------
template <int NT, bool TRANSPOSED>  // N = 16 NT <= 64
__global__ __launch_bounds__(kThreads) void small_in_f32_kernel(const float *__restrict__ A,
                                                                const float *__restrict__ Y,
                                                                float *__restrict__ C, int B, int M, int w, int nblk,
                                                                int64_t asb, int64_t ysb, int64_t ysr, int64_t csb,
                                                                int64_t csr) {
  constexpr int ROWS = 64, N = 16 * NT;
  constexpr int MAXC = TRANSPOSED ? 8 : 4;  // aligned 4-float chunks of band rows per thread (checked on the host)
  extern __shared__ __attribute__((aligned(16))) float lds_f32[];
  const int W = 2 * w + 1;
  const int wp = (w + 1) & ~1, pad = wp - w, P = 2 * wp + 1;
  const int yc = ROWS + 2 * wp + 16;             // sequence positions cv0 .. cv0 + yc - 1 in the Y image
  const int SYT = (((yc + 3) >> 2) | 1) << 2;    // pitch of a Yt row: SYT / 4 odd keeps 16 rows in 16 bank groups
  float *aimg = lds_f32;
  float *yimg = lds_f32 + ROWS * P + 32;

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int i0 = blk * ROWS;
  const float *Ab = A + (int64_t)b * asb, *Yb = Y + (int64_t)b * ysb;
  const int cv0 = i0 - wp;

  // band rows r_s .. r_e, flat: aligned chunks of four floats, all requested before any is used
  const int r_s = TRANSPOSED ? max(i0 - w, 0) : i0;
  const int r_e = min(TRANSPOSED ? i0 + ROWS - 1 + w : i0 + ROWS - 1, M - 1);
  const float *rows = Ab + (int64_t)r_s * W;
  const int n_el = (r_e - r_s + 1) * W;
  const int dg = (int)((reinterpret_cast<uintptr_t>(rows) >> 2) & 3);
  const int n_chunks = (dg + n_el + 3) >> 2;
  f32x4 band[MAXC];
#pragma unroll
  for (int u = 0; u < MAXC; ++u) {
    const int q = tid + kThreads * u;
    band[u] = *reinterpret_cast<const f32x4 *>(q < n_chunks ? rows - dg + 4 * q : A);
  }
  // Y rows: an instruction takes 16 consecutive positions x 4 consecutive pieces, so that its four
  // scalar LDS writes are free of bank conflicts (positions run along a Yt row)
  const int y_items = ((yc + 15) >> 4) * 16 * (N / 4);  // whole blocks of 16 positions; positions >= yc are skipped
  for (int base = 0; base < y_items; base += 4 * kThreads) {
    f32x4 yv[4];
    int yrow[4], ycol[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int q = base + kThreads * u + tid;
      const int grp = q >> 6, l = q & 63;
      const int cc = 16 * (grp / NT) + (l & 15), piece = 4 * (grp % NT) + (l >> 4);
      const int c = cv0 + cc;
      const bool ok = (q < y_items) & (cc < yc) & (c >= 0) & (c < M);
      yv[u] = *reinterpret_cast<const f32x4 *>(ok ? Yb + (int64_t)c * ysr + 4 * piece : Y);
      yrow[u] = (q < y_items) & (cc < yc) ? 4 * piece : -1;
      ycol[u] = ok ? cc : -1 - cc;  // negative: position outside the sequence, stored as zeros
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (yrow[u] < 0) continue;
      const bool ok = ycol[u] >= 0;
      const int cc = ok ? ycol[u] : -1 - ycol[u];
#pragma unroll
      for (int e = 0; e < 4; ++e) yimg[(yrow[u] + e) * SYT + cc] = ok ? yv[u][e] : 0.f;
    }
  }
  // band chunks -> image
#pragma unroll
  for (int u = 0; u < MAXC; ++u) {
    const int q = tid + kThreads * u;
    if (q >= n_chunks) continue;
    const int first = 4 * q - dg;  // flat index (r W + j, r from r_s) of the chunk's element 0
    const int s0 = max(first, 0);
    int r = s0 / W, j = s0 - r * W;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int id = first + e;
      if (id >= 0 && id < n_el) {
        if (TRANSPOSED) {
          const int c = r_s + r + j - w - i0;  // output row, relative to the block
          if (c >= 0 && c < ROWS) aimg[c * P + 2 * w - j + pad] = band[u][e];
        } else {
          aimg[r * P + j + pad] = band[u][e];
        }
        if (++j == W) j = 0, ++r;
      }
    }
  }
  __syncthreads();

  const int r0 = 16 * wave, r = lane & 15, kq = lane >> 4;
  const int R = r0 + r, i = i0 + R;
  const int nks = (16 + 2 * wp + 15) >> 4;
  f32x4 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  // image column off + e of row R is band column j' = off + e - r (j' - pad in the band), contraction
  // position cv0 + r0 + off + e; element index R P + j' = R 2wp + r0 + off + e
  const float *trow = aimg + R * 2 * wp + r0 + 4 * kq;
  const float *yrow0 = yimg + r * SYT + r0 + 4 * kq;
  for (int ks = 0; ks < nks; ++ks) {
    const int off = 16 * ks + 4 * kq;
    f32x4 bop = *reinterpret_cast<const f32x4 *>(trow + 16 * ks);
    const int pos = cv0 + r0 + off;  // contraction position of element 0
    const int e_lo = max(pad + r - off, -pos);
    const int e_hi = i < M ? min(pad + 2 * w + r - off, M - 1 - pos) : -1;
#pragma unroll
    for (int e = 0; e < 4; ++e) bop[e] = (e >= e_lo) & (e <= e_hi) ? bop[e] : 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const f32x4 aop = *reinterpret_cast<const f32x4 *>(yrow0 + 16 * t * SYT + 16 * ks);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(aop[e], bop[e], acc[t], 0, 0, 0);
    }
  }
  // acc[t][v]: column 16 t + 4 (lane / 16) + v of row i
  if (i < M) {
    float *crow = C + (int64_t)b * csb + (int64_t)i * csr + 4 * kq;
#pragma unroll
    for (int t = 0; t < NT; ++t) __builtin_nontemporal_store(acc[t], reinterpret_cast<f32x4 *>(crow + 16 * t));
  }
}

// ------------------------------------------------------------------------------------------
// Band rows for windows that are not a multiple of 4.  The MFMA reads of the band-in kernels
// need an image whose 8-column groups are 16-byte aligned in every row, i.e. a row pitch of
// 1 (mod 8) elements, which the flat band has only when w % 4 == 0.  For the other windows the
// rows are re-pitched on their way into LDS: entry (r, j) goes to img[r * pitch + j], with the
// pitch of the next window wp that is a multiple of 4 and the row centred in it, so that the
// image is the band of window wp with the outer wp - w entries on either side missing (they are
// masked like every other invalid entry).  The rows are fetched as aligned 16-byte chunks, all
// issued together, and scattered element by element.
// ------------------------------------------------------------------------------------------
template <int MAXC>
__device__ __forceinline__ void fetch_band_rows(u32x4 (&reg)[MAXC], const uint16_t *rows, int n_el,
                                                const uint16_t *safe, int tid) {
  const int dg = (int)((reinterpret_cast<uintptr_t>(rows) >> 1) & 7);
  const int n = n_el > 0 ? (dg + n_el + 7) >> 3 : 0;  // <= MAXC * kThreads (checked on the host)
#pragma unroll
  for (int u = 0; u < MAXC; ++u) {
    const int q = tid + kThreads * u;
    reg[u] = *reinterpret_cast<const u32x4 *>(q < n ? rows - dg + 8 * q : safe);
  }
}
template <int MAXC>
__device__ __forceinline__ void scatter_band_rows(const u32x4 (&reg)[MAXC], const uint16_t *rows, int n_el, int W,
                                                  uint16_t *img, int pitch, int tid) {
  const int dg = (int)((reinterpret_cast<uintptr_t>(rows) >> 1) & 7);
  const int n = n_el > 0 ? (dg + n_el + 7) >> 3 : 0;
  // (Lanes 16 apart meet in one LDS bank here; an element order rotated per 16-lane group avoids
  // that and was measured 15-30 % slower: the address arithmetic, not the bank, is what costs.)
#pragma unroll
  for (int u = 0; u < MAXC; ++u) {
    const int q = tid + kThreads * u;
    if (q >= n) continue;
    const int first = 8 * q - dg;  // flat index (r W + j) of the chunk's element 0
    const int s = max(first, 0);
    int r = s / W, j = s - r * W;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int id = first + e;
      if (id >= 0 && id < n_el) {
        img[r * pitch + j] = (uint16_t)(reg[u][e >> 1] >> (16 * (e & 1)));
        if (++j == W) j = 0, ++r;
      }
    }
  }
}
constexpr int kRepitchChunksP2 = 4, kRepitchChunksP3 = 6;  // per thread: 128 and 192 rows of up to 63 entries

// ------------------------------------------------------------------------------------------
// P2 narrow: C[b,i,h] = sum_j A[b,i,j] * Y[b,i+j-w,h]
// ------------------------------------------------------------------------------------------
template <typename T, int NT, int RW, bool RP>  // N <= 32 NT; RW rows per wave; RP: w % 4 != 0, re-pitched image
__global__ __launch_bounds__(kThreads) void small_p2_kernel(const uint16_t *__restrict__ A,
                                                            const uint16_t *__restrict__ Y,
                                                            uint16_t *__restrict__ C, int B, int M, int N, int w,
                                                            int nblk, int64_t asb, int64_t ysb, int64_t ysr,
                                                            int64_t csb, int64_t csr) {
  constexpr int ROWS = 4 * RW;
  constexpr int SY = lds_stride_tr(32 * NT);
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  const int W = 2 * w + 1;
  const int wp = RP ? (w + 3) & ~3 : w, pad = wp - w;    // the image is laid out for window wp
  const int a_elems = ((ROWS * (2 * wp + 1) + 16 + 7) >> 3) << 3;  // band image, whole 16-byte chunks
  uint16_t *aimg = lds;
  uint16_t *yimg = lds + a_elems;  // rows c = cv0 .. cv0 + ROWS + 2w + 32, stride SY; all initialised

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int i0 = blk * ROWS;
  const int nrows = min(ROWS, M - i0);
  const uint16_t *Ab = A + (int64_t)b * asb + (int64_t)i0 * W;
  const uint16_t *Yb = Y + (int64_t)b * ysb;
  const int delta = RP ? 0 : (int)((reinterpret_cast<uintptr_t>(Ab) >> 1) & 7);

  // band rows, flat: aligned chunks; the first and last chunk may hold neighbours' entries
  // (inside the tensor's pages: aligned 16-byte chunks never straddle a page)
  const int n_el = nrows * W;
  const int chunks = RP ? 0 : (delta + n_el + 7) >> 3;
  u32x4 band[RP ? kRepitchChunksP2 : 1];
  if constexpr (RP) fetch_band_rows(band, Ab, n_el, A, tid);
  // Y rows, row-major, zero outside the sequence
  const int cv0 = i0 - wp - 8;
  const int yrows = ROWS + 2 * wp + 32, ncg = N >> 3;  // every row a 16-column step can reach
  const int ychunks = yrows * ncg;
  // loads go out in batches of 8 per thread before any of them is used
  constexpr int BATCH = 8;
  for (int base = 0; base < chunks + ychunks; base += BATCH * kThreads) {
    u32x4 reg[BATCH];
#pragma unroll
    for (int s = 0; s < BATCH; ++s) {
      const int q = base + s * kThreads + tid;
      const int qy = q - chunks, yr = qy / ncg, hg = qy - yr * ncg, c = cv0 + yr;
      const uint16_t *src = q < chunks ? Ab - delta + 8 * q : Yb + (int64_t)c * ysr + 8 * hg;
      const bool ok = q < chunks || (q < chunks + ychunks && c >= 0 && c < M);
      reg[s] = *reinterpret_cast<const u32x4 *>(ok ? src : A);  // (band and Y share the loop: plain loads)
    }
#pragma unroll
    for (int s = 0; s < BATCH; ++s) {
      const int q = base + s * kThreads + tid;
      const int qy = q - chunks, yr = qy / ncg, hg = qy - yr * ncg, c = cv0 + yr;
      if (q < chunks)
        *reinterpret_cast<u32x4 *>(aimg + 8 * q) = reg[s];
      else if (q < chunks + ychunks)
        *reinterpret_cast<u32x4 *>(yimg + yr * SY + 8 * hg) = mask_row_chunk(reg[s], (c >= 0) & (c < M));
    }
  }
  if constexpr (RP) scatter_band_rows(band, Ab, n_el, W, aimg + pad, 2 * wp + 1, tid);
  __syncthreads();

  const int nks = (32 + 2 * wp + delta + 15) >> 4;  // 16-column steps covering one 32-row tile's band
  u32x2 outp[RW / 32][NT][4];
#pragma unroll
  for (int nt = 0; nt < RW / 32; ++nt) {
    const int r0 = RW * wave + 32 * nt;  // first row of the tile, relative to i0 (multiple of 32)
    const int r = lane & 31, i = i0 + r0 + r;
    f32x16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;
    // dense columns start at c_al = i0 + r0 - wp - delta, which makes every 8-column group of every
    // row an aligned chunk of the image: element index (r0 + r) 2wp + r0 + 16 ks + 8 kg
    const uint16_t *trow = aimg + (r0 + r) * 2 * wp + r0 + 8 * (lane >> 5);
    for (int ks = 0; ks < nks; ++ks) {
      const int off = 16 * ks + 8 * (lane >> 5);    // column offset of this lane's group from c_al
      const int c_g = i0 + r0 - wp - delta + off;    // sequence position of its first element
      u32x4 bop = *reinterpret_cast<const u32x4 *>(trow + 16 * ks);
      // element e is image column off + e - delta - r of row i, band column j = that - pad:
      // valid iff 0 <= j <= 2w and 0 <= c < M
      const int e_lo = max(pad + delta + r - off, -c_g);
      const int e_hi = i < M ? min(pad + 2 * w + delta + r - off, M - 1 - c_g) : -1;
      bop = mask_band_chunk(bop, e_lo, e_hi);
      const int k0 = r0 - delta + 8 + 16 * ks;  // row of yimg holding sequence position c_al + 16 ks
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const u32x4 aop = lds_read_transposed(yimg, SY, k0, 32 * t, lane);
        acc[t] = Mma<T>::run(aop, bop, acc[t]);
      }
    }
    // park the tile's result in registers until every wave is done with the LDS images
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        outp[nt][t][q4][0] = Mma<T>::pack2(acc[t][4 * q4], acc[t][4 * q4 + 1]);
        outp[nt][t][q4][1] = Mma<T>::pack2(acc[t][4 * q4 + 2], acc[t][4 * q4 + 3]);
      }
  }
  // results leave through LDS as row-contiguous 16-byte stores (whole 128-byte lines) instead
  // of 8 bytes per lane scattered over 32 rows; the staging area reuses the images
  __syncthreads();
  constexpr int SO = 32 * NT + 8;
  uint16_t *stage = lds + wave * (RW * SO);
#pragma unroll
  for (int nt = 0; nt < RW / 32; ++nt)
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *reinterpret_cast<u32x2 *>(stage + (32 * nt + (lane & 31)) * SO + 32 * t + 8 * q4 + 4 * (lane >> 5)) =
            outp[nt][t][q4];
  wave_sync_lds();
  const int per_row = N >> 3;  // 16-byte chunks per output row
  for (int q = lane; q < RW * per_row; q += 64) {
    const int r = q / per_row, hg = q - r * per_row;
    const int i = i0 + RW * wave + r;
    if (i < M)  // whole 128-byte lines, written once and not read again here: non-temporal
      store_chunk_streaming(C + (int64_t)b * csb + (int64_t)i * csr + 8 * hg,
                            *reinterpret_cast<const u32x4 *>(stage + r * SO + 8 * hg));
  }
}

// ------------------------------------------------------------------------------------------
// P3 narrow: C[b,c,h] = sum_r A[b,r,c-r+w] * Y[b,r,h]
// ------------------------------------------------------------------------------------------
// Output-stationary like the wide kernel, staged like the narrow P2: a workgroup owns ROWS
// output rows c and copies the band rows r in [c_first - w, c_last + w] flat into LDS, plus
// the Y rows of the same range.  Band entry (r, c) has flat element index r*2w + c + w (+ base),
// so with 2w a multiple of 8 the image is a matrix Mat[r][c] with row stride 2w whose 16-byte
// chunk grid along c is the same in every row: output tiles are laid on that grid (shifted by
// `shift` = (base + w) mod 8 against c = 0, the same for all workgroups of a batch element) and
// ds_read_b64_tr_b16 then delivers, per lane c, the entries of 8 consecutive r: the B operand.
// For w % 4 != 0 (RP) the image is re-pitched to the next multiple of 4, wp, and its grid is free:
// Mat has row stride 2wp, starts on a chunk boundary and the tiles start at c = 0.
template <typename T, int NT, int RW, bool RP>  // N <= 32 NT; RW output rows per wave
__global__ __launch_bounds__(kThreads) void small_p3_kernel(const uint16_t *__restrict__ A,
                                                            const uint16_t *__restrict__ Y,
                                                            uint16_t *__restrict__ C, int B, int M, int N, int w,
                                                            int nblk, int64_t asb, int64_t ysb, int64_t ysr,
                                                            int64_t csb, int64_t csr) {
  constexpr int ROWS = 4 * RW;
  constexpr int SY = lds_stride_tr(32 * NT);
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  const int W = 2 * w + 1;
  const int wp = RP ? (w + 3) & ~3 : w, pad = wp - w;    // the image is laid out for window wp
  const int span = ROWS + 2 * wp;                        // band / Y rows a workgroup can touch
  const int a_elems = ((span * (2 * wp + 1) + 16 + 7) >> 3) << 3;  // band image, whole 16-byte chunks
  uint16_t *aimg = lds;
  // Y rows r_org .. r_org + span + 15 (the last 16-row step may run past the span), stride SY, zero
  // outside the sequence and all initialised: they meet masked zeros of the band inside the MFMA
  uint16_t *yimg = lds + a_elems;

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t base_el = (int64_t)(reinterpret_cast<uintptr_t>(A) >> 1) + (int64_t)b * asb;
  const int shift = RP ? 0 : (int)((base_el + w) & 7);
  const int c_first = blk * ROWS - shift;  // first output row of this workgroup (may be < 0)
  if (c_first >= M) return;
  const int r_org = c_first - wp;          // band row that image row 0 stands for (may be < 0)
  const int r_s = max(r_org, 0), r_e = min(r_org + span - 1, M - 1);  // rows that exist
  const uint16_t *Yb = Y + (int64_t)b * ysb;
  // global element index of image element 0, rounded down to a chunk: g0 = base + r_org * W - delta
  const int64_t g_org = base_el + (int64_t)r_org * W;
  const int delta = RP ? 0 : (int)(g_org & 7);
  const uint16_t *img_src = A + ((g_org - delta) - (int64_t)(reinterpret_cast<uintptr_t>(A) >> 1));

  // flat band rows r_s..r_e: whole aligned chunks (neighbours' entries at both ends are masked later)
  const int q_lo = (delta + (r_s - r_org) * W) >> 3;
  const int q_hi = (delta + (r_e + 1 - r_org) * W + 7) >> 3;  // exclusive
  const int chunks = RP ? 0 : max(q_hi - q_lo, 0);
  const uint16_t *band_rows = A + (int64_t)b * asb + (int64_t)r_s * W;  // RP: rows r_s..r_e, re-pitched
  const int band_el = (r_e - r_s + 1) * W;
  u32x4 band[RP ? kRepitchChunksP3 : 1];
  if constexpr (RP) fetch_band_rows(band, band_rows, band_el, A, tid);
  const int ncg = N >> 3;
  const int ychunks = (span + 16) * ncg;
  constexpr int BATCH = 8;
  for (int base = 0; base < chunks + ychunks; base += BATCH * kThreads) {
    u32x4 reg[BATCH];
#pragma unroll
    for (int s = 0; s < BATCH; ++s) {
      const int q = base + s * kThreads + tid;
      const int qy = q - chunks, yr = qy / ncg, hg = qy - yr * ncg, r = r_org + yr;
      const uint16_t *src = q < chunks ? img_src + 8 * (int64_t)(q_lo + q) : Yb + (int64_t)r * ysr + 8 * hg;
      const bool ok = q < chunks || (q < chunks + ychunks && r >= 0 && r < M);
      reg[s] = *reinterpret_cast<const u32x4 *>(ok ? src : A);
    }
#pragma unroll
    for (int s = 0; s < BATCH; ++s) {
      const int q = base + s * kThreads + tid;
      const int qy = q - chunks, yr = qy / ncg, hg = qy - yr * ncg, r = r_org + yr;
      if (q < chunks)
        *reinterpret_cast<u32x4 *>(aimg + 8 * (q_lo + q)) = reg[s];
      else if (q < chunks + ychunks)
        *reinterpret_cast<u32x4 *>(yimg + yr * SY + 8 * hg) = mask_row_chunk(reg[s], (r >= 0) & (r < M));
    }
  }
  if constexpr (RP)
    scatter_band_rows(band, band_rows, band_el, W, aimg + (r_s - r_org) * (2 * wp + 1) + pad, 2 * wp + 1, tid);
  __syncthreads();

  const int nks = (32 + 2 * wp + 15) >> 4;  // 16-row steps covering the band rows of one 32-row output tile
  u32x2 outp[RW / 32][NT][4];
#pragma unroll
  for (int nt = 0; nt < RW / 32; ++nt) {
    const int t0 = RW * wave + 32 * nt;        // first output row of the tile, relative to c_first
    const int c = c_first + t0 + (lane & 31);  // this lane's output row
    f32x16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;
    // Mat[k][x]: k = r - r_org, x = c - r_org + wp = t0 + (lane & 31) + 2wp; element delta + k*2wp + x
    for (int ks = 0; ks < nks; ++ks) {
      const int k0 = t0 + 16 * ks;                       // image row of band row c_tile - wp + 16 ks
      const int r_g = r_org + k0 + 8 * (lane >> 5);      // band row of this lane's element 0
      u32x4 bop = lds_read_transposed(aimg + delta, 2 * wp, k0, t0 + 2 * wp, lane);
      // element e is band row r_g + e: valid iff |r - c| <= w and 0 <= r < M
      const int e_lo = max(c - w - r_g, -r_g);
      const int e_hi = min(c + w - r_g, M - 1 - r_g);
      bop = mask_band_chunk(bop, e_lo, e_hi);
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const u32x4 aop = lds_read_transposed(yimg, SY, k0, 32 * t, lane);
        acc[t] = Mma<T>::run(aop, bop, acc[t]);
      }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        outp[nt][t][q4][0] = Mma<T>::pack2(acc[t][4 * q4], acc[t][4 * q4 + 1]);
        outp[nt][t][q4][1] = Mma<T>::pack2(acc[t][4 * q4 + 2], acc[t][4 * q4 + 3]);
      }
  }
  // results leave through LDS as row-contiguous 16-byte stores; the staging area reuses the images
  __syncthreads();
  constexpr int SO = 32 * NT + 8;
  uint16_t *stage = lds + wave * (RW * SO);
#pragma unroll
  for (int nt = 0; nt < RW / 32; ++nt)
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *reinterpret_cast<u32x2 *>(stage + (32 * nt + (lane & 31)) * SO + 32 * t + 8 * q4 + 4 * (lane >> 5)) =
            outp[nt][t][q4];
  wave_sync_lds();
  const int per_row = N >> 3;
  for (int q = lane; q < RW * per_row; q += 64) {
    const int r = q / per_row, hg = q - r * per_row;
    const int c = c_first + RW * wave + r;
    if (c >= 0 && c < M)
      store_chunk_streaming(C + (int64_t)b * csb + (int64_t)c * csr + 8 * hg,
                            *reinterpret_cast<const u32x4 *>(stage + r * SO + 8 * hg));
  }
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
bool small_shape_ok(int64_t M, int64_t N, int64_t w, int dtype) {
  if (dtype != WM_DTYPE_BF16 && dtype != WM_DTYPE_F16) return false;
  if (N < 16 || N > 128 || N % 16 != 0) return false;
  return M >= 1 && M <= (1 << 30) && w >= 1 && w <= SMALL_MAX_W;
}
// The band-out kernel reaches further when its operands are small enough for the registers: the
// image of 256 band rows fits 64 KB of LDS up to w = 63.
#ifndef WM_SMALL_P1_MAX_W
#define WM_SMALL_P1_MAX_W 63
#endif
bool small_p1_shape_ok(int64_t M, int64_t N, int64_t w, int dtype) {
  if (dtype != WM_DTYPE_BF16 && dtype != WM_DTYPE_F16) return false;
  if (N < 16 || N > 128 || N % 16 != 0) return false;
  return M >= 1 && M <= (1 << 30) && w >= 1 && w <= (N <= 64 ? WM_SMALL_P1_MAX_W : SMALL_MAX_W);
}

unsigned small_grid(int64_t B, int64_t nblk) { return (unsigned)tiled_grid(B, nblk); }

template <typename T>
hipError_t launch_small_p1(const Problem &p, const View &x, const View &y, const View &c) {
  const int nblk = (int)((p.M + 255) / 256);
  const dim3 grid(small_grid(p.B, nblk)), block(kThreads);
  const size_t lds = (size_t)(256 * (2 * p.w + 1) + 24) * 2;
#define WM_SP1(NK, NYT)                                                                                      \
  hipLaunchKernelGGL((small_p1_kernel<T, NK, NYT>), grid, block, lds, p.stream, (const uint16_t *)x.data,      \
                     (const uint16_t *)y.data, (uint16_t *)c.data, (int)p.B, (int)p.M, (int)p.w, nblk, x.sb,   \
                     x.sr, y.sb, y.sr, c.sb)
#define WM_SP1_N(NYT)                    \
  switch (p.N / 16) {                    \
    case 1: WM_SP1(1, NYT); break;       \
    case 2: WM_SP1(2, NYT); break;       \
    case 3: WM_SP1(3, NYT); break;       \
    case 4: WM_SP1(4, NYT); break;       \
    case 5: WM_SP1(5, NYT); break;       \
    case 6: WM_SP1(6, NYT); break;       \
    case 7: WM_SP1(7, NYT); break;       \
    default: WM_SP1(8, NYT); break;      \
  }
  if (p.w <= 8) {  // 16-row tiles of Y that cover 64 + 2w rows
    WM_SP1_N(5)
  } else if (p.w <= 16) {
    WM_SP1_N(6)
  } else if (p.w <= 24) {
    WM_SP1_N(7)
  } else if (p.w <= 32) {
    WM_SP1_N(8)
  } else {  // N <= 64 only
#define WM_SP1_W(NYT)                    \
  switch (p.N / 16) {                    \
    case 1: WM_SP1(1, NYT); break;       \
    case 2: WM_SP1(2, NYT); break;       \
    case 3: WM_SP1(3, NYT); break;       \
    default: WM_SP1(4, NYT); break;      \
  }
    if (p.w <= 48) {
      WM_SP1_W(10)
    } else {
      WM_SP1_W(12)
    }
#undef WM_SP1_W
  }
#undef WM_SP1_N
#undef WM_SP1
  return hipGetLastError();
}

// float32 band-out kernel: N a multiple of 16 up to 64 (the operands live in registers), w up to
// SMALL_F32_MAX_W (the float image of 256 band rows must fit 64 KB of LDS).
#ifndef WM_SMALL_F32_MAX_W
#define WM_SMALL_F32_MAX_W 31
#endif
hipError_t launch_small_p1_f32(const Problem &p, const View &x, const View &y, const View &c) {
  const int nblk = (int)((p.M + 255) / 256);
  const dim3 grid(small_grid(p.B, nblk)), block(kThreads);
  const size_t lds = (size_t)(256 * (2 * p.w + 1) + 12) * 4;
#define WM_SPF(NK, NYT)                                                                                      \
  hipLaunchKernelGGL((small_p1_f32_kernel<NK, NYT>), grid, block, lds, p.stream, (const float *)x.data,      \
                     (const float *)y.data, (float *)c.data, (int)p.B, (int)p.M, (int)p.w, nblk, x.sb, x.sr, \
                     y.sb, y.sr, c.sb)
#define WM_SPF_N(NYT)                    \
  switch (p.N / 16) {                    \
    case 1: WM_SPF(1, NYT); break;       \
    case 2: WM_SPF(2, NYT); break;       \
    case 3: WM_SPF(3, NYT); break;       \
    default: WM_SPF(4, NYT); break;      \
  }
  if (p.w <= 8) {
    WM_SPF_N(5)
  } else if (p.w <= 16) {
    WM_SPF_N(6)
  } else if (p.w <= 24) {
    WM_SPF_N(7)
  } else {
    WM_SPF_N(8)
  }
#undef WM_SPF_N
#undef WM_SPF
  return hipGetLastError();
}

// float32 band-in kernels: N a multiple of 16 up to 64; w limited by the two LDS images.
// Range (B96 M16384, alternating builds, P2 / P3 in us): against the vector-ALU kernels, which stop at
// w = 14: N = 64, w = 12: 225 / 245 against 280 / 293, w = 8: 197 / 221 against 204 / 217, w = 4: 203 / 229
// against 182 / 183; N = 32, w = 12: 111 / 141 against 98 / 128.  Against the float32 MFMA family: N = 64,
// w = 16: 226 / 247 against 366 / 344, w = 28: 338 / 373 against 441 / 408, w = 31: 413 / 487 against
// 441 / 410; N = 16, w = 16: 88 / 116 against 208 / 229.
#ifndef WM_SMALL_F32_IN_MAX_W
#define WM_SMALL_F32_IN_MAX_W 28
#endif
int64_t small_in_f32_min_w(int64_t N) { return N >= 48 ? 12 : 15; }
size_t small_in_f32_lds(int64_t w, int64_t N) {
  const int64_t wp = (w + 1) & ~(int64_t)1, yc = 64 + 2 * wp + 16, syt = (((yc + 3) >> 2) | 1) << 2;
  return (size_t)(64 * (2 * wp + 1) + 32 + N * syt) * 4;
}
template <bool TRANSPOSED>
hipError_t launch_small_in_f32(const Problem &p, const View &a, const View &y, const View &c) {
  const int nblk = (int)((p.M + 63) / 64);
  const dim3 grid(small_grid(p.B, nblk)), block(kThreads);
  const size_t lds = small_in_f32_lds(p.w, p.N);
#define WM_SIF(NT)                                                                                              \
  hipLaunchKernelGGL((small_in_f32_kernel<NT, TRANSPOSED>), grid, block, lds, p.stream, (const float *)a.data,  \
                     (const float *)y.data, (float *)c.data, (int)p.B, (int)p.M, (int)p.w, nblk, a.sb, y.sb,    \
                     y.sr, c.sb, c.sr)
  switch (p.N / 16) {
    case 1: WM_SIF(1); break;
    case 2: WM_SIF(2); break;
    case 3: WM_SIF(3); break;
    default: WM_SIF(4); break;
  }
#undef WM_SIF
  return hipGetLastError();
}

// Window the LDS images of the band-in kernels are laid out for: w itself or the next multiple of 4.
int64_t image_window(int64_t w) { return (w + 3) & ~(int64_t)3; }

// LDS bytes of the P2 kernel: band image of `rows` rows plus the Y rows they reach.
size_t small_p2_lds(int64_t rows, int64_t w, int64_t NT) {
  const int64_t W = 2 * w + 1;
  const size_t a_elems = (size_t)(((rows * W + 16 + 7) >> 3) << 3);
  return (a_elems + (size_t)(rows + 2 * w + 32) * (32 * NT + 16)) * 2;
}
constexpr size_t kSmallLdsLimit = 65536;  // default limit for dynamic LDS
// Rows per wave.  64 (256-row workgroups) were measured 20-30 % slower than 32 at every narrow
// window: the LDS images of a 256-row workgroup allow two workgroups per CU, and these kernels
// (load everything, barrier, multiply, barrier, store) need more of them in flight to overlap.
int small_p2_rows_per_wave(int64_t, int64_t) { return 32; }

template <typename T>
hipError_t launch_small_p2(const Problem &p, const View &a, const View &y, const View &c) {
  const int NT = (int)((p.N + 31) / 32);
  const int RW = small_p2_rows_per_wave(p.w, NT);
  const int rows = 4 * RW;
  const int nblk = (int)((p.M + rows - 1) / rows);
  const dim3 grid(small_grid(p.B, nblk)), block(kThreads);
  const size_t lds = small_p2_lds(rows, image_window(p.w), NT);
#define WM_SP2(NT_, RW_, RP_)                                                                                  \
  hipLaunchKernelGGL((small_p2_kernel<T, NT_, RW_, RP_>), grid, block, lds, p.stream, (const uint16_t *)a.data, \
                     (const uint16_t *)y.data, (uint16_t *)c.data, (int)p.B, (int)p.M, (int)p.N, (int)p.w, nblk, \
                     a.sb, y.sb, y.sr, c.sb, c.sr)
#define WM_SP2_N(RP_)                   \
  switch (NT) {                         \
    case 1: WM_SP2(1, 32, RP_); break;  \
    case 2: WM_SP2(2, 32, RP_); break;  \
    case 3: WM_SP2(3, 32, RP_); break;  \
    default: WM_SP2(4, 32, RP_); break; \
  }
  if (p.w % 4 == 0) {
    WM_SP2_N(false)
  } else {
    WM_SP2_N(true)
  }
#undef WM_SP2_N
#undef WM_SP2
  return hipGetLastError();
}

// LDS bytes of the P3 kernel: flat image of rows + 2w band rows plus as many Y rows.
size_t small_p3_lds(int64_t rows, int64_t w, int64_t NT) {
  const int64_t W = 2 * w + 1, span = rows + 2 * w;
  const size_t a_elems = (size_t)(((span * W + 16 + 7) >> 3) << 3);
  return (a_elems + (size_t)(span + 16) * (32 * NT + 16)) * 2;
}
int small_p3_rows_per_wave(int64_t, int64_t) { return 32; }

template <typename T>
hipError_t launch_small_p3(const Problem &p, const View &a, const View &y, const View &c) {
  const int NT = (int)((p.N + 31) / 32);
  const int RW = small_p3_rows_per_wave(p.w, NT);
  const int rows = 4 * RW;
  const int nblk = (int)((p.M + 7 + rows - 1) / rows);  // output tiles start up to 7 rows before row 0
  const dim3 grid(small_grid(p.B, nblk)), block(kThreads);
  const size_t lds = small_p3_lds(rows, image_window(p.w), NT);
#define WM_SP3(NT_, RW_, RP_)                                                                                  \
  hipLaunchKernelGGL((small_p3_kernel<T, NT_, RW_, RP_>), grid, block, lds, p.stream, (const uint16_t *)a.data, \
                     (const uint16_t *)y.data, (uint16_t *)c.data, (int)p.B, (int)p.M, (int)p.N, (int)p.w, nblk, \
                     a.sb, y.sb, y.sr, c.sb, c.sr)
#define WM_SP3_N(RP_)                   \
  switch (NT) {                         \
    case 1: WM_SP3(1, 32, RP_); break;  \
    case 2: WM_SP3(2, 32, RP_); break;  \
    case 3: WM_SP3(3, 32, RP_); break;  \
    default: WM_SP3(4, 32, RP_); break; \
  }
  if (p.w % 4 == 0) {
    WM_SP3_N(false)
  } else {
    WM_SP3_N(true)
  }
#undef WM_SP3_N
#undef WM_SP3
  return hipGetLastError();
}

bool band_contiguous(const View &v, int64_t W) { return v.sc == 1 && v.sr == W && ((uintptr_t)v.data % 16) == 0; }

}  // namespace

bool small_f32_p1_supports(int64_t M, int64_t N, int64_t w) {
  return M >= 1 && M <= (1 << 30) && N >= 16 && N <= 64 && N % 16 == 0 && w >= 1 && w <= WM_SMALL_F32_MAX_W;
}

bool small_f32_in_supports(int64_t M, int64_t N, int64_t w) {
  // band chunks per thread: 64 rows (P2) or 64 + 2w rows (P3) of 2w + 1 floats, 4 / 8 chunks of 4 floats x 256 threads
  return M >= 1 && M <= (1 << 30) && N >= 16 && N <= 64 && N % 16 == 0 && w >= small_in_f32_min_w(N) && w <= WM_SMALL_F32_IN_MAX_W &&
         (64 + 2 * w) * (2 * w + 1) + 6 <= 8 * 4 * 256 && small_in_f32_lds(w, N) <= kSmallLdsLimit;
}

// Windows at which the wide-band band-in kernels that load their tiles straight into LDS were
// measured faster than the kernels of this file (16-bit tensors of 100 M elements at M = 16384, both
// directions of each product; e.g. N = 64, w = 24: 110-128 us against 131-150 us; N = 48, w = 28,
// P3: 143-151 against 172-184; N = 128, w = 12: 88-92 against 101-107).
bool wide_band_in_is_faster(int op, int64_t N, int64_t w) {
  switch (N) {
    case 32: return op == 3 && w >= 28;
    case 48: return op == 3 ? w >= 24 : w >= 28;
    case 64: return op == 3 ? w >= 13 : w >= 16;
    case 112: return op == 3 ? w >= 12 : (w >= 16 && w <= 24);
    case 128: return w >= 12 && w <= 16;
    default: return false;
  }
}

bool small_supports(int op, int64_t M, int64_t N, int64_t w, int dtype, unsigned flags) {
  if (dtype == WM_DTYPE_F32) return op == 1 ? small_f32_p1_supports(M, N, w) : small_f32_in_supports(M, N, w);
  if (op == 1) return small_p1_shape_ok(M, N, w, dtype);
  if (!small_shape_ok(M, N, w, dtype)) return false;
  if (!(flags & WM_FLAG_NO_LDS_DIRECT) && w >= 8 && wide_band_in_is_faster(op, N, w)) return false;
  if (op == 2) {
    // the two LDS images must fit the default 64 KB dynamic limit; wider cases go to the wide-band family
    const int64_t NT = (N + 31) / 32;
    return small_p2_lds(4 * small_p2_rows_per_wave(w, NT), image_window(w), NT) <= kSmallLdsLimit;
  }
  if (op == 3) {
    const int64_t NT = (N + 31) / 32;
    // re-pitched images of w = 29..31 (two workgroups per CU) were measured slower than the wide-band
    // kernel: 198-202 us against 156-161 us at B96 M16384 N64
    if (w % 4 != 0 && w > 28) return false;
    return small_p3_lds(4 * small_p3_rows_per_wave(w, NT), image_window(w), NT) <= kSmallLdsLimit;
  }
  return false;
}

bool try_launch_small_p1(const Problem &p, const View &x, const View &y, const View &c, hipError_t *err) {
  if (!small_supports(1, p.M, p.N, p.w, p.dtype, p.flags)) return false;
  if (!fast_layout(x, p.dtype) || !fast_layout(y, p.dtype) || !band_contiguous(c, 2 * p.w + 1)) return false;
  if (p.dtype == WM_DTYPE_F32) {
    *err = launch_small_p1_f32(p, x, y, c);
    return true;
  }
  *err = p.dtype == WM_DTYPE_BF16 ? launch_small_p1<bf16_t>(p, x, y, c) : launch_small_p1<f16_t>(p, x, y, c);
  return true;
}

bool try_launch_small_p2(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  // a window is left to the wide-band kernels only where the ones that were measured faster, those
  // with tiles straight into LDS, take this layout
  const unsigned flags = lds_direct_layout_ok(p, a, y) ? p.flags : p.flags | WM_FLAG_NO_LDS_DIRECT;
  if (!small_supports(2, p.M, p.N, p.w, p.dtype, flags)) return false;
  if (!band_contiguous(a, 2 * p.w + 1) || !fast_layout(y, p.dtype) || !fast_layout(c, p.dtype)) return false;
  if (p.dtype == WM_DTYPE_F32) {
    *err = launch_small_in_f32<false>(p, a, y, c);
    return true;
  }
  *err = p.dtype == WM_DTYPE_BF16 ? launch_small_p2<bf16_t>(p, a, y, c) : launch_small_p2<f16_t>(p, a, y, c);
  return true;
}

bool try_launch_small_p3(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  // a window is left to the wide-band kernels only where the ones that were measured faster, those
  // with tiles straight into LDS, take this layout
  const unsigned flags = lds_direct_layout_ok(p, a, y) ? p.flags : p.flags | WM_FLAG_NO_LDS_DIRECT;
  if (!small_supports(3, p.M, p.N, p.w, p.dtype, flags)) return false;
  if (!band_contiguous(a, 2 * p.w + 1) || !fast_layout(y, p.dtype) || !fast_layout(c, p.dtype)) return false;
  if (p.dtype == WM_DTYPE_F32) {
    *err = launch_small_in_f32<true>(p, a, y, c);
    return true;
  }
  *err = p.dtype == WM_DTYPE_BF16 ? launch_small_p3<bf16_t>(p, a, y, c) : launch_small_p3<f16_t>(p, a, y, c);
  return true;
}

}  // namespace wm
