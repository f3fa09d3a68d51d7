// MFMA kernel family for 16-bit storage (bf16 / f16, float32 accumulate) on gfx950.
//
// All three primitives are tiled GEMMs over a "skewed" tile T of the band:
//     T[r][c] = band[r, c - r + w]   (row r of the sequence, dense column c)
// For one block of 128 sequence rows (P1, P2) or 128 output rows (P3) a workgroup
// of four 64-lane waves walks the dense columns (P1, P2) or the band rows (P3) in
// chunks of 64, double-buffering the chunk operands in LDS, and feeds
// v_mfma_f32_32x32x16_{bf16,f16}.  Each wave owns 32 rows of the block.
//
//   P1  S^T(c, r) = Y[c,:] . X[r,:]      A-operand Y chunk (LDS, k = h contiguous)
//                                         B-operand X rows (registers, loaded once)
//       the 32 x 64 result is staged per wave in LDS and leaves as row-contiguous
//       16-byte stores straight into the band (band entry (r, c-r+w)).
//   P2  O^T(h, r) = sum_c Y[c,h] T[r][c]  A-operand Y chunk via ds_read_b64_tr_b16
//                                         B-operand T tile (LDS, k = c contiguous)
//   P3  C^T(h, c) = sum_r Y[r,h] T[r][c]  both operands via ds_read_b64_tr_b16
//       (output-stationary over c: no atomics).
//
// Band rows have odd length 2w+1, so a band row is never 16-byte aligned as a
// whole; but element (r, c) sits at flat index  b*sb + r*2w + c + w, hence when
// w % 4 == 0 every group of 8 dense columns starting at c8 = -(b*sb + w) (mod 8)
// is one aligned 16-byte chunk in every row.  The ALIGNED instantiation picks
// its column groups that way; the other instantiation issues the same 16-byte
// accesses at 2-byte alignment (legal on gfx950, somewhat slower).
//
// Masking is done on bits, never by multiplying with zero: invalid entries of an
// input band are cleared before they reach LDS, and out-of-sequence entries of an
// output band are stored as +0.0 whatever the operands hold.
#include "wm_mfma_common.hpp"

#include <algorithm>
#include <type_traits>

namespace wm {
namespace {

// ------------------------------------------------------------------------------------------
// P2: C[b,i,h] = sum_c T[i][c] * Y[b,c,h]
// ------------------------------------------------------------------------------------------
template <typename T, int NT, bool ALIGNED, int KCH>
__global__ __launch_bounds__(kThreads, NT <= 2 ? 3 : 2) void mfma_p2_kernel(const uint16_t *__restrict__ A,
                                                              const uint16_t *__restrict__ Y,
                                                              uint16_t *__restrict__ C, int B, int M, int N, int w,
                                                              int nblk, int galign, int64_t asb, int64_t ysb,
                                                              int64_t ysr, int64_t csb, int64_t csr) {
  constexpr int KC = KCH;                 // chunk length of this kernel (shadows the family default)
  constexpr int TS = TM * KC / 8 / kThreads;  // band chunks per thread per tile
  constexpr int GPR = KC / 8;              // 8-column groups per tile row
  constexpr int YS = (KC * NT + 63) / 64;  // Y chunks per thread per tile
  constexpr int NP = 32 * NT;
  // T tile rows are not padded (LDS is what limits the workgroups per CU); the 16-byte chunk g of
  // row r lives at chunk position g ^ (r mod GPR), which keeps the b128 operand reads of 8
  // consecutive rows in different banks
  constexpr int ST = KC;
  constexpr int SY = lds_stride_tr(NP);
  __shared__ __attribute__((aligned(16))) uint16_t t_lds[2][TM * ST];
  __shared__ __attribute__((aligned(16))) uint16_t y_lds[2][KC * SY];  // columns NP.. of a row are padding

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int W = 2 * w + 1;
  const int i0 = blk * TM;
  const int rows = min(TM, M - i0);
  const int c_lo = max(i0 - w, 0), c_hi = min(i0 + rows - 1 + w, M - 1);
  const uint16_t *Ab = A + (int64_t)b * asb;
  const uint16_t *Yb = Y + (int64_t)b * ysb;
  const int c_start = ALIGNED ? c_lo - (int)(((int64_t)c_lo + (int64_t)b * asb + w) & (galign - 1)) : c_lo;
  const int nk = (c_hi - c_start + KC) / KC;

  // per-thread chunk coordinates (loop invariant)
  int t_lo[TS], t_hi[TS];        // valid dense-column range of the chunk's row
  const uint16_t *t_ptr[TS];    // address of dense column 0 of the row (may be virtual)
#pragma unroll
  for (int s = 0; s < TS; ++s) {
    const int q = tid + kThreads * s, r = q / GPR;
    const int i = i0 + r;
    t_lo[s] = max(i - w, 0);
    t_hi[s] = i < M ? min(i + w, M - 1) : -1;
    t_ptr[s] = Ab + (int64_t)i * W + (w - i);
  }
  const int ychunks = KC * (N >> 3), ncg = N >> 3;
  int y_r[YS], y_h[YS], y_off[YS];
#pragma unroll
  for (int s = 0; s < YS; ++s) {
    const int q = tid + kThreads * s;
    y_r[s] = q < ychunks ? q / ncg : KC;  // KC = no row: loads nothing real ...
    y_h[s] = q < ychunks ? (q % ncg) * 8 : 0;
    y_off[s] = q < ychunks ? y_r[s] * SY + y_h[s] : NP;  // ... and writes into the padding of row 0
  }

  // Register-staged prefetch PF chunks deep: chunk k+PF is requested before chunk k is
  // multiplied, so PF chunks of band and Y rows are in flight per workgroup at any time.
  u32x4 t_reg[PF][TS], y_reg[PF][YS];
  auto fetch = [&](int k, u32x4(&tr)[TS], u32x4(&yr)[YS]) {  // loads only
    const int cb = c_start + k * KC;
#pragma unroll
    for (int s = 0; s < TS; ++s) {
      const int c8 = cb + 8 * ((tid + kThreads * s) & (GPR - 1));
      tr[s] = fetch_band_chunk<ALIGNED>(t_ptr[s] + c8, A, t_lo[s] - c8, t_hi[s] - c8);
    }
#pragma unroll
    for (int s = 0; s < YS; ++s) {
      const int c = cb + y_r[s];
      yr[s] = fetch_row_chunk(Yb + (int64_t)c * ysr + y_h[s], Y, (y_r[s] < KC) & (c >= 0) & (c <= c_hi));
    }
  };
  // A chunk is interior when every element of its T tile and every Y row is valid; its masks
  // are skipped (most chunks of a wide band).
  const int in_lo = rows == TM ? max(i0 + TM - 1 - w, 0) : 0x7fffffff, in_hi = min(i0 + w, c_hi);
  auto stash = [&](int k, const u32x4(&tr)[TS], const u32x4(&yr)[YS]) {  // mask, then to LDS buffer k & 1
    const int cb = c_start + k * KC, buf = k & 1;
    u32x4 tv[TS], yv[YS];
#pragma unroll
    for (int s = 0; s < TS; ++s) tv[s] = pin(tr[s]);
#pragma unroll
    for (int s = 0; s < YS; ++s) yv[s] = pin(yr[s]);
    if (!(cb >= in_lo && cb + KC - 1 <= in_hi)) {
#pragma unroll
      for (int s = 0; s < TS; ++s) {
        const int c8 = cb + 8 * ((tid + kThreads * s) & (GPR - 1));
        const int e_lo = t_lo[s] - c8, e_hi = t_hi[s] - c8;
        // the 64 chunks of one wave instruction are 8 consecutive rows: in an edge chunk half of
        // these groups are whole (nothing to mask) or empty (one select), wave-uniformly
        const bool whole = (e_lo <= 0) & (e_hi >= 7), any = band_chunk_any(e_lo, e_hi);
        if (__builtin_amdgcn_ballot_w64(!whole) == 0) continue;
        if (__builtin_amdgcn_ballot_w64(any & !whole) == 0) {
          tv[s] = mask_row_chunk(tv[s], any);
        } else {
          tv[s] = mask_band_chunk(tv[s], e_lo, e_hi);
        }
      }
#pragma unroll
      for (int s = 0; s < YS; ++s) {
        const int c = cb + y_r[s];
        yv[s] = mask_row_chunk(yv[s], (c >= 0) & (c <= c_hi));
      }
    }
#pragma unroll
    for (int s = 0; s < TS; ++s) {
      const int q = tid + kThreads * s;
      *reinterpret_cast<u32x4 *>(&t_lds[buf][(q / GPR) * ST + (((q ^ (q / GPR)) & (GPR - 1)) << 3)]) = tv[s];
    }
#pragma unroll
    for (int s = 0; s < YS; ++s) *reinterpret_cast<u32x4 *>(&y_lds[buf][y_off[s]]) = yv[s];
  };

  f32x16 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[nt][v] = 0.f;

#pragma unroll
  for (int s = 0; s < PF; ++s) fetch(s, t_reg[s], y_reg[s]);
  __builtin_amdgcn_sched_barrier(0);
  stash(0, t_reg[0], y_reg[0]);
  __syncthreads();
  // One pipeline slot: request chunk k+PF into register set `mine`, multiply chunk k out of
  // LDS, then move chunk k+1 (register set `next`, requested PF-1 slots ago) into LDS.
  // The prefetch is unconditional -- chunks past the end are invalid by their coordinates and
  // read the safe address -- and the slots are chained by explicit loop exits, so that the
  // compiler can count outstanding loads exactly and waits only for the set it stores.
  auto slot = [&](int k, u32x4(&mine_t)[TS], u32x4(&mine_y)[YS], u32x4(&next_t)[TS], u32x4(&next_y)[YS]) {
    const int buf = k & 1;
    fetch(k + PF, mine_t, mine_y);
    __builtin_amdgcn_sched_barrier(0);
    const int trow = wave * 32 + (lane & 31);
    const uint16_t *tl = &t_lds[buf][trow * ST];
#pragma unroll
    for (int ks = 0; ks < KC / 16; ++ks) {
      const u32x4 bop = *reinterpret_cast<const u32x4 *>(tl + (((2 * ks + (lane >> 5)) ^ trow) & (GPR - 1)) * 8);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const u32x4 aop = lds_read_transposed(y_lds[buf], SY, ks * 16, 32 * nt, lane);
        acc[nt] = Mma<T>::run(aop, bop, acc[nt]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    stash(k + 1, next_t, next_y);
    __syncthreads();
  };
  static_assert(PF == 2, "the slot chain below is written out for two register sets");
  // Slots run in pairs inside the loop, an odd last one after it: one loop exit, one back edge,
  // so the state of the memory counters is the same on every way into a slot.
  int k = 0;
  for (; k + 1 < nk; k += 2) {
    slot(k, t_reg[0], y_reg[0], t_reg[1], y_reg[1]);
    slot(k + 1, t_reg[1], y_reg[1], t_reg[0], y_reg[0]);
  }
  if (k < nk) slot(k, t_reg[0], y_reg[0], t_reg[1], y_reg[1]);

  // acc[nt][v]: h = 32 nt + 8 (v / 4) + 4 (lane / 32) + v % 4, row = wave * 32 + lane % 32; every
  // wave is past the last barrier, so the tile buffers are free
  static_assert(4 * RowStage<NT>::ELEMS <= 2 * TM * KC, "the four staging areas must fit the band tile buffers");
  store_wave_rows<T, NT>(&t_lds[0][0] + wave * RowStage<NT>::ELEMS, acc, 1.0f, C + (int64_t)b * csb, csr,
                         i0 + wave * 32, M, N, lane);
}

// ------------------------------------------------------------------------------------------
// P3: C[b,c,h] = sum_r T[r][c] * Y[b,r,h]
// ------------------------------------------------------------------------------------------
template <typename T, int NT, bool ALIGNED>
__global__ __launch_bounds__(kThreads, NT <= 2 ? 3 : 2) void mfma_p3_kernel(const uint16_t *__restrict__ A,
                                                              const uint16_t *__restrict__ Y,
                                                              uint16_t *__restrict__ C, int B, int M, int N, int w,
                                                              int nblk, int galign, int64_t asb, int64_t ysb,
                                                              int64_t ysr, int64_t csb, int64_t csr) {
  constexpr int NP = 32 * NT;
  constexpr int ST = TM;  // T tile [KC rows r][TM cols c], unpadded and swizzled (see lds_read_transposed_swz)
  constexpr int SY = lds_stride_tr(NP);
  __shared__ __attribute__((aligned(16))) uint16_t t_lds[2][KC * ST];
  __shared__ __attribute__((aligned(16))) uint16_t y_lds[2][KC * SY];  // columns NP.. of a row are padding

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int W = 2 * w + 1;
  // block origin: aligned variant shifts it left so that every 8-column group is an aligned chunk
  const int c0 = blk * TM - (ALIGNED ? (int)(((int64_t)b * asb + w) & (galign - 1)) : 0);
  const int c_first = max(c0, 0), c_last = min(c0 + TM, M) - 1;
  if (c_first > c_last) return;
  const int r_lo = max(c_first - w, 0), r_hi = min(c_last + w, M - 1);
  const int nk = (r_hi - r_lo + KC) / KC;
  const uint16_t *Ab = A + (int64_t)b * asb;
  const uint16_t *Yb = Y + (int64_t)b * ysb;

  const int ychunks = KC * (N >> 3), ncg = N >> 3;
  int y_r[NT], y_h[NT], y_off[NT];
#pragma unroll
  for (int s = 0; s < NT; ++s) {
    const int q = tid + kThreads * s;
    y_r[s] = q < ychunks ? q / ncg : KC;  // KC = no row: loads nothing real ...
    y_h[s] = q < ychunks ? (q % ncg) * 8 : 0;
    y_off[s] = q < ychunks ? y_r[s] * SY + y_h[s] : NP;  // ... and writes into the padding of row 0
  }

  u32x4 t_reg[PF][4], y_reg[PF][NT];
  auto fetch = [&](int k, u32x4(&tr)[4], u32x4(&yr)[NT]) {  // loads only
    const int rb = r_lo + k * KC;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int q = tid + kThreads * s;
      const int r = rb + (q >> 4), c8 = c0 + 8 * (q & 15);
      const int lo = max(r - w, 0), hi = r <= r_hi ? min(r + w, M - 1) : -1;  // r > r_hi also covers k >= nk
      tr[s] = fetch_band_chunk<ALIGNED>(Ab + (int64_t)r * W + (w - r) + c8, A, lo - c8, hi - c8);
    }
#pragma unroll
    for (int s = 0; s < NT; ++s) {
      const int r = rb + y_r[s];
      yr[s] = fetch_row_chunk(Yb + (int64_t)r * ysr + y_h[s], Y, (y_r[s] < KC) & (r <= r_hi));
    }
  };
  // Interior chunk: all KC band rows exist and each covers all TM columns of the block.
  const bool block_whole = c0 >= 0 && c0 + TM <= M;
  auto stash = [&](int k, const u32x4(&tr)[4], const u32x4(&yr)[NT]) {  // mask, then to LDS buffer k & 1
    const int rb = r_lo + k * KC, buf = k & 1;
    u32x4 tv[4], yv[NT];
#pragma unroll
    for (int s = 0; s < 4; ++s) tv[s] = pin(tr[s]);
#pragma unroll
    for (int s = 0; s < NT; ++s) yv[s] = pin(yr[s]);
    if (!(block_whole && rb + KC - 1 <= r_hi && rb + KC - 1 - w <= c0 && c0 + TM - 1 <= rb + w)) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int q = tid + kThreads * s;
        const int r = rb + (q >> 4), c8 = c0 + 8 * (q & 15);
        const int lo = max(r - w, 0), hi = r <= r_hi ? min(r + w, M - 1) : -1;
        tv[s] = mask_band_chunk(tv[s], lo - c8, hi - c8);
      }
#pragma unroll
      for (int s = 0; s < NT; ++s) yv[s] = mask_row_chunk(yv[s], rb + y_r[s] <= r_hi);
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int q = tid + kThreads * s;
      *reinterpret_cast<u32x4 *>(&t_lds[buf][(q >> 4) * ST + swz32((q & 15) * 8, q >> 4)]) = tv[s];
    }
#pragma unroll
    for (int s = 0; s < NT; ++s) *reinterpret_cast<u32x4 *>(&y_lds[buf][y_off[s]]) = yv[s];
  };

  f32x16 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[nt][v] = 0.f;

#pragma unroll
  for (int s = 0; s < PF; ++s) fetch(s, t_reg[s], y_reg[s]);
  __builtin_amdgcn_sched_barrier(0);
  stash(0, t_reg[0], y_reg[0]);
  __syncthreads();
  // same slot chain as in the band-in kernel above
  auto slot = [&](int k, u32x4(&mine_t)[4], u32x4(&mine_y)[NT], u32x4(&next_t)[4], u32x4(&next_y)[NT]) {
    const int buf = k & 1;
    fetch(k + PF, mine_t, mine_y);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < KC / 16; ++ks) {
      const u32x4 bop = lds_read_transposed_swz(t_lds[buf], ST, ks * 16, wave * 32, lane);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const u32x4 aop = lds_read_transposed(y_lds[buf], SY, ks * 16, 32 * nt, lane);
        acc[nt] = Mma<T>::run(aop, bop, acc[nt]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    stash(k + 1, next_t, next_y);
    __syncthreads();
  };
  static_assert(PF == 2, "the slot chain below is written out for two register sets");
  // Slots run in pairs inside the loop, an odd last one after it: one loop exit, one back edge,
  // so the state of the memory counters is the same on every way into a slot.
  int k = 0;
  for (; k + 1 < nk; k += 2) {
    slot(k, t_reg[0], y_reg[0], t_reg[1], y_reg[1]);
    slot(k + 1, t_reg[1], y_reg[1], t_reg[0], y_reg[0]);
  }
  if (k < nk) slot(k, t_reg[0], y_reg[0], t_reg[1], y_reg[1]);

  static_assert(4 * RowStage<NT>::ELEMS <= 2 * TM * KC, "the four staging areas must fit the band tile buffers");
  store_wave_rows<T, NT>(&t_lds[0][0] + wave * RowStage<NT>::ELEMS, acc, 1.0f, C + (int64_t)b * csb, csr,
                         c0 + wave * 32, M, N, lane);
}

// ------------------------------------------------------------------------------------------
// P1: band[b,i,c-i+w] = sum_h X[b,i,h] * Y[b,c,h]   (+0.0 where c is outside the sequence)
// ------------------------------------------------------------------------------------------
// RING (16-byte column groups that are not whole lines, w % 4 == 0 but w % 32 != 0): row i's 128-byte
// lines begin at a column offset of its own, so a chunk of 64 columns on a common grid would leave
// every row as two partial lines, completed a chunk apart, which neither plain nor non-temporal
// stores do well (200 and 250 us against 85 us for the whole-line case at B96 M4096 N64, w = 260
// against 256).  Here the staging area of a wavefront keeps the last two chunks (a ring of 128
// columns per row), and after every chunk each row stores the one line of its own grid that has
// just been completed: whole lines for every row, one chunk step late at most, plus one closing
// step for the lines that end after the last chunk.  RING = 2 is the same for windows that are not a
// multiple of 4: the rows' lines then begin at any even column offset, a 16-byte piece of a line is
// no longer one piece of the ring, and the staging area is read in 4-byte units.
// LINES: the column groups are whole lines (galign == 64); a compile-time fact on purpose: a store
// path chosen at run time puts the stores into a branch, after which the compiler no longer knows
// how many memory operations are in flight and turns its next wait into a wait for all of them
// (85 -> 130 us at config 3).
template <typename T, int NK, bool ALIGNED, int RING = 0, bool LINES = false>  // NK = N / 16
__global__ __launch_bounds__(kThreads, RING && NK <= 4 ? 3 : 2) void mfma_p1_kernel(const uint16_t *__restrict__ X,
                                                              const uint16_t *__restrict__ Y,
                                                              uint16_t *__restrict__ C, int B, int M, int w,
                                                              int nblk, int galign, int64_t xsb, int64_t xsr,
                                                              int64_t ysb, int64_t ysr, int64_t csb) {
  constexpr int N = 16 * NK;
  constexpr int SY = N + 8;   // Y chunk rows: 16 (mod 128) bytes apart in banks -> conflict-free b128 reads
  // per-wave staging rows: one chunk, padded; or a ring of two chunks, unpadded, the 16-byte piece p
  // of row r at position p ^ (r % 16)
  constexpr int SS = RING ? 2 * KC : KC + 8;
  static_assert(!RING || ALIGNED, "the ring stores pieces that are 16-byte aligned in memory, with the seam logic");
  constexpr int kMaxShift = RING == 2 ? 62 : 56;  // largest column offset of a row's lines
  constexpr int YS = (KC * N / 8 + kThreads - 1) / kThreads;
  __shared__ __attribute__((aligned(16))) uint16_t y_lds[2][(KC + 1) * SY];  // row KC: sink for idle loader slots
  __shared__ __attribute__((aligned(16))) uint16_t s_lds[4][32 * SS];
  // Seam buffer.  The 16-byte chunk that holds the first band entries of row i also holds the
  // last entries of row i-1 (band rows have odd length).  The head piece is parked here when
  // its tile is produced; when the tail piece of the row above turns up, many column chunks
  // later, the two are merged and leave as one aligned 16-byte store.
  __shared__ __attribute__((aligned(16))) uint16_t seam[TM * 8];

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int W = 2 * w + 1;
  const int i0 = blk * TM;
  const int rows = min(TM, M - i0);
  const int c_lo = i0 - w, c_hi = i0 + rows - 1 + w;  // not clipped: out-of-sequence entries are written as zeros
  int c_start = ALIGNED ? c_lo - (int)(((int64_t)c_lo + (int64_t)b * csb + w) & (galign - 1)) : c_lo;
  int nk = (c_hi - c_start + KC) / KC;
  // A launch with too few tiles for the chip gives every tile to gridDim.y workgroups, each with a
  // contiguous share of the tile's chunks; the shares write disjoint column ranges of the band rows.
  // Without the ring nothing is computed twice.  With it a row's line k spans chunks k - 1 and k, so a
  // share that owns lines [first, last) also computes chunk first - 1, stores nothing after it (the
  // rows' valid ranges below begin at the share's first line) and leaves the closing step, line
  // `last`, to the next share.
  const bool shared_tile = gridDim.y > 1;
  bool first_share = true, last_share = true;
  if (shared_tile) {
    const int total = RING ? nk + 1 : nk;  // lines (the closing step stores line nk) or chunks
    const int first = (int)((int64_t)total * blockIdx.y / gridDim.y), last = (int)((int64_t)total * (blockIdx.y + 1) / gridDim.y);
    first_share = first == 0, last_share = last == total;
    const int k0 = RING && !first_share ? first - 1 : first;
    c_start += k0 * KC;
    nk = (RING && last_share ? last - 1 : last) - k0;
  }
  const uint16_t *Yb = Y + (int64_t)b * ysb;
  uint16_t *Cb = C + (int64_t)b * csb;
  // Head and tail pieces of neighbouring rows meet through the seam buffer when both rows belong
  // to this wave, or to any wave of the workgroup if a workgroup barrier is certain to separate
  // the two tiles (the tail is produced 2w-1 columns after the head: at least two chunks later).
  // (ring: a row's tail line is stored (2w + d' - d) / 64 steps after the head line of the row below,
  // d, d' <= kMaxShift the rows' line offsets: at least one step from 2w - kMaxShift >= 64 on)
  // In a shared tile head and tail fall into different workgroups: both leave element by element.
  const bool seam_in_tile = ALIGNED && !shared_tile;
  const bool seam_across_waves = seam_in_tile && (RING ? 2 * w - kMaxShift >= KC : 2 * w - 1 >= 2 * KC);

  // B-operand: this wave's 32 rows of X, all of N, kept in registers
  u32x4 xop[NK];
  {
    const int i = i0 + wave * 32 + (lane & 31);
    const uint16_t *xr = X + (int64_t)b * xsb + (int64_t)i * xsr + 8 * (lane >> 5);
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) xop[ks] = load_row_chunk(xr + 16 * ks, X, i < M);
  }

  // Everything that does not change from chunk to chunk is worked out once per lane here: the
  // kernel is bound by instruction issue, and per-chunk address and range arithmetic was most of it.
  // Y loader slots: row y_c0 + 64 k of the sequence, 8 columns from y_h; sink slots never valid.
  int y_c0[YS], y_lds_off[YS];
  const uint16_t *y_run[YS];  // address of the slot's chunk in the next chunk to be requested
  const int y_cmax = min(M - 1, c_hi);
#pragma unroll
  for (int s = 0; s < YS; ++s) {
    const int q = tid + kThreads * s;
    const bool real = q < KC * N / 8;
    const int yr = real ? q / (N / 8) : KC, yh = real ? (q % (N / 8)) * 8 : 0;  // row KC of the LDS tile is a sink
    y_c0[s] = real ? c_start + yr : -0x40000000;
    y_lds_off[s] = yr * SY + yh;
    y_run[s] = Yb + (int64_t)(c_start + yr) * ysr + yh;
  }
  const int64_t y_step = (int64_t)KC * ysr;
  u32x4 y_reg[PF][YS];
  auto fetch = [&](int k, u32x4(&yr)[YS]) {  // loads only, called for k = 0, 1, 2, ... in order
#pragma unroll
    for (int s = 0; s < YS; ++s) {
      const unsigned c = (unsigned)(y_c0[s] + k * KC);  // valid iff 0 <= c <= y_cmax
      yr[s] = fetch_row_chunk(y_run[s], Y, c <= (unsigned)y_cmax);
      y_run[s] += y_step;
    }
  };
  auto stash = [&](int k, const u32x4(&yr)[YS]) {
    uint16_t *dst = y_lds[k & 1];
#pragma unroll
    for (int s = 0; s < YS; ++s) {
      const unsigned c = (unsigned)(y_c0[s] + k * KC);
      *reinterpret_cast<u32x4 *>(dst + y_lds_off[s]) = mask_row_chunk(pin(yr[s]), c <= (unsigned)y_cmax);
    }
  };

  uint16_t *stage = s_lds[wave];
  // Store slots: lane -> row r = lane / 8 + 8 s of the wave's 32 rows, column group g = lane % 8.
  const int iw_first = i0 + wave * 32;
  int st_lo[4], st_hi[4];   // chunk-relative valid element range is [st_lo - cb, st_hi - cb]
  uint16_t *st_dst[4];      // address of dense column 8 g of the row (add cb)
  const uint16_t *st_src[4];  // (ring: the row's staging area)
  int st_shift[4], st_piece[4];  // ring: the row's lines begin at columns c_start + st_shift (mod 64); first piece of a line
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int r = (lane >> 3) + 8 * s, g = lane & 7;
    const int i = iw_first + r;
    st_lo[s] = i - w - 8 * g;
    st_hi[s] = i < M ? i + w - 8 * g : -0x40000000;
    st_dst[s] = Cb + (int64_t)i * W + (w - i) + 8 * g;
    st_src[s] = RING ? stage + r * SS : stage + r * SS + 8 * g;
    // element address of (i, c_start) modulo a line: the line that contains it begins that many columns earlier
    st_shift[s] = RING ? (int)((0 - (reinterpret_cast<uintptr_t>(Cb + (int64_t)i * W + (w - i) + c_start) >> 1)) & 63) : 0;
    st_piece[s] = (st_shift[s] >> 3) + g;
    // a later share of a tile owns the row from the line that its second chunk completes
    if (RING && !first_share) st_lo[s] = max(i - w, c_start + st_shift[s]) - 8 * g;
  }
  uint16_t *stage_wr = stage + (lane & 31) * SS + 4 * (lane >> 5);
  const int y_rd_off = (lane & 31) * SY + 8 * (lane >> 5);

  // The stores that follow chunk k (k = nk: the closing step of the ring).  Row-contiguous: 8 lanes
  // cover 64 dense columns of one row, the chunk's own or, with the ring, the row's line that chunk k
  // completed: columns cb + shift - 64 ... cb + shift - 1, which begin in the half of the ring that
  // chunk k - 1 filled.
  auto store_lines = [&](int k) __attribute__((always_inline)) {
    const int cb = c_start + k * KC;
    auto cb_of = [&](int s) { return RING ? cb + st_shift[s] - KC : cb; };
    auto piece_of = [&](int s) {  // the lane's 16 bytes of slot s
      const int r = (lane >> 3) + 8 * s;
      if (RING == 2) {
        u32x4 v;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int e = (KC * ((k + 1) & 1) + st_shift[s] + 8 * (lane & 7) + 2 * j) & (2 * KC - 1);
          v[j] = *reinterpret_cast<const uint32_t *>(st_src[s] + (((e >> 3) ^ (r & 15)) << 3) + (e & 7));
        }
        return v;
      }
      if (RING) return *reinterpret_cast<const u32x4 *>(st_src[s] + ((((st_piece[s] + 8 * ((k + 1) & 1)) & 15) ^ (r & 15)) << 3));
      return *reinterpret_cast<const u32x4 *>(st_src[s]);
    };
    if (cb - (RING ? KC : 0) >= iw_first + 31 - w && cb + (RING ? kMaxShift : KC) - 1 <= iw_first + w && iw_first + 31 < M &&
        (!RING || first_share || k > 0)) {
      // every chunk of the wave's tile lies inside the band: nothing to decide, and each group of 8
      // lanes writes one whole 128-byte line, which is what makes the streaming store pay
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const u32x4 val = piece_of(s);
        if (ALIGNED && (RING || LINES))
          store_chunk_streaming(st_dst[s] + cb_of(s), val);
        else
          store_chunk<ALIGNED>(st_dst[s] + cb_of(s), val);  // (pieces of two lines: plain, see store_chunk_streaming)
      }
      wave_sync_lds();
    } else {
      // pass A: whole chunks go out; head pieces are parked in the seam buffer.
      u32x4 v[4];
      int tail_hi[4];  // >= 0: this slot holds a tail piece with elements 0..tail_hi, handled in pass B
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int rw = wave * 32 + (lane >> 3) + 8 * s, r = rw & 31;
        const int e_lo = st_lo[s] - cb_of(s), e_hi = st_hi[s] - cb_of(s);
        tail_hi[s] = -1;
        if (e_hi >= 0 && e_lo <= 7) {
          v[s] = piece_of(s);
          uint16_t *dst = st_dst[s] + cb_of(s);
          if (e_lo <= 0 && e_hi >= 7) {
            store_chunk<ALIGNED>(dst, v[s]);  // (plain: lines of edge tiles are completed piecewise)
          } else if (e_lo > 0) {  // head piece: elements e_lo..7 (W >= 17, so it reaches the chunk's end)
            if (seam_in_tile && rw > 0 && (r > 0 || seam_across_waves))
              *reinterpret_cast<u32x4 *>(&seam[rw * 8]) = v[s];
            else
              store_chunk_elements(dst, v[s], e_lo, 7);
          } else {
            tail_hi[s] = e_hi;
          }
        }
      }
      wave_sync_lds();
      // pass B: tail pieces pick up the head piece of the row below and leave as whole chunks.
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        if (tail_hi[s] >= 0) {
          const int rw = wave * 32 + (lane >> 3) + 8 * s, r = rw & 31;
          uint16_t *dst = st_dst[s] + cb_of(s);
          if (seam_in_tile && rw + 1 < TM && i0 + rw + 1 < M && (r < 31 || seam_across_waves)) {
            const u32x4 head = *reinterpret_cast<const u32x4 *>(&seam[(rw + 1) * 8]);
            const u32x4 mine_part = keep_range(v[s], 0, tail_hi[s]);
            const u32x4 head_part = keep_range(head, tail_hi[s] + 1, 7);
            u32x4 merged = {mine_part[0] | head_part[0], mine_part[1] | head_part[1], mine_part[2] | head_part[2],
                            mine_part[3] | head_part[3]};
            store_chunk<true>(dst, merged);
          } else {
            store_chunk_elements(dst, v[s], 0, tail_hi[s]);
          }
        }
      }
    }
  };

  // One slot: request Y chunk k+PF, multiply chunk k, stage the 32 x 64 result, store it, then move
  // chunk k+1 into LDS.  The stores are issued before the wait for chunk k+1, which was requested
  // a whole slot earlier, so the wait leaves them (and the newest loads) in flight.
  auto slot = [&](int k, u32x4(&mine)[YS], u32x4(&next)[YS]) {
    const int buf = k & 1;
    const int cb = c_start + k * KC;
    fetch(k + PF, mine);
    __builtin_amdgcn_sched_barrier(0);
    // multiply and stage; the version for chunks with columns outside the sequence forces those
    // columns to +0.0 (by definition, whatever X holds) and is kept out of the common path
    auto multiply_and_stage = [&](auto edge) {
#pragma unroll
      for (int mt = 0; mt < KC / 32; ++mt) {
        f32x16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
        const uint16_t *yl = y_lds[buf] + y_rd_off + 32 * mt * SY;
#pragma unroll
        for (int ks = 0; ks < NK; ++ks)
          acc = Mma<T>::run(*reinterpret_cast<const u32x4 *>(yl + 16 * ks), xop[ks], acc);
        // acc[v]: dense column = 32 mt + 8 (v / 4) + 4 (lane / 32) + v % 4, row = lane % 32
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          uint32_t lo = Mma<T>::pack2(acc[4 * q4], acc[4 * q4 + 1]);
          uint32_t hi = Mma<T>::pack2(acc[4 * q4 + 2], acc[4 * q4 + 3]);
          if (decltype(edge)::value) {
            const int c = cb + 32 * mt + 8 * q4 + 4 * (lane >> 5);
            if (c < 0 || c >= M) lo &= 0xffff0000u;
            if (c + 1 < 0 || c + 1 >= M) lo &= 0x0000ffffu;
            if (c + 2 < 0 || c + 2 >= M) hi &= 0xffff0000u;
            if (c + 3 < 0 || c + 3 >= M) hi &= 0x0000ffffu;
          }
          u32x2 o = {lo, hi};
          if (RING)
            *reinterpret_cast<u32x2 *>(stage_wr + (((8 * buf + 4 * mt + q4) ^ (lane & 15)) << 3)) = o;
          else
            *reinterpret_cast<u32x2 *>(stage_wr + 32 * mt + 8 * q4) = o;
        }
      }
    };
    if (cb < 0 || cb + KC > M)
      multiply_and_stage(std::true_type{});
    else
      multiply_and_stage(std::false_type{});
    wave_sync_lds();
    store_lines(k);
    __builtin_amdgcn_sched_barrier(0);
    stash(k + 1, next);
    __syncthreads();
  };

#pragma unroll
  for (int s = 0; s < PF; ++s) fetch(s, y_reg[s]);
  __builtin_amdgcn_sched_barrier(0);
  stash(0, y_reg[0]);
  __syncthreads();
  static_assert(PF == 2, "the slot chain below is written out for two register sets");
  int k = 0;
  for (; k + 1 < nk; k += 2) {
    slot(k, y_reg[0], y_reg[1]);
    slot(k + 1, y_reg[1], y_reg[0]);
  }
  if (k < nk) slot(k, y_reg[0], y_reg[1]);
  if (RING && last_share) store_lines(nk);  // every wavefront is past the last barrier; lines that end after the last chunk
}

// ------------------------------------------------------------------------------------------
// P1 at N = 128 with the Y chunks loaded straight into LDS
// ------------------------------------------------------------------------------------------
// The kernel above with one change: a Y chunk does not pass through registers on its way to LDS.
// Buffer loads with the lds modifier write it into an unpadded, swizzled tile (wm_mfma_common.hpp),
// one chunk ahead; rows past the end of the sequence read as zeros, rows before its start are
// replaced by row 0 (the columns they would produce are forced to +0.0 anyway).  Without the two
// register sets of the staged prefetch and the padding of the tile, three workgroups fit a CU
// where the kernel above places two, which is what lets the multiplications of one workgroup run
// under the band stores of another.  The kernel counts its own loads: a wavefront waits until its
// part of the next chunk has landed while leaving the stores it has just issued in flight.
template <typename T, int NK, bool ALIGNED>  // NK = N / 16
__global__ __launch_bounds__(kThreads, 3) void mfma_p1_dma_kernel(const uint16_t *__restrict__ X,
                                                              const uint16_t *__restrict__ Y,
                                                              uint16_t *__restrict__ C, int B, int M, int w,
                                                              int nblk, int galign, int64_t xsb, int64_t xsr,
                                                              int64_t ysb, int64_t ysr, int64_t csb) {
  constexpr int N = 16 * NK, PPR = 2 * NK, ROWB = 2 * N;  // 16-byte pieces and bytes per tile row
  constexpr int SS = KC + 8;  // per-wave staging rows
  constexpr int LOADS = PPR / 4;  // loads per wavefront and chunk
  static_assert(NK == 4 || NK == 8, "tile rows of 128 or 256 bytes");
  __shared__ __attribute__((aligned(1024))) uint16_t y_lds[2][KC * N];
  __shared__ __attribute__((aligned(16))) uint16_t s_lds[4][32 * SS];
  // Seam buffer.  The 16-byte chunk that holds the first band entries of row i also holds the
  // last entries of row i-1 (band rows have odd length).  The head piece is parked here when
  // its tile is produced; when the tail piece of the row above turns up, many column chunks
  // later, the two are merged and leave as one aligned 16-byte store.
  __shared__ __attribute__((aligned(16))) uint16_t seam[TM * 8];

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  const int W = 2 * w + 1;
  const int i0 = blk * TM;
  const int rows = min(TM, M - i0);
  const int c_lo = i0 - w, c_hi = i0 + rows - 1 + w;  // not clipped: out-of-sequence entries are written as zeros
  const int c_start = ALIGNED ? c_lo - (int)(((int64_t)c_lo + (int64_t)b * csb + w) & (galign - 1)) : c_lo;
  const int nk = (c_hi - c_start + KC) / KC;
  const uint16_t *Yb = Y + (int64_t)b * ysb;
  uint16_t *Cb = C + (int64_t)b * csb;
  // Head and tail pieces of neighbouring rows meet through the seam buffer when both rows belong
  // to this wave, or to any wave of the workgroup if a workgroup barrier is certain to separate
  // the two tiles (the tail is produced 2w-1 columns after the head: at least two chunks later).
  const bool seam_across_waves = ALIGNED && (2 * w - 1 >= 2 * KC);

  // B-operand: this wave's 32 rows of X, all of N, kept in registers
  u32x4 xop[NK];
  {
    const int i = i0 + wave * 32 + (lane & 31);
    const uint16_t *xr = X + (int64_t)b * xsb + (int64_t)i * xsr + 8 * (lane >> 5);
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) xop[ks] = load_row_chunk(xr + 16 * ks, X, i < M);
  }

  // Y chunk k into tile k & 1: the chunk position is a scalar offset of the loads; only a chunk that
  // starts before the sequence needs per-lane addresses (row 0 stands in for the rows before it)
  const u32x4 y_rsrc = make_rsrc(Yb, (uint32_t)((int64_t)(M - 1) * ysr * 2 + ROWB));
  const uint32_t y_voff = dma_lane_offset<PPR>(wave_s, lane, ysr);
  const uint32_t y_step = (uint32_t)(256 / PPR * ysr * 2), y_row_bytes = (uint32_t)(ysr * 2);
  auto request = [&](int k) {
    const int cb = c_start + k * KC;
    if (cb >= 0) {
      dma_chunk<PPR>(y_rsrc, y_lds[k & 1], wave_s, y_voff, (uint32_t)cb * y_row_bytes, y_step);
    } else {
      const uint32_t base = lds_address(y_lds[k & 1]) + 1024 * wave_s;
#pragma unroll
      for (int j = 0; j < LOADS; ++j) {
        const int slot = 64 * (wave_s + 4 * j) + lane, row = slot / PPR, piece = (slot % PPR) ^ swz<PPR>(row);
        dma_piece(y_rsrc, base + 4096 * j, (uint32_t)max(cb + row, 0) * y_row_bytes + 16 * piece, 0);
      }
    }
  };

  uint16_t *stage = s_lds[wave];
  // Store slots: lane -> row r = lane / 8 + 8 s of the wave's 32 rows, column group g = lane % 8.
  const int iw_first = i0 + wave * 32;
  int st_lo[4], st_hi[4];   // chunk-relative valid element range is [st_lo - cb, st_hi - cb]
  uint16_t *st_dst[4];      // address of dense column 8 g of the row (add cb)
  const uint16_t *st_src[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int r = (lane >> 3) + 8 * s, g = lane & 7;
    const int i = iw_first + r;
    st_lo[s] = i - w - 8 * g;
    st_hi[s] = i < M ? i + w - 8 * g : -0x40000000;
    st_dst[s] = Cb + (int64_t)i * W + (w - i) + 8 * g;
    st_src[s] = stage + r * SS + 8 * g;
  }
  uint16_t *stage_wr = stage + (lane & 31) * SS + 4 * (lane >> 5);
  const uint32_t y_at = (uint32_t)((lane & 31) * ROWB + (((lane >> 5) ^ swz<PPR>(lane & 31)) << 4));  // byte offset, piece of ks = 0

  // One slot: multiply chunk k, stage the 32 x 64 result and store it.  Returns whether the slot
  // issued exactly the four whole-line stores per lane of a chunk inside the band.
  auto slot = [&](int k) {
    const int buf = k & 1;
    const int cb = c_start + k * KC;
    bool four_stores = false;
    // chunks of the workgroup's column range that no row of this wavefront reaches
    if (cb + KC - 1 < iw_first - w || cb > iw_first + 31 + w) return false;
    // multiply and stage; the version for chunks with columns outside the sequence forces those
    // columns to +0.0 (by definition, whatever X holds) and is kept out of the common path
    auto multiply_and_stage = [&](auto edge) {
#pragma unroll
      for (int mt = 0; mt < KC / 32; ++mt) {
        f32x16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
        const char *yl = reinterpret_cast<const char *>(y_lds[buf]) + 32 * mt * ROWB;
#pragma unroll
        for (int ks = 0; ks < NK; ++ks)
          acc = Mma<T>::run(*reinterpret_cast<const u32x4 *>(yl + (y_at ^ (32 * ks))), xop[ks], acc);
        // acc[v]: dense column = 32 mt + 8 (v / 4) + 4 (lane / 32) + v % 4, row = lane % 32
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          uint32_t lo = Mma<T>::pack2(acc[4 * q4], acc[4 * q4 + 1]);
          uint32_t hi = Mma<T>::pack2(acc[4 * q4 + 2], acc[4 * q4 + 3]);
          if (decltype(edge)::value) {
            const int c = cb + 32 * mt + 8 * q4 + 4 * (lane >> 5);
            if (c < 0 || c >= M) lo &= 0xffff0000u;
            if (c + 1 < 0 || c + 1 >= M) lo &= 0x0000ffffu;
            if (c + 2 < 0 || c + 2 >= M) hi &= 0xffff0000u;
            if (c + 3 < 0 || c + 3 >= M) hi &= 0x0000ffffu;
          }
          u32x2 o = {lo, hi};
          *reinterpret_cast<u32x2 *>(stage_wr + 32 * mt + 8 * q4) = o;
        }
      }
    };
    if (cb < 0 || cb + KC > M)
      multiply_and_stage(std::true_type{});
    else
      multiply_and_stage(std::false_type{});
    wave_sync_lds();
    // Row-contiguous stores: 8 lanes cover the 64 dense columns of one row.
    if (cb >= iw_first + 31 - w && cb + KC - 1 <= iw_first + w && iw_first + 31 < M) {
      // every chunk of the wave's tile lies inside the band: nothing to decide, and each group of 8
      // lanes writes one whole 128-byte line, which is what makes the streaming store pay
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const u32x4 val = *reinterpret_cast<const u32x4 *>(st_src[s]);
        if (ALIGNED)  // (this kernel is launched for whole-line column groups only)
          store_chunk_streaming(st_dst[s] + cb, val);
        else
          store_chunk<false>(st_dst[s] + cb, val);
      }
      wave_sync_lds();
      four_stores = true;
    } else {
      // pass A: whole chunks go out; head pieces are parked in the seam buffer.
      u32x4 v[4];
      int tail_hi[4];  // >= 0: this slot holds a tail piece with elements 0..tail_hi, handled in pass B
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int rw = wave * 32 + (lane >> 3) + 8 * s, r = rw & 31;
        const int e_lo = st_lo[s] - cb, e_hi = st_hi[s] - cb;
        tail_hi[s] = -1;
        if (e_hi >= 0 && e_lo <= 7) {
          v[s] = *reinterpret_cast<const u32x4 *>(st_src[s]);
          uint16_t *dst = st_dst[s] + cb;
          if (e_lo <= 0 && e_hi >= 7) {
            store_chunk<ALIGNED>(dst, v[s]);  // (plain: lines of edge tiles are completed piecewise)
          } else if (e_lo > 0) {  // head piece: elements e_lo..7 (W >= 17, so it reaches the chunk's end)
            if (ALIGNED && rw > 0 && (r > 0 || seam_across_waves))
              *reinterpret_cast<u32x4 *>(&seam[rw * 8]) = v[s];
            else
              store_chunk_elements(dst, v[s], e_lo, 7);
          } else {
            tail_hi[s] = e_hi;
          }
        }
      }
      wave_sync_lds();
      // pass B: tail pieces pick up the head piece of the row below and leave as whole chunks.
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        if (tail_hi[s] >= 0) {
          const int rw = wave * 32 + (lane >> 3) + 8 * s, r = rw & 31;
          uint16_t *dst = st_dst[s] + cb;
          if (ALIGNED && rw + 1 < TM && i0 + rw + 1 < M && (r < 31 || seam_across_waves)) {
            const u32x4 head = *reinterpret_cast<const u32x4 *>(&seam[(rw + 1) * 8]);
            const u32x4 mine_part = keep_range(v[s], 0, tail_hi[s]);
            const u32x4 head_part = keep_range(head, tail_hi[s] + 1, 7);
            u32x4 merged = {mine_part[0] | head_part[0], mine_part[1] | head_part[1], mine_part[2] | head_part[2],
                            mine_part[3] | head_part[3]};
            store_chunk<true>(dst, merged);
          } else {
            store_chunk_elements(dst, v[s], 0, tail_hi[s]);
          }
        }
      }
    }
    return four_stores;
  };

  request(0);
  bool four_stores = false;  // scalar: every lane of a wavefront takes the same store path
  for (int k = 0; k < nk; ++k) {
    // This wavefront's loads of chunk k are older than the stores of the slot before: when that slot
    // issued exactly four of them they stay in flight, otherwise everything is waited for.  All LDS
    // traffic of the wavefront (staging, seam buffer) is complete as well before the barrier, after
    // which chunk k is in LDS for everyone and nobody reads chunk k - 1 any more.
    if (four_stores)
      wait_vmcnt_lgkm0<4>();
    else
      wait_vmcnt_lgkm0<0>();
    __builtin_amdgcn_s_barrier();
    request(k + 1);  // past the last chunk: zeros into a tile nobody reads
    four_stores = slot(k);
  }
  wait_vmcnt<0>();  // the load past the last chunk must not outlive the workgroup's LDS
}


// ------------------------------------------------------------------------------------------
// P3 with band tile and Y chunk loaded straight into LDS (whole-line column groups, N = 64 or 128)
// ------------------------------------------------------------------------------------------
// Same tiling and arithmetic as mfma_p3_kernel.  Nothing passes through registers on its way to LDS:
// when the column groups are whole 128-byte lines every row of the skewed tile is 256 aligned bytes
// of memory, 2w elements below the row before it, so the tile is a strided block that buffer loads
// with the lds modifier copy as it is (swizzled through which piece a lane fetches).  What the
// register path did to a chunk before storing it to LDS -- clearing the entries that belong to a
// neighbouring band row or lie past the sequence -- is done on the operand after it is read from
// LDS, and only in the chunks of a wavefront's 32 columns that need it; chunks that lie wholly
// outside those columns' band are not multiplied at all.  Rows of Y past the sequence read as zeros
// (buffer range check); DEPTH chunks are in flight per workgroup, counted by the kernel itself.
#ifndef WM_P3_DMA_KC
#define WM_P3_DMA_KC 64
#endif
#ifndef WM_P3_SHALLOW_BELOW
#define WM_P3_SHALLOW_BELOW 136
#endif
constexpr int kShallowChunksBelow = WM_P3_SHALLOW_BELOW;  // window sizes below this take the 32-row chunks
#ifndef WM_P3_DMA_STAGES
#define WM_P3_DMA_STAGES 2
#endif
template <typename T, int NK, int KCH, int STAGES>
__global__ __launch_bounds__(kThreads, (160 * 1024 / (STAGES * KCH * (2 * TM + (NK <= 4 ? 128 : 256))) >= 4
                                           ? 4
                                           : 160 * 1024 / (STAGES * KCH * (2 * TM + (NK <= 4 ? 128 : 256))) >= 3
                                                 ? 3
                                                 : 160 * 1024 / (STAGES * KCH * (2 * TM + (NK <= 4 ? 128 : 256))) >= 2 ? 2 : 1)) void mfma_p3_dma_kernel(
    const uint16_t *__restrict__ A, const uint16_t *__restrict__ Y, uint16_t *__restrict__ C, int B, int M, int n_total, int w,
    int nblk, int galign, int64_t asb, int64_t ysb, int64_t ysr, int64_t csb, int64_t csr) {
  constexpr int N = 16 * NK, NT = (NK + 1) / 2, CH = KCH, DEPTH = STAGES - 1;
  using TT = LdsTile<CH, TM / 8>;            // [CH rows r][TM columns c]
  using YT = LdsTile<CH, NK <= 4 ? 8 : 16>;  // [CH rows r][64 or 128 columns, of which N are fetched]
  constexpr int LOADS = TT::LOADS + YT::LOADS;
  static_assert(NK >= 1 && NK <= 8, "N = 16 ... 128");
  static_assert(CH % 16 == 0 && STAGES >= 2 && DEPTH * LOADS < 64, "vmcnt holds 6 bits");
  __shared__ __attribute__((aligned(1024))) uint16_t t_lds[STAGES][TT::ELEMS];
  __shared__ __attribute__((aligned(1024))) uint16_t y_lds[STAGES][YT::ELEMS];

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int W = 2 * w + 1;
  const int64_t a0 = (int64_t)b * asb;
  const int a_rem = (int)(a0 & 63);
  // element (r, c0) of this batch element starts a 128-byte line (galign 64) or a 16-byte piece (8)
  const int c0 = blk * TM - ((a_rem + w) & (galign - 1));
  const int c_first = max(c0, 0), c_last = min(c0 + TM, M) - 1;
  if (c_first > c_last) return;
  const int r_lo = max(c_first - w, 0), r_hi = min(c_last + w, M - 1);
  const int nk = (r_hi - r_lo + CH) / CH;

  // band: the buffer starts at the 128-byte line that holds the batch element's first entry and ends
  // with the batch element; tile row r, column c0 is at element a_rem + r 2w + c0 + w of it
  const u32x4 t_rsrc = make_rsrc(A + (a0 - a_rem), (uint32_t)(((int64_t)a_rem + (int64_t)M * W) * 2));
  // whole-line column groups: the band is streamed (non-temporal), each line is fetched by one load
  const bool lines = galign == 64;
  const uint32_t t_voff = TT::lane_offset(wave, lane, 2 * w), t_step = TT::step(2 * w);
  const uint32_t t_col0 = (uint32_t)(a_rem + c0 + w) * 2, t_row = (uint32_t)(4 * w);  // bytes
  // blockIdx.y selects which N columns of Y and C this workgroup works on (launches with few tiles
  // give every block of columns workgroups of its own; otherwise there is one block)
  const int h0 = N * (int)blockIdx.y;
  const int n_cols = min(N, n_total - h0);  // (the last block of a width that is no multiple of N is narrower)
  const u32x4 y_rsrc = make_rsrc(Y + (int64_t)b * ysb + h0, (uint32_t)(((int64_t)(M - 1) * ysr + n_cols) * 2));
  // (pieces of the Y tile beyond column N are requested out of range: zeros, no memory traffic)
  const uint32_t y_voff = YT::load_piece(wave, lane) < n_cols / 8 ? YT::lane_offset(wave, lane, ysr) : 0x80000000u;
  const uint32_t y_step = YT::step(ysr), y_row = (uint32_t)(ysr * 2);
  // A piece of the band tile (8 columns from c8 of band row r) holds an entry of the band only if
  // c8 - r lies in [-w - 7, w]; the others are requested beyond the end of the buffer, which costs no
  // memory traffic (a quarter of the tile's pieces at w = 2 TM).  c8 - r falls by CH per chunk.
  int t_skew[TT::LOADS];
#pragma unroll
  for (int j = 0; j < TT::LOADS; ++j)
    t_skew[j] = c0 + 8 * TT::load_piece(wave, lane) - (r_lo + TT::load_row(wave, lane, j)) + w + 7;
  auto request = [&](int k, int stage) {  // chunks past the last one read zeros or rows nobody multiplies
    const uint32_t rb = (uint32_t)(r_lo + k * CH);
    uint32_t voff[TT::LOADS];
#pragma unroll
    for (int j = 0; j < TT::LOADS; ++j)
      voff[j] = (uint32_t)(t_skew[j] - k * CH) <= (uint32_t)(2 * w + 7) ? t_voff : 0x80000000u;
    TT::request_some(t_rsrc, t_lds[stage], wave, voff, t_col0 + rb * t_row, t_step, lines);
    YT::request(y_rsrc, y_lds[stage], wave, y_voff, rb * y_row, y_step);
  };

  f32x16 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[nt][v] = 0.f;

  // this wavefront's columns and, per lane, the band rows that hold an entry of its column
  const int cw0 = c0 + 32 * wave;
  const int c_mine = cw0 + (lane & 31);
  const int row_lo = c_mine - w, row_hi = min(c_mine + w, M - 1);
  const uint32_t t_at = TT::tr_at(lane), y_at = YT::tr_at(lane);
  auto multiply = [&](int rb, int stage, auto edge) {
    u32x4 bop[CH / 16], aop[CH / 16][NT];
#pragma unroll
    for (int ks = 0; ks < CH / 16; ++ks) {
      bop[ks] = TT::cols(t_lds[stage], t_at, 16 * ks, wave);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) aop[ks][nt] = YT::cols(y_lds[stage], y_at, 16 * ks, nt);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < CH / 16; ++ks) {
      if (decltype(edge)::value) bop[ks] = keep_rows_tr(bop[ks], rb + 16 * ks + 4 * (lane >> 5), row_lo, row_hi);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[nt] = Mma<T>::run(aop[ks][nt], bop[ks], acc[nt]);
    }
  };

#pragma unroll
  for (int s = 0; s < DEPTH; ++s) request(s, s);
  int stage = 0, ahead = DEPTH % STAGES;  // stage of chunk k, stage of chunk k + DEPTH
  for (int k = 0; k < nk; ++k) {
    // this wavefront's part of chunk k has landed; after the barrier all of it has, and nobody reads
    // chunk k - 1 any more, whose stage the next request overwrites
    wait_vmcnt<(DEPTH - 1) * LOADS>();
    __builtin_amdgcn_s_barrier();
    request(k + DEPTH, ahead);
    const int rb = r_lo + k * CH;
    if (rb - w <= cw0 + 31 && cw0 <= rb + CH - 1 + w) {  // else: no row of the chunk reaches these columns
      if (rb + CH - 1 - w <= cw0 && cw0 + 31 <= rb + w && rb + CH - 1 <= M - 1)
        multiply(rb, stage, std::false_type{});
      else
        multiply(rb, stage, std::true_type{});
    }
    stage = stage + 1 == STAGES ? 0 : stage + 1;
    ahead = ahead + 1 == STAGES ? 0 : ahead + 1;
  }
  // the loads past the last chunk must have landed before the tiles are reused for the result rows
  wait_vmcnt<0>();
  __syncthreads();
  static_assert(4 * RowStage<NT>::ELEMS <= STAGES * TT::ELEMS, "the four staging areas must fit the band tile buffers");
  store_wave_rows<T, NT>(&t_lds[0][0] + wave * RowStage<NT>::ELEMS, acc, 1.0f, C + (int64_t)b * csb + h0, csr, cw0, M,
                         n_cols, lane);
}

// ------------------------------------------------------------------------------------------
// P2 with band tile and Y chunk loaded straight into LDS (aligned column groups, N = 64 or 128)
// ------------------------------------------------------------------------------------------
// mfma_p2_kernel organised like mfma_p3_dma_kernel above: the band tile [128 rows][64 dense columns]
// is a strided block of 128-byte rows in memory, 2w elements apart.  The first chunk of a tile may
// begin before dense column 0: its position goes into the lanes' offsets, so that exactly the
// pieces before the buffer read as zeros.
template <typename T, int NK, int STAGES>
__global__ __launch_bounds__(kThreads, (160 * 1024 / (STAGES * KC * (2 * TM + (NK <= 4 ? 128 : 256))) >= 3
                                           ? 3
                                           : 160 * 1024 / (STAGES * KC * (2 * TM + (NK <= 4 ? 128 : 256))) >= 2 ? 2 : 1)) void mfma_p2_dma_kernel(
    const uint16_t *__restrict__ A, const uint16_t *__restrict__ Y, uint16_t *__restrict__ C, int B, int M, int n_total, int w,
    int nblk, int galign, int64_t asb, int64_t ysb, int64_t ysr, int64_t csb, int64_t csr) {
  constexpr int N = 16 * NK, NT = (NK + 1) / 2, DEPTH = STAGES - 1;
  using TT = LdsTile<TM, KC / 8>;            // [TM rows i][KC dense columns c]
  using YT = LdsTile<KC, NK <= 4 ? 8 : 16>;  // [KC rows c][64 or 128 columns, of which N are fetched]
  constexpr int LOADS = TT::LOADS + YT::LOADS;
  static_assert(NK >= 1 && NK <= 8, "N = 16 ... 128");
  static_assert(KC == 64 && STAGES >= 2 && DEPTH * LOADS < 64, "band tile rows of 128 bytes; vmcnt holds 6 bits");
  __shared__ __attribute__((aligned(1024))) uint16_t t_lds[STAGES][TT::ELEMS];
  __shared__ __attribute__((aligned(1024))) uint16_t y_lds[STAGES][YT::ELEMS];

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int W = 2 * w + 1;
  const int i0 = blk * TM;
  const int rows = min(TM, M - i0);
  const int c_lo = max(i0 - w, 0), c_hi = min(i0 + rows - 1 + w, M - 1);
  const int64_t a0 = (int64_t)b * asb;
  const int a_rem = (int)(a0 & 63);
  const int c_start = c_lo - ((c_lo + a_rem + w) & (galign - 1));
  const int nk = (c_hi - c_start + KC) / KC;

  // band: buffer from the 128-byte line that holds the batch element's first entry to the end of the
  // batch element; tile row i, dense column c is at element a_rem + i 2w + c + w of it
  const u32x4 t_rsrc = make_rsrc(A + (a0 - a_rem), (uint32_t)(((int64_t)a_rem + (int64_t)M * W) * 2));
  const bool lines = galign == 64;  // whole-line column groups: the band is streamed (non-temporal)
  const uint32_t t_voff = TT::lane_offset(wave, lane, 2 * w) + (uint32_t)(a_rem + (int64_t)i0 * 2 * w + w) * 2;
  const uint32_t t_step = TT::step(2 * w);
  // blockIdx.y selects which N columns of Y and C this workgroup works on (launches with few tiles
  // give every block of columns workgroups of its own; otherwise there is one block)
  const int h0 = N * (int)blockIdx.y;
  const int n_cols = min(N, n_total - h0);  // (the last block of a width that is no multiple of N is narrower)
  const u32x4 y_rsrc = make_rsrc(Y + (int64_t)b * ysb + h0, (uint32_t)(((int64_t)(M - 1) * ysr + n_cols) * 2));
  const bool y_piece = YT::load_piece(wave, lane) < n_cols / 8;  // else: beyond the block's columns, requested out of range
  const uint32_t y_voff = YT::lane_offset(wave, lane, ysr), y_step = YT::step(ysr), y_row = (uint32_t)(ysr * 2);
  // pieces of the band tile that hold no entry of the band (8 columns from c8 of row i with c8 - i
  // outside [-w - 7, w]) are requested beyond the end of the buffer: no memory traffic for them
  int t_skew[TT::LOADS];
#pragma unroll
  for (int j = 0; j < TT::LOADS; ++j)
    t_skew[j] = c_start + 8 * TT::load_piece(wave, lane) - (i0 + TT::load_row(wave, lane, j)) + w + 7;
  auto request = [&](int k, int stage) {  // 32-bit wrap-around on purpose: rows before the buffer are out of range
    const int cb = c_start + k * KC;
    uint32_t voff[TT::LOADS];
#pragma unroll
    for (int j = 0; j < TT::LOADS; ++j)
      voff[j] = (uint32_t)(t_skew[j] + k * KC) <= (uint32_t)(2 * w + 7)
                    ? t_voff + (uint32_t)(2 * cb) + t_step * j
                    : 0x80000000u;
    TT::request_some(t_rsrc, t_lds[stage], wave, voff, 0, 0, lines);
    YT::request_at(y_rsrc, y_lds[stage], wave, y_piece ? y_voff + (uint32_t)cb * y_row : 0x80000000u, y_piece ? y_step : 0u);
  };

  f32x16 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[nt][v] = 0.f;

  // this wavefront's rows and, per lane, the dense columns that its row's band holds
  const int iw0 = i0 + 32 * wave;
  const int i_mine = iw0 + (lane & 31);
  const int col_lo = max(i_mine - w, 0), col_hi = i_mine < M ? min(i_mine + w, M - 1) : -1;
  const uint32_t t_at = TT::row_at(lane), y_at = YT::tr_at_seq(lane);
  auto multiply = [&](int cb, int stage, auto edge) {
    u32x4 bop[KC / 16], aop[KC / 16][NT];
#pragma unroll
    for (int ks = 0; ks < KC / 16; ++ks) {
      bop[ks] = TT::rows(t_lds[stage], t_at, wave, ks);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) aop[ks][nt] = YT::cols_seq(y_lds[stage], y_at, 16 * ks, nt);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < KC / 16; ++ks) {
      if (decltype(edge)::value) {
        const int c8 = cb + 16 * ks + 8 * (lane >> 5);
        bop[ks] = mask_band_chunk(bop[ks], col_lo - c8, col_hi - c8);
      }
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[nt] = Mma<T>::run(aop[ks][nt], bop[ks], acc[nt]);
    }
  };

#pragma unroll
  for (int s = 0; s < DEPTH; ++s) request(s, s);
  int stage = 0, ahead = DEPTH % STAGES;
  for (int k = 0; k < nk; ++k) {
    wait_vmcnt<(DEPTH - 1) * LOADS>();
    __builtin_amdgcn_s_barrier();
    request(k + DEPTH, ahead);
    const int cb = c_start + k * KC;
    if (cb <= iw0 + 31 + w && iw0 - w <= cb + KC - 1) {  // else: no column of the chunk lies in these rows' bands
      if (cb >= max(iw0 + 31 - w, 0) && cb + KC - 1 <= min(iw0 + w, M - 1) && iw0 + 31 <= M - 1)
        multiply(cb, stage, std::false_type{});
      else
        multiply(cb, stage, std::true_type{});
    }
    stage = stage + 1 == STAGES ? 0 : stage + 1;
    ahead = ahead + 1 == STAGES ? 0 : ahead + 1;
  }
  wait_vmcnt<0>();
  __syncthreads();
  static_assert(4 * RowStage<NT>::ELEMS <= STAGES * TT::ELEMS, "the four staging areas must fit the band tile buffers");
  store_wave_rows<T, NT>(&t_lds[0][0] + wave * RowStage<NT>::ELEMS, acc, 1.0f, C + (int64_t)b * csb + h0, csr, iw0, M,
                         n_cols, lane);
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
bool shape_ok(int64_t M, int64_t N, int64_t w, int dtype) {
  if (dtype != WM_DTYPE_BF16 && dtype != WM_DTYPE_F16) return false;
  if (N < 16 || N > 128 || N % 16 != 0) return false;
  if (M < 1 || w < 8) return false;  // partial band chunks are read whole, which needs w >= 7
  if (M > (1 << 30) || w > (1 << 28)) return false;
  return true;
}

bool band_ok(const View &v, int64_t W) { return v.sc == 1 && v.sr == W && ((uintptr_t)v.data % 2) == 0; }
bool band_aligned(const View &v, int64_t w, unsigned flags) {
  return !(flags & WM_FLAG_NO_ALIGNED_BAND) && (w % 4 == 0) && ((uintptr_t)v.data % 16) == 0;
}
// Column-group alignment (elements) of the ALIGNED kernels: whole 128-byte lines when the
// skew per row (2w elements) keeps them aligned, 16-byte chunks otherwise.
int band_group(const View &v, int64_t w) { return (w % 32 == 0 && ((uintptr_t)v.data % 128) == 0) ? 64 : 8; }

unsigned grid_size(int64_t B, int64_t nblk) { return (unsigned)tiled_grid(B, nblk); }

// Workgroups per tile for a launch of `tiles` tiles whose chunk loops are `chunks` long: one while
// the tiles fill the chip's 256 CUs, otherwise enough to keep about three per CU resident, each with
// at least four chunks.
constexpr int kCUs = 256;
unsigned tile_shares(int64_t tiles, int64_t chunks) {
  if (tiles >= kCUs || chunks < 8) return 1;
  const int64_t want = (3 * kCUs + tiles - 1) / tiles;
  return (unsigned)std::max<int64_t>(1, std::min<int64_t>({want, chunks / 4, 64}));
}

// Column blocks of the band-in kernels that load their tiles straight into LDS.  A workgroup alone on
// its CU is bound by its own chunk step (operand reads, then the MFMAs of every column block, one
// wavefront per SIMD with nothing to overlap them), not by its bytes, so a launch with few tiles gives
// every two to four 16-column groups of Y workgroups of their own (`blockIdx.y`; the last block may be
// narrower); the band tile is then fetched once per block, from L2 after the first.  Measured under
// graph replay, bf16, band-in / transposed, us, with / without: 32 tiles N128 w256 9.4 / 14.7 and 10.3 /
// 14.4; 128 tiles N128 w1024 31.5 / 38.5; 160 tiles N128 w512 19.5 / 22.7; 168 tiles N80 w1500 38.6 /
// 43.9 and 37.1 / 43.0; 192 tiles N128 w256 13.5 / 15.4; level at 224 tiles N128 w512; at N = 64 level up
// to 192 tiles and 13 % slower at 224 tiles w1024, 40 % slower at 384.  Returns the width of a block in
// units of 16 columns.
int band_in_column_block(int64_t tiles, int64_t N) {
  const int nk = (int)(N / 16);
  if (tiles > (N > 64 ? 200 : kCUs / 2) || nk < 4) return nk;
  const int blocks = 4 * tiles > kCUs ? 2 : 4;
  return std::max(2, (nk + blocks - 1) / blocks);
}

// Shapes the kernels that load their tiles straight into LDS accept (band-in products): 32-bit byte
// offsets inside a batch element of the band and of Y (chunks past the end included), and band rows
// that can be cut into 16-byte pieces at 4-byte aligned addresses.  Returns the column-group
// alignment to launch with (64, 8 or 2 elements), 0 if the shape is not accepted.
template <bool ALIGNED>
int lds_direct_group(const Problem &p, const View &a, const View &y) {
  if (!lds_direct_layout_ok(p, a, y)) return 0;
  return ALIGNED ? band_group(a, p.w) : 2;
}

// Chunk length of P2 (64: the result rows are staged in the band tile buffers, which 32 would make
// too small; 32 and 128 were measured slower before that).
#ifndef WM_P2_KC
#define WM_P2_KC 64
#endif
template <typename T, bool ALIGNED>
hipError_t launch_p2(const Problem &p, const View &a, const View &y, const View &c) {
  const int nblk = (int)((p.M + TM - 1) / TM);
  const int galign = band_group(a, p.w);
  const dim3 grid(grid_size(p.B, nblk)), block(kThreads);
  // Tiles straight into LDS (N = 64 / 128, 16-byte column groups, 32-bit byte offsets inside a batch
  // element of the band and of Y, chunks past the end included).  Measured against the kernel below
  // at B = 96, M = 4096, N = 64: 28 % faster at w = 36, 30 % at w = 100, 6-13 % at w = 256, 19 % at
  // w = 260; 14 % at B = 32, M = 32768, w = 64; 4-7 % at config 4, 10 % at N = 128 and w = 260.  Once
  // the band outgrows the last-level cache the kernel below, with two chunks per workgroup in flight,
  // is 2-4 % faster at N = 64 (B = 384 at w = 256; B = 32, M = 32768 at w = 512): not worth a rule.
  if (const int g = lds_direct_group<ALIGNED>(p, a, y)) {
    const int nkb = band_in_column_block(p.B * nblk, p.N);
    const dim3 grid_c(grid.x, (unsigned)((p.N / 16 + nkb - 1) / nkb));
#define WM_P2_DMA(NK, STAGES)                                                                                  \
  case NK:                                                                                                     \
    hipLaunchKernelGGL((mfma_p2_dma_kernel<T, NK, STAGES>), grid_c, block, 0, p.stream, (const uint16_t *)a.data, \
                       (const uint16_t *)y.data, (uint16_t *)c.data, (int)p.B, (int)p.M, (int)p.N, (int)p.w,   \
                       nblk, g, a.sb, y.sb, y.sr, c.sb, c.sr);                                                 \
    break;
    switch (nkb) {
      WM_P2_DMA(1, 2) WM_P2_DMA(2, 2) WM_P2_DMA(3, 2) WM_P2_DMA(4, 2) WM_P2_DMA(5, 2) WM_P2_DMA(6, 2) WM_P2_DMA(7, 2)
      WM_P2_DMA(8, 2)
    }
#undef WM_P2_DMA
    return hipGetLastError();
  }
#define WM_P2(NT)                                                                                              \
  hipLaunchKernelGGL((mfma_p2_kernel<T, NT, ALIGNED, WM_P2_KC>), grid, block, 0, p.stream, (const uint16_t *)a.data,     \
                     (const uint16_t *)y.data, (uint16_t *)c.data, (int)p.B, (int)p.M, (int)p.N, (int)p.w, nblk, \
                     galign, a.sb, y.sb, y.sr, c.sb, c.sr)
  switch ((p.N + 31) / 32) {
    case 1: WM_P2(1); break;
    case 2: WM_P2(2); break;
    case 3: WM_P2(3); break;
    default: WM_P2(4); break;
  }
#undef WM_P2
  return hipGetLastError();
}

template <typename T, bool ALIGNED>
hipError_t launch_p3(const Problem &p, const View &a, const View &y, const View &c) {
  const int galign = band_group(a, p.w);
  const int nblk = (int)((p.M + (ALIGNED ? galign - 1 : 0) + TM - 1) / TM);
  const dim3 grid(grid_size(p.B, nblk)), block(kThreads);
  // Tiles straight into LDS, as for the band-in product above.  Measured against the kernel below at
  // B = 96, M = 4096, N = 64: 35 % faster at w = 36, 30 % at w = 100, 12-15 % at w = 256 and 260;
  // 23 % at B = 32, M = 32768, w = 64; 9-13 % at config 4; 4 % at B = 384, w = 256; equal at B = 32,
  // M = 32768, w = 512.
  if (const int g = lds_direct_group<ALIGNED>(p, a, y)) {
    const int nblk_g = (int)((p.M + g - 1 + TM - 1) / TM);
    const int nkb = band_in_column_block(p.B * ((p.M + TM - 1) / TM), p.N);
    const dim3 grid_g(grid_size(p.B, nblk_g), (unsigned)((p.N / 16 + nkb - 1) / nkb));
#define WM_P3_DMA(NK, KCH, STAGES)                                                                             \
  case NK:                                                                                                     \
    hipLaunchKernelGGL((mfma_p3_dma_kernel<T, NK, KCH, STAGES>), grid_g, block, 0, p.stream,                   \
                       (const uint16_t *)a.data, (const uint16_t *)y.data, (uint16_t *)c.data, (int)p.B,       \
                       (int)p.M, (int)p.N, (int)p.w, nblk_g, g, a.sb, y.sb, y.sr, c.sb, c.sr);                 \
    break;
    // A band of a few chunks only: chunks of 32 rows, three deep, fit four workgroups on a CU up to
    // N = 64 and overfetch less at the band's edges (B96 M16384 N64, 32- against 64-row chunks: 119
    // against 140 us at w = 33, 130 against 145 at w = 48, 175 against 188 at w = 96, 206 against 216
    // at w = 128, 349 against 329 at w = 200).
    if (p.N <= 64 && p.w < kShallowChunksBelow) {
      switch (nkb) { WM_P3_DMA(1, 32, 3) WM_P3_DMA(2, 32, 3) WM_P3_DMA(3, 32, 3) WM_P3_DMA(4, 32, 3) }
    } else {
      switch (nkb) {
        WM_P3_DMA(1, WM_P3_DMA_KC, WM_P3_DMA_STAGES) WM_P3_DMA(2, WM_P3_DMA_KC, WM_P3_DMA_STAGES)
        WM_P3_DMA(3, WM_P3_DMA_KC, WM_P3_DMA_STAGES) WM_P3_DMA(4, WM_P3_DMA_KC, WM_P3_DMA_STAGES)
        WM_P3_DMA(5, WM_P3_DMA_KC, WM_P3_DMA_STAGES) WM_P3_DMA(6, WM_P3_DMA_KC, WM_P3_DMA_STAGES)
        WM_P3_DMA(7, WM_P3_DMA_KC, WM_P3_DMA_STAGES) WM_P3_DMA(8, WM_P3_DMA_KC, WM_P3_DMA_STAGES)
      }
    }
#undef WM_P3_DMA
    return hipGetLastError();
  }
#define WM_P3(NT)                                                                                              \
  hipLaunchKernelGGL((mfma_p3_kernel<T, NT, ALIGNED>), grid, block, 0, p.stream, (const uint16_t *)a.data,     \
                     (const uint16_t *)y.data, (uint16_t *)c.data, (int)p.B, (int)p.M, (int)p.N, (int)p.w, nblk, \
                     galign, a.sb, y.sb, y.sr, c.sb, c.sr)
  switch ((p.N + 31) / 32) {
    case 1: WM_P3(1); break;
    case 2: WM_P3(2); break;
    case 3: WM_P3(3); break;
    default: WM_P3(4); break;
  }
#undef WM_P3
  return hipGetLastError();
}

template <typename T, bool ALIGNED>
hipError_t launch_p1(const Problem &p, const View &x, const View &y, const View &c) {
  const int nblk = (int)((p.M + TM - 1) / TM);
  const int galign = band_group(c, p.w);
  const dim3 block(kThreads);
  dim3 grid(grid_size(p.B, nblk));
  // 16-byte column groups: every row is stored as two partial lines per chunk.  While the band fits
  // the last-level cache (256 MB) the halves meet there and plain stores do (B96 M4096 N64 w = 100,
  // 158 MB: 62 us, against 67 us with the ring of whole lines); beyond it the ring wins: 91 against
  // 116 us at w = 164 (259 MB), 119 against 200 us at w = 260, 327 against 747 us at w = 1028.
  // Fewer tiles than CUs (a wide band over a short sequence, few batch elements): a workgroup alone
  // on its CU is bound by the latency of its chunk loop, about 1.3 us per chunk whatever runs beside
  // it, so the tiles are shared out until about three workgroups per CU are resident, each with at
  // least four chunks (B7 M3001 N80 w1500 bf16, 168 tiles: 65 -> 40 us).
  // A launch with fewer tiles than CUs shares its tiles out and then runs several times as many
  // workgroups as before, whose partial lines no longer meet in the caches: ring there as well
  // (B7 M3001 N80 w1500, 126 MB: 40 against 45 us into one buffer, 40 against 65 us into a rotation of nine).
  const unsigned shares = tile_shares(p.B * nblk, (TM + 2 * p.w) / KC + 1);
  const bool ring_pays = p.B * p.M * (2 * p.w + 1) * 2 >= (int64_t)220 << 20 || shares > 1;
  // windows that are not a multiple of 4: the same with lines at any even column offset, which needs
  // the band 4-byte aligned (138-150 against 205 us at B96 M4096 N64, w = 255, 257, 258)
  const bool ring_unaligned = !(p.flags & WM_FLAG_NO_ALIGNED_BAND) && ((uintptr_t)c.data % 4) == 0;
  grid.y = shares;
#define WM_P1_LAUNCH(NK, AL, RING, LINES, G)                                                                 \
  hipLaunchKernelGGL((mfma_p1_kernel<T, NK, AL, RING, LINES>), grid, block, 0, p.stream,                     \
                     (const uint16_t *)x.data, (const uint16_t *)y.data, (uint16_t *)c.data, (int)p.B,       \
                     (int)p.M, (int)p.w, nblk, G, x.sb, x.sr, y.sb, y.sr, c.sb)
#define WM_P1(NK)                                                                                            \
  if (!ALIGNED && ring_pays && ring_unaligned)                                                               \
    WM_P1_LAUNCH(NK, true, 2, false, 2);                                                                     \
  else if (ALIGNED && galign != 64 && ring_pays)                                                             \
    WM_P1_LAUNCH(NK, ALIGNED, (ALIGNED ? 1 : 0), false, galign);                                             \
  else if (ALIGNED && galign == 64)                                                                          \
    WM_P1_LAUNCH(NK, ALIGNED, 0, ALIGNED, galign);                                                           \
  else                                                                                                       \
    WM_P1_LAUNCH(NK, ALIGNED, 0, false, galign)
  // N = 128 with whole-line band stores: Y chunks straight into LDS, three workgroups per CU (32-bit
  // byte offsets inside a batch element).  With 16-byte column groups most slots take the piecewise
  // store path, whose stores this kernel waits for: 10 % slower there than the kernel above.
  // It runs one workgroup per tile: with few tiles the kernel above, which shares them out, is ahead
  // (fp16/bf16, this kernel / the one above: B1 M8192 w2048, 64 tiles: 72 / 28 us; B2 M4096 w1024: 41 /
  // 18; B4 M4096 w256, 128 tiles: 17.9 / 14.6; B6 M4096 w128, 192 tiles: 14.0 / 15.0; B7 M4096 w512,
  // 224 tiles: 25.9 / 26.5).
  if (ALIGNED && galign == 64 && !(p.flags & WM_FLAG_NO_LDS_DIRECT) && y.sr > 0 &&
      (p.M + 2 * KC) * y.sr * 2 < 0x7fffffff && p.N == 128 && (shares == 1 || p.B * nblk >= 160)) {
    // (at N = 64, where the kernel above already places four workgroups on a CU, this variant measured
    // equal at w = 256 and 512 and 8 % slower at w = 64)
    hipLaunchKernelGGL((mfma_p1_dma_kernel<T, 8, ALIGNED>), dim3(grid.x), block, 0, p.stream, (const uint16_t *)x.data,
                       (const uint16_t *)y.data, (uint16_t *)c.data, (int)p.B, (int)p.M, (int)p.w, nblk, galign, x.sb,
                       x.sr, y.sb, y.sr, c.sb);
    return hipGetLastError();
  }
  switch (p.N / 16) {
    case 1: WM_P1(1); break;
    case 2: WM_P1(2); break;
    case 3: WM_P1(3); break;
    case 4: WM_P1(4); break;
    case 5: WM_P1(5); break;
    case 6: WM_P1(6); break;
    case 7: WM_P1(7); break;
    default: WM_P1(8); break;
  }
#undef WM_P1
#undef WM_P1_LAUNCH
  return hipGetLastError();
}

template <bool ALIGNED>
hipError_t by_dtype(int op, const Problem &p, const View &a, const View &y, const View &c) {
  if (p.dtype == WM_DTYPE_BF16) {
    if (op == 1) return launch_p1<bf16_t, ALIGNED>(p, a, y, c);
    if (op == 2) return launch_p2<bf16_t, ALIGNED>(p, a, y, c);
    return launch_p3<bf16_t, ALIGNED>(p, a, y, c);
  }
  if (op == 1) return launch_p1<f16_t, ALIGNED>(p, a, y, c);
  if (op == 2) return launch_p2<f16_t, ALIGNED>(p, a, y, c);
  return launch_p3<f16_t, ALIGNED>(p, a, y, c);
}

}  // namespace

bool lds_direct_layout_ok(const Problem &p, const View &a, const View &y) {
  if ((p.flags & WM_FLAG_NO_LDS_DIRECT) || y.sr <= 0 || ((uintptr_t)a.data % 4) != 0) return false;
  return (p.M + 4 * KC) * (2 * p.w + 1) * 2 + 256 < 0x7fffffff && (p.M + 4 * KC) * y.sr * 2 < 0x7fffffff;
}

bool mfma_supports(int op, int64_t B, int64_t M, int64_t N, int64_t w, int dtype) {
  (void)op;
  (void)B;
  return shape_ok(M, N, w, dtype);
}

bool try_launch_mfma_p1(const Problem &p, const View &x, const View &y, const View &c, hipError_t *err) {
  if (!shape_ok(p.M, p.N, p.w, p.dtype)) return false;
  if (!fast_layout(x, p.dtype) || !fast_layout(y, p.dtype) || !band_ok(c, 2 * p.w + 1)) return false;
  *err = band_aligned(c, p.w, p.flags) ? by_dtype<true>(1, p, x, y, c) : by_dtype<false>(1, p, x, y, c);
  return true;
}

bool try_launch_mfma_p2(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  if (!shape_ok(p.M, p.N, p.w, p.dtype)) return false;
  if (!band_ok(a, 2 * p.w + 1) || !fast_layout(y, p.dtype) || !fast_layout(c, p.dtype)) return false;
  *err = band_aligned(a, p.w, p.flags) ? by_dtype<true>(2, p, a, y, c) : by_dtype<false>(2, p, a, y, c);
  return true;
}

bool try_launch_mfma_p3(const Problem &p, const View &a, const View &y, const View &c, hipError_t *err) {
  if (!shape_ok(p.M, p.N, p.w, p.dtype)) return false;
  if (!band_ok(a, 2 * p.w + 1) || !fast_layout(y, p.dtype) || !fast_layout(c, p.dtype)) return false;
  *err = band_aligned(a, p.w, p.flags) ? by_dtype<true>(3, p, a, y, c) : by_dtype<false>(3, p, a, y, c);
  return true;
}

}  // namespace wm
