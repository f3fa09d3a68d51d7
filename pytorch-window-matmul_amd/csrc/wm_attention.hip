// Fused window attention, forward:  O = unwindow_matmul(softmax(scale * window_matmul(Q, K^T)), V)
// in one kernel, without the (B, M, 2w+1) band ever reaching memory.  It reproduces the chain the
// reference's callers write (reference tests/test_attention.py:57-63), including its treatment of
// band entries outside the sequence: window_matmul leaves +0.0 there, so without masking they take
// part in the softmax with score 0 (and contribute nothing to the output); with masking they are
// left out.  Besides O the kernel stores the log-sum-exp of every row, which is all a recomputing
// backward needs.
//
// One workgroup owns 128 queries (32 per wavefront) and walks over the keys its band can reach in
// chunks of 64, staged in LDS (K and V, double buffered) and shared by its four wavefronts.
// Per wavefront and block of 32 keys:
//   S^T = K_blk . Q^T         v_mfma_f32_32x32x16, A = key rows from LDS, B = the wavefront's
//                             queries, held in registers for the whole kernel.  In the result a
//                             lane owns ONE query (lane % 32) and 16 of the 32 keys, so the row
//                             maximum and sum of the softmax are in-lane loops plus one exchange
//                             with lane ^ 32.
//   P^T = exp2(c S^T - m)     online softmax; the running maximum m is only raised when a block
//                             exceeds it by more than 8 (in log2 units), so most blocks skip the
//                             rescaling of O.  Rounded to 16 bits, P^T is already laid out as the
//                             B operand of the next product.
//   O^T += V_blk^T . P^T      A = V columns, fetched from the row-major LDS tile with
//                             ds_read_b64_tr_b16.
// Blocks that lie entirely outside a wavefront's band are skipped, blocks entirely inside it run
// without any masking arithmetic.
#include "wm_mfma_common.hpp"

#include <type_traits>

namespace wm {
namespace {

constexpr int AT_TM = 128;  // queries per workgroup
constexpr int AT_KC = 64;   // keys per chunk
constexpr float kRaiseStep = 8.0f;
constexpr float kLn2F = 0.6931471805599453f;

// Transposed operand fetch like lds_read_transposed, but for the k order that the accumulator
// layout of the first product dictates: the lane with half = lane / 32 gets rows
// k0 + 4 half + {0..3} and k0 + 8 + 4 half + {0..3}.
__device__ __forceinline__ u32x4 lds_read_transposed_split(const uint16_t *mat, int stride, int k0, int x0, int lane) {
  const int s = lane & 15, grp = lane >> 4;
  const int xb = x0 + 16 * (grp & 1) + 4 * (s & 3);
  const int kb = k0 + 4 * (grp >> 1) + (s >> 2);
  typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
  const uint16_t *p0 = mat + kb * stride + xb;
  const uint16_t *p1 = p0 + 8 * stride;
  const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0));
  const s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p1));
  const u32x2 ua = __builtin_bit_cast(u32x2, a), ub = __builtin_bit_cast(u32x2, b);
  u32x4 r = {ua[0], ua[1], ub[0], ub[1]};
  return r;
}

// Value of the same register in lane ^ 32 combined with the own one.
__device__ __forceinline__ float across_halves_max(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float across_halves_sum(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <typename T, int NK, bool MASK>  // N = 16 NK
__global__ __launch_bounds__(kThreads, NK <= 4 ? 4 : 2) void attention_forward_kernel(
    const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
    uint16_t *__restrict__ O, float *__restrict__ L, int B, int M, int w, int nblk, float c, int64_t qsb, int64_t qsr,
    int64_t ksb, int64_t ksr, int64_t vsb, int64_t vsr, int64_t osb, int64_t osr) {
  constexpr int N = 16 * NK, NB = (NK + 1) / 2;  // NB blocks of 32 output columns; the last may be half used
  constexpr int KS = N + 8;         // key rows 16 (mod 128) bytes apart in banks: conflict-free b128 reads
  constexpr int VS = 32 * NB + 16;  // value rows 32 or 96 (mod 128) bytes apart: what the transposed reads want
  constexpr int PIECES = AT_KC * N / 8;                       // 16-byte pieces of a chunk, per tensor
  constexpr int SLOTS = (PIECES + kThreads - 1) / kThreads;   // pieces per thread (the last slot may be idle)
  __shared__ __attribute__((aligned(16))) uint16_t k_lds[2][AT_KC * KS];
  __shared__ __attribute__((aligned(16))) uint16_t v_lds[2][AT_KC * VS];

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5;
  const int i0 = blk * AT_TM;
  const int qw0 = i0 + 32 * wave;     // first query of this wavefront
  const int qi = qw0 + (lane & 31);   // this lane's query
  const uint16_t *Kb = K + (int64_t)b * ksb;
  const uint16_t *Vb = V + (int64_t)b * vsb;

  // B operand of the first product: the wavefront's 32 queries, all of N, in registers
  u32x4 qf[NK];
  {
    const uint16_t *qr = Q + (int64_t)b * qsb + (int64_t)qi * qsr + 8 * half;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) qf[ks] = load_row_chunk(qr + 16 * ks, Q, qi < M);
  }

  const int kc_lo = max(i0 - w, 0) / AT_KC;
  const int kc_hi = min(i0 + AT_TM - 1 + w, M - 1) / AT_KC;

  // loader slots: row and column of the 16-byte piece this thread moves, per chunk
  int l_row[SLOTS], l_col[SLOTS];
#pragma unroll
  for (int u = 0; u < SLOTS; ++u) {
    const int p = min(tid + kThreads * u, PIECES - 1);  // an idle slot repeats the last piece
    l_row[u] = p / (N / 8);
    l_col[u] = (p % (N / 8)) * 8;
  }
  u32x4 kreg[SLOTS], vreg[SLOTS];
  // Loads only.  Rows past the end of the sequence (and the chunk after the last one) are clamped
  // to the last row instead of being zero-filled: every key they stand for is masked out by the
  // edge logic below, so only finite stand-in data is needed.
  auto fetch = [&](int kc) {
    const int base = min(kc, kc_hi) * AT_KC;
#pragma unroll
    for (int u = 0; u < SLOTS; ++u) {
      const int key = min(base + l_row[u], M - 1);
      kreg[u] = *reinterpret_cast<const u32x4 *>(Kb + (int64_t)key * ksr + l_col[u]);
      vreg[u] = *reinterpret_cast<const u32x4 *>(Vb + (int64_t)key * vsr + l_col[u]);
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int u = 0; u < SLOTS; ++u) {
      *reinterpret_cast<u32x4 *>(&k_lds[buf][l_row[u] * KS + l_col[u]]) = kreg[u];
      *reinterpret_cast<u32x4 *>(&v_lds[buf][l_row[u] * VS + l_col[u]]) = vreg[u];
    }
  };

  f32x16 o[NB];
#pragma unroll
  for (int hb = 0; hb < NB; ++hb)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[hb][v] = 0.0f;
  float m_used = -1.0e30f;  // running maximum in log2 units (finite, so that -inf scores give exp2(-inf) = 0)
  float l_part = 0.0f;      // this lane's share of the running sum
  const float ninf = -__builtin_huge_valf();

  auto block = [&](int buf, int kb, int c0, auto edge) {
    constexpr bool EDGE = decltype(edge)::value;
    f32x16 s;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = 0.0f;
    const uint16_t *krow = &k_lds[buf][(32 * kb + (lane & 31)) * KS + 8 * half];
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) s = Mma<T>::run(*reinterpret_cast<const u32x4 *>(krow + 16 * ks), qf[ks], s);
    // accumulator v of this lane: key c0 + 8 (v / 4) + 4 half + v % 4, query qi
    if (EDGE) {
      // key offset ofs = 8 (v / 4) + v % 4 of this lane is inside the band and the sequence iff
      // first <= ofs <= last; one unsigned comparison per element after this per-lane setup
      const int d0 = c0 + 4 * half - qi;  // key - query at ofs = 0
      const int first = -w - d0, last = min(w - d0, M - 1 - c0 - 4 * half);
      const int origin = last < first ? 0x100000 : first;
      const unsigned span = last < first ? 0u : (unsigned)(last - first);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int ofs = 8 * (v / 4) + v % 4;
        s[v] = (unsigned)(ofs - origin) <= span ? s[v] : ninf;
      }
    }
    float bm = s[0];
#pragma unroll
    for (int v = 1; v < 16; ++v) bm = fmaxf(bm, s[v]);
    bm = across_halves_max(bm) * c;
    const bool raise = bm > m_used + kRaiseStep;
    if (__builtin_amdgcn_ballot_w64(raise) != 0) {
      const float m_new = raise ? bm : m_used;
      const float alpha = __builtin_amdgcn_exp2f(m_used - m_new);
      m_used = m_new;
      l_part *= alpha;
#pragma unroll
      for (int hb = 0; hb < NB; ++hb)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[hb][v] *= alpha;
    }
    float p[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) p[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], c, -m_used));
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const u32x4 pf = {Mma<T>::pack2(p[8 * t + 0], p[8 * t + 1]), Mma<T>::pack2(p[8 * t + 2], p[8 * t + 3]),
                        Mma<T>::pack2(p[8 * t + 4], p[8 * t + 5]), Mma<T>::pack2(p[8 * t + 6], p[8 * t + 7])};
      // the row sum is taken over the rounded probabilities, the ones that multiply V
#pragma unroll
      for (int d = 0; d < 4; ++d) l_part = Mma<T>::add_pair(pf[d], l_part);
#pragma unroll
      for (int hb = 0; hb < NB; ++hb) {
        const u32x4 vf = lds_read_transposed_split(v_lds[buf], VS, 32 * kb + 16 * t, 32 * hb, lane);
        o[hb] = Mma<T>::run(vf, pf, o[hb]);
      }
    }
  };

  fetch(kc_lo);
  stash(0);
  __syncthreads();
  for (int kc = kc_lo; kc <= kc_hi; ++kc) {
    const int buf = (kc - kc_lo) & 1;
    fetch(kc + 1);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int c0 = kc * AT_KC + 32 * kb;
      // wave-uniform: skip blocks outside this wavefront's band or the sequence
      if (c0 + 31 < qw0 - w || c0 > qw0 + 31 + w || c0 >= M) continue;
      const bool interior = c0 >= qw0 + 31 - w && c0 + 31 <= qw0 + w && c0 + 31 < M;
      if (interior)
        block(buf, kb, c0, std::false_type());
      else
        block(buf, kb, c0, std::true_type());
    }
    stash(buf ^ 1);
    __syncthreads();
  }

  float l = across_halves_sum(l_part);
  float alpha = 1.0f;  // what the accumulated O still has to be scaled by (folded into the division by l)
  if (!MASK) {
    // Band entries outside the sequence: score 0 each, no value row.  Branch-free, see
    // attention_forward_dma_kernel.
    const int n_out = max(0, w - qi) + max(0, qi + w - (M - 1));
    const float m_new = n_out > 0 ? fmaxf(m_used, 0.0f) : m_used;
    alpha = __builtin_amdgcn_exp2f(m_used - m_new);
    l = l * alpha + (float)n_out * __builtin_amdgcn_exp2f(-m_new);
    m_used = m_new;
  }
  if (qi >= M) l = 1.0f;  // rows past the end: keep the arithmetic finite, nothing is stored
  const float inv = alpha / l;
  if (L != nullptr && half == 0 && qi < M) L[(int64_t)b * M + qi] = (m_used + __builtin_amdgcn_logf(l)) * kLn2F;
  // every wave is past the last barrier: the value buffers are free and stage the result rows
  static_assert(4 * RowStage<NB>::ELEMS <= 2 * AT_KC * VS, "the four staging areas must fit the value buffers");
  store_wave_rows<T, NB>(&v_lds[0][0] + wave * RowStage<NB>::ELEMS, o, inv, O + (int64_t)b * osb, osr, qw0, M, N, lane);
}

// ---------------------------------------------------------------------------------------------
// Narrow windows (w <= 16 (NKB - 1)): one pass, no key loop
// ---------------------------------------------------------------------------------------------
// A wavefront's 32 queries reach at most 32 NKB keys, so all of S^T (NKB tiles) sits in registers
// at once and the softmax is the plain two-pass one.  Queries go straight from memory into MFMA
// operand registers; the key and value rows of the workgroup are fetched as coalesced 16-byte
// pieces, every load in flight before the first use, and pass through one LDS region in turn
// (keys for S^T, then values for the second product, then the output rows, which leave as whole
// non-temporal lines).  What bounds this kernel is HBM: it reads q, k, v and writes o, nothing else.
template <typename T, int NK, int NKB, bool MASK>
__global__ __launch_bounds__(kThreads, 2) void attention_forward_narrow_kernel(
    const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
    uint16_t *__restrict__ O, float *__restrict__ L, int B, int M, int w, int nblk, float c, int64_t qsb, int64_t qsr,
    int64_t ksb, int64_t ksr, int64_t vsb, int64_t vsr, int64_t osb, int64_t osr) {
  constexpr int N = 16 * NK, NB = (NK + 1) / 2;
  constexpr int PADW = 16 * (NKB - 1);         // keys staged before the first and after the last query
  constexpr int ROWS = AT_TM + 2 * PADW;       // key / value rows of the workgroup
  constexpr int KS = N + 8;                    // key tile: plain b128 operand reads
  constexpr int VS = 32 * NB + 16;             // value tile: transposed reads
  constexpr int PIECES = ROWS * N / 8, SLOTS = (PIECES + kThreads - 1) / kThreads;
  // one LDS region, used three times: key tile, then value tile, then output staging
  __shared__ __attribute__((aligned(16))) uint16_t tile[ROWS * VS];
  static_assert(KS <= VS, "the key tile must fit the region of the value tile");

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5;
  const int i0 = blk * AT_TM;
  const int qw0 = i0 + 32 * wave, qi = qw0 + (lane & 31);
  const int kw0 = qw0 - PADW;  // first key of this wavefront's tiles

  // every load of the workgroup is issued before the first use: queries in operand layout, key and
  // value rows as coalesced 16-byte pieces (rows outside the sequence read a safe address, zeroed later)
  u32x4 qf[NK], kreg[SLOTS], vreg[SLOTS];
  {
    const uint16_t *qr = Q + (int64_t)b * qsb + (int64_t)qi * qsr + 8 * half;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) qf[ks] = fetch_row_chunk(qr + 16 * ks, Q, qi < M);
    const uint16_t *Kb = K + (int64_t)b * ksb, *Vb = V + (int64_t)b * vsb;
#pragma unroll
    for (int u = 0; u < SLOTS; ++u) {
      const int p = min(tid + kThreads * u, PIECES - 1);
      const int key = i0 - PADW + p / (N / 8), col = (p % (N / 8)) * 8;
      const bool ok = (key >= 0) & (key < M);
      kreg[u] = fetch_row_chunk(Kb + (int64_t)key * ksr + col, K, ok);
      vreg[u] = fetch_row_chunk(Vb + (int64_t)key * vsr + col, V, ok);
    }
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) qf[ks] = mask_row_chunk(qf[ks], qi < M);
#pragma unroll
    for (int u = 0; u < SLOTS; ++u) {
      const int p = min(tid + kThreads * u, PIECES - 1);
      const int row = p / (N / 8), key = i0 - PADW + row;
      *reinterpret_cast<u32x4 *>(&tile[row * KS + (p % (N / 8)) * 8]) = mask_row_chunk(kreg[u], (key >= 0) & (key < M));
    }
  }
  __syncthreads();

  // S^T tiles: accumulator v of tile j: key kw0 + 32 j + 8 (v / 4) + 4 half + v % 4, query qi
  const float ninf = -__builtin_huge_valf();
  f32x16 s[NKB];
  float top = ninf;
#pragma unroll
  for (int j = 0; j < NKB; ++j) {
#pragma unroll
    for (int v = 0; v < 16; ++v) s[j][v] = 0.0f;
    const uint16_t *krow = &tile[(32 * wave + 32 * j + (lane & 31)) * KS + 8 * half];
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) s[j] = Mma<T>::run(*reinterpret_cast<const u32x4 *>(krow + 16 * ks), qf[ks], s[j]);
    // valid key offsets of this lane in tile j: first..last (band and sequence), as in the wide kernel
    const int k0 = kw0 + 32 * j + 4 * half;  // key at offset 0
    const int first = max(qi - w, 0) - k0, last = min(qi + w, M - 1) - k0;
    const int origin = last < first ? 0x100000 : first;
    const unsigned span = last < first ? 0u : (unsigned)(last - first);
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int ofs = 8 * (v / 4) + v % 4;
      s[j][v] = (unsigned)(ofs - origin) <= span ? s[j][v] : ninf;
      top = fmaxf(top, s[j][v]);
    }
  }
  __syncthreads();  // the key tile has been read by everyone: the value tile takes its place
#pragma unroll
  for (int u = 0; u < SLOTS; ++u) {
    const int p = min(tid + kThreads * u, PIECES - 1);
    const int row = p / (N / 8), key = i0 - PADW + row;
    *reinterpret_cast<u32x4 *>(&tile[row * VS + (p % (N / 8)) * 8]) = mask_row_chunk(vreg[u], (key >= 0) & (key < M));
  }
  __syncthreads();
  top = across_halves_max(top) * c;  // log2 units
  const int n_out = MASK ? 0 : max(0, w - qi) + max(0, qi + w - (M - 1));  // zero-score entries outside the sequence
  if (n_out > 0) top = fmaxf(top, 0.0f);
  if (qi >= M) top = 0.0f;  // rows past the end: keep the arithmetic finite, nothing is stored
  float l_part = 0.0f;
  f32x16 o[NB];
#pragma unroll
  for (int hb = 0; hb < NB; ++hb)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[hb][v] = 0.0f;
#pragma unroll
  for (int j = 0; j < NKB; ++j) {
    float p[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) p[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[j][v], c, -top));
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const u32x4 pf = {Mma<T>::pack2(p[8 * t + 0], p[8 * t + 1]), Mma<T>::pack2(p[8 * t + 2], p[8 * t + 3]),
                        Mma<T>::pack2(p[8 * t + 4], p[8 * t + 5]), Mma<T>::pack2(p[8 * t + 6], p[8 * t + 7])};
#pragma unroll
      for (int d = 0; d < 4; ++d) l_part = Mma<T>::add_pair(pf[d], l_part);
#pragma unroll
      for (int hb = 0; hb < NB; ++hb) {
        const u32x4 vf = lds_read_transposed_split(tile, VS, 32 * wave + 32 * j + 16 * t, 32 * hb, lane);
        o[hb] = Mma<T>::run(vf, pf, o[hb]);
      }
    }
  }
  float l = across_halves_sum(l_part);
  if (n_out > 0) l += (float)n_out * __builtin_amdgcn_exp2f(-top);
  const float inv = 1.0f / l;
  if (L != nullptr && half == 0 && qi < M) L[(int64_t)b * M + qi] = (top + __builtin_amdgcn_logf(l)) * kLn2F;
  // The result leaves through LDS (the value tile is no longer needed) as row-contiguous,
  // non-temporal 16-byte stores: whole 128-byte lines instead of 8 bytes per lane over 32 rows.
  __syncthreads();
  constexpr int SO = 32 * NB + 8;
  static_assert(4 * 32 * SO <= ROWS * VS, "output staging must fit the value tile");
  uint16_t *stage = tile + wave * (32 * SO);
#pragma unroll
  for (int hb = 0; hb < NB; ++hb)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const u32x2 out = {Mma<T>::pack2(o[hb][4 * g] * inv, o[hb][4 * g + 1] * inv),
                         Mma<T>::pack2(o[hb][4 * g + 2] * inv, o[hb][4 * g + 3] * inv)};
      *reinterpret_cast<u32x2 *>(stage + (lane & 31) * SO + 32 * hb + 8 * g + 4 * half) = out;
    }
  wave_sync_lds();
  constexpr int PER_ROW = N / 8;
  for (int p = lane; p < 32 * PER_ROW; p += 64) {
    const int r = p / PER_ROW, hg = p - r * PER_ROW;
    if (qw0 + r < M)
      store_chunk_streaming(O + (int64_t)b * osb + (int64_t)(qw0 + r) * osr + 8 * hg,
                            *reinterpret_cast<const u32x4 *>(stage + r * SO + 8 * hg));
  }
}


// ---------------------------------------------------------------------------------------------
// Key and value chunks go from memory straight into LDS
// ---------------------------------------------------------------------------------------------
// Same tiling and arithmetic as attention_forward_kernel.  What differs is how the wavefronts are
// kept busy:
//   * K and V chunks are written into LDS by the memory system itself (buffer loads with the lds
//     modifier, swizzled tiles, see wm_mfma_common.hpp): no staging registers, no LDS stores, no
//     address arithmetic per chunk (the chunk position is a scalar offset of the load), rows past
//     the sequence read as zeros, and chunks are requested DEPTH iterations before their use.
//   * Everything that decides what a wavefront does with a chunk is scalar (the wavefront's first
//     query is read with readfirstlane), so skipped blocks cost a scalar branch.
//   * A chunk whose two 32-key blocks both lie inside the wavefront's band is processed as a pair:
//     both score tiles are formed by two independent MFMA chains, one row maximum serves both, and
//     the exponentials of one block run on the vector ALU while the matrix pipe multiplies the
//     other block's probabilities with V.
template <typename T, int NK, bool MASK>
__global__ __launch_bounds__(kThreads, NK <= 4 ? 4 : 2) void attention_forward_dma_kernel(
    const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
    uint16_t *__restrict__ O, float *__restrict__ L, int B, int M, int w, int nblk, float c, int64_t qsb, int64_t qsr,
    int64_t ksb, int64_t ksr, int64_t vsb, int64_t vsr, int64_t osb, int64_t osr) {
  // tile rows of 128 bytes (N <= 64) or 256 bytes; the pieces of a row beyond column N are never
  // fetched (requested out of range: zeros, no memory traffic)
  constexpr int N = 16 * NK, NB = (NK + 1) / 2, ROWB = NK <= 4 ? 128 : 256, PPR = ROWB / 16;
  constexpr int STAGES = 2, DEPTH = STAGES - 1;
  constexpr int TILE = AT_KC * ROWB / 2;   // elements per tile
  constexpr int LOADS = 2 * (PPR / 4);     // loads per wavefront and chunk (K and V)
  static_assert(NK >= 1 && NK <= 8, "N = 16 ... 128");
  __shared__ __attribute__((aligned(1024))) uint16_t kv_lds[2 * STAGES][TILE];  // key tiles, then value tiles
  uint16_t (*const k_lds)[TILE] = kv_lds, (*const v_lds)[TILE] = kv_lds + STAGES;

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i0 = blk * AT_TM;
  const int qw0 = i0 + 32 * wave;     // first query of this wavefront (scalar)
  const int qi = qw0 + (lane & 31);   // this lane's query

  const u32x4 k_rsrc = make_rsrc(K + (int64_t)b * ksb, (uint32_t)((M - 1) * ksr * 2 + 2 * N));
  const u32x4 v_rsrc = make_rsrc(V + (int64_t)b * vsb, (uint32_t)((M - 1) * vsr * 2 + 2 * N));
  const bool piece_in_row = (((64 * wave + lane) % PPR) ^ swz<PPR>((64 * wave + lane) / PPR)) < N / 8;
  const uint32_t k_voff = piece_in_row ? dma_lane_offset<PPR>(wave, lane, ksr) : 0x80000000u;
  const uint32_t v_voff = piece_in_row ? dma_lane_offset<PPR>(wave, lane, vsr) : 0x80000000u;
  const uint32_t k_step = (uint32_t)(256 / PPR * ksr * 2), v_step = (uint32_t)(256 / PPR * vsr * 2);
  const uint32_t k_chunk = (uint32_t)(AT_KC * ksr * 2), v_chunk = (uint32_t)(AT_KC * vsr * 2);
  auto request = [&](int kc, int stage) {
    dma_chunk<PPR>(k_rsrc, k_lds[stage], wave, k_voff, k_chunk * (uint32_t)kc, k_step);
    dma_chunk<PPR>(v_rsrc, v_lds[stage], wave, v_voff, v_chunk * (uint32_t)kc, v_step);
  };

  const int kc_lo = max(i0 - w, 0) / AT_KC;
  const int kc_hi = min(i0 + AT_TM - 1 + w, M - 1) / AT_KC;
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) request(kc_lo + d, d);

  // B operand of the first product: the wavefront's 32 queries, all of N, in registers
  u32x4 qf[NK];
  {
    const uint16_t *qr = Q + (int64_t)b * qsb + (int64_t)qi * qsr + 8 * half;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) qf[ks] = load_row_chunk(qr + 16 * ks, Q, qi < M);
  }

  // LDS byte offsets inside a tile.  Key rows as A operand: row lane % 32 of a block, pieces
  // 2 ks + half; value columns through the transposing read: rows 4 (grp / 2) + s / 4 (+ 8),
  // 8 bytes at column 32 hb + 16 (grp % 2) + 4 (s % 4).  The swizzle only touches address bits
  // that the ks / hb terms do not carry into, so those terms are XORed in at the point of use.
  const int r32 = lane & 31;
  const uint32_t k_at = (uint32_t)(r32 * ROWB + ((half ^ swz<PPR>(r32)) << 4));
  const int s16 = lane & 15, grp = lane >> 4, rowl = 4 * (grp >> 1) + (s16 >> 2);
  const uint32_t v_at = (uint32_t)(rowl * ROWB + (((2 * (grp & 1) + ((s16 & 3) >> 1)) ^ swz<PPR>(rowl)) << 4) + 8 * (s16 & 1));
  typedef s16x4 __attribute__((address_space(3))) * lds_tr_ptr;
  auto key_operand = [&](const uint16_t *tile, int kb, int ks) {
    return *reinterpret_cast<const u32x4 *>(reinterpret_cast<const char *>(tile) + 32 * kb * ROWB + (k_at ^ (32 * ks)));
  };
  auto value_operand = [&](const uint16_t *tile, int kb, int t, int hb) {
    const char *p = reinterpret_cast<const char *>(tile) + (32 * kb + 16 * t) * ROWB;
    const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(p + (v_at ^ (64 * hb)))));
    const u32x2 hi = __builtin_bit_cast(  // eight rows further down the swizzle differs in bit 1
        u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(p + 8 * ROWB + (v_at ^ 32 ^ (64 * hb)))));
    const u32x4 r = {lo[0], lo[1], hi[0], hi[1]};
    return r;
  };

  f32x16 o[NB];
#pragma unroll
  for (int hb = 0; hb < NB; ++hb)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[hb][v] = 0.0f;
  float m_used = -1.0e30f;  // running maximum in log2 units (finite, so that -inf scores give exp2(-inf) = 0)
  float l_part = 0.0f;      // this lane's share of the running sum
  const float ninf = -__builtin_huge_valf();

  // The LDS reads of a product are all issued before its first MFMA: left to itself the compiler
  // reuses one register set for consecutive operands, one LDS latency in front of every MFMA.
  auto scores = [&](const uint16_t *kt, int kb) {
    f32x16 s;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = 0.0f;
    u32x4 ka[NK];
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) ka[ks] = key_operand(kt, kb, ks);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) s = Mma<T>::run(ka[ks], qf[ks], s);
    return s;
  };
  auto block_max = [&](const f32x16 &s) {
    float bm = s[0];
#pragma unroll
    for (int v = 1; v < 16; ++v) bm = fmaxf(bm, s[v]);
    return bm;
  };
  // raises the running maximum to bm (log2 units, already exchanged between the half-waves) when
  // some row of the wavefront exceeds it by more than kRaiseStep
  auto raise_to = [&](float bm) {
    const bool raise = bm > m_used + kRaiseStep;
    if (__builtin_amdgcn_ballot_w64(raise) != 0) {
      const float m_new = raise ? bm : m_used;
      const float alpha = __builtin_amdgcn_exp2f(m_used - m_new);
      m_used = m_new;
      l_part *= alpha;
#pragma unroll
      for (int hb = 0; hb < NB; ++hb)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[hb][v] *= alpha;
    }
  };
  // P^T = exp2(c S^T - m), rounded; row sums over the rounded values; O^T += V_blk^T P^T
  auto accumulate = [&](const uint16_t *vt, int kb, const f32x16 &s) {
    u32x4 va[2][NB];  // in flight while the exponentials run
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int hb = 0; hb < NB; ++hb) va[t][hb] = value_operand(vt, kb, t, hb);
    __builtin_amdgcn_sched_barrier(0);
    float p[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) p[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], c, -m_used));
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const u32x4 pf = {Mma<T>::pack2(p[8 * t + 0], p[8 * t + 1]), Mma<T>::pack2(p[8 * t + 2], p[8 * t + 3]),
                        Mma<T>::pack2(p[8 * t + 4], p[8 * t + 5]), Mma<T>::pack2(p[8 * t + 6], p[8 * t + 7])};
#pragma unroll
      for (int d = 0; d < 4; ++d) l_part = Mma<T>::add_pair(pf[d], l_part);
#pragma unroll
      for (int hb = 0; hb < NB; ++hb) o[hb] = Mma<T>::run(va[t][hb], pf, o[hb]);
    }
  };
  // accumulator v of a lane: key c0 + 8 (v / 4) + 4 half + v % 4, query qi; offsets first..last are
  // inside the band and the sequence
  auto mask_edge = [&](f32x16 &s, int c0) {
    const int d0 = c0 + 4 * half - qi;
    const int first = -w - d0, last = min(w - d0, M - 1 - c0 - 4 * half);
    const int origin = last < first ? 0x100000 : first;
    const unsigned span = last < first ? 0u : (unsigned)(last - first);
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int ofs = 8 * (v / 4) + v % 4;
      s[v] = (unsigned)(ofs - origin) <= span ? s[v] : ninf;
    }
  };

  int stage = 0;
  // Start of an iteration: this wavefront's pieces of chunk kc have landed (the DEPTH - 1 younger
  // chunks may still be in flight); after the barrier so have everyone's, and nobody reads chunk
  // kc - 1 any more, whose tile takes chunk kc + DEPTH (beyond the sequence: zeros nobody reads).
  auto open_chunk = [&](int kc) {
    wait_vmcnt<(DEPTH - 1) * LOADS>();
    __builtin_amdgcn_s_barrier();
    int st = stage + DEPTH;
    st = st >= STAGES ? st - STAGES : st;
    request(kc + DEPTH, st);
  };
  auto close_chunk = [&]() { stage = stage + 1 == STAGES ? 0 : stage + 1; };
  // chunk with a block that is outside the band or the sequence, or crosses their edge
  auto edge_chunk = [&](int kc) {
    open_chunk(kc);
    const uint16_t *kt = k_lds[stage], *vt = v_lds[stage];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int cb = kc * AT_KC + 32 * kb;
      if (cb + 31 < qw0 - w || cb > qw0 + 31 + w || cb >= M) continue;  // scalar
      f32x16 s = scores(kt, kb);
      mask_edge(s, cb);  // also where the block happens to need no mask: one code path, no register shuffling
      raise_to(across_halves_max(block_max(s)) * c);
      accumulate(vt, kb, s);
    }
    close_chunk();
  };
  // The wavefront's chunks [pair_lo, pair_hi] lie wholly inside its band and the sequence; every
  // wavefront of the workgroup passes the same number of barriers, whichever loop it is in.
  const int pair_lo = max(kc_lo, (qw0 + 31 - w + 63) >> 6);
  const int pair_hi = min(kc_hi, (min(qw0 + w, M - 1) - 63) >> 6);
  const int lead_end = pair_lo <= pair_hi ? pair_lo : kc_hi + 1;
  int kc = kc_lo;
  for (; kc < lead_end; ++kc) edge_chunk(kc);
  for (; kc <= pair_hi; ++kc) {
    open_chunk(kc);
    const uint16_t *kt = k_lds[stage], *vt = v_lds[stage];
    const f32x16 s0 = scores(kt, 0), s1 = scores(kt, 1);
    raise_to(across_halves_max(fmaxf(block_max(s0), block_max(s1))) * c);
    accumulate(vt, 0, s0);
    accumulate(vt, 1, s1);
    close_chunk();
  }
  for (; kc <= kc_hi; ++kc) edge_chunk(kc);

  float l = across_halves_sum(l_part);
  float alpha = 1.0f;  // what the accumulated O still has to be scaled by (folded into the division by l)
  if (!MASK) {
    // Band entries outside the sequence: score 0 each, no value row.  Branch-free: a row without such
    // entries keeps its maximum, alpha = 1 and adds 0 to the sum.
    const int n_out = max(0, w - qi) + max(0, qi + w - (M - 1));
    const float m_new = n_out > 0 ? fmaxf(m_used, 0.0f) : m_used;
    alpha = __builtin_amdgcn_exp2f(m_used - m_new);
    l = l * alpha + (float)n_out * __builtin_amdgcn_exp2f(-m_new);
    m_used = m_new;
  }
  if (qi >= M) l = 1.0f;  // rows past the end: keep the arithmetic finite, nothing is stored
  const float inv = alpha / l;
  if (L != nullptr && half == 0 && qi < M) L[(int64_t)b * M + qi] = (m_used + __builtin_amdgcn_logf(l)) * kLn2F;
  // The chunks requested past the last one must have landed before their tiles are reused, and
  // every wavefront must be done with the last chunk: then the tiles stage the result rows.
  wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  static_assert(4 * RowStage<NB>::ELEMS <= 2 * STAGES * TILE, "the four staging areas must fit the tiles");
  store_wave_rows<T, NB>(&k_lds[0][0] + wave * RowStage<NB>::ELEMS, o, inv, O + (int64_t)b * osb, osr, qw0, M, N, lane);
}

template <typename T, int NK>
hipError_t launch_forward(const Problem &p, const View &q, const View &k, const View &v, const View &o, float *lse,
                          double scale, int mask) {
  const int nblk = (int)((p.M + AT_TM - 1) / AT_TM);
  if (tiled_grid(p.B, nblk) > 0x7fffffff) return hipErrorInvalidValue;
  const dim3 grid((unsigned)tiled_grid(p.B, nblk)), block(kThreads);
  const float c = (float)(scale * 1.4426950408889634);
#define WM_AT(KERNEL)                                                                                              \
  hipLaunchKernelGGL(KERNEL, grid, block, 0, p.stream, (const uint16_t *)q.data, (const uint16_t *)k.data,         \
                     (const uint16_t *)v.data, (uint16_t *)o.data, lse, (int)p.B, (int)p.M, (int)p.w, nblk, c,     \
                     q.sb, q.sr, k.sb, k.sr, v.sb, v.sr, o.sb, o.sr)
  // narrow windows take the one-pass kernel (two key tiles per wavefront up to w = 16, three up to 32)
  if (p.w <= 16 && !(p.flags & WM_FLAG_NO_NARROW_BAND)) {
    if (mask)
      WM_AT((attention_forward_narrow_kernel<T, NK, 2, true>));
    else
      WM_AT((attention_forward_narrow_kernel<T, NK, 2, false>));
  } else if (p.w <= 32 && NK <= 4 && !(p.flags & WM_FLAG_NO_NARROW_BAND)) {
    if (mask)
      WM_AT((attention_forward_narrow_kernel<T, NK, 3, true>));
    else
      WM_AT((attention_forward_narrow_kernel<T, NK, 3, false>));
  } else {
    // the buffer loads of the LDS-direct kernel address a batch element with 32-bit byte offsets
    const int64_t lim = 0x7fffffff;
    const bool fits = (p.M + 3 * AT_KC) * k.sr * 2 < lim && (p.M + 3 * AT_KC) * v.sr * 2 < lim && k.sr > 0 && v.sr > 0;
    if (fits && !(p.flags & WM_FLAG_NO_LDS_DIRECT)) {
      if (mask)
        WM_AT((attention_forward_dma_kernel<T, NK, true>));
      else
        WM_AT((attention_forward_dma_kernel<T, NK, false>));
    } else if (mask) {
      WM_AT((attention_forward_kernel<T, NK, true>));
    } else {
      WM_AT((attention_forward_kernel<T, NK, false>));
    }
  }
#undef WM_AT
  return hipGetLastError();
}

template <typename T>
hipError_t forward_by_width(const Problem &p, const View &q, const View &k, const View &v, const View &o, float *lse,
                            double scale, int mask) {
  switch (p.N / 16) {
    case 1: return launch_forward<T, 1>(p, q, k, v, o, lse, scale, mask);
    case 2: return launch_forward<T, 2>(p, q, k, v, o, lse, scale, mask);
    case 3: return launch_forward<T, 3>(p, q, k, v, o, lse, scale, mask);
    case 4: return launch_forward<T, 4>(p, q, k, v, o, lse, scale, mask);
    case 5: return launch_forward<T, 5>(p, q, k, v, o, lse, scale, mask);
    case 6: return launch_forward<T, 6>(p, q, k, v, o, lse, scale, mask);
    case 7: return launch_forward<T, 7>(p, q, k, v, o, lse, scale, mask);
    default: return launch_forward<T, 8>(p, q, k, v, o, lse, scale, mask);
  }
}

}  // namespace

bool attention_supports(int64_t M, int64_t N, int64_t w, int dtype, double scale) {
  if (dtype != WM_DTYPE_BF16 && dtype != WM_DTYPE_F16) return false;
  if (N % 16 != 0 || N < 16 || N > 128) return false;
  if (M < 1 || w < 1 || w > 0x3fffffff) return false;
  if (M > 0x7fffffff - w - 2 * AT_TM) return false;  // row and key indices are 32-bit in the kernels
  return scale > 0.0 && scale < 1.0e30;
}

bool try_launch_attention_forward(const Problem &p, const View &q, const View &k, const View &v, const View &o,
                                  float *lse, double scale, int mask, hipError_t *err) {
  if (p.flags & WM_FLAG_FORCE_STRIDED) return false;
  if (!attention_supports(p.M, p.N, p.w, p.dtype, scale)) return false;
  if (!fast_layout(q, p.dtype) || !fast_layout(k, p.dtype) || !fast_layout(v, p.dtype) || !fast_layout(o, p.dtype))
    return false;
  *err = p.dtype == WM_DTYPE_BF16 ? forward_by_width<bf16_t>(p, q, k, v, o, lse, scale, mask)
                                  : forward_by_width<f16_t>(p, q, k, v, o, lse, scale, mask);
  return true;
}

}  // namespace wm
