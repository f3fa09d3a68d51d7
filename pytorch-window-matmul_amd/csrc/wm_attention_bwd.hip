// Fused window attention, backward, by recomputation from the saved log-sum-exp L of every row:
//   P[i,c]  = exp(scale * q_i . k_c - L_i)            for |i - c| <= w, 0 <= c < M
//   D_i     = sum_h dO[i,h] * O[i,h]                   (= sum_c P[i,c] * dP[i,c])
//   dP[i,c] = dO_i . v_c
//   dS[i,c] = scale * P[i,c] * (dP[i,c] - D_i)
//   dQ_i = sum_c dS[i,c] k_c      dK_c = sum_i dS[i,c] q_i      dV_c = sum_i P[i,c] dO_i
// Band entries outside the sequence need no special case here: they only enter through L (the
// forward counted them there when asked to) and their own gradients are dropped by the chain of
// separate ops as well.
//
// Two output-stationary kernels, no atomics:
//   query kernel  a workgroup owns 128 queries and walks over the key chunks of its band
//                 (K and V staged in LDS): S^T, dP^T, then dQ^T += K^T dS^T.  It also writes D.
//   key kernel    a workgroup owns 128 keys and walks over the query chunks of their band
//                 (Q, dO, L, D staged in LDS): S, dP, then dV^T += dO^T P and dK^T += Q^T dS.
// Both use the layout of the forward kernel: in every 32x32 score tile a lane owns one row of the
// stationary side (lane % 32) and 16 rows of the streamed side, so P and dS come out of the
// arithmetic already arranged as B operands of the products that consume them, and the streamed
// tiles are read from LDS both by rows (first products) and transposed (second products).
// Narrow windows of heads up to 64 wide take a third kernel that does the work of both at once
// (attention_backward_narrow_kernel below).
#include "wm_mfma_common.hpp"

#include <type_traits>

namespace wm {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int AB_TM = 128;  // stationary rows per workgroup (32 per wavefront)
constexpr int AB_KC = 64;   // streamed rows per chunk

// See wm_attention.hip: rows k0 + 4 half + {0..3} and k0 + 8 + 4 half + {0..3}.
__device__ __forceinline__ u32x4 lds_tr_split(const uint16_t *mat, int stride, int k0, int x0, int lane) {
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

__device__ __forceinline__ float halves_sum(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <typename T>
__device__ __forceinline__ float dot8(u32x4 a, u32x4 b) {
  float acc = 0.0f;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    T a0, a1, b0, b1;
    const uint16_t al = (uint16_t)a[d], ah = (uint16_t)(a[d] >> 16), bl = (uint16_t)b[d], bh = (uint16_t)(b[d] >> 16);
    __builtin_memcpy(&a0, &al, 2), __builtin_memcpy(&a1, &ah, 2);
    __builtin_memcpy(&b0, &bl, 2), __builtin_memcpy(&b1, &bh, 2);
    acc += to_acc<T>(a0) * to_acc<T>(b0) + to_acc<T>(a1) * to_acc<T>(b1);
  }
  return acc;
}

template <typename T>
__device__ __forceinline__ u32x4 pack8(const float *x) {
  const u32x4 r = {Mma<T>::pack2(x[0], x[1]), Mma<T>::pack2(x[2], x[3]), Mma<T>::pack2(x[4], x[5]),
                   Mma<T>::pack2(x[6], x[7])};
  return r;
}

// ---------------------------------------------------------------------------------------------
// query kernel: dQ and D
// ---------------------------------------------------------------------------------------------
template <typename T, int NK, bool WITH_DQ>  // N = 16 NK; WITH_DQ false: only D is wanted (grad_q not requested)
__global__ __launch_bounds__(kThreads, NK <= 4 ? 3 : 1) void attention_backward_query_kernel(
    const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
    const uint16_t *__restrict__ O, const uint16_t *__restrict__ dO, const float *__restrict__ L,
    uint16_t *__restrict__ dQ, float *__restrict__ D, int B, int M, int w, int nblk, float scale, int64_t qsb,
    int64_t qsr, int64_t ksb, int64_t ksr, int64_t vsb, int64_t vsr, int64_t osb, int64_t osr, int64_t gsb, int64_t gsr,
    int64_t dqsb, int64_t dqsr) {
  constexpr int N = 16 * NK, NB = (NK + 1) / 2;
  constexpr int TS = 32 * NB + 16;  // tile rows 32 or 96 (mod 128) bytes apart: row reads and transposed reads
  constexpr int PIECES = AB_KC * N / 8;
  constexpr int SLOTS = (PIECES + kThreads - 1) / kThreads;  // the last slot may be idle
  __shared__ __attribute__((aligned(16))) uint16_t k_lds[2][AB_KC * TS];
  __shared__ __attribute__((aligned(16))) uint16_t v_lds[2][AB_KC * TS];

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5;
  const int i0 = blk * AB_TM;
  const int qw0 = i0 + 32 * wave;
  const int qi = qw0 + (lane & 31);
  const bool q_ok = qi < M;
  const uint16_t *Kb = K + (int64_t)b * ksb;
  const uint16_t *Vb = V + (int64_t)b * vsb;
  const float c = scale * 1.4426950408889634f;

  // stationary side in registers: the query rows and their upstream gradient rows (B operands)
  u32x4 qf[NK], gf[NK];
  float delta = 0.0f;
  {
    const uint16_t *qr = Q + (int64_t)b * qsb + (int64_t)qi * qsr + 8 * half;
    const uint16_t *gr = dO + (int64_t)b * gsb + (int64_t)qi * gsr + 8 * half;
    const uint16_t *orow = O + (int64_t)b * osb + (int64_t)qi * osr + 8 * half;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      qf[ks] = load_row_chunk(qr + 16 * ks, Q, q_ok);
      gf[ks] = load_row_chunk(gr + 16 * ks, dO, q_ok);
      delta += dot8<T>(gf[ks], load_row_chunk(orow + 16 * ks, O, q_ok));
    }
  }
  delta = halves_sum(delta);
  if (q_ok && half == 0) D[(int64_t)b * M + qi] = delta;
  if (!WITH_DQ) return;
  const float l2 = (q_ok ? L[(int64_t)b * M + qi] : 0.0f) * 1.4426950408889634f;
  const float delta_s = delta * scale;

  const int kc_lo = max(i0 - w, 0) / AB_KC;
  const int kc_hi = min(i0 + AB_TM - 1 + w, M - 1) / AB_KC;
  int l_row[SLOTS], l_col[SLOTS];
#pragma unroll
  for (int u = 0; u < SLOTS; ++u) {
    // an idle slot repeats the last piece; widths that fill every slot keep the plain affine index
    const int p = PIECES % kThreads == 0 ? tid + kThreads * u : min(tid + kThreads * u, PIECES - 1);
    l_row[u] = p / (N / 8);
    l_col[u] = (p % (N / 8)) * 8;
  }
  u32x4 kreg[SLOTS], vreg[SLOTS];
  // loads only; rows past the sequence are clamped to its last row (they are masked out below)
  auto fetch = [&](int kc) {
    const int base = min(kc, kc_hi) * AB_KC;
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
      *reinterpret_cast<u32x4 *>(&k_lds[buf][l_row[u] * TS + l_col[u]]) = kreg[u];
      *reinterpret_cast<u32x4 *>(&v_lds[buf][l_row[u] * TS + l_col[u]]) = vreg[u];
    }
  };

  f32x16 dq[NB];
#pragma unroll
  for (int hb = 0; hb < NB; ++hb)
#pragma unroll
    for (int v = 0; v < 16; ++v) dq[hb][v] = 0.0f;
  const float ninf = -__builtin_huge_valf();

  auto block = [&](int buf, int kb, int c0, auto edge) {
    constexpr bool EDGE = decltype(edge)::value;
    f32x16 s, dp;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = 0.0f, dp[v] = 0.0f;
    const int at = (32 * kb + (lane & 31)) * TS + 8 * half;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      s = Mma<T>::run(*reinterpret_cast<const u32x4 *>(&k_lds[buf][at + 16 * ks]), qf[ks], s);
      dp = Mma<T>::run(*reinterpret_cast<const u32x4 *>(&v_lds[buf][at + 16 * ks]), gf[ks], dp);
    }
    // accumulator v of this lane: key c0 + 8 (v / 4) + 4 half + v % 4, query qi
    if (EDGE) {
      const int d0 = c0 + 4 * half - qi;  // key - query at offset 0; valid offsets: first..last
      const int first = -w - d0, last = min(w - d0, M - 1 - c0 - 4 * half);
      const int origin = last < first ? 0x100000 : first;
      const unsigned span = last < first ? 0u : (unsigned)(last - first);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int ofs = 8 * (v / 4) + v % 4;
        s[v] = (unsigned)(ofs - origin) <= span ? s[v] : ninf;
      }
    }
    float ds[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], c, -l2));
      ds[v] = p * __builtin_fmaf(dp[v], scale, -delta_s);
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const u32x4 dsf = pack8<T>(ds + 8 * t);
#pragma unroll
      for (int hb = 0; hb < NB; ++hb)
        dq[hb] = Mma<T>::run(lds_tr_split(k_lds[buf], TS, 32 * kb + 16 * t, 32 * hb, lane), dsf, dq[hb]);
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
      const int c0 = kc * AB_KC + 32 * kb;
      if (c0 + 31 < qw0 - w || c0 > qw0 + 31 + w || c0 >= M) continue;  // wave-uniform
      const bool interior = c0 >= qw0 + 31 - w && c0 + 31 <= qw0 + w && c0 + 31 < M;
      if (interior)
        block(buf, kb, c0, std::false_type());
      else
        block(buf, kb, c0, std::true_type());
    }
    stash(buf ^ 1);
    __syncthreads();
  }
  // every wave is past the last barrier: the key buffers are free and stage the result rows
  static_assert(4 * RowStage<NB>::ELEMS <= 2 * AB_KC * TS, "the four staging areas must fit the key buffers");
  store_wave_rows<T, NB>(&k_lds[0][0] + wave * RowStage<NB>::ELEMS, dq, 1.0f, dQ + (int64_t)b * dqsb, dqsr, qw0, M, N,
                         lane);
}

// ---------------------------------------------------------------------------------------------
// key kernel: dK and dV
// ---------------------------------------------------------------------------------------------
template <typename T, int NK>  // N = 16 NK
__global__ __launch_bounds__(kThreads, NK <= 4 ? 2 : 1) void attention_backward_key_kernel(
    const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
    const uint16_t *__restrict__ dO, const float *__restrict__ L, const float *__restrict__ D,
    uint16_t *__restrict__ dK, uint16_t *__restrict__ dV, int B, int M, int w, int nblk, float scale, int64_t qsb,
    int64_t qsr, int64_t ksb, int64_t ksr, int64_t vsb, int64_t vsr, int64_t gsb, int64_t gsr, int64_t dksb,
    int64_t dksr, int64_t dvsb, int64_t dvsr) {
  constexpr int N = 16 * NK, NB = (NK + 1) / 2;
  constexpr int TS = 32 * NB + 16;
  constexpr int PIECES = AB_KC * N / 8;
  constexpr int SLOTS = (PIECES + kThreads - 1) / kThreads;
  __shared__ __attribute__((aligned(16))) uint16_t q_lds[2][AB_KC * TS];
  __shared__ __attribute__((aligned(16))) uint16_t g_lds[2][AB_KC * TS];
  __shared__ __attribute__((aligned(16))) float l_lds[2][AB_KC];  // L * log2(e) of the chunk's queries
  __shared__ __attribute__((aligned(16))) float d_lds[2][AB_KC];  // D * scale

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5;
  const int c0 = blk * AB_TM;
  const int kw0 = c0 + 32 * wave;     // first key of this wavefront
  const int kj = kw0 + (lane & 31);   // this lane's key
  const bool k_ok = kj < M;
  const uint16_t *Qb = Q + (int64_t)b * qsb;
  const uint16_t *Gb = dO + (int64_t)b * gsb;
  const float *Lb = L + (int64_t)b * M;
  const float *Db = D + (int64_t)b * M;
  const float c = scale * 1.4426950408889634f;

  u32x4 kf[NK], vf[NK];
  {
    const uint16_t *kr = K + (int64_t)b * ksb + (int64_t)kj * ksr + 8 * half;
    const uint16_t *vr = V + (int64_t)b * vsb + (int64_t)kj * vsr + 8 * half;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      kf[ks] = load_row_chunk(kr + 16 * ks, K, k_ok);
      vf[ks] = load_row_chunk(vr + 16 * ks, V, k_ok);
    }
  }

  const int qc_lo = max(c0 - w, 0) / AB_KC;
  const int qc_hi = min(c0 + AB_TM - 1 + w, M - 1) / AB_KC;
  int l_row[SLOTS], l_col[SLOTS];
#pragma unroll
  for (int u = 0; u < SLOTS; ++u) {
    // an idle slot repeats the last piece; widths that fill every slot keep the plain affine index
    const int p = PIECES % kThreads == 0 ? tid + kThreads * u : min(tid + kThreads * u, PIECES - 1);
    l_row[u] = p / (N / 8);
    l_col[u] = (p % (N / 8)) * 8;
  }
  u32x4 qreg[SLOTS], greg[SLOTS];
  float stat = 0.0f;  // threads 0..63 carry L of one query of the chunk, threads 64..127 carry D
  auto fetch = [&](int qc) {
    const int base = min(qc, qc_hi) * AB_KC;
#pragma unroll
    for (int u = 0; u < SLOTS; ++u) {
      const int r = min(base + l_row[u], M - 1);
      qreg[u] = *reinterpret_cast<const u32x4 *>(Qb + (int64_t)r * qsr + l_col[u]);
      greg[u] = *reinterpret_cast<const u32x4 *>(Gb + (int64_t)r * gsr + l_col[u]);
    }
    const int r = min(base + (tid & 63), M - 1);
    stat = (tid < 64 ? Lb : Db)[r];
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int u = 0; u < SLOTS; ++u) {
      *reinterpret_cast<u32x4 *>(&q_lds[buf][l_row[u] * TS + l_col[u]]) = qreg[u];
      *reinterpret_cast<u32x4 *>(&g_lds[buf][l_row[u] * TS + l_col[u]]) = greg[u];
    }
    if (tid < 64) l_lds[buf][tid] = stat * 1.4426950408889634f;
    else if (tid < 128) d_lds[buf][tid - 64] = stat * scale;
  };

  f32x16 dk[NB], dv[NB];
#pragma unroll
  for (int hb = 0; hb < NB; ++hb)
#pragma unroll
    for (int v = 0; v < 16; ++v) dk[hb][v] = 0.0f, dv[hb][v] = 0.0f;
  const float ninf = -__builtin_huge_valf();

  auto block = [&](int buf, int qb, int r0, auto edge) {
    constexpr bool EDGE = decltype(edge)::value;
    f32x16 s, dp;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = 0.0f, dp[v] = 0.0f;
    const int at = (32 * qb + (lane & 31)) * TS + 8 * half;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      s = Mma<T>::run(*reinterpret_cast<const u32x4 *>(&q_lds[buf][at + 16 * ks]), kf[ks], s);
      dp = Mma<T>::run(*reinterpret_cast<const u32x4 *>(&g_lds[buf][at + 16 * ks]), vf[ks], dp);
    }
    // accumulator v of this lane: query r0 + 8 (v / 4) + 4 half + v % 4, key kj
    if (EDGE) {
      const int d0 = r0 + 4 * half - kj;  // query - key at offset 0; valid offsets: first..last
      const int first = -w - d0, last = min(w - d0, M - 1 - r0 - 4 * half);
      const int origin = last < first ? 0x100000 : first;
      const unsigned span = last < first ? 0u : (unsigned)(last - first);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int ofs = 8 * (v / 4) + v % 4;
        s[v] = (unsigned)(ofs - origin) <= span ? s[v] : ninf;
      }
    }
    float p[16], ds[16];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 l2 = *reinterpret_cast<const f32x4 *>(&l_lds[buf][32 * qb + 8 * g + 4 * half]);
      const f32x4 dl = *reinterpret_cast<const f32x4 *>(&d_lds[buf][32 * qb + 8 * g + 4 * half]);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int v = 4 * g + r;
        p[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], c, -l2[r]));
        ds[v] = p[v] * __builtin_fmaf(dp[v], scale, -dl[r]);
      }
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const u32x4 pf = pack8<T>(p + 8 * t), dsf = pack8<T>(ds + 8 * t);
#pragma unroll
      for (int hb = 0; hb < NB; ++hb) {
        dv[hb] = Mma<T>::run(lds_tr_split(g_lds[buf], TS, 32 * qb + 16 * t, 32 * hb, lane), pf, dv[hb]);
        dk[hb] = Mma<T>::run(lds_tr_split(q_lds[buf], TS, 32 * qb + 16 * t, 32 * hb, lane), dsf, dk[hb]);
      }
    }
  };

  fetch(qc_lo);
  stash(0);
  __syncthreads();
  for (int qc = qc_lo; qc <= qc_hi; ++qc) {
    const int buf = (qc - qc_lo) & 1;
    fetch(qc + 1);
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const int r0 = qc * AB_KC + 32 * qb;
      if (r0 + 31 < kw0 - w || r0 > kw0 + 31 + w || r0 >= M) continue;  // wave-uniform
      const bool interior = r0 >= kw0 + 31 - w && r0 + 31 <= kw0 + w && r0 + 31 < M;
      if (interior)
        block(buf, qb, r0, std::false_type());
      else
        block(buf, qb, r0, std::true_type());
    }
    stash(buf ^ 1);
    __syncthreads();
  }
  // every wave is past the last barrier: the query buffers are free and stage the result rows;
  // either output may be absent (gradient not requested)
  static_assert(4 * RowStage<NB>::ELEMS <= 2 * AB_KC * TS, "the four staging areas must fit the query buffers");
  uint16_t *stage = &q_lds[0][0] + wave * RowStage<NB>::ELEMS;
  if (dK != nullptr) store_wave_rows<T, NB>(stage, dk, 1.0f, dK + (int64_t)b * dksb, dksr, kw0, M, N, lane);
  if (dV != nullptr) store_wave_rows<T, NB>(stage, dv, 1.0f, dV + (int64_t)b * dvsb, dvsr, kw0, M, N, lane);
}


// ---------------------------------------------------------------------------------------------
// N = 64 and N = 128: the streamed tiles go from memory straight into LDS
// ---------------------------------------------------------------------------------------------
// Same arithmetic as the two kernels above, organised like attention_forward_dma_kernel
// (wm_attention.hip): swizzled tiles filled by buffer loads with the lds modifier, requested DEPTH
// chunks ahead and counted by the kernel itself; scalar control flow; one branch-free loop for the
// chunks that lie wholly inside a wavefront's band and a general one for the chunks at its edges.
// The workspace holds two float32 values per row: -D = -sum_h dO * O at [b * M + i] (negated: the dP
// accumulators of the key kernel start from it) and the row's log-sum-exp in log2 units at
// [B * M + b * M + i]; the query kernel writes both, the key kernel streams both.  dS is formed
// without the factor `scale`, which multiplies the finished dQ and dK.
constexpr float kLog2e = 1.4426950408889634f;

template <int NK>
struct BwdTile {
  // tile rows of 128 bytes (N <= 64) or 256 bytes; pieces of a row beyond column N are never fetched
  static constexpr int N = 16 * NK, NB = (NK + 1) / 2, ROWB = NK <= 4 ? 128 : 256, PPR = ROWB / 16, TILE = AB_KC * ROWB / 2;
  // byte offset of the lane's piece for the loads of a chunk (dma_chunk), out of range for pieces beyond N
  static __device__ __forceinline__ uint32_t load_offset(int wave, int lane, int64_t row_stride) {
    const int slot = 64 * wave + lane;
    return ((slot % PPR) ^ swz<PPR>(slot / PPR)) < N / 8 ? dma_lane_offset<PPR>(wave, lane, row_stride) : 0x80000000u;
  }
  static constexpr int STAGES = NK <= 4 ? 3 : 2, DEPTH = STAGES - 1;
  typedef s16x4 __attribute__((address_space(3))) * lds_tr_ptr;
  // byte offsets inside a tile for the two ways a tile is read (see attention_forward_dma_kernel)
  static __device__ __forceinline__ uint32_t row_at(int lane) {
    const int r32 = lane & 31, half = lane >> 5;
    return (uint32_t)(r32 * ROWB + ((half ^ swz<PPR>(r32)) << 4));
  }
  static __device__ __forceinline__ uint32_t tr_at(int lane) {
    const int s16 = lane & 15, grp = lane >> 4, rowl = 4 * (grp >> 1) + (s16 >> 2);
    return (uint32_t)(rowl * ROWB + (((2 * (grp & 1) + ((s16 & 3) >> 1)) ^ swz<PPR>(rowl)) << 4) + 8 * (s16 & 1));
  }
  // rows 32 blk + lane % 32 of the tile, pieces 2 ks + half: A operand of a product contracted over N
  static __device__ __forceinline__ u32x4 rows(const uint16_t *tile, uint32_t at, int blk, int ks) {
    return *reinterpret_cast<const u32x4 *>(reinterpret_cast<const char *>(tile) + 32 * blk * ROWB + (at ^ (32 * ks)));
  }
  // columns 32 hb .. + 31 of rows 32 blk + 16 t .. + 15, transposed: A operand of a product contracted over rows
  static __device__ __forceinline__ u32x4 cols(const uint16_t *tile, uint32_t at, int blk, int t, int hb) {
    const char *p = reinterpret_cast<const char *>(tile) + (32 * blk + 16 * t) * ROWB;
    const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(p + (at ^ (64 * hb)))));
    const u32x2 hi = __builtin_bit_cast(  // eight rows further down the swizzle differs in bit 1
        u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(p + 8 * ROWB + (at ^ 32 ^ (64 * hb)))));
    const u32x4 r = {lo[0], lo[1], hi[0], hi[1]};
    return r;
  }
};


// D and the log-sum-exp in log2 units for the key kernel when grad_q is not wanted.
template <typename T, int NK>
__global__ __launch_bounds__(kThreads) void attention_backward_stats_kernel(
    const uint16_t *__restrict__ O, const uint16_t *__restrict__ dO, const float *__restrict__ L, float *__restrict__ D,
    int B, int M, int nblk, int64_t osb, int64_t osr, int64_t gsb, int64_t gsr) {
  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int lane = threadIdx.x & 63, half = lane >> 5;
  const int qi = blk * AB_TM + 32 * (threadIdx.x >> 6) + (lane & 31);
  const bool q_ok = qi < M;
  const uint16_t *gr = dO + (int64_t)b * gsb + (int64_t)qi * gsr + 8 * half;
  const uint16_t *orow = O + (int64_t)b * osb + (int64_t)qi * osr + 8 * half;
  float delta = 0.0f;
#pragma unroll
  for (int ks = 0; ks < NK; ++ks)
    delta += dot8<T>(load_row_chunk(gr + 16 * ks, dO, q_ok), load_row_chunk(orow + 16 * ks, O, q_ok));
  delta = halves_sum(delta);
  if (q_ok && half == 0) {
    D[(int64_t)b * M + qi] = -delta;
    D[((int64_t)B + b) * M + qi] = L[(int64_t)b * M + qi] * kLog2e;
  }
}

// (Three workgroups per CU up to N = 64: the kernel needs about 157 registers.  Forced into the 128 of a
// fourth workgroup it spills 35 of them and takes 237 instead of 104 us at B96 M4096 N64 w256; with
// three workgroups two stages do as well as three, 101 against 104 us, and are what it uses.)
template <typename T, int NK>
__global__ __launch_bounds__(kThreads, NK <= 4 ? 3 : 2) void attention_backward_query_dma_kernel(
    const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
    const uint16_t *__restrict__ O, const uint16_t *__restrict__ dO, const float *__restrict__ L,
    uint16_t *__restrict__ dQ, float *__restrict__ D, int B, int M, int w, int nblk, float scale, int64_t qsb,
    int64_t qsr, int64_t ksb, int64_t ksr, int64_t vsb, int64_t vsr, int64_t osb, int64_t osr, int64_t gsb, int64_t gsr,
    int64_t dqsb, int64_t dqsr) {
  typedef BwdTile<NK> TL;
  constexpr int N = TL::N, NB = TL::NB, PPR = TL::PPR, ROWB = TL::ROWB, TILE = TL::TILE;
  constexpr int STAGES = 2, DEPTH = STAGES - 1;
  constexpr int LOADS = 2 * (PPR / 4);  // loads per wavefront and chunk (K and V)
  __shared__ __attribute__((aligned(1024))) uint16_t kv_lds[2 * STAGES][TILE];  // key tiles, then value tiles
  uint16_t (*const k_lds)[TILE] = kv_lds, (*const v_lds)[TILE] = kv_lds + STAGES;

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i0 = blk * AB_TM;
  const int qw0 = i0 + 32 * wave;  // scalar
  const int qi = qw0 + (lane & 31);
  const bool q_ok = qi < M;
  const float c = scale * kLog2e;

  const u32x4 k_rsrc = make_rsrc(K + (int64_t)b * ksb, (uint32_t)((M - 1) * ksr * 2 + 2 * N));
  const u32x4 v_rsrc = make_rsrc(V + (int64_t)b * vsb, (uint32_t)((M - 1) * vsr * 2 + 2 * N));
  const uint32_t k_voff = TL::load_offset(wave, lane, ksr), v_voff = TL::load_offset(wave, lane, vsr);
  const uint32_t k_step = (uint32_t)(256 / PPR * ksr * 2), v_step = (uint32_t)(256 / PPR * vsr * 2);
  const uint32_t k_chunk = (uint32_t)(AB_KC * ksr * 2), v_chunk = (uint32_t)(AB_KC * vsr * 2);
  auto request = [&](int kc, int stage) {
    dma_chunk<PPR>(k_rsrc, k_lds[stage], wave, k_voff, k_chunk * (uint32_t)kc, k_step);
    dma_chunk<PPR>(v_rsrc, v_lds[stage], wave, v_voff, v_chunk * (uint32_t)kc, v_step);
  };
  const int kc_lo = max(i0 - w, 0) / AB_KC;
  const int kc_hi = min(i0 + AB_TM - 1 + w, M - 1) / AB_KC;
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) request(kc_lo + d, d);

  // stationary side in registers: the query rows and their upstream gradient rows (B operands)
  u32x4 qf[NK], gf[NK];
  float delta = 0.0f;
  {
    const uint16_t *qr = Q + (int64_t)b * qsb + (int64_t)qi * qsr + 8 * half;
    const uint16_t *gr = dO + (int64_t)b * gsb + (int64_t)qi * gsr + 8 * half;
    const uint16_t *orow = O + (int64_t)b * osb + (int64_t)qi * osr + 8 * half;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      qf[ks] = load_row_chunk(qr + 16 * ks, Q, q_ok);
      gf[ks] = load_row_chunk(gr + 16 * ks, dO, q_ok);
      delta += dot8<T>(gf[ks], load_row_chunk(orow + 16 * ks, O, q_ok));
    }
  }
  delta = halves_sum(delta);
  const float l2 = (q_ok ? L[(int64_t)b * M + qi] : 0.0f) * kLog2e;
  if (q_ok && half == 0) {
    D[(int64_t)b * M + qi] = -delta;  // the key kernel's dP accumulators start from it
    D[((int64_t)B + b) * M + qi] = l2;
  }

  const uint32_t row_at = TL::row_at(lane), tr_at = TL::tr_at(lane);
  f32x16 dq[NB];
#pragma unroll
  for (int hb = 0; hb < NB; ++hb)
#pragma unroll
    for (int v = 0; v < 16; ++v) dq[hb][v] = 0.0f;
  const float ninf = -__builtin_huge_valf();

  // one block of 32 keys: S^T, dP^T, dS^T, dQ^T += K^T dS^T (LDS reads hoisted as in the key kernel below)
  auto block = [&](const uint16_t *kt, const uint16_t *vt, int kb, int c0, auto edge) {
    constexpr bool EDGE = decltype(edge)::value;
    f32x16 s, dp;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = 0.0f, dp[v] = 0.0f;
    u32x4 ka[NK], va[NK];
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) ka[ks] = TL::rows(kt, row_at, kb, ks), va[ks] = TL::rows(vt, row_at, kb, ks);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      s = Mma<T>::run(ka[ks], qf[ks], s);
      dp = Mma<T>::run(va[ks], gf[ks], dp);
    }
    u32x4 kc[2][NB];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int hb = 0; hb < NB; ++hb) kc[t][hb] = TL::cols(kt, tr_at, kb, t, hb);
    __builtin_amdgcn_sched_barrier(0);
    if (EDGE) {
      const int d0 = c0 + 4 * half - qi;  // key - query at offset 0; valid offsets: first..last
      const int first = -w - d0, last = min(w - d0, M - 1 - c0 - 4 * half);
      const int origin = last < first ? 0x100000 : first;
      const unsigned span = last < first ? 0u : (unsigned)(last - first);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int ofs = 8 * (v / 4) + v % 4;
        s[v] = (unsigned)(ofs - origin) <= span ? s[v] : ninf;
      }
    }
    float ds[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) ds[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], c, -l2)) * (dp[v] - delta);
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const u32x4 dsf = pack8<T>(ds + 8 * t);
#pragma unroll
      for (int hb = 0; hb < NB; ++hb) dq[hb] = Mma<T>::run(kc[t][hb], dsf, dq[hb]);
    }
  };

  int stage = 0;
  auto open_chunk = [&](int kc) {
    wait_vmcnt<(DEPTH - 1) * LOADS>();
    __builtin_amdgcn_s_barrier();
    int st = stage + DEPTH;
    st = st >= STAGES ? st - STAGES : st;
    request(kc + DEPTH, st);
  };
  auto close_chunk = [&]() { stage = stage + 1 == STAGES ? 0 : stage + 1; };
  auto edge_chunk = [&](int kc) {
    open_chunk(kc);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int cb = kc * AB_KC + 32 * kb;
      if (cb + 31 < qw0 - w || cb > qw0 + 31 + w || cb >= M) continue;  // scalar
      // one instantiation for every block of an edge chunk, masked whether it needs it or not: two
      // code paths that update the accumulators make the compiler copy them between register sets
      block(k_lds[stage], v_lds[stage], kb, cb, std::true_type());
    }
    close_chunk();
  };
  const int pair_lo = max(kc_lo, (qw0 + 31 - w + 63) >> 6);
  const int pair_hi = min(kc_hi, (min(qw0 + w, M - 1) - 63) >> 6);
  const int lead_end = pair_lo <= pair_hi ? pair_lo : kc_hi + 1;
  int kc = kc_lo;
  for (; kc < lead_end; ++kc) edge_chunk(kc);
  for (; kc <= pair_hi; ++kc) {
    open_chunk(kc);
    block(k_lds[stage], v_lds[stage], 0, 0, std::false_type());
    block(k_lds[stage], v_lds[stage], 1, 0, std::false_type());
    close_chunk();
  }
  for (; kc <= kc_hi; ++kc) edge_chunk(kc);

  wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  static_assert(4 * RowStage<NB>::ELEMS <= 2 * STAGES * TILE, "the four staging areas must fit the tiles");
  store_wave_rows<T, NB>(&k_lds[0][0] + wave * RowStage<NB>::ELEMS, dq, scale, dQ + (int64_t)b * dqsb, dqsr, qw0, M, N,
                         lane);
}

template <typename T, int NK>
__global__ __launch_bounds__(kThreads, NK <= 4 ? 2 : 1) void attention_backward_key_dma_kernel(
    const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
    const uint16_t *__restrict__ dO, const float *__restrict__ D, uint16_t *__restrict__ dK,
    uint16_t *__restrict__ dV, int B, int M, int w, int nblk, float scale, int64_t qsb, int64_t qsr, int64_t ksb,
    int64_t ksr, int64_t vsb, int64_t vsr, int64_t gsb, int64_t gsr, int64_t dksb, int64_t dksr, int64_t dvsb,
    int64_t dvsr) {
  typedef BwdTile<NK> TL;
  constexpr int N = TL::N, NB = TL::NB, PPR = TL::PPR, ROWB = TL::ROWB, TILE = TL::TILE;
  constexpr int STAGES = TL::STAGES, DEPTH = TL::DEPTH;
  constexpr int LOADS = 2 * (PPR / 4) + 1;  // loads per wavefront and chunk: Q, dO and one row statistic
  __shared__ __attribute__((aligned(1024))) uint16_t q_lds[STAGES][TILE];
  __shared__ __attribute__((aligned(1024))) uint16_t g_lds[STAGES][TILE];
  __shared__ __attribute__((aligned(256))) float stat_lds[STAGES][2][AB_KC];  // [0] -D, [1] log-sum-exp (log2 units)

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c0 = blk * AB_TM;
  const int kw0 = c0 + 32 * wave;  // first key of this wavefront (scalar)
  const int kj = kw0 + (lane & 31);
  const bool k_ok = kj < M;
  const float c = scale * kLog2e;

  const u32x4 q_rsrc = make_rsrc(Q + (int64_t)b * qsb, (uint32_t)((M - 1) * qsr * 2 + 2 * N));
  const u32x4 g_rsrc = make_rsrc(dO + (int64_t)b * gsb, (uint32_t)((M - 1) * gsr * 2 + 2 * N));
  // waves 0 and 2 fetch D, waves 1 and 3 the log-sum-exp (twice the same 256 bytes each: every
  // wavefront then has the same number of loads in flight, which is what the waits count)
  const u32x4 s_rsrc = make_rsrc(D + ((int64_t)(wave & 1) * B + b) * M, (uint32_t)(M * 4));
  const uint32_t q_voff = TL::load_offset(wave, lane, qsr), g_voff = TL::load_offset(wave, lane, gsr);
  const uint32_t q_step = (uint32_t)(256 / PPR * qsr * 2), g_step = (uint32_t)(256 / PPR * gsr * 2);
  const uint32_t q_chunk = (uint32_t)(AB_KC * qsr * 2), g_chunk = (uint32_t)(AB_KC * gsr * 2);
  auto request = [&](int qc, int stage) {
    dma_chunk<PPR>(q_rsrc, q_lds[stage], wave, q_voff, q_chunk * (uint32_t)qc, q_step);
    dma_chunk<PPR>(g_rsrc, g_lds[stage], wave, g_voff, g_chunk * (uint32_t)qc, g_step);
    dma_dword(s_rsrc, lds_address(stat_lds[stage][wave & 1]), 4 * lane, (uint32_t)(qc * AB_KC * 4));
  };
  const int qc_lo = max(c0 - w, 0) / AB_KC;
  const int qc_hi = min(c0 + AB_TM - 1 + w, M - 1) / AB_KC;
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) request(qc_lo + d, d);

  u32x4 kf[NK], vf[NK];
  {
    const uint16_t *kr = K + (int64_t)b * ksb + (int64_t)kj * ksr + 8 * half;
    const uint16_t *vr = V + (int64_t)b * vsb + (int64_t)kj * vsr + 8 * half;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      kf[ks] = load_row_chunk(kr + 16 * ks, K, k_ok);
      vf[ks] = load_row_chunk(vr + 16 * ks, V, k_ok);
    }
  }

  const uint32_t row_at = TL::row_at(lane), tr_at = TL::tr_at(lane);
  f32x16 dk[NB], dv[NB];
#pragma unroll
  for (int hb = 0; hb < NB; ++hb)
#pragma unroll
    for (int v = 0; v < 16; ++v) dk[hb][v] = 0.0f, dv[hb][v] = 0.0f;
  const float ninf = -__builtin_huge_valf();

  // one block of 32 queries: S, dP, then dV^T += dO^T P and dK^T += Q^T dS.  The LDS reads of a
  // phase are all issued before its first product (left to itself the compiler reuses one register
  // set for consecutive operands, which puts one LDS latency in front of every MFMA), and those of
  // the second phase are in flight while the exponentials run.
  auto block = [&](const uint16_t *qt, const uint16_t *gt, const float *st, int qb, int r0, auto edge) {
    constexpr bool EDGE = decltype(edge)::value;
    f32x16 s, dp;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = 0.0f;
    u32x4 qa[NK], ga[NK];
    f32x4 l2[4];
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) qa[ks] = TL::rows(qt, row_at, qb, ks), ga[ks] = TL::rows(gt, row_at, qb, ks);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      // the dP accumulator starts from -D of its sixteen queries: dP - D comes out of the matrix pipe
      const f32x4 nd = *reinterpret_cast<const f32x4 *>(st + 32 * qb + 8 * g + 4 * half);
      dp[4 * g] = nd[0], dp[4 * g + 1] = nd[1], dp[4 * g + 2] = nd[2], dp[4 * g + 3] = nd[3];
      l2[g] = *reinterpret_cast<const f32x4 *>(st + AB_KC + 32 * qb + 8 * g + 4 * half);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      s = Mma<T>::run(qa[ks], kf[ks], s);
      dp = Mma<T>::run(ga[ks], vf[ks], dp);
    }
    u32x4 gc[2][NB], qc[2][NB];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int hb = 0; hb < NB; ++hb) gc[t][hb] = TL::cols(gt, tr_at, qb, t, hb), qc[t][hb] = TL::cols(qt, tr_at, qb, t, hb);
    __builtin_amdgcn_sched_barrier(0);
    // accumulator v of this lane: query r0 + 8 (v / 4) + 4 half + v % 4, key kj
    if (EDGE) {
      const int d0 = r0 + 4 * half - kj;  // query - key at offset 0; valid offsets: first..last
      const int first = -w - d0, last = min(w - d0, M - 1 - r0 - 4 * half);
      const int origin = last < first ? 0x100000 : first;
      const unsigned span = last < first ? 0u : (unsigned)(last - first);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int ofs = 8 * (v / 4) + v % 4;
        s[v] = (unsigned)(ofs - origin) <= span ? s[v] : ninf;
      }
    }
    float p[16], ds[16];
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int v = 4 * g + r;
        p[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], c, -l2[g][r]));
        ds[v] = p[v] * dp[v];
      }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const u32x4 pf = pack8<T>(p + 8 * t), dsf = pack8<T>(ds + 8 * t);
#pragma unroll
      for (int hb = 0; hb < NB; ++hb) {
        dv[hb] = Mma<T>::run(gc[t][hb], pf, dv[hb]);
        dk[hb] = Mma<T>::run(qc[t][hb], dsf, dk[hb]);
      }
    }
  };

  int stage = 0;
  auto open_chunk = [&](int qc) {
    wait_vmcnt<(DEPTH - 1) * LOADS>();
    __builtin_amdgcn_s_barrier();
    int st = stage + DEPTH;
    st = st >= STAGES ? st - STAGES : st;
    request(qc + DEPTH, st);
  };
  auto close_chunk = [&]() { stage = stage + 1 == STAGES ? 0 : stage + 1; };
  auto edge_chunk = [&](int qc) {
    open_chunk(qc);
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const int rb = qc * AB_KC + 32 * qb;
      if (rb + 31 < kw0 - w || rb > kw0 + 31 + w || rb >= M) continue;  // scalar
      block(q_lds[stage], g_lds[stage], stat_lds[stage][0], qb, rb, std::true_type());  // see the query kernel
    }
    close_chunk();
  };
  const int pair_lo = max(qc_lo, (kw0 + 31 - w + 63) >> 6);
  const int pair_hi = min(qc_hi, (min(kw0 + w, M - 1) - 63) >> 6);
  const int lead_end = pair_lo <= pair_hi ? pair_lo : qc_hi + 1;
  int qc = qc_lo;
  for (; qc < lead_end; ++qc) edge_chunk(qc);
  for (; qc <= pair_hi; ++qc) {
    open_chunk(qc);
    block(q_lds[stage], g_lds[stage], stat_lds[stage][0], 0, 0, std::false_type());
    block(q_lds[stage], g_lds[stage], stat_lds[stage][0], 1, 0, std::false_type());
    close_chunk();
  }
  for (; qc <= qc_hi; ++qc) edge_chunk(qc);

  wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  static_assert(4 * RowStage<NB>::ELEMS <= STAGES * TILE, "the four staging areas must fit the query tiles");
  uint16_t *stage_rows = &q_lds[0][0] + wave * RowStage<NB>::ELEMS;
  if (dK != nullptr) store_wave_rows<T, NB>(stage_rows, dk, scale, dK + (int64_t)b * dksb, dksr, kw0, M, N, lane);
  if (dV != nullptr) store_wave_rows<T, NB>(stage_rows, dv, 1.0f, dV + (int64_t)b * dvsb, dvsr, kw0, M, N, lane);
}

// ---------------------------------------------------------------------------------------------
// Narrow windows (w <= 16 (NKB - 1), N <= 64): one kernel for all three gradients
// ---------------------------------------------------------------------------------------------
// With a band of at most 65 entries the two kernels above read q, k, v and dO twice and exchange D
// through memory.  Here a workgroup owns 128 rows both as keys and as queries; the rows it needs
// from its neighbours (w on either side) come with the tiles:
//   1. Q and dO rows [i0 - w, i0 + 127 + w] go straight into two LDS tiles (rows further out, up to
//      the tile's 16 (NKB - 1) on either side, are not fetched); D = dO . O and the log-sum-exp of
//      those rows go into a small LDS array; the wavefront's own k and v rows into registers.
//   2. As keys: S, dP against the 32 NKB query rows a wavefront's keys can reach, dV^T += dO^T P,
//      dK^T += Q^T dS; dK and dV leave through LDS as whole lines.
//   3. K and V rows replace Q and dO in the two tiles, the wavefront's own q and dO rows go into
//      registers; as queries: S^T, dP^T, dQ^T += K^T dS^T; dQ leaves the same way.
// Memory sees q, k, v, dO, O once each (plus the halo, which the neighbouring workgroup has
// usually just brought into the L2) and dQ, dK, dV once: nothing else bounds this kernel.
template <typename T, int NK, int NKB>
__global__ __launch_bounds__(kThreads, NKB >= 4 || (NK >= 3 && NKB == 3) ? 2 : 3) void attention_backward_narrow_kernel(
    const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
    const uint16_t *__restrict__ O, const uint16_t *__restrict__ dO, const float *__restrict__ L,
    uint16_t *__restrict__ dQ, uint16_t *__restrict__ dK, uint16_t *__restrict__ dV, int B, int M, int w, int nblk,
    float scale, int64_t qsb, int64_t qsr, int64_t ksb, int64_t ksr, int64_t vsb, int64_t vsr, int64_t osb, int64_t osr,
    int64_t gsb, int64_t gsr, int64_t dqsb, int64_t dqsr, int64_t dksb, int64_t dksr, int64_t dvsb, int64_t dvsr) {
  static_assert(NK <= 4, "rows of 128 bytes: two tiles and the staging must fit 64 KB of LDS");
  constexpr int N = 16 * NK, NB = (NK + 1) / 2;
  constexpr int PADW = 16 * (NKB - 1);     // tile rows before the first and after the last own row
  constexpr int ROWS = AB_TM + 2 * PADW;   // rows of a tile
  typedef LdsTile<ROWS, 8> TL;
  constexpr int LOADS = TL::LOADS;
  // Two tiles (Q then K; dO then V) and the row statistics ([0] D, [1] log-sum-exp in log2 units).  With
  // five row blocks per wavefront they take 66 KB, more than a kernel can declare: that instantiation
  // gets them as dynamic LDS, which the launcher asks for (narrow_lds_bytes).
  constexpr bool DYN = NKB >= 5;
  __shared__ __attribute__((aligned(1024))) uint16_t tiles_declared[DYN ? 8 : 2 * TL::ELEMS];
  __shared__ __attribute__((aligned(16))) float stat_declared[DYN ? 4 : 2 * ROWS];
  extern __shared__ __attribute__((aligned(1024))) unsigned char narrow_dynamic_lds[];
  uint16_t *const tile_a = DYN ? reinterpret_cast<uint16_t *>(narrow_dynamic_lds) : tiles_declared;
  uint16_t *const tile_b = tile_a + TL::ELEMS;
  float(*const stat)[ROWS] = reinterpret_cast<float(*)[ROWS]>(
      DYN ? reinterpret_cast<float *>(narrow_dynamic_lds + 4 * TL::ELEMS) : stat_declared);
  static_assert(4 * RowStage<NB>::ELEMS <= TL::ELEMS, "the four staging areas must fit one tile");

  int b, blk;
  if (!decode_block(nblk, B, &b, &blk)) return;
  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i0 = blk * AB_TM;
  const int t0 = i0 - PADW;         // sequence row of tile row 0 (negative in the first workgroup)
  const int rw0 = i0 + 32 * wave;   // first own row of this wavefront (scalar)
  const int ri = rw0 + (lane & 31);
  const bool r_ok = ri < M;
  const float c = scale * kLog2e;
  const int need_lo = max(i0 - w, 0), need_hi = min(i0 + AB_TM - 1 + w, M - 1);  // rows anybody reads

  // one tile from a tensor: tile row r = sequence row t0 + r; rows nobody reads and pieces beyond
  // column N are requested out of range (zeros, no traffic)
  const int piece = TL::load_piece(wave, lane);
  auto request = [&](const uint16_t *base, int64_t sr, const uint16_t *tile) __attribute__((always_inline)) {
    const u32x4 rsrc = make_rsrc(base, (uint32_t)((M - 1) * sr * 2 + 2 * N));
    const uint32_t lds = lds_address(tile) + 1024 * wave;
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
      const int row = t0 + TL::load_row(wave, lane, j);
      const bool wanted = row >= need_lo && row <= need_hi && piece < N / 8;
      dma_piece(rsrc, lds + 4096 * j, wanted ? (uint32_t)(row * sr * 2 + piece * 16) : 0x80000000u, 0);
    }
  };
  request(Q + (int64_t)b * qsb, qsr, tile_a);
  request(dO + (int64_t)b * gsb, gsr, tile_b);

  const uint32_t row_at = TL::row_at(lane), tr_at = TL::tr_at(lane);
  const float ninf = -__builtin_huge_valf();
  const int r32 = lane & 31;
  const bool want_kv = dK != nullptr || dV != nullptr;
  // a group of 32 tile rows that starts at row `first` (a multiple of 16) as B operand: row lane % 32,
  // pieces 2 ks + lane / 32
  auto own_rows = [&](const uint16_t *tile, int first, uint32_t at, int ks) __attribute__((always_inline)) {
    return *reinterpret_cast<const u32x4 *>(reinterpret_cast<const char *>(tile) + first * TL::ROWB + (at ^ (32 * ks)));
  };

  // For D = dO . O the rows of O come in operand layout (lane pair per row) and meet the rows of dO
  // in the tile: the wavefront's own 32 rows, and in the first and last wavefronts the rows before
  // and after the workgroup's own.
  const int own_first = PADW + 32 * wave;                            // tile row of the wavefront's first own row
  constexpr int HP = (PADW + 31) / 32;                               // wavefronts per side of the halo (32 rows each)
  const bool halo_wave = wave < HP || wave >= 4 - HP;                // scalar
  const int hp = wave < HP ? wave : wave - (4 - HP);
  const int halo_first = (wave < HP ? 0 : PADW + AB_TM) + 32 * hp;   // first halo row of this wavefront
  const int halo_rows = min(32, PADW - 32 * hp);
  const int h32 = r32 < halo_rows ? r32 : 0;                         // lanes beyond the halo repeat its first row
  const uint32_t halo_at = TL::row_at(32 * half + h32);
  u32x4 o_own[NK], o_halo[NK];
  float l_own, l_halo = 0.0f;
  {
    const int row = t0 + own_first + r32;
    const bool ok = row >= need_lo && row <= need_hi;
    const uint16_t *orow = O + (int64_t)b * osb + (int64_t)row * osr + 8 * half;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) o_own[ks] = load_row_chunk(orow + 16 * ks, O, ok);
    l_own = ok ? L[(int64_t)b * M + row] * kLog2e : 0.0f;
  }
  if (halo_wave) {
    const int row = t0 + halo_first + h32;
    const bool ok = row >= need_lo && row <= need_hi;
    const uint16_t *orow = O + (int64_t)b * osb + (int64_t)row * osr + 8 * half;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) o_halo[ks] = load_row_chunk(orow + 16 * ks, O, ok);
    l_halo = ok ? L[(int64_t)b * M + row] * kLog2e : 0.0f;
  }
  // own rows as keys: B operands of the first two products
  u32x4 kf[NK], vf[NK];
  if (want_kv) {
    const uint16_t *kr = K + (int64_t)b * ksb + (int64_t)ri * ksr + 8 * half;
    const uint16_t *vr = V + (int64_t)b * vsb + (int64_t)ri * vsr + 8 * half;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      kf[ks] = load_row_chunk(kr + 16 * ks, K, r_ok);
      vf[ks] = load_row_chunk(vr + 16 * ks, V, r_ok);
    }
  }
  wait_vmcnt<0>();
  __syncthreads();

  {
    float d = 0.0f;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) d += dot8<T>(own_rows(tile_b, own_first, row_at, ks), o_own[ks]);
    d = halves_sum(d);
    if (half == 0) stat[0][own_first + r32] = d, stat[1][own_first + r32] = l_own;
  }
  if (halo_wave) {
    float d = 0.0f;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) d += dot8<T>(own_rows(tile_b, halo_first, halo_at, ks), o_halo[ks]);
    d = halves_sum(d);
    if (half == 0 && r32 < halo_rows) stat[0][halo_first + r32] = d, stat[1][halo_first + r32] = l_halo;
  }
  __syncthreads();

  f32x16 dk[NB], dv[NB];
  if (want_kv) {
#pragma unroll
    for (int hb = 0; hb < NB; ++hb)
#pragma unroll
      for (int v = 0; v < 16; ++v) dk[hb][v] = 0.0f, dv[hb][v] = 0.0f;
#pragma unroll
    for (int j = 0; j < NKB; ++j) {
      const int rb = wave + j;          // 32-row block of the tiles
      const int r0 = t0 + 32 * rb;      // its first sequence row
      if (r0 + 31 < rw0 - w || r0 > rw0 + 31 + w || r0 >= M || r0 + 31 < 0) continue;  // scalar
      f32x16 s, dp;
#pragma unroll
      for (int v = 0; v < 16; ++v) s[v] = 0.0f, dp[v] = 0.0f;
      u32x4 qa[NK], ga[NK];
#pragma unroll
      for (int ks = 0; ks < NK; ++ks) qa[ks] = TL::rows(tile_a, row_at, rb, ks), ga[ks] = TL::rows(tile_b, row_at, rb, ks);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < NK; ++ks) {
        s = Mma<T>::run(qa[ks], kf[ks], s);
        dp = Mma<T>::run(ga[ks], vf[ks], dp);
      }
      {
        // accumulator v of this lane: query r0 + 4 half + 8 (v / 4) + v % 4, key ri
        const int d0 = r0 + 4 * half - ri;  // query - key at offset 0; valid offsets: first..last
        const int first = max(-w - d0, -(r0 + 4 * half)), last = min(w - d0, M - 1 - r0 - 4 * half);
        const int origin = last < first ? 0x100000 : first;
        const unsigned span = last < first ? 0u : (unsigned)(last - first);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int ofs = 8 * (v / 4) + v % 4;
          s[v] = (unsigned)(ofs - origin) <= span ? s[v] : ninf;
        }
      }
      // by halves of the block (16 query rows each): the operands of the second products and the row
      // statistics of a half are read when its turn comes, which keeps three workgroups on a CU
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        u32x4 gc[NB], qc[NB];
#pragma unroll
        for (int hb = 0; hb < NB; ++hb)
          gc[hb] = TL::cols(tile_b, tr_at, 32 * rb + 16 * t, hb), qc[hb] = TL::cols(tile_a, tr_at, 32 * rb + 16 * t, hb);
        float p[8], ds[8];
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          const f32x4 dl = *reinterpret_cast<const f32x4 *>(&stat[0][32 * rb + 16 * t + 8 * g + 4 * half]);
          const f32x4 l2 = *reinterpret_cast<const f32x4 *>(&stat[1][32 * rb + 16 * t + 8 * g + 4 * half]);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int v = 8 * t + 4 * g + r;
            p[4 * g + r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], c, -l2[r]));
            ds[4 * g + r] = p[4 * g + r] * (dp[v] - dl[r]);
          }
        }
        const u32x4 pf = pack8<T>(p), dsf = pack8<T>(ds);
#pragma unroll
        for (int hb = 0; hb < NB; ++hb) {
          dv[hb] = Mma<T>::run(gc[hb], pf, dv[hb]);
          dk[hb] = Mma<T>::run(qc[hb], dsf, dk[hb]);
        }
      }
    }
  }
  // own rows as queries: B operands of the other side, taken from the tiles before they go
  u32x4 qf[NK], gf[NK];
  float delta = 0.0f, lse2 = 0.0f;
  if (dQ != nullptr) {
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) qf[ks] = own_rows(tile_a, own_first, row_at, ks), gf[ks] = own_rows(tile_b, own_first, row_at, ks);
    delta = stat[0][own_first + r32], lse2 = stat[1][own_first + r32];
  }
  __syncthreads();  // nobody reads the tiles any more
  // K replaces Q while dK and dV leave through the other tile; V follows when those rows are out
  if (dQ != nullptr) request(K + (int64_t)b * ksb, ksr, tile_a);
  uint16_t *stage_rows = tile_b + wave * RowStage<NB>::ELEMS;
  if (dK != nullptr) store_wave_rows<T, NB>(stage_rows, dk, scale, dK + (int64_t)b * dksb, dksr, rw0, M, N, lane);
  if (dV != nullptr) store_wave_rows<T, NB>(stage_rows, dv, 1.0f, dV + (int64_t)b * dvsb, dvsr, rw0, M, N, lane);
  if (dQ == nullptr) return;
  __syncthreads();
  request(V + (int64_t)b * vsb, vsr, tile_b);
  f32x16 dq[NB];
#pragma unroll
  for (int hb = 0; hb < NB; ++hb)
#pragma unroll
    for (int v = 0; v < 16; ++v) dq[hb][v] = 0.0f;
  wait_vmcnt<0>();
  __syncthreads();
#pragma unroll
  for (int j = 0; j < NKB; ++j) {
    const int rb = wave + j;
    const int c0 = t0 + 32 * rb;  // first key of the block
    if (c0 + 31 < rw0 - w || c0 > rw0 + 31 + w || c0 >= M || c0 + 31 < 0) continue;  // scalar
    f32x16 s, dp;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = 0.0f, dp[v] = 0.0f;
    u32x4 ka[NK], va[NK];
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) ka[ks] = TL::rows(tile_a, row_at, rb, ks), va[ks] = TL::rows(tile_b, row_at, rb, ks);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      s = Mma<T>::run(ka[ks], qf[ks], s);
      dp = Mma<T>::run(va[ks], gf[ks], dp);
    }
    u32x4 kc[2][NB];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int hb = 0; hb < NB; ++hb) kc[t][hb] = TL::cols(tile_a, tr_at, 32 * rb + 16 * t, hb);
    __builtin_amdgcn_sched_barrier(0);
    {
      // accumulator v of this lane: key c0 + 4 half + 8 (v / 4) + v % 4, query ri
      const int d0 = c0 + 4 * half - ri;
      const int first = max(-w - d0, -(c0 + 4 * half)), last = min(w - d0, M - 1 - c0 - 4 * half);
      const int origin = last < first ? 0x100000 : first;
      const unsigned span = last < first ? 0u : (unsigned)(last - first);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int ofs = 8 * (v / 4) + v % 4;
        s[v] = (unsigned)(ofs - origin) <= span ? s[v] : ninf;
      }
    }
    float ds[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) ds[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], c, -lse2)) * (dp[v] - delta);
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const u32x4 dsf = pack8<T>(ds + 8 * t);
#pragma unroll
      for (int hb = 0; hb < NB; ++hb) dq[hb] = Mma<T>::run(kc[t][hb], dsf, dq[hb]);
    }
  }
  __syncthreads();
  store_wave_rows<T, NB>(tile_a + wave * RowStage<NB>::ELEMS, dq, scale, dQ + (int64_t)b * dqsb, dqsr, rw0, M, N, lane);
}

template <typename T, int NK>
hipError_t launch_backward(const Problem &p, const View &q, const View &k, const View &v, const View &o,
                           const View &go, const float *lse, float *delta, const View &gq, const View &gk,
                           const View &gv, double scale) {
  const int nblk = (int)((p.M + AB_TM - 1) / AB_TM);
  if (tiled_grid(p.B, nblk) > 0x7fffffff) return hipErrorInvalidValue;
  const dim3 grid((unsigned)tiled_grid(p.B, nblk)), block(kThreads);
  typedef const uint16_t *in_t;
  typedef uint16_t *out_t;
  {
    // the LDS-direct kernels address a batch element with 32-bit byte offsets
    const int64_t lim = 0x7fffffff;
    bool fits = !(p.flags & WM_FLAG_NO_LDS_DIRECT) && (p.M + 3 * AB_KC) * 4 < lim;
    for (const View *t : {&q, &k, &v, &go}) fits = fits && t->sr > 0 && (p.M + 3 * AB_KC) * t->sr * 2 < lim;
    if constexpr (NK <= 4) {
      // narrow windows: one kernel for all three gradients (two row blocks per wavefront up to w = 16, three up
      // to 32, four up to 48, five up to 64 where it still pays: B96 M16384 N64 w = 64: 490 against 555 us for
      // the two kernels, N = 48: 552 against 592, N = 32: 633 against 603)
      if (fits && (p.w <= 48 || (p.w <= 64 && NK >= 3)) && !(p.flags & WM_FLAG_NO_NARROW_BAND)) {
#define WM_ABN(NKB, LDS_BYTES)                                                                                        \
  hipLaunchKernelGGL((attention_backward_narrow_kernel<T, NK, NKB>), grid, block, LDS_BYTES, p.stream, (in_t)q.data,  \
                     (in_t)k.data, (in_t)v.data, (in_t)o.data, (in_t)go.data, lse, (out_t)gq.data, (out_t)gk.data,    \
                     (out_t)gv.data, (int)p.B, (int)p.M, (int)p.w, nblk, (float)scale, q.sb, q.sr, k.sb, k.sr, v.sb,  \
                     v.sr, o.sb, o.sr, go.sb, go.sr, gq.sb, gq.sr, gk.sb, gk.sr, gv.sb, gv.sr)
        if (p.w <= 16) {
          WM_ABN(2, 0);
          return hipGetLastError();
        } else if (p.w <= 32) {
          WM_ABN(3, 0);
          return hipGetLastError();
        } else if (p.w <= 48) {
          WM_ABN(4, 0);
          return hipGetLastError();
        } else {
          // 66 KB of LDS: above what a kernel gets without asking (the call changes an attribute of the
          // function, it allocates nothing); if the runtime refuses, the two kernels below take over
          constexpr int rows = AB_TM + 2 * 64, bytes = 2 * rows * 128 + 2 * rows * 4;
          const auto kernel = attention_backward_narrow_kernel<T, NK, 5>;
          if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  bytes) == hipSuccess) {
            WM_ABN(5, bytes);
            return hipGetLastError();
          }
          (void)hipGetLastError();
        }
#undef WM_ABN
      }
    }
    if (fits) {
      if (gq.data != nullptr)
        hipLaunchKernelGGL((attention_backward_query_dma_kernel<T, NK>), grid, block, 0, p.stream, (in_t)q.data,
                           (in_t)k.data, (in_t)v.data, (in_t)o.data, (in_t)go.data, lse, (out_t)gq.data, delta, (int)p.B,
                           (int)p.M, (int)p.w, nblk, (float)scale, q.sb, q.sr, k.sb, k.sr, v.sb, v.sr, o.sb, o.sr, go.sb,
                           go.sr, gq.sb, gq.sr);
      else
        hipLaunchKernelGGL((attention_backward_stats_kernel<T, NK>), grid, block, 0, p.stream, (in_t)o.data,
                           (in_t)go.data, lse, delta, (int)p.B, (int)p.M, nblk, o.sb, o.sr, go.sb, go.sr);
      hipError_t err = hipGetLastError();
      if (err != hipSuccess || (gk.data == nullptr && gv.data == nullptr)) return err;
      hipLaunchKernelGGL((attention_backward_key_dma_kernel<T, NK>), grid, block, 0, p.stream, (in_t)q.data,
                         (in_t)k.data, (in_t)v.data, (in_t)go.data, (const float *)delta, (out_t)gk.data,
                         (out_t)gv.data, (int)p.B, (int)p.M, (int)p.w, nblk, (float)scale, q.sb, q.sr, k.sb, k.sr, v.sb,
                         v.sr, go.sb, go.sr, gk.sb, gk.sr, gv.sb, gv.sr);
      return hipGetLastError();
    }
  }
#define WM_ABQ(WITH_DQ)                                                                                              \
  hipLaunchKernelGGL((attention_backward_query_kernel<T, NK, WITH_DQ>), grid, block, 0, p.stream, (in_t)q.data,      \
                     (in_t)k.data, (in_t)v.data, (in_t)o.data, (in_t)go.data, lse, (out_t)gq.data, delta, (int)p.B,  \
                     (int)p.M, (int)p.w, nblk, (float)scale, q.sb, q.sr, k.sb, k.sr, v.sb, v.sr, o.sb, o.sr, go.sb,  \
                     go.sr, gq.sb, gq.sr)
  // D is needed by the key kernel even when grad_q is not: the query kernel then stops after writing it
  if (gq.data != nullptr)
    WM_ABQ(true);
  else if (gk.data != nullptr || gv.data != nullptr)
    WM_ABQ(false);
#undef WM_ABQ
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  if (gk.data == nullptr && gv.data == nullptr) return hipSuccess;
  hipLaunchKernelGGL((attention_backward_key_kernel<T, NK>), grid, block, 0, p.stream, (in_t)q.data, (in_t)k.data,
                     (in_t)v.data, (in_t)go.data, lse, (const float *)delta, (out_t)gk.data, (out_t)gv.data, (int)p.B,
                     (int)p.M, (int)p.w, nblk, (float)scale, q.sb, q.sr, k.sb, k.sr, v.sb, v.sr, go.sb, go.sr, gk.sb,
                     gk.sr, gv.sb, gv.sr);
  return hipGetLastError();
}

template <typename T>
hipError_t backward_by_width(const Problem &p, const View &q, const View &k, const View &v, const View &o,
                             const View &go, const float *lse, float *delta, const View &gq, const View &gk,
                             const View &gv, double scale) {
  switch (p.N / 16) {
    case 1: return launch_backward<T, 1>(p, q, k, v, o, go, lse, delta, gq, gk, gv, scale);
    case 2: return launch_backward<T, 2>(p, q, k, v, o, go, lse, delta, gq, gk, gv, scale);
    case 3: return launch_backward<T, 3>(p, q, k, v, o, go, lse, delta, gq, gk, gv, scale);
    case 4: return launch_backward<T, 4>(p, q, k, v, o, go, lse, delta, gq, gk, gv, scale);
    case 5: return launch_backward<T, 5>(p, q, k, v, o, go, lse, delta, gq, gk, gv, scale);
    case 6: return launch_backward<T, 6>(p, q, k, v, o, go, lse, delta, gq, gk, gv, scale);
    case 7: return launch_backward<T, 7>(p, q, k, v, o, go, lse, delta, gq, gk, gv, scale);
    default: return launch_backward<T, 8>(p, q, k, v, o, go, lse, delta, gq, gk, gv, scale);
  }
}

}  // namespace

bool try_launch_attention_backward(const Problem &p, const View &q, const View &k, const View &v, const View &o,
                                   const View &go, const float *lse, float *delta, const View &gq, const View &gk,
                                   const View &gv, double scale, hipError_t *err) {
  if (p.flags & WM_FLAG_FORCE_STRIDED) return false;
  if (!attention_supports(p.M, p.N, p.w, p.dtype, scale)) return false;
  const View *all[] = {&q, &k, &v, &o, &go, &gq, &gk, &gv};
  for (const View *t : all)
    if (t->data != nullptr && !fast_layout(*t, p.dtype)) return false;  // absent outputs have no layout
  *err = p.dtype == WM_DTYPE_BF16 ? backward_by_width<bf16_t>(p, q, k, v, o, go, lse, delta, gq, gk, gv, scale)
                                  : backward_by_width<f16_t>(p, q, k, v, o, go, lse, delta, gq, gk, gv, scale);
  return true;
}

}  // namespace wm
