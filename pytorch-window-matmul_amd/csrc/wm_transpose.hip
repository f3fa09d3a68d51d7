// Batched transpose of the last two dimensions: (B, R, C) with unit column stride -> contiguous
// (B, C, R).  It serves one caller: keys that arrive as a contiguous (B, N, M) tensor.  The banded
// kernels want key rows contiguous (the reference makes the same copy on entry,
// reference cuda/window_matmul_cuda.cu:236, 285), and this kernel makes that copy at memory speed
// where a general strided copy reaches a quarter of it.
//
// A workgroup moves a tile of 64 rows x 64 columns through LDS: 16-byte pieces along the columns come
// in (whole lines of the source; single elements, consecutive lanes along a row, where the rows of
// the source are not 16-byte aligned, e.g. a sequence length that is not a multiple of 8), 16-byte
// pieces along the rows go out (the 64 destination rows of a
// tile are 64 R elements apart in a contiguous region, so the writes are whole lines too).  The tile's
// row pitch is odd in 4-byte (8-byte) words, which spreads the gathered reads over the banks.
#include "wm_common.hpp"

namespace wm {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int TR_T = 64;  // tile edge in elements

template <typename E, bool VEC_IN>  // E: an unsigned integer of the element's size; VEC_IN: source rows are 16-byte aligned
__global__ __launch_bounds__(256) void transpose_kernel(const E *__restrict__ src, E *__restrict__ dst, int R, int C,
                                                        int64_t ssb, int64_t ssr) {
  constexpr int ES = sizeof(E), PER = 16 / ES;                // elements per 16-byte piece
  constexpr int PITCH = TR_T * ES + (ES == 8 ? 8 : 4);        // bytes per tile row
  constexpr int PPR = TR_T / PER;                             // pieces per tile row (either way)
  __shared__ __attribute__((aligned(16))) unsigned char tile[TR_T * PITCH];
  const int c0 = blockIdx.x * TR_T, r0 = blockIdx.y * TR_T;
  const int64_t b = blockIdx.z;
  const E *sb = src + b * ssb;
  E *db = dst + b * (int64_t)R * C;

  if (VEC_IN) {
    // in: piece p = (row p / PPR, columns PER (p % PPR) ...)
#pragma unroll
    for (int u = 0; u < TR_T * PPR / 256; ++u) {
      const int p = threadIdx.x + 256 * u;
      const int r = p / PPR, cp = p % PPR;
      const int gr = r0 + r, gc = c0 + cp * PER;
      union {
        u32x4 v;
        E e[PER];
      } in;
      in.v = u32x4{0u, 0u, 0u, 0u};
      if (gr < R) {
        const E *g = sb + (int64_t)gr * ssr + gc;
        if (gc + PER <= C) {
          in.v = *reinterpret_cast<const u32x4 *>(g);
        } else {
#pragma unroll
          for (int j = 0; j < PER; ++j)
            if (gc + j < C) in.e[j] = g[j];
        }
      }
      unsigned char *t = tile + r * PITCH + cp * 16;
      if (ES == 8) {
        reinterpret_cast<uint64_t *>(t)[0] = ((uint64_t)in.v[1] << 32) | in.v[0];
        reinterpret_cast<uint64_t *>(t)[1] = ((uint64_t)in.v[3] << 32) | in.v[2];
      } else {
#pragma unroll
        for (int d = 0; d < 4; ++d) reinterpret_cast<uint32_t *>(t)[d] = in.v[d];
      }
    }
  } else {
    // source rows start at any element: one element per lane, consecutive lanes along the row
    E e[TR_T * TR_T / 256];
#pragma unroll
    for (int u = 0; u < TR_T * TR_T / 256; ++u) {
      const int idx = threadIdx.x + 256 * u, r = idx / TR_T, c = idx % TR_T;
      const bool ok = r0 + r < R && c0 + c < C;
      e[u] = ok ? sb[(int64_t)(r0 + r) * ssr + c0 + c] : E(0);
    }
#pragma unroll
    for (int u = 0; u < TR_T * TR_T / 256; ++u) {
      const int idx = threadIdx.x + 256 * u, r = idx / TR_T, c = idx % TR_T;
      *reinterpret_cast<E *>(tile + r * PITCH + c * ES) = e[u];
    }
  }
  __syncthreads();
  // out: piece p = (column p / PPR of the tile = destination row, rows PER (p % PPR) ... of the tile)
#pragma unroll
  for (int u = 0; u < TR_T * PPR / 256; ++u) {
    const int p = threadIdx.x + 256 * u;
    const int c = p / PPR, rp = p % PPR;
    const int gc = c0 + c, gr = r0 + rp * PER;
    union {
      u32x4 v;
      E e[PER];
    } out;
#pragma unroll
    for (int j = 0; j < PER; ++j) out.e[j] = *reinterpret_cast<const E *>(tile + (rp * PER + j) * PITCH + c * ES);
    if (gc < C && gr < R)  // R is a multiple of PER: a piece is inside or outside as a whole
      __builtin_nontemporal_store(out.v, reinterpret_cast<u32x4 *>(db + (int64_t)gc * R + gr));
  }
}

template <typename E>
hipError_t launch(const void *src, void *dst, int64_t B, int64_t R, int64_t C, int64_t ssb, int64_t ssr, bool vec_in,
                  hipStream_t stream) {
  const dim3 grid((unsigned)((C + TR_T - 1) / TR_T), (unsigned)((R + TR_T - 1) / TR_T), (unsigned)B);
  if (vec_in)
    hipLaunchKernelGGL((transpose_kernel<E, true>), grid, dim3(256), 0, stream, static_cast<const E *>(src),
                       static_cast<E *>(dst), (int)R, (int)C, ssb, ssr);
  else
    hipLaunchKernelGGL((transpose_kernel<E, false>), grid, dim3(256), 0, stream, static_cast<const E *>(src),
                       static_cast<E *>(dst), (int)R, (int)C, ssb, ssr);
  return hipGetLastError();
}

}  // namespace

// false: the layout is not one this kernel takes (nothing launched)
bool try_launch_transpose(const void *src, void *dst, int64_t B, int64_t R, int64_t C, int64_t ssb, int64_t ssr,
                          int elem_size, hipStream_t stream, hipError_t *err) {
  if (elem_size != 2 && elem_size != 4 && elem_size != 8) return false;
  const int64_t per = 16 / elem_size;
  // the destination leaves as 16-byte pieces along R; the source comes in as such pieces along C where
  // its rows allow it, element by element otherwise
  if (reinterpret_cast<uintptr_t>(dst) % 16 != 0 || R % per != 0 || reinterpret_cast<uintptr_t>(src) % elem_size != 0) return false;
  const bool vec_in = reinterpret_cast<uintptr_t>(src) % 16 == 0 && ssb % per == 0 && ssr % per == 0;
  if (ssr < C || B > 65535 || (R + TR_T - 1) / TR_T > 65535 || C > 0x7fffffff - TR_T || R > 0x7fffffff - TR_T) return false;
  *err = hipSuccess;
  if (B == 0 || R == 0 || C == 0) return true;
  *err = elem_size == 2   ? launch<uint16_t>(src, dst, B, R, C, ssb, ssr, vec_in, stream)
         : elem_size == 4 ? launch<uint32_t>(src, dst, B, R, C, ssb, ssr, vec_in, stream)
                          : launch<uint64_t>(src, dst, B, R, C, ssb, ssr, vec_in, stream);
  return true;
}

}  // namespace wm
