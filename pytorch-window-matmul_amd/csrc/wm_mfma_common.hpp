// Device helpers shared by the MFMA kernel families (16-bit storage, float32 accumulate).
#pragma once

#include "wm_common.hpp"
#include "wm_types.hpp"

namespace wm {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int TM = 128;  // rows per workgroup (32 per wave)
constexpr int KC = 64;   // chunk length along the contraction (P2, P3) / dense columns (P1)
constexpr int PF = 2;    // chunks requested ahead of the one being multiplied (P2, P3)

struct __attribute__((packed, aligned(2))) Chunk2 {
  u32x4 v;
};

// Band chunks are read exactly once per kernel: the aligned variant loads them non-temporal so
// that the stream does not evict the operand rows that neighbouring workgroups share in L2.
template <bool ALIGNED>
__device__ __forceinline__ u32x4 load_chunk(const uint16_t *p) {
  if (ALIGNED) return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
  return reinterpret_cast<const Chunk2 *>(p)->v;
}
template <bool ALIGNED>
__device__ __forceinline__ void store_chunk(uint16_t *p, u32x4 v) {
  if (ALIGNED)
    *reinterpret_cast<u32x4 *>(p) = v;
  else
    reinterpret_cast<Chunk2 *>(p)->v = v;
}
// Streaming store for data that is written once and not read again by this kernel (the band):
// marked non-temporal so that it does not push the operand rows other workgroups still need
// out of the L2.
__device__ __forceinline__ void store_chunk_streaming(uint16_t *p, u32x4 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p));
}

// Keeps elements e_lo..e_hi (inclusive, in 0..7) of a chunk of eight 16-bit values, clears the rest.
__device__ __forceinline__ u32x4 keep_range(u32x4 v, int e_lo, int e_hi) {
  u32x4 r;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const uint32_t lo = (2 * d >= e_lo && 2 * d <= e_hi) ? 0x0000ffffu : 0u;
    const uint32_t hi = (2 * d + 1 >= e_lo && 2 * d + 1 <= e_hi) ? 0xffff0000u : 0u;
    r[d] = v[d] & (lo | hi);
  }
  return r;
}

// Band chunk = 8 consecutive dense columns of one row of the skewed tile, of which only
// elements [e_lo, e_hi] are valid.  Loading is split in two branch-free halves so that the
// prefetch contains nothing but loads (a use of the loaded value, or a load inside a branch,
// makes the compiler wait for memory on the spot and serialises the pipeline):
//   fetch_band_chunk  issues the 16-byte load; from `safe` (any readable, suitably aligned
//                     address) when no element is valid;
//   mask_band_chunk   clears the invalid elements, later, when the chunk goes to LDS.
// A partially valid chunk is read whole: with w >= 7 the up-to-7 elements on either side of a
// row's valid range are band entries of the same or the neighbouring row, i.e. inside the
// tensor (the kernels are only used for w >= 8).
__device__ __forceinline__ bool band_chunk_any(int e_lo, int e_hi) { return (e_hi >= 0) & (e_lo <= 7) & (e_lo <= e_hi); }
template <bool ALIGNED>
__device__ __forceinline__ u32x4 fetch_band_chunk(const uint16_t *p, const uint16_t *safe, int e_lo, int e_hi) {
  return load_chunk<ALIGNED>(band_chunk_any(e_lo, e_hi) ? p : safe);
}
__device__ __forceinline__ u32x4 mask_band_chunk(u32x4 v, int e_lo, int e_hi) {
  return keep_range(v, band_chunk_any(e_lo, e_hi) ? e_lo : 8, e_hi);
}

// Row chunk of a dense operand; rows outside the sequence are fetched from `safe` and zeroed later.
__device__ __forceinline__ u32x4 fetch_row_chunk(const uint16_t *p, const uint16_t *safe, bool valid) {
  return *reinterpret_cast<const u32x4 *>(valid ? p : safe);
}
__device__ __forceinline__ u32x4 mask_row_chunk(u32x4 v, bool valid) {
  const uint32_t m = valid ? 0xffffffffu : 0u;
  u32x4 r = {v[0] & m, v[1] & m, v[2] & m, v[3] & m};
  return r;
}
__device__ __forceinline__ u32x4 load_row_chunk(const uint16_t *p, const uint16_t *safe, bool valid) {
  return mask_row_chunk(fetch_row_chunk(p, safe, valid), valid);
}

template <typename T>
struct Mma;
template <>
struct Mma<bf16_t> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
  }
  // 16x16x32: lane = row/column lane % 16, eight consecutive k from 8 (lane / 16); c[v] = row 4 (lane / 16) + v
  static __device__ __forceinline__ f32x4 run16(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));  // v_cvt_pk_bf16_f32, RNE
  }
  // acc + lo + hi of a packed pair (v_dot2c_f32_bf16 with a pair of ones)
  static __device__ __forceinline__ float add_pair(uint32_t pair, float acc) {
    const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pair), ones, acc, false);
  }
};
template <>
struct Mma<f16_t> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                  0, 0);
  }
  static __device__ __forceinline__ f32x4 run16(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                  0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));  // v_cvt_pk_f16_f32, RNE (one instruction, not three)
  }
  static __device__ __forceinline__ float add_pair(uint32_t pair, float acc) {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    const f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, pair), ones, acc, false);
  }
};

// Operand fetch for a matrix stored in LDS as Mat[k][x] (x contiguous) when the MFMA
// wants, per lane, x = lane % 32 and eight consecutive k starting at 8 * (lane / 32).
// ds_read_b64_tr_b16 works on 16-lane groups: lane s of a group supplies the address of
// 4 consecutive x in row s/4 and receives, for x = its own position in the group, the
// 4 values of rows 0..3.  Two such reads cover the 8 k's.
__device__ __forceinline__ u32x4 lds_read_transposed(const uint16_t *mat, int stride, int k0, int x0, int lane) {
  const int s = lane & 15, grp = lane >> 4;
  const int xb = x0 + 16 * (grp & 1) + 4 * (s & 3);
  const int kb = k0 + 8 * (grp >> 1) + (s >> 2);
  typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
  const uint16_t *p0 = mat + kb * stride + xb;
  const uint16_t *p1 = p0 + 4 * stride;
  const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0));
  const s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p1));
  const u32x2 ua = __builtin_bit_cast(u32x2, a), ub = __builtin_bit_cast(u32x2, b);
  u32x4 r = {ua[0], ua[1], ub[0], ub[1]};
  return r;
}

// Same fetch from a matrix stored WITHOUT row padding (row length a multiple of 128 elements) and
// swizzled instead: the 32-byte block b of row k lives at block position b ^ ((k & 3) << 1).  The
// four rows a 16-lane group touches (k = 4n .. 4n+3) then fall into four different bank groups.
__device__ __forceinline__ int swz32(int x, int k) { return (((x >> 4) ^ ((k & 3) << 1)) << 4) | (x & 15); }
__device__ __forceinline__ u32x4 lds_read_transposed_swz(const uint16_t *mat, int stride, int k0, int x0, int lane) {
  const int s = lane & 15, grp = lane >> 4;
  const int xb = x0 + 16 * (grp & 1) + 4 * (s & 3);
  const int kb = k0 + 8 * (grp >> 1) + (s >> 2);  // k0 is a multiple of 8: kb & 3 == s >> 2, same for kb + 4
  typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
  const uint16_t *p0 = mat + kb * stride + swz32(xb, kb);
  const uint16_t *p1 = p0 + 4 * stride;
  const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0));
  const s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p1));
  const u32x2 ua = __builtin_bit_cast(u32x2, a), ub = __builtin_bit_cast(u32x2, b);
  u32x4 r = {ua[0], ua[1], ub[0], ub[1]};
  return r;
}

// Pins a prefetched register at this point of the program: the compiler may not use the value
// (and therefore may not wait for its load) any earlier than here.
__device__ __forceinline__ u32x4 pin(u32x4 v) {
  asm volatile("" : "+v"(v));
  return v;
}

__device__ __forceinline__ void wave_sync_lds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Result rows of a wave that holds 32 rows x 32 NB columns transposed: lane = row (lane % 32),
// accumulator v of block hb = column 32 hb + 8 (v / 4) + 4 (lane / 32) + v % 4.  Stored from
// there a row would leave as 8-byte pieces, sixteen per 128 bytes.  The rows go through a
// wave-private LDS area instead (RowStage<NB>::ELEMS elements, e.g. part of the operand buffers
// once the last chunk is multiplied) and leave as 16-byte pieces, consecutive lanes on
// consecutive pieces of a row: whole 128-byte lines per 8 lanes, non-temporal so that they do
// not displace streamed operands on their way through the caches.  `mul` scales the lane's row.
template <int NB>
struct RowStage {
  static constexpr int SW = NB == 1 ? 32 : 64;  // columns staged at a time
  static constexpr int STRIDE = SW + 8;         // staged rows 16 bytes apart mod 128 (SW = 64)
  static constexpr int ELEMS = 32 * STRIDE;     // per wave
};
template <typename T, int NB>
__device__ __forceinline__ void store_wave_rows(uint16_t *stage, const f32x16 (&acc)[NB], float mul, uint16_t *Cb,
                                                int64_t csr, int row0, int M, int N, int lane) {
  constexpr int SW = RowStage<NB>::SW, STRIDE = RowStage<NB>::STRIDE;
  constexpr int CPR = SW / 8, RPP = 64 / CPR;  // 16-byte pieces per staged row, rows per 64-lane pass
  const int r = lane & 31, half = lane >> 5;
#pragma unroll
  for (int n0 = 0; n0 < NB; n0 += SW / 32) {
    wave_sync_lds();  // whatever the wave still reads from the area has been read
#pragma unroll
    for (int hb = n0; hb < n0 + SW / 32 && hb < NB; ++hb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const u32x2 o = {Mma<T>::pack2(acc[hb][4 * g] * mul, acc[hb][4 * g + 1] * mul),
                         Mma<T>::pack2(acc[hb][4 * g + 2] * mul, acc[hb][4 * g + 3] * mul)};
        *reinterpret_cast<u32x2 *>(stage + r * STRIDE + 32 * (hb - n0) + 8 * g + 4 * half) = o;
      }
    wave_sync_lds();
#pragma unroll
    for (int s = 0; s < 32 / RPP; ++s) {
      const int rr = lane / CPR + RPP * s, piece = lane % CPR;
      const int row = row0 + rr, h = 32 * n0 + 8 * piece;
      if (row >= 0 && row < M && h < N)
        __builtin_nontemporal_store(*reinterpret_cast<const u32x4 *>(stage + rr * STRIDE + 8 * piece),
                                    reinterpret_cast<u32x4 *>(Cb + (int64_t)row * csr + h));
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Tiles that global memory writes straight into LDS (buffer_load ... lds), no registers in between
// ---------------------------------------------------------------------------------------------
// One wave-level load moves 64 pieces of 16 bytes; lane l's piece lands at LDS base + 16 l, so a
// tile of R rows x PPR pieces is a flat, unpadded row-major array of 16-byte slots and WHICH piece
// a lane fetches is the only freedom.  Rows of 128 or 256 bytes (PPR 8 or 16) would put a column of
// the tile into one bank group, so the piece that lives in slot p of row r is piece p ^ swz<PPR>(r).
// LDS reads are served 256 bytes per cycle from 64 banks (ds_read_b128: 16 lanes a cycle,
// ds_read_b64_tr_b16: 32 lanes a cycle), and a cycle's lanes must fall into 16 different 16-byte
// bank groups:
//   rows r..r+15, same piece (ds_read_b128 of an operand with the contraction along the row)
//   rows 4n..4n+3, the four pieces of a 64-byte block (ds_read_b64_tr_b16, two 16-lane groups)
// 256-byte rows start in the same bank, so the swizzle alone tells 16 rows apart: row bits 0-1 go
// to piece bits 2-3 (the rows of a transposing read), row bits 2-3 to piece bits 0-1.  128-byte
// rows alternate between the two halves of the banks, which takes care of row bit 0: row bit 1
// goes to piece bit 2, row bits 2-3 to piece bits 0-1.  In both, a row 4 further down has bit 0 of
// the swizzle flipped and a row 8 further down bit 1; 16 rows further down nothing changes.
// (Measured per instruction with the swizzle (r & 3) << 1 | (r >> 2) & 1, which tells only 8 rows
// apart: 8 instead of 4 cycles per ds_read_b128, and 4 instead of 2 per transposing read of 256-byte rows.)
template <int PPR>
__device__ __forceinline__ int swz(int r) {
  static_assert(PPR == 8 || PPR == 16, "rows of 128 or 256 bytes");
  return PPR == 16 ? ((r & 3) << 2) | ((r >> 2) & 3) : (((r >> 1) & 1) << 2) | (((r >> 3) & 1) << 1) | ((r >> 2) & 1);
}

// s_waitcnt vmcnt(n) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// s_waitcnt vmcnt(n) lgkmcnt(0): additionally all of the wave's LDS traffic is complete.
template <int N>
__device__ __forceinline__ void wait_vmcnt_lgkm0() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (0 << 8));
}

// Raw buffer descriptor (four scalar registers) over `bytes` bytes at p: loads beyond the end
// return zeros.
__device__ __forceinline__ u32x4 make_rsrc(const void *p, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  const u32x4 r = {(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, bytes, 0x00020000u};
  return r;
}

// One wave-level load of 64 x 16 bytes into LDS at byte address lds_base (+ 16 lane, added by the
// hardware); lane l fetches buffer offset voff + soff.  Written as assembly on purpose: the
// compiler would make every later LDS read wait for all such loads in flight (it cannot tell the
// tiles apart), which is exactly the wait a multi-stage pipeline must not have.  The kernels
// count these loads themselves (wait_vmcnt) before the barrier that publishes a tile.  M0 is
// written here and named as clobbered, so that a use of M0 the compiler makes itself (dynamic
// register indexing, its own LDS-direct loads) is set up again after this statement.
__device__ __forceinline__ void dma_piece(u32x4 rsrc, uint32_t lds_base, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds"
               :
               : "v"(voff), "s"(rsrc), "s"(soff), "s"(lds_base)
               : "memory", "m0");
}
// The same marked non-temporal, for data that is read exactly once and in whole cache lines (a band
// whose column groups are lines): it should not push the rows that neighbouring workgroups share out
// of the L2.  Not for pieces whose line-mates are fetched by another load: those would miss again.
__device__ __forceinline__ void dma_piece_streaming(u32x4 rsrc, uint32_t lds_base, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen nt lds"
               :
               : "v"(voff), "s"(rsrc), "s"(soff), "s"(lds_base)
               : "memory", "m0");
}
// The same with 4 bytes per lane: 256 consecutive bytes of LDS per wave-level load.
__device__ __forceinline__ void dma_dword(u32x4 rsrc, uint32_t lds_base, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dword %0, %1, %2 offen lds"
               :
               : "v"(voff), "s"(rsrc), "s"(soff), "s"(lds_base)
               : "memory", "m0");
}
__device__ __forceinline__ uint32_t lds_address(const void *p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
}

// Loads the chunk of 64 rows that starts `row_bytes0` bytes into the buffer into a tile at `tile`
// (LDS, 64 * PPR slots).  `voff` is the lane's byte offset inside a chunk for the first of the
// wave's loads (row and swizzled piece of slot 64 wave + lane); the wave's further loads are
// 256 / PPR rows apart, which is `step` bytes in memory and 4096 bytes in LDS.
template <int PPR>
__device__ __forceinline__ void dma_chunk(u32x4 rsrc, const uint16_t *tile, int wave, uint32_t voff,
                                          uint32_t row_bytes0, uint32_t step) {
  constexpr int LOADS = PPR / 4;  // per wave: 64 PPR pieces / 64 lanes / 4 waves
  const uint32_t base = lds_address(tile) + 1024 * wave;
#pragma unroll
  for (int j = 0; j < LOADS; ++j) dma_piece(rsrc, base + 4096 * j, voff, row_bytes0 + step * j);
}
// The lane's offset for the above: slot 64 wave + lane of the tile -> row, logical piece.
template <int PPR>
__device__ __forceinline__ uint32_t dma_lane_offset(int wave, int lane, int64_t row_stride_elems) {
  const int slot = 64 * wave + lane, row = slot / PPR, piece = (slot % PPR) ^ swz<PPR>(row);
  return (uint32_t)(row * row_stride_elems * 2 + piece * 16);
}

// A swizzled tile of ROWS rows x PPR pieces as the loads above fill it, generalised to any row count
// whose pieces divide evenly over the four wavefronts: the loading side (which piece a lane
// fetches, how the wave's loads step through the rows) and the two ways the MFMA kernels read it.
template <int ROWS, int PPR>
struct LdsTile {
  static_assert((ROWS * PPR) % 256 == 0 && (PPR == 8 || PPR == 16), "whole wave-level loads; rows of 128 or 256 bytes");
  static constexpr int LOADS = ROWS * PPR / 256;  // wave-level loads per wavefront and tile
  static constexpr int ROWB = 16 * PPR;           // bytes per row
  static constexpr int ELEMS = ROWS * PPR * 8;    // 16-bit elements per tile
  typedef s16x4 __attribute__((address_space(3))) * lds_tr_ptr;
  // the lane's byte offset inside a tile's memory image for the first of the wave's loads
  static __device__ __forceinline__ uint32_t lane_offset(int wave, int lane, int64_t row_stride_elems) {
    return dma_lane_offset<PPR>(wave, lane, row_stride_elems);
  }
  // row of the tile that the lane's j-th load fills, and which 16 bytes of that row it fetches
  static __device__ __forceinline__ int load_row(int wave, int lane, int j) { return (64 * wave + lane) / PPR + 256 / PPR * j; }
  static __device__ __forceinline__ int load_piece(int wave, int lane) {
    const int slot = 64 * wave + lane;
    return (slot % PPR) ^ swz<PPR>(slot / PPR);
  }
  // bytes in memory between two of the wave's loads (256 / PPR rows)
  static __device__ __forceinline__ uint32_t step(int64_t row_stride_elems) {
    return (uint32_t)(256 / PPR * row_stride_elems * 2);
  }
  static __device__ __forceinline__ void request(u32x4 rsrc, const uint16_t *tile, int wave, uint32_t voff,
                                                 uint32_t bytes0, uint32_t step_bytes) {
    const uint32_t base = lds_address(tile) + 1024 * wave;
#pragma unroll
    for (int j = 0; j < LOADS; ++j) dma_piece(rsrc, base + 4096 * j, voff, bytes0 + step_bytes * j);
  }
  // `request` for a tile of which a lane needs only some pieces: load j is made from voff[j], which
  // the caller sets beyond the end of the buffer for pieces nobody will read (such a load returns
  // zeros without touching memory).  `streaming` (uniform over the wavefront) marks the loads
  // non-temporal.
  static __device__ __forceinline__ void request_some(u32x4 rsrc, const uint16_t *tile, int wave,
                                                      const uint32_t (&voff)[LOADS], uint32_t bytes0,
                                                      uint32_t step_bytes, bool streaming) {
    const uint32_t base = lds_address(tile) + 1024 * wave;
    if (streaming) {
#pragma unroll
      for (int j = 0; j < LOADS; ++j) dma_piece_streaming(rsrc, base + 4096 * j, voff[j], bytes0 + step_bytes * j);
    } else {
#pragma unroll
      for (int j = 0; j < LOADS; ++j) dma_piece(rsrc, base + 4096 * j, voff[j], bytes0 + step_bytes * j);
    }
  }
  // Reading.  row_at: lane -> row lane % 32, piece lane / 32 (add 32 r0 ROWB for other rows, XOR
  // 32 ks for pieces 2 ks + lane / 32): operand with the contraction along the row.
  static __device__ __forceinline__ uint32_t row_at(int lane) {
    const int r32 = lane & 31, half = lane >> 5;
    return (uint32_t)(r32 * ROWB + ((half ^ swz<PPR>(r32)) << 4));
  }
  static __device__ __forceinline__ u32x4 rows(const uint16_t *tile, uint32_t at, int blk, int ks) {
    return *reinterpret_cast<const u32x4 *>(reinterpret_cast<const char *>(tile) + 32 * blk * ROWB + (at ^ (32 * ks)));
  }
  // tr_at / cols: operand with the contraction along the rows of the tile, read transposed.  The
  // lane gets column 32 cb + lane % 32 of rows r0 + 4 (lane / 32) + {0, 1, 2, 3, 8, 9, 10, 11},
  // r0 a multiple of 16.
  static __device__ __forceinline__ uint32_t tr_at(int lane) {
    const int s16 = lane & 15, grp = lane >> 4, rowl = 4 * (grp >> 1) + (s16 >> 2);
    return (uint32_t)(rowl * ROWB + (((2 * (grp & 1) + ((s16 & 3) >> 1)) ^ swz<PPR>(rowl)) << 4) + 8 * (s16 & 1));
  }
  static __device__ __forceinline__ u32x4 cols(const uint16_t *tile, uint32_t at, int r0, int cb) {
    const char *p = reinterpret_cast<const char *>(tile) + r0 * ROWB;
    // eight rows further down the swizzle differs in bit 1
    const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(p + (at ^ (64 * cb)))));
    const u32x2 hi = __builtin_bit_cast(
        u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(p + 8 * ROWB + (at ^ 32 ^ (64 * cb)))));
    const u32x4 r = {lo[0], lo[1], hi[0], hi[1]};
    return r;
  }
  // tr_at_seq / cols_seq: the same read with the lane's eight rows consecutive,
  // r0 + 8 (lane / 32) + {0 .. 7}: the order in which `rows` of another tile delivers its pieces.
  static __device__ __forceinline__ uint32_t tr_at_seq(int lane) {
    const int s16 = lane & 15, grp = lane >> 4, rowl = 8 * (grp >> 1) + (s16 >> 2);
    return (uint32_t)(rowl * ROWB + (((2 * (grp & 1) + ((s16 & 3) >> 1)) ^ swz<PPR>(rowl)) << 4) + 8 * (s16 & 1));
  }
  static __device__ __forceinline__ u32x4 cols_seq(const uint16_t *tile, uint32_t at, int r0, int cb) {
    const char *p = reinterpret_cast<const char *>(tile) + r0 * ROWB;
    // four rows further down the swizzle differs in its lowest bit
    const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(p + (at ^ (64 * cb)))));
    const u32x2 hi = __builtin_bit_cast(
        u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(p + 4 * ROWB + (at ^ 16 ^ (64 * cb)))));
    const u32x4 r = {lo[0], lo[1], hi[0], hi[1]};
    return r;
  }
  // `request` with the position of the tile folded into the lane's offset: a tile that begins
  // before the buffer then has its first rows out of range (zeros) instead of all of them
  static __device__ __forceinline__ void request_at(u32x4 rsrc, const uint16_t *tile, int wave, uint32_t voff,
                                                    uint32_t step_bytes) {
    const uint32_t base = lds_address(tile) + 1024 * wave;
#pragma unroll
    for (int j = 0; j < LOADS; ++j) dma_piece(rsrc, base + 4096 * j, voff + step_bytes * j, 0);
  }
};

// Clears the elements of a transposed-read operand (LdsTile::cols) whose row lies outside [lo, hi];
// r_first is the row of the lane's element 0.
__device__ __forceinline__ u32x4 keep_rows_tr(u32x4 v, int r_first, int lo, int hi) {
  u32x4 r;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int ra = r_first + 2 * (d & 1) + 8 * (d >> 1);
    const uint32_t l = (ra >= lo && ra <= hi) ? 0x0000ffffu : 0u;
    const uint32_t h = (ra + 1 >= lo && ra + 1 <= hi) ? 0xffff0000u : 0u;
    r[d] = v[d] & (l | h);
  }
  return r;
}

// Row stride (elements) of matrices read with lds_read_transposed: the byte stride must be
// 32 or 96 (mod 128) so that the 4 rows touched by a 16-lane group fall into distinct banks.
#ifndef WM_PAD_TR
#define WM_PAD_TR 16
#endif
constexpr int lds_stride_tr(int n_padded) { return n_padded + WM_PAD_TR; }

// Element-wise store of elements [e_lo, e_hi] of a chunk (the slow path for chunk pieces that
// cannot be completed with their neighbour row's piece).
__device__ __forceinline__ void store_chunk_elements(uint16_t *dst, u32x4 v, int e_lo, int e_hi) {
#pragma unroll
  for (int e = 0; e < 8; ++e)
    if (e >= e_lo && e <= e_hi) dst[e] = (uint16_t)(v[e >> 1] >> (16 * (e & 1)));
}


}  // namespace
}  // namespace wm
