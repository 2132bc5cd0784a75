// MFMA building blocks for gfx950 (CDNA4), 64-lane wavefronts.
//
// v_mfma_f32_32x32x16_{bf16,f16}: D(32x32) += A(32x16) * B(16x32).
//   A operand, lane l: row l%32, k = 8*(l/32) .. +7      (8 x 16-bit, one 16-byte word)
//   B operand, lane l: col l%32, k = 8*(l/32) .. +7
//   accumulator, lane l, register r (0..15): col l%32, row 8*(r/4) + 4*(l/32) + r%4
// (layouts verified on hardware with an integer-valued GEMM.)
//
// ds_read_tr16_b64 (LDS transpose read): inside each group of 16 lanes, lane i
// supplies the address of four consecutive 16-bit values S[i][0..3] and
// receives S[4j + (i>>2)][i&3] for j = 0..3.  Pointing lane i at
// M[n0 + (i>>2)][d0 + 4*(i&3)] of a row-major matrix therefore returns
// M[n0 .. n0+3][d0 + i]: a column slice, i.e. the k-contiguous MFMA operand of
// the transposed matrix, without ever storing the transpose.
#pragma once

#include <type_traits>
#include <hip/hip_runtime.h>

#include "device_common.h"

namespace dk {

// Head dims the MFMA kernels take: multiples of 8 up to 256.  They run at a
// tile width of 64, 128 or 256; narrower rows are zero-padded on chip.  (The
// split-KV decode kernels stop at 128.)
__host__ __device__ inline bool mfma_head_dim_ok(int d) { return d >= 8 && d <= 256 && d % 8 == 0; }
// the kernels keep a row's byte stride in 32 bits (16-bit elements)
template <typename View>
inline bool mfma_row_bytes_ok(const View &t) { return t.st >= 0 && t.st < (int64_t(1) << 31); }
__host__ __device__ inline int mfma_tile_width(int d) { return d <= 64 ? 64 : d <= 128 ? 128 : 256; }


typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef short shortx8 __attribute__((ext_vector_type(8)));

template <typename T>
struct Mma;  // 16-bit element type -> operand vector, MFMA, conversion

template <>
struct Mma<bf16_t> {
  using vec8 = bf16x8;
  using elem = __bf16;
  static __device__ __forceinline__ floatx16 mma(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ vec8 pack(const float *x) {
    vec8 r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = (__bf16)x[i];
    return r;
  }
};

template <>
struct Mma<f16_t> {
  using vec8 = f16x8;
  using elem = _Float16;
  static __device__ __forceinline__ floatx16 mma(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ vec8 pack(const float *x) {
    vec8 r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = (_Float16)x[i];
    return r;
  }
};

// Four floats to four 16-bit values (round to nearest even) with the hardware conversions
// (v_cvt_pk_bf16_f32 / v_cvt_f16_f32), 8 bytes ready to store.  The generic `from_float` for
// bf16 is integer arithmetic with a NaN branch, some ten instructions per value: at 64 values
// per lane that was the larger part of the forward's close-down.
template <typename T>
__device__ __forceinline__ uint2 pack4(float a, float b, float c, float d) {
  using E = typename Mma<T>::elem;
  typedef E v4 __attribute__((ext_vector_type(4)));
  const v4 r = {(E)a, (E)b, (E)c, (E)d};
  return __builtin_bit_cast(uint2, r);
}

// acc + dot product of two 16-byte groups of eight 16-bit values (exact fp32 products)
template <typename T>
__device__ __forceinline__ float dot8(uint4 a, uint4 b, float acc);
template <>
__device__ __forceinline__ float dot8<bf16_t>(uint4 a, uint4 b, float acc) {
  typedef __bf16 v2 __attribute__((ext_vector_type(2)));
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2, a.x), __builtin_bit_cast(v2, b.x), acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2, a.y), __builtin_bit_cast(v2, b.y), acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2, a.z), __builtin_bit_cast(v2, b.z), acc, false);
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2, a.w), __builtin_bit_cast(v2, b.w), acc, false);
}
template <>
__device__ __forceinline__ float dot8<f16_t>(uint4 a, uint4 b, float acc) {
  typedef _Float16 v2 __attribute__((ext_vector_type(2)));
  acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(v2, a.x), __builtin_bit_cast(v2, b.x), acc, false);
  acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(v2, a.y), __builtin_bit_cast(v2, b.y), acc, false);
  acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(v2, a.z), __builtin_bit_cast(v2, b.z), acc, false);
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2, a.w), __builtin_bit_cast(v2, b.w), acc, false);
}

template <typename V>
__device__ __forceinline__ V as_vec8(uint4 w) {
  return __builtin_bit_cast(V, w);
}

// 16-byte LDS read of 8 consecutive 16-bit values.
template <typename V>
__device__ __forceinline__ V lds_read8(const char *p) {
  return as_vec8<V>(*reinterpret_cast<const uint4 *>(p));
}

// The same reads from 32-bit LDS byte addresses.  Loop-invariant per-lane addresses are kept as
// such integers and passed through opaque_lds_address once: left as pointer arithmetic the
// compiler splits them into a row part and a chunk part and adds the two again in front of
// every read (8 + 16 additions per 64 x 64 block in the forward).
__device__ __forceinline__ uint32_t opaque_lds_address(uint32_t a) {
  asm volatile("" : "+v"(a));
  return a;
}
template <typename V>
__device__ __forceinline__ V lds_read8_at(uint32_t addr) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef const u32x4 __attribute__((address_space(3))) * lds_ptr;
  return __builtin_bit_cast(V, *(lds_ptr)(uintptr_t)addr);
}
template <typename V>
__device__ __forceinline__ V lds_read_tr8_at(uint32_t a0, uint32_t a1) {
  typedef shortx4 __attribute__((address_space(3))) * lds_ptr;
  shortx4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(uintptr_t)a0);
  shortx4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(uintptr_t)a1);
  shortx8 r = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(V, r);
}

__device__ __forceinline__ uint32_t lds_address(const void *p);  // below

// Loop-invariant operand addresses of a kernel with D-wide tiles: opaque 32-bit LDS addresses
// up to the 128-wide tile; at the 256-wide tile (32 addresses next to 128 accumulator
// registers) plain pointers, which the compiler may rebuild instead of keeping them live.
template <int D>
struct OperandAddress {
  static constexpr bool kOpaque = D <= 128;
  using type = typename std::conditional<kOpaque, uint32_t, const char *>::type;
  static __device__ __forceinline__ type make(char *smem, int offset) {
    if constexpr (kOpaque)
      return opaque_lds_address(lds_address(smem) + offset);
    else
      return smem + offset;
  }
};

// Two transpose reads -> the 8 k-values of one operand lane.
template <typename V>
__device__ __forceinline__ V lds_read_tr8(const char *p0, const char *p1) {
  typedef shortx4 __attribute__((address_space(3))) * lds_ptr;
  shortx4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0));
  shortx4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p1));
  shortx8 r = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(V, r);
}

// Either kind of address (OperandAddress<D>::type)
template <typename V>
__device__ __forceinline__ V lds_operand(const char *p) { return lds_read8<V>(p); }
template <typename V>
__device__ __forceinline__ V lds_operand(uint32_t a) { return lds_read8_at<V>(a); }
template <typename V>
__device__ __forceinline__ V lds_operand_tr(const char *p0, const char *p1) { return lds_read_tr8<V>(p0, p1); }
template <typename V>
__device__ __forceinline__ V lds_operand_tr(uint32_t a0, uint32_t a1) { return lds_read_tr8_at<V>(a0, a1); }

// ---------------------------------------------------------------------------
// 64-row x D tile of 16-bit elements in LDS, row-major, with an XOR swizzle of
// the 16-byte chunks that is conflict-free both for 16-byte row reads (16 lanes
// on 16 consecutive rows) and for transpose reads (4 rows x 64 bytes per
// half-wave).  The swizzle only depends on row & 15.
// ---------------------------------------------------------------------------
template <int D>
struct Tile {
  static constexpr int kRowBytes = D * 2;
  static constexpr int kBytes = 64 * kRowBytes;
  static constexpr int kChunksPerRow = D / 8;
  static __device__ __forceinline__ int swz(int row) {
    if constexpr (D >= 128)
      return ((row & 3) << 2) | ((row >> 2) & 3);
    else
      return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
  }
  // byte offset of 16-byte chunk `chunk` of `row`
  static __device__ __forceinline__ int off(int row, int chunk) {
    return row * kRowBytes + ((chunk ^ swz(row)) << 4);
  }
};

// Per-lane byte offsets of the two transpose reads of d-tile dt, relative to
// row0 of the tile, for row0 a multiple of 16; loop invariants, so no address
// arithmetic is left in the inner loops (the row0 part becomes an immediate).
// The lane (d = 32*dt + lane%32, k-group g) receives rows
// row0 + {4g..4g+3, 8+4g..8+4g+3} of column d.
template <int D>
__device__ __forceinline__ void transposed_offsets(int lane, int (&off)[D / 32][2]) {
  const int i16 = lane & 15, dgrp = (lane >> 4) & 1, g = lane >> 5;
  const int r0 = 4 * g + (i16 >> 2);
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt) {
    const int chunk = 4 * dt + 2 * dgrp + ((i16 & 3) >> 1);
    off[dt][0] = Tile<D>::off(r0, chunk) + (i16 & 1) * 8;
    off[dt][1] = Tile<D>::off(r0 + 8, chunk) + (i16 & 1) * 8;
  }
}

// LDS DMA (global_load_lds): each active lane i of the wave copies `bytes`
// (16 or 4) from gbase + voff to LDS address lds_base + i * bytes; gbase and
// lds_base are wave-uniform.  Issued as inline assembly on purpose: for the
// builtin the compiler places "s_waitcnt vmcnt(0)" in front of every later
// LDS read (it cannot tell which LDS bytes a copy in flight will write), which
// serialises a prefetch with the reads of the tile before it.  Here the caller
// owns the ordering: wait_tile_loads / wait_tiles_ahead, then a barrier,
// before anything reads what was copied.  Vector memory operations complete in
// order, so the compiler's own vmcnt bookkeeping for ordinary loads stays
// conservative (it can only wait for more than it asked for).
__device__ __forceinline__ uint32_t lds_address(const void *p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char *)p;
}
// M0 (the LDS base of the copy) is written without telling the compiler: it
// rejects M0 as a clobber, and nothing else in these kernels uses M0 (on gfx950
// only LDS DMA, lane-indexed moves and messages read it).  Invariant for every
// kernel that calls these helpers: no v_readlane / v_writelane / v_movrel with a
// run-time lane or register index, and no s_sendmsg, anywhere in the kernel
// (readfirstlane and DPP / permute exchanges do not touch M0).
__device__ __forceinline__ uint64_t uniform_address(const void *p) {
  // the builtin returns a signed int: narrow to 32 unsigned bits before widening
  const uint64_t a = (uint64_t)p;
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)a);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  return ((uint64_t)hi << 32) | (uint64_t)lo;
}
// Read one int32 of a look-up table at a wave-uniform address through the scalar
// unit.  A vector load here would make the compiler wait for every vector
// memory operation in flight (vmcnt(0)), tile copies included, before the
// value can be used.
__device__ __forceinline__ int scalar_load(const int32_t *p) {
  int v;
  asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(uniform_address(p)) : "memory");
  return v;
}
// Two table reads in flight together: one round trip instead of two.
__device__ __forceinline__ void scalar_load2(const int32_t *p0, const int32_t *p1, int &v0, int &v1) {
  asm volatile("s_load_dword %0, %2, 0x0\n\ts_load_dword %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)"
               : "=&s"(v0), "=&s"(v1)
               : "s"(uniform_address(p0)), "s"(uniform_address(p1))
               : "memory");
}
// base + rows * row_bytes for a wave-uniform, non-negative row count: one 32 x 32 -> 64 bit
// unsigned multiply (two scalar instructions) where `base + (int64_t)rows * stride` takes a
// signed 64 x 64 bit one (six).
__device__ __forceinline__ const char *row_address(const char *base, int rows, uint32_t row_bytes) {
  return base + (uint64_t)(uint32_t)rows * (uint64_t)row_bytes;
}
__device__ __forceinline__ void lds_dma16(const char *gbase, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(voff), "s"(uniform_address(gbase)), "s"(__builtin_amdgcn_readfirstlane(lds_base))
               : "memory");
}
__device__ __forceinline__ void lds_dma4(const char *gbase, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
               :
               : "v"(voff), "s"(uniform_address(gbase)), "s"(__builtin_amdgcn_readfirstlane(lds_base))
               : "memory");
}
// The same with a full address per lane (lanes of one copy may read different arrays).
__device__ __forceinline__ void lds_dma4_lane(const void *lane_ptr, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
               :
               : "v"(lane_ptr), "s"(__builtin_amdgcn_readfirstlane(lds_base))
               : "memory");
}

// Asynchronous global -> LDS copy of one tile by NT threads, straight into LDS
// (LDS DMA: no staging registers, no ds_write): a wave instruction moves 64 x 16 bytes
// to 1 KB of consecutive LDS; the swizzle is realised by choosing which global
// chunk each lane fetches (lane position p of row r fetches chunk p ^ swz(r)).
// TileLoader::init computes the per-thread global byte offsets once.  Rows
// outside [lo, hi) are zero-filled with ordinary LDS stores.  The caller
// waits (wait_tile_loads) and synchronises before reading the tile.
//
// PAD: the rows in memory hold fewer than D elements (a head_dim that is a
// multiple of 8 below the tile width).  Lanes whose chunk lies beyond the real
// width copy nothing; their LDS slots are never written by any copy, so a
// tile area that was zeroed once (zero_tiles) keeps zeros there for good.
// Every row has chunks inside the real width, so every wave still issues
// exactly kChunks load instructions per tile.
//
// ROWS: rows of the tile (64, or 32 for half tiles; the swizzle only depends on row & 15).
template <int D, int NT, bool PAD = false, int ROWS = 64>
struct TileLoader {
  static constexpr int kCPR = D / 8;
  static constexpr int kChunks = ROWS * kCPR / NT;
  static_assert(kChunks >= 1 && ROWS * kCPR % NT == 0, "every thread copies the same number of chunks");
  uint32_t goff[kChunks];  // global byte offset of this thread's chunk c inside the 64-row block
  int row0;                // first row this thread's wave covers with chunk 0 (wave-uniform)
  int lane_row, lane_byte;
  uint32_t inside;         // PAD: bit c set when this thread's chunk c lies inside the real width

  __device__ __forceinline__ void init(int tid, int64_t row_stride_elems, int real_d = D) {
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    row0 = wave * (64 / kCPR);
    lane_row = lane / kCPR;
    lane_byte = lane * 16;
    inside = 0;
#pragma unroll
    for (int c = 0; c < kChunks; ++c) {
      const int r = row0 + c * (NT / kCPR) + lane_row;
      const int pos = lane % kCPR;
      const int chunk = pos ^ Tile<D>::swz(r);
      goff[c] = (uint32_t)(r * row_stride_elems) * 2u + (uint32_t)(chunk << 4);
      if (chunk * 8 < real_d) inside |= 1u << c;
    }
  }
  // The whole tile lies inside the tensor: kChunks load instructions per wave and nothing else.
  // Callers test for this case with scalar arithmetic and take it on the main path: the general
  // `issue` below costs some thirty scalar instructions per tile in range tests and selects,
  // which all waves of a CU execute behind the same barrier.
  __device__ __forceinline__ void issue_full(const char *gblk, char *tile) const {
    const uint32_t base = lds_address(tile) + row0 * Tile<D>::kRowBytes;
#pragma unroll
    for (int c = 0; c < kChunks; ++c)
      if (!PAD || ((inside >> c) & 1)) lds_dma16(gblk, goff[c], base + c * (NT / kCPR) * Tile<D>::kRowBytes);
  }
  // rows [lo, hi) of the block are copied, the others zero-filled.  Returns true when the
  // whole tile was copied, i.e. when every wave issued exactly kChunks load instructions.
  // gblk (first byte of the 64-row block) is wave-uniform.
  __device__ __forceinline__ bool issue(const char *gblk, int lo, int hi, char *tile) const {
    const uint32_t base = lds_address(tile) + row0 * Tile<D>::kRowBytes;
    if (lo <= 0 && hi >= ROWS) {
#pragma unroll
      for (int c = 0; c < kChunks; ++c)
        if (!PAD || ((inside >> c) & 1)) lds_dma16(gblk, goff[c], base + c * (NT / kCPR) * Tile<D>::kRowBytes);
      return true;
    } else {
#pragma unroll
      for (int c = 0; c < kChunks; ++c) {
        char *wbase = tile + (row0 + c * (NT / kCPR)) * Tile<D>::kRowBytes;
        const int r = row0 + c * (NT / kCPR) + lane_row;
        if (r >= lo && r < hi) {
          if (!PAD || ((inside >> c) & 1)) lds_dma16(gblk, goff[c], base + c * (NT / kCPR) * Tile<D>::kRowBytes);
        } else {
          *reinterpret_cast<uint4 *>(wbase + lane_byte) = make_uint4(0, 0, 0, 0);
        }
      }
      return false;
    }
  }
};

// Write a wave's 32 x D accumulator tile (registers hold acc^T: lane = row m, register = dim) as
// rows of `T` scaled by `row_scale`: the tile goes through `stage` (32 rows of LDS in the tile
// layout, owned by this wave) and leaves as 16-byte pieces, CPR consecutive lanes covering one
// whole row, with the non-temporal hint.  Whole rows written around the L2 measure faster in
// the forward than the 8-byte pieces a lane holds after the multiply (-3 % on the headline
// workload, -8 % at 8 blocks per row); either change alone does not (coalescing alone: no
// change; the hint on 8-byte pieces: much slower).  The backward kernels use it from the
// 128-wide tile on (-1 % there; at the 64-wide tile direct stores are 0.5 % faster).
// Rows outside [row_lo, row_hi) are not written.  The caller makes sure that no wave still
// reads `stage` (a barrier after the last tile read).
template <typename T, int D, bool PAD, int ROWS>
__device__ __forceinline__ void store_staged_rows(const char *stage, T *g_row0, int64_t row_stride, int lane,
                                                  int row_lo, int row_hi, int real_d) {
  // rows 0 .. ROWS-1 of `stage` (tile layout) to g_row0 + row * row_stride, by one wave
  using TL = Tile<D>;
  constexpr int CPR = D / 8, RPI = 64 / CPR;
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  // (the lane number passes through an empty asm statement: the addresses below are then
  // computed here, not hoisted to the start of the kernel, where they would occupy registers
  // through the main loop)
  asm volatile("" : "+v"(lane));
#pragma unroll
  for (int j = 0; j < ROWS / RPI; ++j) {
    const int r = j * RPI + lane / CPR, c = lane % CPR;
    const u32x4 w = *reinterpret_cast<const u32x4 *>(stage + TL::off(r, c));
    // (the hint is unconditional on purpose: behind a run-time test with a plain store in the
    // other branch the compiler merges the two stores into one plain store)
    if (r >= row_lo && r < row_hi && (!PAD || c * 8 < real_d))
      __builtin_nontemporal_store(w, reinterpret_cast<u32x4 *>(g_row0 + (int64_t)r * row_stride + c * 8));
  }
}

template <typename T, int D, bool PAD>
__device__ __forceinline__ void store_tile_rows(char *stage, const floatx16 (&acc)[D / 32], float row_scale, T *g_row0,
                                                int64_t row_stride, int lane, int row_lo, int row_hi, int real_d) {
  using TL = Tile<D>;
  constexpr int DT = D / 32;
  asm volatile("" : "+v"(lane));  // as in store_staged_rows
  const int m = lane & 31, g = lane >> 5;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      // registers 4*r4 .. 4*r4+3 are dims 32dt + 8r4 + 4g + {0..3}
      *reinterpret_cast<uint2 *>(stage + TL::off(m, dt * 4 + r4) + g * 8) =
          pack4<T>(acc[dt][r4 * 4] * row_scale, acc[dt][r4 * 4 + 1] * row_scale, acc[dt][r4 * 4 + 2] * row_scale,
                   acc[dt][r4 * 4 + 3] * row_scale);
    }
  // The rows read back below were written by other lanes of this wave: LDS operations of a wave
  // execute in order, so no hardware wait is needed, but the compiler must not move the reads
  // above the writes (it cannot prove the swizzled addresses disjoint today; this says so).
  asm volatile("" ::: "memory");
  store_staged_rows<T, D, PAD, 32>(stage, g_row0, row_stride, lane, row_lo, row_hi, real_d);
}

// Zero `bytes` (a multiple of 16) of LDS with NT threads; the caller synchronises afterwards.
template <int NT>
__device__ __forceinline__ void zero_tiles(char *lds, int bytes, int tid) {
  for (int off = tid * 16; off < bytes; off += NT * 16) *reinterpret_cast<uint4 *>(lds + off) = make_uint4(0, 0, 0, 0);
}

// All asynchronous tile loads (and any other vector memory loads) of this wave have landed.
__device__ __forceinline__ void wait_tile_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Multi-stage pipelines: wait until at most `ahead` later tiles (LPT vector
// memory instructions per wave each) are still in flight, i.e. until the
// oldest tile has landed.  Vector memory loads return in order.  `ahead` is
// wave-uniform and at most 3.
template <int LPT>
__device__ __forceinline__ void wait_tiles_ahead(int ahead) {
  static_assert(3 * LPT <= 63, "vmcnt is a 6-bit counter");
  if (ahead <= 0)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  else if (ahead == 1)
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LPT) : "memory");
  else if (ahead == 2)
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * LPT) : "memory");
  else
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * LPT) : "memory");
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Maxima without the quieting step.  For fmaxf the compiler first passes every operand that
// might be a signalling NaN through v_max_f32 x, x: 32 extra instructions for the 32 scores of
// a softmax row share, more than the reduction itself.  The matrix unit does not produce
// signalling NaNs, so the instructions are used directly.
__device__ __forceinline__ float max2(float a, float b) {
  float d;
  asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
}
__device__ __forceinline__ float max3(float a, float b, float c) {
  float d;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
  return d;
}
// Maximum of a lane's value and the one of the lane 32 away (one VALU exchange, no LDS round
// trip: v_permlane32_swap of (x, x) leaves the lower half's values in one result and the upper
// half's in the other).
__device__ __forceinline__ float max_with_other_half(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return max2(__builtin_bit_cast(float, r[0]), __builtin_bit_cast(float, r[1]));
}

// Exchange with the lane 32 away (the other half-wave that holds the rest of
// an accumulator row).
__device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32); }

// The same exchange as one VALU instruction (no LDS round trip): v_permlane32_swap
// trades the upper half of its first operand for the lower half of its second,
// so (x, x) yields {lo, lo} and {hi, hi}; a lane's partner value is the one that
// differs from its own.  Returned for use in a symmetric reduction: the result is
// max/sum-equivalent to xor32 when combined with the lane's own value.
__device__ __forceinline__ float xor32_swap(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  // lanes 0..31 hold their own value in r[0] and the partner's in r[1]; lanes 32..63 the reverse
  return __builtin_bit_cast(float, (threadIdx.x & 32) ? r[0] : r[1]);
}

}  // namespace dk
