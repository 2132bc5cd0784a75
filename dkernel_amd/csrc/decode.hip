// Split-KV decode kernels for gfx950: one new query token per sequence over
// padded (left or right), unpadded, packed or paged K/V, bf16 / fp16 (paged
// pools also fp8), head_dim a multiple of 8 up to 256, 64 x 64 tiles,
// grouped-query attention with all q heads of a kv head sharing the
// look-up-table row.  The step is HBM-bound (every attended K/V byte is read
// exactly once, for all q heads of the group together), so the design goal is
// bytes in flight, not FLOPs:
//
//   work unit = one wave = consecutive entries of the row of (sequence, kv
//               head); the number of units of a row and the even split of its
//               entries follow from its length on the device, so waves stream
//               similar amounts of K/V whatever the sequence lengths are;
//   workgroup = kDecodeWaves consecutive units of one row (workgroups beyond a
//               row's unit count exit at once; a row that needs several
//               workgroups is cut into a whole number of them, so that none
//               holds LDS and wave slots for idle waves);
//   wave      = per block: computes S^T = K Q^T (the q heads of the group are the MFMA
//               columns), softmax, O^T += V^T P^T with LDS transpose reads,
//               keeping a running (max, sum, O) in registers;
//   epilogue  = a row whose units all sit in one workgroup is merged there
//               through LDS and written as O / LSE; otherwise one fp32
//               partial (O unnormalised, max, sum) per (sequence, q head,
//               unit) goes to the caller's workspace and decode_combine_kernel
//               merges those rows.
// A wave works on half blocks (32 keys): 2 x 8.5 KB of private LDS tiles and
// the next half block prefetched into registers, so 8 waves are resident per
// CU (2 per SIMD, <= 256 VGPRs each): one wave's loads overlap the other's
// multiplies on the same SIMD.  (Head dims above 128: 256-wide tiles, 2 x 33 KB per wave, one
// workgroup of four waves per CU and one wave per SIMD.)
#include <algorithm>
#include <type_traits>

#include "common.h"
#include "device_common.h"
#include "mfma_common.h"

namespace dk {

constexpr int kDecodeWaves = 4;  // units (waves) per workgroup

// Upper bound on the entries of one table row: the caller's hint when given,
// else the number of column blocks.
static int decode_max_row_entries(const FwdParams &p) {
  return p.csr.max_row_entries > 0 ? p.csr.max_row_entries : p.csr.num_rows;
}

// Table entries per work unit (one wave).  With enough rows (sequences x kv heads) to fill the
// machine, a row is cut into as many units as a workgroup has waves, so that it is finished
// inside one workgroup and the merge kernel is not launched at all; with few rows, into more
// units (about 1024 waves in total).  At most 16 (the paged path keeps a unit's page numbers in
// the lanes of one register).
static int decode_unit_blocks(const FwdParams &p) {
  const int rows = p.seqs.batch * p.Hkv;
  const int units_per_row = std::max(kDecodeWaves, cdiv(1024, rows > 0 ? rows : 1));
  return std::min(16, std::max(2, cdiv(decode_max_row_entries(p), units_per_row)));
}

// Units a row of n table entries is cut into: as many as the unit size asks for, and at least
// the waves of one workgroup (one entry each at worst), so that every wave of the workgroup that
// finishes a row streams a share of it.  A row that needs more than one workgroup gets a whole
// number of them: a workgroup with a single busy wave would hold the LDS and the wave slots of
// four.  Used by both kernels.
__host__ __device__ inline int decode_row_units(int n, int unit_blocks, int waves) {
  const int by_size = (n + unit_blocks - 1) / unit_blocks;
  const int by_waves = n < waves ? n : waves;
  const int units = by_size > by_waves ? by_size : by_waves;
  return units > waves ? (units + waves - 1) / waves * waves : units;
}

template <int D>
struct DecSmem {  // per wave: one 32-key half block of K and of V, plus q of the group
  static constexpr int kStride = D * 2 + 16;   // bytes per row
  static constexpr int kHalf = 32 * kStride;   // one half-block tile
  // followed by q of the group's heads, row-major: ratio * D * 2 bytes
  static int wave_bytes(int ratio) { return 2 * kHalf + ratio * D * 2; }
};

// workspace layout: [batch][Hq][max_units][D + 2] floats (O[D] unnormalised, max, sum)
// Eight OCP e4m3 bytes -> eight elements of T.  Exact (e4m3 has 3 mantissa bits), so bf16 is
// the upper half of the fp32 value and fp16 needs no rounding mode: one convert and one pack per
// two elements.
template <typename T>
__device__ __forceinline__ uint32_t pack2_exact(float a, float b);
template <>
__device__ __forceinline__ uint32_t pack2_exact<bf16_t>(float a, float b) {
  return __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);  // hi16(b) : hi16(a)
}
template <>
__device__ __forceinline__ uint32_t pack2_exact<f16_t>(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}
template <typename T>
__device__ __forceinline__ uint4 fp8x8_to(uint2 w) {
  typedef float float2_ __attribute__((ext_vector_type(2)));
  const float2_ a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w.x, false), b = __builtin_amdgcn_cvt_pk_f32_fp8((int)w.x, true);
  const float2_ c = __builtin_amdgcn_cvt_pk_f32_fp8((int)w.y, false), d = __builtin_amdgcn_cvt_pk_f32_fp8((int)w.y, true);
  return make_uint4(pack2_exact<T>(a[0], a[1]), pack2_exact<T>(b[0], b[1]), pack2_exact<T>(c[0], c[1]),
                    pack2_exact<T>(d[0], d[1]));
}

// KV8 (with PAGED): the K/V pools hold fp8 bytes, converted to T on the way into LDS.
// W waves per workgroup = W consecutive units of one row.  A row whose units all sit in one
// workgroup is finished here (the waves exchange their partials through LDS and write O / LSE);
// longer rows leave their partials in the workspace for decode_combine_kernel.
template <typename T, int D, bool PAD, bool SUB, bool PAGED, bool KV8, int W>
__global__ __launch_bounds__(64 * W) __attribute__((amdgpu_waves_per_eu(D == 256 ? 1 : 2, D == 256 ? 1 : 2))) void decode_partial_kernel(
    const FwdParams p, float *ws, int unit_blocks, int max_units) {
  using M = Mma<T>;
  using vec8 = typename M::vec8;
  using S = DecSmem<D>;
  constexpr int KS = D / 16, DT = D / 32, CPR = D / 8;
  // SUB: table entries are (column, bit mask over the pattern blocks inside the 64 x 64 tile)
  constexpr int EW = SUB ? 2 : 1;  // ints per table entry
  extern __shared__ __align__(16) char smem_all[];

  const int kvh = blockIdx.y, b = blockIdx.z;
  const SeqInfo sq = load_seq(p.seqs, b, p.causal);
  if (sq.q_len <= 0) return;
  const int ratio = __builtin_amdgcn_readfirstlane(p.Hq / p.Hkv);  // integer division runs on the VALU
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int wave_bytes = 2 * S::kHalf + ratio * D * 2;
  char *smem = smem_all + wave * wave_bytes;  // this wave's private tiles and q copy
  const int m = lane & 31, g = lane >> 5;  // m = q head inside the group (MFMA column)
  const int pos = sq.past;                 // absolute position of the single query token
  const int rb = pos / 64;
  const int h0 = kvh * ratio;
  const int lh = lut_head(p.csr, h0, p.Hq, p.Hkv);
  // table reads go through the scalar unit (wave-uniform addresses, no vector-memory wait)
  int row0 = 0, row1 = 0;
  if (sq.k_len > 0 && rb < p.csr.num_rows)
    scalar_load2(p.csr.ptr + lh * p.csr.ptr_sh + rb, p.csr.ptr + lh * p.csr.ptr_sh + rb + 1, row0, row1);
  // the row's entries are split evenly over as many units as the unit size asks for
  const int n_ent = row1 - row0;
  // never more than the host sized the grid and the workspace for: a row longer than the caller's
  // max_row_entries hint said is still cut into max_units units, each with a larger share
  const int u_cnt = min(decode_row_units(n_ent, unit_blocks, W), max_units);
  if ((int)blockIdx.x * W >= u_cnt && blockIdx.x > 0) return;  // nothing for this workgroup
  const bool merge_here = u_cnt <= W;  // (a row without entries is written here too: O = 0, LSE = -inf)
  const int per = u_cnt > 0 ? (n_ent + u_cnt - 1) / u_cnt : 0;
  const int unit = blockIdx.x * W + wave;
  const bool active = unit < u_cnt;
  if (!active && !merge_here) return;
  const int e0 = row0 + unit * per;
  const int e1 = active ? min(e0 + per, row1) : e0;
  const int32_t *cols = p.csr.idx + lh * p.csr.idx_sh;
  // SUB: the query's row of pattern blocks inside its tile selects f of the entry's f x f mask
  // bits; half block hb & 1 holds key parts [hb & 1, hb & 1 + 1) * f / 2 of them
  const int lb = SUB ? (p.csr.sub_block == 16 ? 4 : 5) : 6, f = 64 >> lb;
  const int row_shift = ((pos & 63) >> lb) * f;
  auto half_bits = [&](int bits, int hb) { return (bits >> (row_shift + (hb & 1) * (f >> 1))) & ((1 << (f >> 1)) - 1); };
  // contiguous K/V: the sequence's first key; paged K/V: the pools (pages are added per half block)
  static_assert(!KV8 || PAGED, "fp8 K/V comes through the paged entry");
  using KV = typename std::conditional<KV8, uint8_t, T>::type;  // element type of the K/V memory
  const KV *kbase = (const KV *)p.k.ptr + kvh * p.k.sh + (PAGED ? 0 : sq.b * p.k.sb + (int64_t)sq.k_start * p.k.st);
  const KV *vbase = (const KV *)p.v.ptr + kvh * p.v.sh + (PAGED ? 0 : sq.b * p.v.sb + (int64_t)sq.k_start * p.v.st);
  // K/V bytes are read once per step: non-temporal loads keep them from displacing each other in
  // the memory-side cache (measured 44.6 -> 40.5 us per step on 32 sequences of 1K-8K tokens)
  auto load8 = [](const KV *src) -> uint4 {  // 8 head dims starting at src, as T
    if constexpr (KV8) {
      typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
      const u32x2 w = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(src));
      return fp8x8_to<T>(make_uint2(w[0], w[1]));
    } else {
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src));
      return make_uint4(w[0], w[1], w[2], w[3]);
    }
  };

  // PAGED: page numbers of the whole unit in one vector load, four lanes per table entry (a
  // 64-key block spans at most four pages of >= 16 tokens): lane 4 j + s holds the page of keys
  // [s, s + 1) * page_size of entry e0 + j (pages of >= 64 tokens: s = 0 only).  Entries of the
  // page table beyond the sequence's last token are never read; a negative entry inside the
  // sequence (a caller's mistake: such slots mark unused pages) is read as page 0 rather than
  // as an address before the pool.
  // A unit of more than 16 entries (only when the caller's max_row_entries hint understated the
  // row) reloads the register every 16 entries.
  int my_page = 0;
  auto load_pages = [&](int j0) {  // pages of entries e0 + j0 .. e0 + j0 + 15
    int pg = 0;
    const int j = j0 + (lane >> 2), s = lane & 3;
    const int ps = 1 << p.paged.page_shift;
    if (j < e1 - e0) {
      const int col = cols[(e0 + j) * EW];
      const int tok = col * 64 + (ps < 64 ? s * ps : 0);
      if (col >= 0 && tok < sq.k_len && (s == 0 || s * ps < 64))
        pg = max(p.paged.table[b * p.paged.table_sb + (tok >> p.paged.page_shift)], 0);
    }
    return pg;
  };
  if constexpr (PAGED) my_page = load_pages(0);

  // half block hb of this unit = keys cols[e0 + hb/2] * 64 + 32 * (hb & 1) + [0, 32)
  constexpr int HCH = 32 * CPR / 64;  // 16-byte chunks per lane per half tile
  uint4 kreg[HCH], vreg[HCH];
  auto prefetch = [&](int hb, int col, int bits) {
    const int key0 = col * 64 + (hb & 1) * 32;
    if constexpr (PAGED)
      if (hb > 0 && (hb & 31) == 0) my_page = load_pages(hb >> 1);  // (never with the default unit sizes)
    if (SUB && half_bits(bits, hb) == 0) return;  // no attended key in this half: neither read nor used
    // element offset of row r of the half block from kbase / vbase
    int pg_lo = 0, pg_hi = 0, in_page0 = 0;
    if constexpr (PAGED) {
      // the half block's 32 keys lie in one page, or in two pages of 16
      const int psl = p.paged.page_shift, half = hb & 1;
      const int s_lo = psl < 6 ? (half * 32) >> psl : 0, s_hi = psl < 6 ? (half * 32 + 16) >> psl : 0;
      // (lane-indexed reads: the compiler may route the lane number through M0.  Nothing in this
      // file writes M0 behind its back - the LDS DMA helpers of mfma_common.h, which do, are not
      // used by the decode kernels.)
      pg_lo = __builtin_amdgcn_readlane(my_page, (((hb >> 1) & 15) * 4 + s_lo) & 63);
      pg_hi = __builtin_amdgcn_readlane(my_page, (((hb >> 1) & 15) * 4 + s_hi) & 63);
      in_page0 = key0 & ((1 << psl) - 1);
    }
    auto k_off = [&](int r) -> int64_t {
      if constexpr (PAGED) {
        const int in_page = (in_page0 + r) & ((1 << p.paged.page_shift) - 1);
        return (int64_t)(r < 16 ? pg_lo : pg_hi) * p.paged.k_page_stride + (int64_t)in_page * p.k.st;
      } else {
        return (int64_t)(key0 + r) * p.k.st;
      }
    };
    auto v_off = [&](int r) -> int64_t {
      if constexpr (PAGED) {
        const int in_page = (in_page0 + r) & ((1 << p.paged.page_shift) - 1);
        return (int64_t)(r < 16 ? pg_lo : pg_hi) * p.paged.v_page_stride + (int64_t)in_page * p.v.st;
      } else {
        return (int64_t)(key0 + r) * p.v.st;
      }
    };
    if (!PAD && col >= 0 && key0 + 32 <= sq.k_len) {  // whole half inside the sequence: no guards
#pragma unroll
      for (int c = 0; c < HCH; ++c) {
        const int idx = lane + c * 64;
        const int r = idx / CPR, ch = idx % CPR;
        kreg[c] = load8(kbase + k_off(r) + ch * 8);
        vreg[c] = load8(vbase + v_off(r) + ch * 8);
      }
    } else {  // rows beyond the sequence and (PAD) head dims beyond p.D read as zeros
#pragma unroll
      for (int c = 0; c < HCH; ++c) {
        const int idx = lane + c * 64;
        const int r = idx / CPR, ch = idx % CPR;
        kreg[c] = vreg[c] = make_uint4(0, 0, 0, 0);
        if (col >= 0 && key0 + r < sq.k_len && (!PAD || ch * 8 < p.D)) {
          kreg[c] = load8(kbase + k_off(r) + ch * 8);
          vreg[c] = load8(vbase + v_off(r) + ch * 8);
        }
      }
    }
  };
  // the first K/V request goes out before anything else touches memory
  int col_cur = 0, bits_cur = 0;
  if (e0 < e1) {  // (an even split can leave the last units of a row without entries: neutral partials)
    if constexpr (SUB)
      scalar_load2(cols + e0 * EW, cols + e0 * EW + 1, col_cur, bits_cur);
    else
      col_cur = scalar_load(cols + e0);
    prefetch(0, col_cur, bits_cur);
  }

  // q of the group's heads -> LDS (row min(m, ratio-1) feeds MFMA column m;
  // columns >= ratio are duplicates whose results are never stored)
  char *ks_ = smem, *vs_ = smem + S::kHalf, *qs_ = smem + 2 * S::kHalf;
  {
    const int hh = lane / CPR, ch = lane % CPR;  // 64 lanes cover 64 / CPR heads per pass
    for (int h = hh; h < ratio; h += 64 / CPR) {
      const T *qp = (const T *)p.q.ptr + sq.b * p.q.sb + (int64_t)(h0 + h) * p.q.sh + (int64_t)sq.q_start * p.q.st;
      uint4 w = make_uint4(0, 0, 0, 0);
      if (!PAD || ch * 8 < p.D) w = *reinterpret_cast<const uint4 *>(qp + ch * 8);
      *reinterpret_cast<uint4 *>(qs_ + h * D * 2 + ch * 16) = w;
    }
  }
  const int q_read = (m < ratio ? m : ratio - 1) * D * 2 + g * 16;

  floatx16 oacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  const int k_read = m * S::kStride + g * 16;
  const int i16 = lane & 15, dgrp = (lane >> 4) & 1;
  const int v_read = (4 * g + (i16 >> 2)) * S::kStride + (16 * dgrp + 4 * (i16 & 3)) * 2;
  const int nhalf = 2 * (e1 - e0);

  for (int hb = 0; hb < nhalf; ++hb) {
    const int col = col_cur;
    const int hbits = SUB ? half_bits(bits_cur, hb) : 1;
    const int key0 = col * 64 + (hb & 1) * 32;
    // table entry of the next half block (the next block after an odd half)
    if ((hb & 1) && hb + 1 < nhalf) {
      const int32_t *ent = cols + (e0 + ((hb + 1) >> 1)) * EW;
      if constexpr (SUB)
        scalar_load2(ent, ent + 1, col_cur, bits_cur);
      else
        col_cur = scalar_load(ent);
    }
    // The tiles are private to this wave and LDS operations of one wave
    // execute in order, so the previous half block's reads are done; only the
    // compiler must not reorder across these points (a memory fence would
    // also drain the global prefetch issued next).
    asm volatile("" ::: "memory");
    if (hbits != 0) {  // (a half without attended keys was not read)
#pragma unroll
      for (int c = 0; c < HCH; ++c) {
        const int idx = lane + c * 64;
        const int r = idx / CPR, ch = idx % CPR;
        *reinterpret_cast<uint4 *>(ks_ + r * S::kStride + ch * 16) = kreg[c];
        *reinterpret_cast<uint4 *>(vs_ + r * S::kStride + ch * 16) = vreg[c];
      }
    }
    asm volatile("" ::: "memory");
    if (hb + 1 < nhalf) prefetch(hb + 1, col_cur, bits_cur);
    if (hbits == 0 || col < 0 || key0 >= sq.k_len || (p.causal && key0 > pos)) continue;

    floatx16 sacc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
    {
      vec8 a[KS], qb[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        a[ks] = lds_read8<vec8>(ks_ + k_read + ks * 32);
        qb[ks] = lds_read8<vec8>(qs_ + q_read + ks * 32);
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) sacc = M::mma(a[ks], qb[ks], sacc);
    }
    const bool need_mask = (key0 + 31 >= sq.k_len) || (p.causal && key0 + 31 > pos);
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float sv = sacc[r] * p.scale_log2;
      if constexpr (SUB) {
        // key 8 (r / 4) + 4 g + r % 4 of the half: the last two terms stay inside a part of >= 16 keys
        if (!((hbits >> (((r >> 2) * 8) >> lb)) & 1)) sv = -INFINITY;
      }
      if (need_mask) {
        const int key = key0 + (r >> 2) * 8 + g * 4 + (r & 3);
        if (key >= sq.k_len || (p.causal && key > pos)) sv = -INFINITY;
      }
      sacc[r] = sv;
      mx = fmaxf(mx, sv);
    }
    mx = fmaxf(mx, xor32(mx));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_use);
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float pv = fast_exp2(sacc[r] - m_use);
      sacc[r] = pv;
      psum += pv;
    }
    psum += xor32(psum);
    l_run = l_run * alpha + psum;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      float pf[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) pf[i] = sacc[t * 8 + i];
      const vec8 pb = M::pack(pf);
      const char *vrow = vs_ + v_read + t * 16 * S::kStride;
      vec8 a[DT];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) a[dt] = lds_read_tr8<vec8>(vrow + dt * 64, vrow + 8 * S::kStride + dt * 64);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) oacc[dt] = M::mma(a[dt], pb, oacc[dt]);
    }
  }

  // ---- partial result of this unit: lanes (m < ratio) hold head h0 + m ----
  // rows [head][D + 2] floats (O unnormalised, max, sum): in the workspace, or, when the row is
  // finished here, in this wave's own tile area (its tiles are dead by now)
  if (m < ratio) {
    float *dst = merge_here ? reinterpret_cast<float *>(smem) + m * (D + 2)
                            : ws + (((int64_t)b * p.Hq + h0 + m) * max_units + unit) * (D + 2);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4)
        *reinterpret_cast<float4 *>(dst + dt * 32 + r4 * 8 + g * 4) =
            make_float4(oacc[dt][r4 * 4], oacc[dt][r4 * 4 + 1], oacc[dt][r4 * 4 + 2], oacc[dt][r4 * 4 + 3]);
    if (g == 0) {
      dst[D] = m_run;
      dst[D + 1] = l_run;
    }
  }
  {
    if (!merge_here) return;
    __syncthreads();  // every wave of the workgroup gets here (merge_here is workgroup-uniform)
    // heads of the group are dealt to the waves; lane l owns dims l D/64 .. of its head
    constexpr int PER = D / 64;
    for (int h = wave; h < ratio; h += W) {
      float mv[W], lv[W], ov[W][PER];
#pragma unroll
      for (int u = 0; u < W; ++u) {
        const float *row = reinterpret_cast<const float *>(smem_all + u * wave_bytes) + h * (D + 2);
        mv[u] = row[D];
        lv[u] = row[D + 1];
#pragma unroll
        for (int i = 0; i < PER; ++i) ov[u][i] = row[lane * PER + i];
      }
      float mmax = mv[0];
#pragma unroll
      for (int u = 1; u < W; ++u) mmax = fmaxf(mmax, mv[u]);
      const float muse = mmax == -INFINITY ? 0.f : mmax;
      float l = 0.f, o[PER];
#pragma unroll
      for (int i = 0; i < PER; ++i) o[i] = 0.f;
#pragma unroll
      for (int u = 0; u < W; ++u) {
        const float sc = fast_exp2(mv[u] - muse);  // a wave without entries has max = -inf: weight 0
        l += sc * lv[u];
#pragma unroll
        for (int i = 0; i < PER; ++i) o[i] += sc * ov[u][i];
      }
      const float inv = l > 0.f ? (p.paged.table ? p.paged.out_scale : 1.f) / l : 0.f;
      T *op = (T *)p.o.ptr + sq.b * p.o.sb + (int64_t)(h0 + h) * p.o.sh + (int64_t)sq.q_start * p.o.st;
#pragma unroll
      for (int i = 0; i < PER; ++i)
        if (!PAD || lane * PER + i < p.D) op[lane * PER + i] = from_float<T>(o[i] * inv);
      if (p.lse.ptr && lane == 0)
        p.lse.ptr[sq.b * p.lse.sb + (h0 + h) * p.lse.sh + (int64_t)sq.q_start * p.lse.st] =
            l > 0.f ? (mmax + log2f(l)) * kLn2 : -INFINITY;
    }
  }
}

// Merge of the unit partials: one wave per (sequence, q head), lane l owns
// dims {2l, 2l+1} (D = 128) or dim l (D = 64).  All loads of a row are issued
// before the first use (units are few, a dependent load chain per unit would
// make this small kernel latency-bound).
template <typename T, int D, bool PAD>
__global__ __launch_bounds__(64) void decode_combine_kernel(const FwdParams p, const float *ws, int unit_blocks,
                                                            int max_units, int merged_units) {
  constexpr int PER = D / 64;  // dims per lane
  constexpr int MAXU = 8;      // units merged per pass
  const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
  const SeqInfo sq = load_seq(p.seqs, b, p.causal);
  if (sq.q_len <= 0) return;
  int units = 0;
  const int rb = sq.past / 64;
  if (sq.k_len > 0 && rb < p.csr.num_rows) {
    const int lh = lut_head(p.csr, h, p.Hq, p.Hkv);
    const int n = scalar_load(p.csr.ptr + lh * p.csr.ptr_sh + rb + 1) - scalar_load(p.csr.ptr + lh * p.csr.ptr_sh + rb);
    units = min(decode_row_units(n, unit_blocks, merged_units), max_units);  // as the partial kernel
  }
  // rows of at most merged_units units (the waves of a partial-kernel workgroup) were finished there
  if (units <= merged_units) return;
  const float *src = ws + ((int64_t)b * p.Hq + h) * max_units * (D + 2);
  float mmax = -INFINITY, l = 0.f, o[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) o[i] = 0.f;
  for (int s0 = 0; s0 < units; s0 += MAXU) {
    float mv[MAXU], lv[MAXU], ov[MAXU][PER];
#pragma unroll
    for (int s = 0; s < MAXU; ++s) {
      const bool ok = s0 + s < units;
      const float *row = src + (s0 + (ok ? s : 0)) * (D + 2);
      mv[s] = ok ? row[D] : -INFINITY;
      lv[s] = ok ? row[D + 1] : 0.f;
#pragma unroll
      for (int i = 0; i < PER; ++i) ov[s][i] = ok ? row[lane * PER + i] : 0.f;
    }
    float mnew = mmax;
#pragma unroll
    for (int s = 0; s < MAXU; ++s) mnew = fmaxf(mnew, mv[s]);
    const float muse = mnew == -INFINITY ? 0.f : mnew;
    const float alpha = fast_exp2(mmax - muse);  // exp2(-inf) = 0 on the first pass
    l *= alpha;
#pragma unroll
    for (int i = 0; i < PER; ++i) o[i] *= alpha;
#pragma unroll
    for (int s = 0; s < MAXU; ++s) {
      const float sc = fast_exp2(mv[s] - muse);
      l += sc * lv[s];
#pragma unroll
      for (int i = 0; i < PER; ++i) o[i] += sc * ov[s][i];
    }
    mmax = mnew;
  }
  const float inv = l > 0.f ? (p.paged.table ? p.paged.out_scale : 1.f) / l : 0.f;
  T *op = (T *)p.o.ptr + sq.b * p.o.sb + h * p.o.sh + (int64_t)sq.q_start * p.o.st;
#pragma unroll
  for (int i = 0; i < PER; ++i)
    if (!PAD || lane * PER + i < p.D) op[lane * PER + i] = from_float<T>(o[i] * inv);  // inv includes the V scale
  if (p.lse.ptr && lane == 0)
    p.lse.ptr[sq.b * p.lse.sb + h * p.lse.sh + (int64_t)sq.q_start * p.lse.st] =
        l > 0.f ? (mmax + log2f(l)) * kLn2 : -INFINITY;
}

// Unit slots per (sequence, q head) in the workspace: the longest row's units (rows that fit one
// workgroup keep their partials in LDS).
static int decode_max_units(const FwdParams &p) {
  return decode_row_units(decode_max_row_entries(p), decode_unit_blocks(p), kDecodeWaves);
}

bool decode_supported(const FwdParams &p, int dtype) {
  const int ratio = p.Hq / p.Hkv;
  const bool shared_row = p.csr.num_heads == 1 || (p.csr.num_heads == p.Hkv && p.Hkv != p.Hq) || ratio == 1 ||
                          (p.csr.num_heads == p.Hq && p.csr.group % ratio == 0);
  const int width = mfma_tile_width(p.D);
  const int lds = kDecodeWaves * (2 * 32 * (width * 2 + 16) + ratio * width * 2);  // DecSmem<width>::wave_bytes
  return (dtype == DK_BF16 || dtype == DK_F16) && mfma_head_dim_ok(p.D) && lds <= 160 * 1024 && p.csr.block_rows == 64 &&
         p.csr.block_cols == 64 && p.vec_ok &&
         (p.csr.entry_width == 1 || p.csr.sub_block != 0) &&
         (p.seqs.packed ? (p.seqs.packed & 2) != 0 : p.seqs.max_q_len == 1) && ratio <= 32 && shared_row && p.causal &&
         !p.seqs.zero_outside;  // (rows without a query are cleared by the prefill kernels only)
}

size_t decode_workspace_bytes(const FwdParams &p) {
  return (size_t)p.seqs.batch * p.Hq * decode_max_units(p) * (mfma_tile_width(p.D) + 2) * sizeof(float);
}

template <typename T, int D, bool PAD, bool SUB, bool PAGED, bool KV8 = false>
static int launch_decode_td(const FwdParams &p, float *ws, hipStream_t stream) {
  constexpr int W = kDecodeWaves;
  const int smem = W * DecSmem<D>::wave_bytes(p.Hq / p.Hkv);
  const int unit_blocks = decode_unit_blocks(p), max_units = decode_max_units(p);
  const int groups = cdiv(max_units, W);
  DK_REQUIRE(groups <= 65535, "too many decode units");
  DK_REQUIRE(smem <= 160 * 1024, "decode workgroup needs %d bytes of LDS", smem);
  DK_ALLOW_DYNAMIC_LDS((decode_partial_kernel<T, D, PAD, SUB, PAGED, KV8, W>), smem);
  DK_NOTE_KERNEL("decode_partial_kernel");
  hipLaunchKernelGGL((decode_partial_kernel<T, D, PAD, SUB, PAGED, KV8, W>), dim3(groups, p.Hkv, p.seqs.batch),
                     dim3(64 * W), smem, stream, p, ws, unit_blocks, max_units);
  DK_HIP_CHECK(hipGetLastError());
  if (groups == 1) return DK_OK;  // every row was finished inside its workgroup
  DK_NOTE_KERNEL("decode_combine_kernel");
  hipLaunchKernelGGL((decode_combine_kernel<T, D, PAD>), dim3(p.Hq, p.seqs.batch), dim3(64), 0, stream, p, ws,
                     unit_blocks, max_units, W);
  DK_HIP_CHECK(hipGetLastError());
  return DK_OK;
}

template <typename T, bool PAGED>
static int launch_decode_tp(const FwdParams &p, float *ws, hipStream_t stream) {
  if (p.D > 128)  // 256-wide tiles (always the zero-padding instantiation), one wave per SIMD
    return p.csr.sub_block ? launch_decode_td<T, 256, true, true, PAGED>(p, ws, stream)
                           : launch_decode_td<T, 256, true, false, PAGED>(p, ws, stream);
  if (p.csr.sub_block) {  // entries carry a bit mask over the pattern's 16- or 32-token blocks
    if (p.D == 128) return launch_decode_td<T, 128, false, true, PAGED>(p, ws, stream);
    if (p.D == 64) return launch_decode_td<T, 64, false, true, PAGED>(p, ws, stream);
    return p.D > 64 ? launch_decode_td<T, 128, true, true, PAGED>(p, ws, stream)
                    : launch_decode_td<T, 64, true, true, PAGED>(p, ws, stream);
  }
  if (p.D == 128) return launch_decode_td<T, 128, false, false, PAGED>(p, ws, stream);
  if (p.D == 64) return launch_decode_td<T, 64, false, false, PAGED>(p, ws, stream);
  return p.D > 64 ? launch_decode_td<T, 128, true, false, PAGED>(p, ws, stream)
                  : launch_decode_td<T, 64, true, false, PAGED>(p, ws, stream);
}

// head dims below the tile width (64 or 128) run the zero-padded instantiation; K/V come from the
// tensors themselves or, with a page table, from page pools
template <typename T>
static int launch_decode_t(const FwdParams &p, float *ws, hipStream_t stream) {
  if (p.paged.table && p.paged.kv_fp8) {  // fp8 pools: plain tiles only
    if (p.csr.sub_block || (p.D != 64 && p.D != 128))
      return fail(DK_ERR_UNSUPPORTED, "fp8 K/V needs head_dim 64 or 128 and pattern blocks of at least 64");
    return p.D == 128 ? launch_decode_td<T, 128, false, false, true, true>(p, ws, stream)
                      : launch_decode_td<T, 64, false, false, true, true>(p, ws, stream);
  }
  return p.paged.table ? launch_decode_tp<T, true>(p, ws, stream) : launch_decode_tp<T, false>(p, ws, stream);
}

int launch_decode(const FwdParams &p, int dtype, void *workspace, size_t workspace_bytes, hipStream_t stream) {
  DK_REQUIRE(workspace && workspace_bytes >= decode_workspace_bytes(p), "decode workspace too small");
  DK_REQUIRE(((uintptr_t)workspace % 16) == 0, "decode workspace must be 16-byte aligned");
  float *ws = (float *)workspace;
  return dtype == DK_BF16 ? launch_decode_t<bf16_t>(p, ws, stream) : launch_decode_t<f16_t>(p, ws, stream);
}

}  // namespace dk
