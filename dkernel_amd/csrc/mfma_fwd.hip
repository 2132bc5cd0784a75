// MFMA forward kernel for gfx950: bf16 / fp16, head dims up to 256 (tiles of 64, 128 or 256 columns), 64 x 64
// blocks.  Online-softmax attention over the K/V blocks listed in the CSR
// look-up table, with LSE.
//
// Work split
//   workgroup = one 64-row q block x G q heads that share a kv head and a
//               look-up-table row (G = 1, 2 or 4), so a K/V block is fetched
//               from HBM/L2 once for all G heads;
//   wave      = 32 q rows of one head (2 waves per head, 2G waves per group).
// Per listed block a wave computes S^T = K Q^T (n x m) with
// v_mfma_f32_32x32x16: the accumulator layout (lane = q row, registers = keys)
// makes the softmax reductions per-lane plus one exchange with the other
// half-wave, and feeds P^T to the second product O^T += V^T P^T as the B
// operand straight from registers.  V stays row-major in LDS; its transposed
// operand comes from LDS transpose reads.  K/V tiles are double buffered in
// LDS (one barrier per block) and copied HBM -> LDS asynchronously, without
// staging registers, while the current one is being multiplied.
//
// Grid: x = head group (fastest, so that the 8 XCDs, which receive
// workgroups round-robin, each keep a fixed set of kv heads in their L2),
// y = q tile with the longest rows first, z = batch.
#include "common.h"
#include "device_common.h"
#include "mfma_common.h"

namespace dk {

template <int V>
struct Const {  // compile-time integer passed to a generic lambda
  static constexpr int value = V;
};

template <int D>
struct FwdSmem {  // one stage = K tile + V tile, swizzled row-major (mfma_common.h)
  static constexpr int kStage = 2 * Tile<D>::kBytes;
};

// At the 256-wide tile (head dims above 128) a wave needs more than 256 registers: one wave per
// SIMD, workgroups of at most two heads.
// At the 64-wide tile a wave needs ~150 registers, so three waves fit a SIMD (three 4-wave
// workgroups per CU): the softmax of one wave then has two others to hide behind.
template <typename T, int D, int G, bool PAD, bool RP, bool SUB = false>
__global__ __launch_bounds__(128 * G) __attribute__((amdgpu_waves_per_eu(G == 1 || D == 256 ? 1 : 2, D == 64 ? 3 : D == 256 ? 1 : 2))) void mfma_fwd_kernel(const FwdParams p, int tiles_y) {
  using M = Mma<T>;
  using vec8 = typename M::vec8;
  using S = FwdSmem<D>;
  constexpr int NT = 128 * G;   // threads
  constexpr int KS = D / 16;    // k-steps of the QK^T product
  constexpr int DT = D / 32;    // d-tiles of the output
  using TL = Tile<D>;
  extern __shared__ __align__(16) char smem[];

  static_assert(!RP || G == 2, "row pairs: two wave pairs, one q tile each");
  // SUB: table entries are (column, bit mask over the pattern blocks inside the 64 x 64 tile)
  static_assert(!SUB || !RP, "sub-block masks: one q tile per workgroup");
  constexpr int EW = SUB ? 2 : 1;  // ints per table entry
  SeqInfo sq;
  int tile;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: row tests and head indices follow it
  int rb;
  int first_rb = 0, last_rb = 0;  // RP: table rows that hold queries of this sequence
  if constexpr (RP) {
    // workgroup = table rows 2u and 2u + 1 of one head (one per wave pair); tiles_y counts pairs
    int u;
    if (p.seqs.packed) {
      // the sequences share one token dimension: row pairs are counted through all of them (last
      // pair first: within a sequence the longest rows start first, as for unpacked inputs)
      int idx;
      const int b = find_packed_sequence(
          p.seqs, p.causal, tiles_y - 1 - (int)blockIdx.y,
          [](const SeqInfo &t) { return seq_row_pairs(t); }, idx);
      if (b < 0) return;
      sq = load_seq(p.seqs, b, p.causal);
      first_rb = sq.past / 64, last_rb = (sq.past + sq.q_len - 1) / 64;
      u = (first_rb >> 1) + idx;
    } else {
      sq = load_seq(p.seqs, blockIdx.z, p.causal);
      first_rb = sq.past / 64, last_rb = (sq.past + sq.q_len - 1) / 64;
      if (p.csr.pair_order)  // the table's own order, longest pairs first (the grid then covers every pair of it)
        u = scalar_load(p.csr.pair_order + lut_head(p.csr, grid_head(p.csr), p.Hq, p.Hkv) * p.csr.order_sh + blockIdx.y);
      else
        u = (first_rb >> 1) + tiles_y - 1 - (int)blockIdx.y;
      if (sq.q_len <= 0 || u > (last_rb >> 1) || u < (first_rb >> 1)) {  // no rows here: only the share of the padding rows, if asked
        if (p.seqs.zero_outside)
          zero_rows_outside<T>(p.seqs, sq, blockIdx.y, tiles_y, p.o, p.lse, grid_head(p.csr), 1, p.D, p.vec_ok, tid, NT);
        return;
      }
    }
    rb = 2 * u + (wave >> 1);
    tile = rb - first_rb;  // outside [0, last_rb - first_rb]: this wave pair has no rows (row_ok false everywhere)
  } else {
    const int ty = tiles_y - 1 - (int)blockIdx.y;  // longest rows first (of a causal pattern)
    bool has_rows;
    if (p.csr.order && !p.seqs.packed) {  // the table's own order, longest rows first (the grid then covers every row of it)
      sq = load_seq(p.seqs, blockIdx.z, p.causal);
      tile = scalar_load(p.csr.order + lut_head(p.csr, grid_head(p.csr) * G, p.Hq, p.Hkv) * p.csr.order_sh + blockIdx.y) -
             sq.past / 64;
      has_rows = tile >= 0 && tile < seq_row_blocks(sq, 64);
    } else {
      has_rows = resolve_tile(p.seqs, p.causal, 64, 1, ty, blockIdx.z, sq, tile);
    }
    if (!has_rows) {
      if (p.seqs.zero_outside)  // (never with packed inputs, for which sq is not set here)
        zero_rows_outside<T>(p.seqs, sq, blockIdx.y, tiles_y, p.o, p.lse, grid_head(p.csr) * G, G, p.D, p.vec_ok, tid, NT);
      return;
    }
    rb = sq.past / 64 + tile;
  }
  if constexpr (PAD) {  // the slots of the head dims beyond p.D stay zero for the whole kernel
    zero_tiles<NT>(smem, 2 * S::kStage, tid);
    __syncthreads();
  }
  const int hx = grid_head(p.csr);  // head (row pairs) or group of G heads of this workgroup
  const int h = RP ? hx : hx * G + (wave >> 1);
  const int kvh = __builtin_amdgcn_readfirstlane(h / (p.Hq / p.Hkv));  // integer division runs on the VALU
  const int m = lane & 31, g = lane >> 5;
  const int row0 = rb * 64 + (wave & 1) * 32;  // first absolute position of this wave
  const int pos = row0 + m;
  const int qi = pos - sq.past;
  const bool row_ok = qi >= 0 && qi < sq.q_len;

  // ---- Q fragments (B operand of S^T = K Q^T), resident in registers ----
  vec8 qf[KS];
  {
    const T *qp = (const T *)p.q.ptr + sq.b * p.q.sb + h * p.q.sh + (int64_t)(sq.q_start + qi) * p.q.st;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 w = make_uint4(0, 0, 0, 0);
      if (row_ok && (!PAD || ks * 16 + g * 8 < p.D)) w = *reinterpret_cast<const uint4 *>(qp + ks * 16 + g * 8);
      qf[ks] = as_vec8<vec8>(w);
    }
  }

  const int lh = lut_head(p.csr, RP ? hx : hx * G, p.Hq, p.Hkv);
  int e0 = 0, e1 = 0;
  int emid = 0;  // RP: entries [e0, emid) are row 2u, [emid, e1) row 2u + 1 (consecutive rows follow each other)
  if constexpr (RP) {
    const int32_t *rp = p.csr.ptr + lh * p.csr.ptr_sh;
    const int ra = rb & ~1;
    if (ra < p.csr.num_rows) scalar_load2(rp + ra, rp + ra + 1, e0, emid);
    e1 = emid;
    if (ra + 1 < p.csr.num_rows) e1 = scalar_load(rp + ra + 2);
    if (ra < first_rb) e0 = emid;     // a row without queries of this sequence contributes nothing
    if (ra + 1 > last_rb) e1 = emid;
  } else if (rb < p.csr.num_rows) {  // table reads go through the scalar unit (no vector-memory wait)
    scalar_load2(p.csr.ptr + lh * p.csr.ptr_sh + rb, p.csr.ptr + lh * p.csr.ptr_sh + rb + 1, e0, e1);
  }
  const int32_t *cols = p.csr.idx + lh * p.csr.idx_sh;
  const T *kbase = (const T *)p.k.ptr + sq.b * p.k.sb + kvh * p.k.sh + (int64_t)sq.k_start * p.k.st;
  const T *vbase = (const T *)p.v.ptr + sq.b * p.v.sb + kvh * p.v.sh + (int64_t)sq.k_start * p.v.st;

  // ---- asynchronous HBM -> LDS copy of one K/V tile pair (no staging registers) ----
  TileLoader<D, NT, PAD> kload, vload;
  kload.init(tid, p.k.st, p.D);
  vload.init(tid, p.v.st, p.D);
  // blocks whose first key lies in [0, k_full_span) hold 64 keys of the sequence
  const uint32_t k_full_span = sq.k_len >= 64 ? (uint32_t)(sq.k_len - 64) + 1u : 0u;
  const uint32_t k_row_bytes = (uint32_t)p.k.st * 2u, v_row_bytes = (uint32_t)p.v.st * 2u;
  auto issue = [&](int col, int stage) {
    const int key0 = col * 64;
    char *ks = smem + stage * S::kStage;
    // (not at the 256-wide tile, nor for one padded head per workgroup: the extra state pushes
    // those instantiations into scratch spills)
    if (D <= 128 && !(PAD && G == 1) && (uint32_t)key0 < k_full_span) {  // main path (one scalar compare; a padding entry is negative)
      kload.issue_full(row_address(reinterpret_cast<const char *>(kbase), key0, k_row_bytes), ks);
      vload.issue_full(row_address(reinterpret_cast<const char *>(vbase), key0, v_row_bytes), ks + TL::kBytes);
      return;
    }
    const int valid = col < 0 ? 0 : sq.k_len - key0;
    kload.issue(reinterpret_cast<const char *>(kbase + (int64_t)key0 * p.k.st), 0, valid, ks);
    vload.issue(reinterpret_cast<const char *>(vbase + (int64_t)key0 * p.v.st), 0, valid, ks + TL::kBytes);
  };

  floatx16 oacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;  // running max (log2 domain) and sum of row `pos`

  // loop-invariant LDS offsets of this lane's operand reads (row m of a 32-key tile, swizzled
  // chunk 2ks+g; transpose-read pairs of d-tile dt); tile / k-step row offsets are immediates
  // (full pointers, and the stage is a compile-time constant of the loop body, so that stage,
  // tile and k-step offsets all end up as instruction immediates)
  using OA = OperandAddress<D>;
  typename OA::type rd[KS], tr[DT][2];
  {
    int tro[DT][2];
    transposed_offsets<D>(lane, tro);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) rd[ks] = OA::make(smem, TL::off(m, 2 * ks + g));
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) tr[dt][0] = OA::make(smem, tro[dt][0]), tr[dt][1] = OA::make(smem, tro[dt][1]);
  }

  // Table entries: block e in col_cur (scalar register); block e + 1 is requested one block
  // early as a vector load (col_pending) and first used behind the next tile wait, so that no
  // table read ever stalls the loop.
  //
  // RP: the workgroup walks the union of its two rows' entries in column order (both rows are
  // sorted), merging them on the fly: head_a / head_b are the next unconsumed entries (scalar),
  // pend_a / pend_b the entries after them (vector loads, consumed behind a tile wait like
  // col_pending); flg says which rows hold the current column.  A wave pair whose row does not
  // hold it only takes part in the copy and the barrier.
  constexpr int kEnd = 0x7fffffff;
  int col_cur = 0, col_pending = 0;
  int bits_cur = 0, bits_pending = 0;  // SUB: the entry's mask, carried like the column
  int a_pos = e0, b_pos = emid, head_a = kEnd, head_b = kEnd, pend_a = 0, pend_b = 0, flg_cur = 0;
  if constexpr (RP) {
    if (a_pos < emid) head_a = scalar_load(cols + a_pos);
    if (b_pos < e1) head_b = scalar_load(cols + b_pos);
    if (a_pos + 1 < emid) pend_a = cols[a_pos + 1];
    if (b_pos + 1 < e1) pend_b = cols[b_pos + 1];
    col_cur = min(head_a, head_b);
    flg_cur = (head_a == col_cur ? 1 : 0) | (head_b == col_cur ? 2 : 0);
    if (col_cur != kEnd) issue(col_cur, 0);
  } else {
    col_cur = e0 < e1 ? scalar_load(cols + e0 * EW) : 0;
    col_pending = e0 + 1 < e1 ? cols[(e0 + 1) * EW] : 0;
    if constexpr (SUB) {
      bits_cur = e0 < e1 ? scalar_load(cols + e0 * EW + 1) : 0;
      bits_pending = e0 + 1 < e1 ? cols[(e0 + 1) * EW + 1] : 0;
    }
    if (e0 < e1) issue(col_cur, 0);
  }
  auto block_step = [&](int e, auto stage_tag) {
    constexpr int stage = decltype(stage_tag)::value;
    const int col = col_cur;
    const int bits = bits_cur;
    wait_tile_loads();
    __syncthreads();  // tile e is visible; every wave is done with the other stage
    if constexpr (RP) {
      const int flg = flg_cur;
      if (flg & 1) {
        ++a_pos;
        head_a = a_pos < emid ? __builtin_amdgcn_readfirstlane(pend_a) : kEnd;
        if (a_pos + 1 < emid) pend_a = cols[a_pos + 1];
      }
      if (flg & 2) {
        ++b_pos;
        head_b = b_pos < e1 ? __builtin_amdgcn_readfirstlane(pend_b) : kEnd;
        if (b_pos + 1 < e1) pend_b = cols[b_pos + 1];
      }
      const int col_next = min(head_a, head_b);
      flg_cur = (head_a == col_next ? 1 : 0) | (head_b == col_next ? 2 : 0);
      if (col_next != kEnd) issue(col_next, stage ^ 1);
      col_cur = col_next;
      if (!((flg >> __builtin_amdgcn_readfirstlane(wave >> 1)) & 1)) return;  // not in this wave pair's row
    } else {
      const int col_next = __builtin_amdgcn_readfirstlane(col_pending);  // landed before the tile did
      if constexpr (SUB) bits_cur = __builtin_amdgcn_readfirstlane(bits_pending);
      if (e + 2 < e1) {
        col_pending = cols[(e + 2) * EW];
        if constexpr (SUB) bits_pending = cols[(e + 2) * EW + 1];
      }
      if (e + 1 < e1) issue(col_next, stage ^ 1);
      col_cur = col_next;
    }
    const int key0 = col * 64;
    if (col < 0 || key0 >= sq.k_len || (p.causal && key0 > row0 + 31)) return;  // nothing visible (wave-uniform)
    constexpr int ks_ = stage * S::kStage, vs_ = ks_ + TL::kBytes;  // byte offsets of this stage's K and V tiles

    // S^T = K Q^T : two 32-key tiles.  Operand reads run one tile ahead of the
    // multiplies so that LDS latency is hidden behind the MFMA pipe.
    floatx16 sacc[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[nt][r] = 0.f;
    // The scheduler barriers pin the order "issue a batch of LDS reads, then
    // multiply the previous batch": left alone, the compiler sinks every read
    // next to its MFMA and each multiply then waits out the LDS latency.
    vec8 va[2][DT];
    if constexpr (D == 256) {
      // 256-wide tiles: the K operands of a 32-key tile are fetched in two batches of eight, so
      // that they fit the register file next to the 128 accumulator registers
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int kb = 0; kb < KS; kb += 8) {
          vec8 ka[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) ka[i] = lds_operand<vec8>(rd[kb + i] + ks_ + nt * 32 * TL::kRowBytes);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int i = 0; i < 8; ++i) sacc[nt] = M::mma(ka[i], qf[kb + i], sacc[nt]);
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) va[0][dt] = lds_operand_tr<vec8>(tr[dt][0] + vs_, tr[dt][1] + vs_);
    } else {
      vec8 ka[2][KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ka[0][ks] = lds_operand<vec8>(rd[ks] + ks_);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ka[1][ks] = lds_operand<vec8>(rd[ks] + ks_ + 32 * TL::kRowBytes);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) sacc[0] = M::mma(ka[0][ks], qf[ks], sacc[0]);
      // first V^T operands do not depend on the softmax: fetch them behind the multiplies
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) va[0][dt] = lds_operand_tr<vec8>(tr[dt][0] + vs_, tr[dt][1] + vs_);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) sacc[1] = M::mma(ka[1][ks], qf[ks], sacc[1]);
      __builtin_amdgcn_sched_barrier(0);
    }

    // online softmax in the log2 domain.  Register r of tile nt is key
    // 32nt + 8(r/4) + 4g + r%4.  m_run is a reference maximum that is only
    // raised when a row's maximum grows by more than 2^8 (the accumulator
    // and the row sum stay consistent with it, so the result is exact).
    if constexpr (SUB) {
      // pattern blocks of the tile that this row does not attend: bit (row part) * f + (key part)
      const int lb = p.csr.sub_block == 16 ? 4 : 5, f = 64 >> lb;
      const int full = f == 4 ? 0xffff : 0xf;
      if ((bits & full) != full) {  // wave-uniform
        const int row_part = ((wave & 1) * 32 + m) >> lb;
        const int row_bits = bits >> (row_part * f);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            // key 32 nt + 8 (r / 4) + 4 g + r % 4: the last two terms stay inside a part of >= 16 keys
            const int key_part = (nt * 32 + (r >> 2) * 8) >> lb;
            sacc[nt][r] = ((row_bits >> key_part) & 1) ? sacc[nt][r] : -INFINITY;
          }
      }
    }
    const bool need_mask = (key0 + 63 >= sq.k_len) || (p.causal && key0 + 63 > row0);
    if (need_mask) {
      const int lim = p.causal ? min(pos, sq.k_len - 1) : sq.k_len - 1;  // last visible key of this row
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = key0 + nt * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
          sacc[nt][r] = key > lim ? -INFINITY : sacc[nt][r];
        }
    }
    float mx = max2(sacc[0][0], sacc[1][0]);
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = max3(mx, sacc[0][r], sacc[1][r]);
    mx = max_with_other_half(mx) * p.scale_log2;  // scale > 0: max commutes with it
    if (__builtin_amdgcn_ballot_w64(mx > m_run + 8.f) != 0) {  // wave-uniform: some row needs a new reference
      const float m_new = fmaxf(m_run, mx);
      const float alpha = fast_exp2(m_run - (m_new == -INFINITY ? 0.f : m_new));
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
      m_run = m_new;
    }
    const float m_use = m_run == -INFINITY ? 0.f : m_run;
    float psum = 0.f;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pv = fast_exp2(fmaf(sacc[nt][r], p.scale_log2, -m_use));
        sacc[nt][r] = pv;
        psum += pv;
      }
    // fp32 sum of the unrounded probabilities (the LSE has to hold 1e-3); per-lane partial,
    // the two half-waves are added once in the epilogue
    l_run += psum;

    // O^T += V^T P^T : k-step (nt, t) covers keys 32nt + 16t + {4g..4g+3, 8+4g..8+4g+3}
#pragma unroll
    for (int step = 0; step < 4; ++step) {
      const int nt = step >> 1, t = step & 1;
      float pf[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) pf[i] = sacc[nt][t * 8 + i];
      const vec8 pb = M::pack(pf);
      if (step < 3) {
        const int vrow = vs_ + ((step + 1) * 16) * TL::kRowBytes;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) va[(step + 1) & 1][dt] = lds_operand_tr<vec8>(tr[dt][0] + vrow, tr[dt][1] + vrow);
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) oacc[dt] = M::mma(va[step & 1][dt], pb, oacc[dt]);
    }
  };
  if constexpr (RP) {
    while (col_cur != kEnd) {
      block_step(0, Const<0>{});
      if (col_cur == kEnd) break;
      block_step(0, Const<1>{});
    }
  } else {
    for (int e = e0; e < e1; e += 2) {
      block_step(e, Const<0>{});
      if (e + 1 < e1) block_step(e + 1, Const<1>{});
    }
  }

  // l_run holds this lane's share of the row sum (keys with this lane's g)
  l_run += xor32(l_run);

  // ---- epilogue: O = O^T / l, LSE = (m + log2 l) ln 2 ----
  __syncthreads();  // the K / V stages are free: each wave stages its O tile in 32 rows of them
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  {
    const int qi0 = row0 - sq.past;  // may be negative or beyond q_len: those rows are skipped
    T *o_row0 = (T *)p.o.ptr + sq.b * p.o.sb + h * p.o.sh + (int64_t)(sq.q_start + qi0) * p.o.st;
    store_tile_rows<T, D, PAD>(smem + wave * 32 * TL::kRowBytes, oacc, inv, o_row0, p.o.st, lane, -qi0,
                               sq.q_len - qi0, p.D);
  }
  // padded inputs: this workgroup's share of the rows that hold no query, behind its own work (at
  // the start the stores of every workgroup would go out together, ahead of all multiplies)
  if (p.seqs.zero_outside)
    zero_rows_outside<T>(p.seqs, sq, blockIdx.y, tiles_y, p.o, p.lse, RP ? hx : hx * G, RP ? 1 : G, p.D,
                         p.vec_ok, tid, NT);
  if (!row_ok) return;
  if (p.lse.ptr && g == 0) {
    const float lse = l_run > 0.f ? (m_run + log2f(l_run)) * kLn2 : -INFINITY;
    p.lse.ptr[sq.b * p.lse.sb + h * p.lse.sh + (int64_t)(sq.q_start + qi) * p.lse.st] = lse;
  }
}

// Explicit instantiations: with only the implicit ones the fp16 host stubs of
// this kernel are not emitted by this compiler version.
#define DK_INSTANTIATE_FWD(T, D, PAD)                                                  \
  template __global__ void mfma_fwd_kernel<T, D, 2, PAD, false>(const FwdParams, int); \
  template __global__ void mfma_fwd_kernel<T, D, 2, PAD, true>(const FwdParams, int);  \
  template __global__ void mfma_fwd_kernel<T, D, 4, PAD, false>(const FwdParams, int);
#define DK_INSTANTIATE_FWD_SUB(T, D, PAD)                                                    \
  template __global__ void mfma_fwd_kernel<T, D, 1, PAD, false, true>(const FwdParams, int); \
  template __global__ void mfma_fwd_kernel<T, D, 2, PAD, false, true>(const FwdParams, int); \
  template __global__ void mfma_fwd_kernel<T, D, 4, PAD, false, true>(const FwdParams, int);
DK_INSTANTIATE_FWD_SUB(bf16_t, 128, false)
DK_INSTANTIATE_FWD_SUB(bf16_t, 64, false)
DK_INSTANTIATE_FWD_SUB(f16_t, 128, false)
DK_INSTANTIATE_FWD_SUB(f16_t, 64, false)
DK_INSTANTIATE_FWD_SUB(bf16_t, 128, true)
DK_INSTANTIATE_FWD_SUB(bf16_t, 64, true)
DK_INSTANTIATE_FWD_SUB(f16_t, 128, true)
DK_INSTANTIATE_FWD_SUB(f16_t, 64, true)
#undef DK_INSTANTIATE_FWD_SUB
// 256-wide tiles: the zero-padding instantiation only (it also takes head_dim 256 itself)
#define DK_INSTANTIATE_FWD_256(T)                                                            \
  template __global__ void mfma_fwd_kernel<T, 256, 2, true, false, false>(const FwdParams, int); \
  template __global__ void mfma_fwd_kernel<T, 256, 2, true, true, false>(const FwdParams, int);  \
  template __global__ void mfma_fwd_kernel<T, 256, 1, true, false, true>(const FwdParams, int);
DK_INSTANTIATE_FWD_256(bf16_t)
DK_INSTANTIATE_FWD_256(f16_t)
#undef DK_INSTANTIATE_FWD_256
DK_INSTANTIATE_FWD(bf16_t, 128, false)
DK_INSTANTIATE_FWD(bf16_t, 64, false)
DK_INSTANTIATE_FWD(f16_t, 128, false)
DK_INSTANTIATE_FWD(f16_t, 64, false)
DK_INSTANTIATE_FWD(bf16_t, 128, true)
DK_INSTANTIATE_FWD(bf16_t, 64, true)
DK_INSTANTIATE_FWD(f16_t, 128, true)
DK_INSTANTIATE_FWD(f16_t, 64, true)
#undef DK_INSTANTIATE_FWD

// Largest G in {4, 2, 1} such that G consecutive q heads share the kv head and
// the look-up-table row.
static int fwd_group(const FwdParams &p) {
  const int ratio = p.Hq / p.Hkv;
  // a table with one row per q head may differ inside a kv group
  const int same_lut = (p.csr.num_heads == p.Hq && p.Hq != p.Hkv) ? p.csr.group : ratio;
  for (int g = 4; g > 1; g >>= 1)
    if (ratio % g == 0 && same_lut % g == 0) return g;
  return 1;
}

// Packed inputs: running work-item counts of the sequences (q tiles, or pairs of q tiles for the
// row-pair kernel), so that a workgroup finds its sequence by bisection instead of adding up the
// sequences before it.
__global__ __launch_bounds__(1024) void packed_item_offsets_kernel(const SeqView s, int causal, int pairs,
                                                                   int32_t *out) {
  if (pairs)
    write_item_offsets(s, causal, [](const SeqInfo &t) { return seq_row_pairs(t); }, out);
  else
    write_item_offsets(s, causal, [](const SeqInfo &t) { return seq_row_blocks(t, 64); }, out);
}

static int launch_item_offsets(const FwdParams &p, bool pairs, hipStream_t stream) {
  if (!p.seqs.packed || !p.seqs.item_offsets) return DK_OK;
  SeqView s = p.seqs;
  s.item_offsets = nullptr;
  DK_NOTE_KERNEL("packed_item_offsets_kernel");
  hipLaunchKernelGGL(packed_item_offsets_kernel, dim3(1), dim3(1024), 0, stream, s, p.causal, pairs ? 1 : 0,
                     p.seqs.item_offsets);
  DK_HIP_CHECK(hipGetLastError());
  return DK_OK;
}

// Scratch the forward can use: batch + 1 ints for packed inputs.
size_t mfma_fwd_workspace_bytes(const FwdParams &p) {
  return p.seqs.packed ? (((size_t)p.seqs.batch + 1) * sizeof(int32_t) + 15) / 16 * 16 : 0;
}

bool mfma_fwd_supported(const FwdParams &p, int dtype) {
  return (dtype == DK_BF16 || dtype == DK_F16) && mfma_head_dim_ok(p.D) && p.csr.block_rows == 64 &&
         p.csr.block_cols == 64 && p.vec_ok &&
         (p.csr.entry_width == 1 || p.csr.sub_block != 0) && mfma_row_bytes_ok(p.k) && mfma_row_bytes_ok(p.v) &&
         p.scale_log2 > 0.f;  // the row maximum is taken before scaling (a scale <= 0 runs on the generic kernels)
}

// The parameters of a launch of (gx heads or head groups) x (gy work items): tables with uneven
// heads get their head rotation.
static FwdParams for_grid(FwdParams p, int gx, int gy) {
  p.csr.rot = head_rotation(p.csr, gx, gy);
  return p;
}

// Several q heads per workgroup (G = 2 or 4 heads that share a kv head and a table row).
template <typename T, int D, int G, bool PAD>
static int launch_tdg(const FwdParams &p, dim3 grid, int tiles_y, hipStream_t stream) {
  constexpr int smem = 2 * FwdSmem<D>::kStage;
  DK_ALLOW_DYNAMIC_LDS((mfma_fwd_kernel<T, D, G, PAD, false>), smem);
  grid.x = p.Hq / G;
  if (int rc = launch_item_offsets(p, false, stream)) return rc;
  const FwdParams pr = for_grid(p, grid.x, grid.y);
  DK_NOTE_KERNEL(pr.csr.rot ? "mfma_fwd_kernel, heads in rotation" : "mfma_fwd_kernel");
  hipLaunchKernelGGL((mfma_fwd_kernel<T, D, G, PAD, false>), grid, dim3(128 * G), smem, stream,
                     pr, tiles_y);
  DK_HIP_CHECK(hipGetLastError());
  return DK_OK;
}

// One head per workgroup: two adjacent q tiles of a head share a workgroup (and the K/V tiles
// their rows have in common), which gives the two waves per SIMD that a single 64-row tile cannot.
template <typename T, int D, bool PAD>
static int launch_row_pairs(const FwdParams &p, hipStream_t stream) {
  const SeqView &s = p.seqs;
  constexpr int smem = 2 * FwdSmem<D>::kStage;
  DK_ALLOW_DYNAMIC_LDS((mfma_fwd_kernel<T, D, 2, PAD, true>), smem);
  int pairs;
  if (s.packed) {
    // per sequence at most (ceil(q_len / 64) + 1) / 2 + 1 pairs; the ceilings add up to at most
    // total / 64 + batch
    pairs = (cdiv(s.max_q_len, 64) + s.batch) / 2 + 2 * s.batch;
  } else if (s.q_starts) {
    pairs = (cdiv(s.max_q_len, 64) + 1) / 2 + 1;  // a sequence's rows start anywhere inside a pair
  } else {
    const int past = p.causal ? s.max_k_len - s.max_q_len : 0;
    pairs = (((past + s.max_q_len - 1) / 64) >> 1) - ((past / 64) >> 1) + 1;
  }
  if (p.csr.pair_order && !s.packed) pairs = (p.csr.num_rows + 1) / 2;  // handed out in the table's order: all of them
  DK_REQUIRE(pairs <= 65535, "too many q tiles for one launch (%d)", pairs);
  if (int rc = launch_item_offsets(p, true, stream)) return rc;
  const FwdParams pr = for_grid(p, p.Hq, pairs);
  DK_NOTE_KERNEL(pr.csr.rot ? "mfma_fwd_kernel, heads in rotation" : "mfma_fwd_kernel");
  hipLaunchKernelGGL((mfma_fwd_kernel<T, D, 2, PAD, true>), dim3(p.Hq, pairs, s.packed ? 1 : s.batch), dim3(256), smem,
                     stream, pr, pairs);
  DK_HIP_CHECK(hipGetLastError());
  return DK_OK;
}

template <typename T, int D, bool PAD>
static int launch_tdp(const FwdParams &p, dim3 grid, int tiles_y, hipStream_t stream) {
  if (fwd_group(p) == 1) return launch_row_pairs<T, D, PAD>(p, stream);
  // 64-wide tiles: workgroups of 2 heads (4 waves), three of them per CU, beat one of 4 heads
  const int group = D == 64 && fwd_group(p) == 4 ? 2 : fwd_group(p);
  return group == 4 ? launch_tdg<T, D, 4, PAD>(p, grid, tiles_y, stream) : launch_tdg<T, D, 2, PAD>(p, grid, tiles_y, stream);
}

// Tables whose entries carry a bit mask over the pattern's 16- or 32-token blocks inside each
// 64 x 64 tile: the plain kernel with the mask applied to S (no row pairs).
template <typename T, int D, int G, bool PAD>
static int launch_sub_g(const FwdParams &p, dim3 grid, int tiles_y, hipStream_t stream) {
  constexpr int smem = 2 * FwdSmem<D>::kStage;
  DK_ALLOW_DYNAMIC_LDS((mfma_fwd_kernel<T, D, G, PAD, false, true>), smem);
  grid.x = p.Hq / G;
  if (int rc = launch_item_offsets(p, false, stream)) return rc;
  const FwdParams pr = for_grid(p, grid.x, grid.y);
  DK_NOTE_KERNEL(pr.csr.rot ? "mfma_fwd_kernel, heads in rotation" : "mfma_fwd_kernel");
  hipLaunchKernelGGL((mfma_fwd_kernel<T, D, G, PAD, false, true>), grid, dim3(128 * G), smem, stream,
                     pr, tiles_y);
  DK_HIP_CHECK(hipGetLastError());
  return DK_OK;
}

template <typename T, int D, bool PAD>
static int launch_sub(const FwdParams &p, dim3 grid, int tiles_y, hipStream_t stream) {
  const int group = D == 64 && fwd_group(p) == 4 ? 2 : fwd_group(p);  // as in launch_tdp
  switch (group) {
    case 4: return launch_sub_g<T, D, 4, PAD>(p, grid, tiles_y, stream);
    case 2: return launch_sub_g<T, D, 2, PAD>(p, grid, tiles_y, stream);
    default: return launch_sub_g<T, D, 1, PAD>(p, grid, tiles_y, stream);
  }
}

// Head dims above 128: 256-wide tiles, one or two heads per workgroup, plain or sub-block-masked
// tables.
template <typename T, int G, bool SUB>
static int launch_256_g(const FwdParams &p, dim3 grid, int tiles_y, hipStream_t stream) {
  constexpr int smem = 2 * FwdSmem<256>::kStage;
  DK_ALLOW_DYNAMIC_LDS((mfma_fwd_kernel<T, 256, G, true, false, SUB>), smem);
  grid.x = p.Hq / G;
  if (int rc = launch_item_offsets(p, false, stream)) return rc;
  const FwdParams pr = for_grid(p, grid.x, grid.y);
  DK_NOTE_KERNEL(pr.csr.rot ? "mfma_fwd_kernel, heads in rotation" : "mfma_fwd_kernel");
  hipLaunchKernelGGL((mfma_fwd_kernel<T, 256, G, true, false, SUB>), grid, dim3(128 * G), smem, stream,
                     pr, tiles_y);
  DK_HIP_CHECK(hipGetLastError());
  return DK_OK;
}

template <typename T>
static int launch_256(const FwdParams &p, dim3 grid, int tiles_y, hipStream_t stream) {
  if (p.csr.sub_block)  // (with the mask registers two heads per workgroup would spill)
    return launch_256_g<T, 1, true>(p, grid, tiles_y, stream);
  // one head per workgroup: two adjacent q tiles share the workgroup and their K/V tiles
  if (fwd_group(p) < 2) return launch_row_pairs<T, 256, true>(p, stream);
  return launch_256_g<T, 2, false>(p, grid, tiles_y, stream);
}

// head dims below the tile width (64 or 128) run the zero-padded instantiation
template <typename T>
static int launch_t(const FwdParams &p, dim3 grid, int tiles_y, hipStream_t stream) {
  if (p.D > 128) return launch_256<T>(p, grid, tiles_y, stream);
  if (p.csr.sub_block) {  // entries carry a bit mask over the pattern's 16- or 32-token blocks
    if (p.D == 128) return launch_sub<T, 128, false>(p, grid, tiles_y, stream);
    if (p.D == 64) return launch_sub<T, 64, false>(p, grid, tiles_y, stream);
    return p.D > 64 ? launch_sub<T, 128, true>(p, grid, tiles_y, stream) : launch_sub<T, 64, true>(p, grid, tiles_y, stream);
  }
  if (p.D == 128) return launch_tdp<T, 128, false>(p, grid, tiles_y, stream);
  if (p.D == 64) return launch_tdp<T, 64, false>(p, grid, tiles_y, stream);
  return p.D > 64 ? launch_tdp<T, 128, true>(p, grid, tiles_y, stream) : launch_tdp<T, 64, true>(p, grid, tiles_y, stream);
}

int launch_mfma_fwd(const FwdParams &p_in, int dtype, void *workspace, size_t workspace_bytes, hipStream_t stream) {
  FwdParams p = p_in;
  if (p.seqs.packed && workspace && workspace_bytes >= mfma_fwd_workspace_bytes(p) && ((uintptr_t)workspace % 4) == 0)
    p.seqs.item_offsets = (int32_t *)workspace;
  const SeqView &s = p.seqs;
  int tiles;
  if (s.packed)
    // a sequence's queries touch at most ceil(q_len / 64) + 1 row blocks (they may start inside
    // one), and the ceilings add up to at most total / 64 + batch
    tiles = cdiv(s.max_q_len, 64) + 2 * s.batch;
  else if (s.q_starts)
    tiles = cdiv(s.max_q_len, 64) + 1;
  else {
    const int past = p.causal ? s.max_k_len - s.max_q_len : 0;
    tiles = (past + s.max_q_len - 1) / 64 - past / 64 + 1;
  }
  if (p.csr.order && !s.packed) tiles = p.csr.num_rows;  // handed out in the table's order: all of them
  DK_REQUIRE(tiles <= 65535, "too many q tiles for one launch (%d)", tiles);
  dim3 grid(1, tiles, s.packed ? 1 : s.batch);
  return dtype == DK_BF16 ? launch_t<bf16_t>(p, grid, tiles, stream) : launch_t<f16_t>(p, grid, tiles, stream);
}

}  // namespace dk
