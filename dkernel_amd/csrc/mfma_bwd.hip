// MFMA backward kernels for gfx950: bf16 / fp16, head dims up to 256 (tiles of 64, 128 or
// 256 columns), 64 x 64 blocks, equal-length unpadded sequences.  Two passes, no atomics:
//
//   dQ pass    (CSR rows)    workgroup = 64 q rows x one q head, 4 waves = 2 row
//              halves x 2 key halves (2 waves per SIMD; the key halves are
//              summed through LDS at the end).  Per listed K/V block:
//              S^T = K Q^T, dP^T = V dO^T (lane = q row, registers = keys, so
//              lse / delta are per-lane scalars), dS^T = P^T (dP^T - delta),
//              dQ^T += K^T dS^T with dS^T fed from registers as the B operand
//              and K^T from LDS transpose reads.  The pass also computes
//              delta = rowsum(O * dO) - dLSE of its rows and leaves it in
//              memory for the dK/dV pass, which therefore runs second.
//   dK/dV pass (CSC columns) workgroup = 64 keys x one kv head (the q heads of
//              a GQA group are looped inside), 4 waves, two workgroups per
//              CU.  A listed q block is worked on in two steps of 32 q rows;
//              each 32 x 32 quadrant (q rows of the step x key half) has an S
//              wave (S = Q K^T, P, dV^T += dO^T P; K fragments in registers)
//              and a dP wave (dP = dO V^T, dS = P (dP - delta), dK^T += Q^T dS;
//              V fragments in registers).  P / dS feed the second products
//              from registers, dO^T / Q^T come from LDS transpose reads.
//              Every wave owns the whole accumulator of one matrix for its 32
//              keys, so nothing is summed across waves at the end.
//
// Tiles are copied HBM -> LDS asynchronously (LDS DMA, no staging registers)
// into rings of stages, in the swizzled row-major layout of mfma_common.h.
#include <climits>

#include "common.h"
#include "device_common.h"
#include "mfma_common.h"

namespace dk {

template <int V>
struct IntConst {  // compile-time integer passed to a generic lambda
  static constexpr int value = V;
};

template <bool V>
struct BoolConst {
  static constexpr bool value = V;
};


// ---------------------------------------------------------------------------
// dQ pass
// ---------------------------------------------------------------------------
template <typename T, int D, bool PAD, bool SUB>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(D == 256 ? 1 : 2, D == 64 ? 3 : D == 256 ? 1 : 2))) void mfma_dq_kernel(const BwdParams p,
                                                                                                   int tiles_y) {
  using M = Mma<T>;
  using vec8 = typename M::vec8;
  using TL = Tile<D>;
  constexpr int NT = 256;
  constexpr int KS = D / 16, DT = D / 32;
  constexpr int STAGE = 2 * TL::kBytes;
  // SUB: table entries are (column, bit mask over the pattern blocks inside the 64 x 64 tile)
  constexpr int EW = SUB ? 2 : 1;  // ints per table entry
  extern __shared__ __align__(16) char smem[];

  const SeqInfo sq = load_seq(p.seqs, blockIdx.z, p.causal);
  const int h = grid_head(p.csr);
  int tile = tiles_y - 1 - (int)blockIdx.y;  // longest rows first (of a causal pattern)
  if (p.csr.order)  // the table's own order, longest rows first (the grid then covers every row of it)
    tile = scalar_load(p.csr.order + lut_head(p.csr, h, p.Hq, p.Hkv) * p.csr.order_sh + blockIdx.y) - sq.past / 64;
  if (tile < 0 || tile >= seq_row_blocks(sq, 64)) return;
  const int rb = sq.past / 64 + tile;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rh = wave & 1, kh = wave >> 1;  // q-row half, key half
  const int kvh = __builtin_amdgcn_readfirstlane(h / (p.Hq / p.Hkv));  // integer division runs on the VALU
  const int m = lane & 31, g = lane >> 5;
  const int row0 = rb * 64 + rh * 32;
  const int pos = row0 + m;
  const int qi = pos - sq.past;
  const bool row_ok = qi >= 0 && qi < sq.q_len;
  if constexpr (PAD) {  // the slots of the head dims beyond p.D stay zero for the whole kernel
    zero_tiles<NT>(smem, 2 * STAGE, tid);
    __syncthreads();
  }

  // Row data.  Q and dO of the 64 rows come in as two tiles by LDS DMA, into the second K/V stage
  // (free until the loop's first step requests the second block), and the waves take their
  // fragments from there: whole cache lines, fetched once for both key halves.  Loaded straight
  // into the fragment layout (lane = row), every load instruction touches 32 rows with 32 bytes
  // each - 96 such loads per workgroup kept the memory pipeline busy for a fifth of a short
  // row's time.  O is only needed for delta = rowsum(O * dO) - dLSE: each thread loads four
  // 16-byte chunks of it, consecutive lanes along a row, multiplies them with the dO chunks in
  // LDS and the lanes of a row add up.
  constexpr int CPR = D / 8;  // 16-byte chunks per row
  __shared__ float delta_rows[64];
  float lse_raw = -INFINITY, dlse_raw = 0.f;
  uint4 oreg[64 * CPR / NT];
  {
    const int qi0 = rb * 64 - sq.past;  // query index of the tile's first row
    TileLoader<D, NT, PAD> qload, doload;
    qload.init(tid, p.q.st, p.D);
    doload.init(tid, p.dout.st, p.D);
    const T *qb = (const T *)p.q.ptr + sq.b * p.q.sb + h * p.q.sh + (int64_t)qi0 * p.q.st;
    const T *dob = (const T *)p.dout.ptr + sq.b * p.dout.sb + h * p.dout.sh + (int64_t)qi0 * p.dout.st;
    qload.issue(reinterpret_cast<const char *>(qb), -qi0, sq.q_len - qi0, smem + STAGE);
    doload.issue(reinterpret_cast<const char *>(dob), -qi0, sq.q_len - qi0, smem + STAGE + TL::kBytes);
    const T *ob = (const T *)p.o.ptr + sq.b * p.o.sb + h * p.o.sh + (int64_t)qi0 * p.o.st;
#pragma unroll
    for (int j = 0; j < 64 * CPR / NT; ++j) {
      const int r = tid / CPR + j * (NT / CPR), ch = tid % CPR;
      oreg[j] = make_uint4(0, 0, 0, 0);
      if (qi0 + r >= 0 && qi0 + r < sq.q_len && (!PAD || ch * 8 < p.D))
        oreg[j] = *reinterpret_cast<const uint4 *>(ob + (int64_t)r * p.o.st + ch * 8);
    }
    if (row_ok) {
      lse_raw = p.lse.ptr[sq.b * p.lse.sb + h * p.lse.sh + (int64_t)qi * p.lse.st];
      if (p.dlse.ptr) dlse_raw = p.dlse.ptr[sq.b * p.dlse.sb + h * p.dlse.sh + (int64_t)qi * p.dlse.st];
    }
  }

  const int lh = lut_head(p.csr, h, p.Hq, p.Hkv);
  // table reads go through the scalar unit: a vector load would have to be waited for with
  // vmcnt(0), i.e. together with every tile copy in flight
  int e0 = 0, e1 = 0;
  if (rb < p.csr.num_rows) {
    scalar_load2(p.csr.ptr + lh * p.csr.ptr_sh + rb, p.csr.ptr + lh * p.csr.ptr_sh + rb + 1, e0, e1);
  }
  const int32_t *cols = p.csr.idx + lh * p.csr.idx_sh;
  const T *kbase = (const T *)p.k.ptr + sq.b * p.k.sb + kvh * p.k.sh;
  const T *vbase = (const T *)p.v.ptr + sq.b * p.v.sb + kvh * p.v.sh;

  TileLoader<D, NT, PAD> kload, vload;
  kload.init(tid, p.k.st, p.D);
  vload.init(tid, p.v.st, p.D);
  // blocks whose first key lies in [0, k_full_span) hold 64 keys of the sequence
  const uint32_t k_full_span = sq.k_len >= 64 ? (uint32_t)(sq.k_len - 64) + 1u : 0u;
  const uint32_t k_row_bytes = (uint32_t)p.k.st * 2u, v_row_bytes = (uint32_t)p.v.st * 2u;
  auto issue = [&](int col, int stage) {  // asynchronous copy of K/V block `col` into `stage`
    const int key0 = col * 64;
    char *ks = smem + stage * STAGE;
    // (not at the 256-wide tile: the extra scalar state pushes those kernels into scratch spills)
    if (D <= 128 && (uint32_t)key0 < k_full_span) {  // main path (one scalar compare; a padding entry is negative)
      kload.issue_full(row_address(reinterpret_cast<const char *>(kbase), key0, k_row_bytes), ks);
      vload.issue_full(row_address(reinterpret_cast<const char *>(vbase), key0, v_row_bytes), ks + TL::kBytes);
      return;
    }
    const int valid = col < 0 ? 0 : sq.k_len - key0;
    kload.issue(reinterpret_cast<const char *>(kbase + (int64_t)key0 * p.k.st), 0, valid, ks);
    vload.issue(reinterpret_cast<const char *>(vbase + (int64_t)key0 * p.v.st), 0, valid, ks + TL::kBytes);
  };
  // operand read addresses inside this wave's key half (row kh*32 + m, chunk 2ks+g swizzled;
  // transpose-read pairs) for a tile at offset 0: full pointers, and the stage is a compile-time
  // constant of the loop body, so that stage and k-step offsets are instruction immediates
  using OA = OperandAddress<D>;
  typename OA::type rd[KS], tr[DT][2];
  {
    int tro[DT][2];
    transposed_offsets<D>(lane, tro);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) rd[ks] = OA::make(smem, TL::off(kh * 32 + m, 2 * ks + g));
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      tr[dt][0] = OA::make(smem, kh * 32 * TL::kRowBytes + tro[dt][0]);
      tr[dt][1] = OA::make(smem, kh * 32 * TL::kRowBytes + tro[dt][1]);
    }
  }

  floatx16 acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;

  // Table entries: block e in col_cur (scalar register); block e + 1 is requested one block
  // early as a vector load (col_pending) and first used behind the next tile wait, so that no
  // table read ever stalls the loop.
  int col_cur = e0 < e1 ? scalar_load(cols + e0 * EW) : 0;
  int col_pending = e0 + 1 < e1 ? cols[(e0 + 1) * EW] : 0;
  int bits_cur = 0, bits_pending = 0;  // SUB: the entry's mask, carried like the column
  if constexpr (SUB) {
    bits_cur = e0 < e1 ? scalar_load(cols + e0 * EW + 1) : 0;
    bits_pending = e0 + 1 < e1 ? cols[(e0 + 1) * EW + 1] : 0;
  }
  if (e0 < e1) issue(col_cur, 0);  // the first tiles are on their way while the row data is fetched

  // Q and dO fragments, lse in the log2 domain, and delta = rowsum(O * dO) - dLSE, which this
  // kernel computes itself and also leaves in p.delta for the dK/dV pass that follows
  wait_tile_loads();
  __syncthreads();  // the Q and dO tiles (and the first K/V tiles) are visible
  vec8 qf[KS], dof[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    qf[ks] = lds_read8<vec8>(smem + STAGE + TL::off(rh * 32 + m, 2 * ks + g));
    dof[ks] = lds_read8<vec8>(smem + STAGE + TL::kBytes + TL::off(rh * 32 + m, 2 * ks + g));
  }
#pragma unroll
  for (int j = 0; j < 64 * CPR / NT; ++j) {
    const int r = tid / CPR + j * (NT / CPR), ch = tid % CPR;
    const uint4 dow = *reinterpret_cast<const uint4 *>(smem + STAGE + TL::kBytes + TL::off(r, ch));
    float d = dot8<T>(oreg[j], dow, 0.f);
#pragma unroll
    for (int off = CPR / 2; off > 0; off >>= 1) d += __shfl_xor(d, off);
    if (ch == 0) delta_rows[r] = d;
  }
  __syncthreads();  // the row sums are there; every wave has its fragments: the second stage is free
  float lse2 = INFINITY, delta = 0.f;
  if (row_ok) {
    lse2 = lse_raw == -INFINITY ? INFINITY : lse_raw * kLog2e;
    delta = delta_rows[rh * 32 + m] - dlse_raw;
    if (kh == 0 && g == 0) p.delta[((int64_t)sq.b * p.Hq + h) * p.seqs.max_q_len + qi] = delta;
  }

  auto block_step = [&](int e, auto stage_tag) {
    constexpr int stage = decltype(stage_tag)::value;
    const int col = col_cur;
    const int bits = bits_cur;
    wait_tile_loads();
    __syncthreads();  // tile e is visible; every wave is done with the other stage
    const int col_next = __builtin_amdgcn_readfirstlane(col_pending);  // landed before the tile did
    if constexpr (SUB) bits_cur = __builtin_amdgcn_readfirstlane(bits_pending);
    if (e + 2 < e1) {
      col_pending = cols[(e + 2) * EW];
      if constexpr (SUB) bits_pending = cols[(e + 2) * EW + 1];
    }
    if (e + 1 < e1) issue(col_next, stage ^ 1);
    col_cur = col_next;
    const int key0 = col * 64 + kh * 32;  // first key of this wave's half
    if (col < 0 || key0 >= sq.k_len || (p.causal && key0 > row0 + 31)) return;
    constexpr int ks_ = stage * STAGE, vs_ = ks_ + TL::kBytes;  // byte offsets of this stage's K and V tiles

    floatx16 s, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
    // batches of operand reads, then the multiplies (the scheduler barriers keep
    // the compiler from sinking each read next to its MFMA)
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      vec8 ka[KS / 2];
#pragma unroll
      for (int i = 0; i < KS / 2; ++i) ka[i] = lds_operand<vec8>(rd[half * (KS / 2) + i] + ks_);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < KS / 2; ++i) s = M::mma(ka[i], qf[half * (KS / 2) + i], s);
    }
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      vec8 va[KS / 2];
#pragma unroll
      for (int i = 0; i < KS / 2; ++i) va[i] = lds_operand<vec8>(rd[half * (KS / 2) + i] + vs_);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < KS / 2; ++i) dp = M::mma(va[i], dof[half * (KS / 2) + i], dp);
    }
    // K^T operands of the dQ product do not depend on dS: fetch them now
    vec8 kt[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) kt[dt] = lds_operand_tr<vec8>(tr[dt][0] + ks_, tr[dt][1] + ks_);

    const bool need_mask = (key0 + 31 >= sq.k_len) || (p.causal && key0 + 31 > row0);
    const int lim = p.causal ? min(pos, sq.k_len - 1) : sq.k_len - 1;  // last visible key of this row
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = fast_exp2(fmaf(s[r], p.scale_log2, -lse2));
    if (need_mask) {  // wave-uniform: only the diagonal block and the last, partial one pay for masks
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = key0 + (r >> 2) * 8 + g * 4 + (r & 3);
        s[r] = key > lim ? 0.f : s[r];
      }
    }
    if constexpr (SUB) {
      // pattern blocks of the tile that this row does not attend: bit (row part) * f + (key part)
      const int lb = p.csr.sub_block == 16 ? 4 : 5, f = 64 >> lb;
      const int full = f == 4 ? 0xffff : 0xf;
      if ((bits & full) != full) {  // wave-uniform
        const int row_bits = bits >> (((rh * 32 + m) >> lb) * f);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          // key kh 32 + 8 (r / 4) + 4 g + r % 4: the last two terms stay inside a part of >= 16 keys
          const int key_part = (kh * 32 + (r >> 2) * 8) >> lb;
          s[r] = ((row_bits >> key_part) & 1) ? s[r] : 0.f;
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] *= dp[r] - delta;  // dS^T without sm_scale (applied once at the end)
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      float f[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) f[i] = s[t * 8 + i];
      const vec8 dsb = M::pack(f);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        acc[dt] = M::mma(kt[dt], dsb, acc[dt]);
        if (t == 0)  // refill with the second k-step's operand as soon as the register is free
          kt[dt] = lds_operand_tr<vec8>(tr[dt][0] + ks_ + 16 * TL::kRowBytes, tr[dt][1] + ks_ + 16 * TL::kRowBytes);
      }
    }
  };
  for (int e = e0; e < e1; e += 2) {
    block_step(e, IntConst<0>{});
    if (e + 1 < e1) block_step(e + 1, IntConst<1>{});
  }

  // Sum the two key halves.  Each wave finishes half of the head dims of its rows: it hands the
  // d-tiles of the other half to its partner through LDS and adds the partner's share to its own,
  // so that conversions and stores are spread over all four waves.
  __syncthreads();
  float *red = reinterpret_cast<float *>(smem);
  static_assert(DT % 2 == 0, "two halves of the d-tiles");
#pragma unroll
  for (int i = 0; i < DT / 2; ++i) {
    // (kh is wave-uniform but not a compile-time constant: the accumulator is picked by a
    // select between two fixed registers, never by a run-time index)
    const int dt = (1 - kh) * (DT / 2) + i;  // a d-tile of the partner's half
#pragma unroll
    for (int r = 0; r < 16; ++r)
      red[((rh * DT + dt) * 16 + r) * 64 + lane] = kh == 0 ? acc[DT / 2 + i][r] : acc[i][r];
  }
  __syncthreads();
  // From the 128-wide tile on the finished rows go through a 64-row tile behind the exchange
  // area and leave as whole rows with the non-temporal hint (16 rows per wave): -1 % of the
  // backward at head_dim 128, -1.5 % at 192 / 256.  At the 64-wide tile the direct 8-byte
  // stores of the accumulator layout measure 0.5 % faster and stay.
  constexpr bool kStagedStores = D >= 128;
  char *const out_tile = smem + 2 * DT * 16 * 64 * (int)sizeof(float);
  static_assert(2 * DT * 16 * 64 * (int)sizeof(float) + TL::kBytes <= 2 * STAGE, "exchange area and output tile fit the stages");
  if constexpr (!kStagedStores) {
    if (!row_ok) return;
  }
  int lane_late = lane;  // opaque copy: the tile addresses below are computed here, not before the loop
  asm volatile("" : "+v"(lane_late));
  const int m_late = lane_late & 31, g_late = lane_late >> 5;
  T *dqp = (T *)p.dq.ptr + sq.b * p.dq.sb + h * p.dq.sh + (int64_t)qi * p.dq.st;
#pragma unroll
  for (int i = 0; i < DT / 2; ++i) {
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      float f4[4];
      const int dt = kh * (DT / 2) + i;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int r = r4 * 4 + j;
        const float own = kh == 0 ? acc[i][r] : acc[DT / 2 + i][r];
        f4[j] = (own + red[((rh * DT + dt) * 16 + r) * 64 + lane]) * p.sm_scale;
      }
      const uint2 o4 = pack4<T>(f4[0], f4[1], f4[2], f4[3]);
      // registers 4*r4 .. 4*r4+3 are dims 32dt + 8r4 + 4g + {0..3}
      if constexpr (kStagedStores)
        *reinterpret_cast<uint2 *>(out_tile + TL::off(rh * 32 + m_late, dt * 4 + r4) + g_late * 8) = o4;
      else if (!PAD || dt * 32 + r4 * 8 + g * 4 < p.D)
        *reinterpret_cast<uint2 *>(dqp + dt * 32 + r4 * 8 + g * 4) = o4;
    }
  }
  if constexpr (kStagedStores) {
    __syncthreads();
    const int qi0 = rb * 64 + wave * 16 - sq.past;  // query index of this wave's first row
    T *dq_row0 = (T *)p.dq.ptr + sq.b * p.dq.sb + h * p.dq.sh + (int64_t)qi0 * p.dq.st;
    store_staged_rows<T, D, PAD, 16>(out_tile + wave * 16 * TL::kRowBytes, dq_row0, p.dq.st, lane, -qi0, sq.q_len - qi0, p.D);
  }
}

// ---------------------------------------------------------------------------
// dQ pass, two q tiles per workgroup (tiles of 64 and 128 head dims)
// ---------------------------------------------------------------------------
// One workgroup = table rows 2u and 2u + 1 of one q head (128 q rows), 4 waves: wave = 32 q rows
// of one of the two rows, against all 64 keys of a block (two 32-key halves one after the other,
// in the same registers).  The workgroup walks the union of its two table rows, merged on the
// fly from the two sorted rows, and copies every K / V tile once for both: neighbouring rows of
// the local window share 15 of 16 columns and every vertical column, so the tile traffic from
// the L2 into LDS (what the one-tile kernel spent a quarter of its time on) is halved; a wave
// skips the blocks its own row does not hold.  Every wave owns the finished dQ of its rows:
// nothing is summed across waves at the end.
template <typename T, int D, bool PAD, bool SUB>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, D == 64 ? 3 : 2))) void mfma_dq_pair_kernel(const BwdParams p,
                                                                                                      int pairs_y) {
  using M = Mma<T>;
  using vec8 = typename M::vec8;
  using TL = Tile<D>;
  constexpr int NT = 256;
  constexpr int KS = D / 16, DT = D / 32;
  constexpr int STAGE = 2 * TL::kBytes;
  constexpr int EW = SUB ? 2 : 1;  // ints per table entry
  extern __shared__ __align__(16) char smem[];

  const SeqInfo sq = load_seq(p.seqs, blockIdx.z, p.causal);
  if (sq.q_len <= 0) return;
  const int first_rb = sq.past / 64, last_rb = (sq.past + sq.q_len - 1) / 64;
  const int h = grid_head(p.csr);
  int u = (first_rb >> 1) + pairs_y - 1 - (int)blockIdx.y;  // longest rows first (of a causal pattern)
  if (p.csr.pair_order)  // the table's own order, longest pairs first (the grid then covers every pair of it)
    u = scalar_load(p.csr.pair_order + lut_head(p.csr, h, p.Hq, p.Hkv) * p.csr.order_sh + blockIdx.y);
  if (u > (last_rb >> 1) || u < (first_rb >> 1)) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ts = wave >> 1, rh = wave & 1;  // which of the two table rows, which half of its 64 q rows
  const int ra = 2 * u, rb = ra + ts;
  const int kvh = __builtin_amdgcn_readfirstlane(h / (p.Hq / p.Hkv));  // integer division runs on the VALU
  const int m = lane & 31, g = lane >> 5;
  const int row0 = rb * 64 + rh * 32;
  const int pos = row0 + m;
  const int qi = pos - sq.past;
  const bool row_ok = qi >= 0 && qi < sq.q_len;  // (a table row without queries of this sequence: false everywhere)
  if constexpr (PAD) {  // the slots of the head dims beyond p.D stay zero for the whole kernel
    zero_tiles<NT>(smem, 2 * STAGE, tid);
    __syncthreads();
  }

  // Row data: Q and dO of the 128 rows come in as four tiles by LDS DMA (stage 0: first table
  // row, stage 1: second), O as 16-byte chunks along the rows, multiplied with the dO chunks in
  // LDS for delta = rowsum(O * dO) - dLSE.  The first K / V request has to wait until every wave
  // has taken its fragments out of the stages.
  constexpr int CPR = D / 8;  // 16-byte chunks per row
  constexpr int OCH = 128 * CPR / NT;
  __shared__ float delta_rows[128];
  float lse_raw = -INFINITY, dlse_raw = 0.f;
  uint4 oreg[OCH];
  {
    TileLoader<D, NT, PAD> qload, doload;
    qload.init(tid, p.q.st, p.D);
    doload.init(tid, p.dout.st, p.D);
    const int qi0 = ra * 64 - sq.past;  // query index of the first of the 128 rows (may be negative)
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      const int q0 = qi0 + t2 * 64;
      const T *qb = (const T *)p.q.ptr + sq.b * p.q.sb + h * p.q.sh + (int64_t)q0 * p.q.st;
      const T *dob = (const T *)p.dout.ptr + sq.b * p.dout.sb + h * p.dout.sh + (int64_t)q0 * p.dout.st;
      qload.issue(reinterpret_cast<const char *>(qb), -q0, sq.q_len - q0, smem + t2 * STAGE);
      doload.issue(reinterpret_cast<const char *>(dob), -q0, sq.q_len - q0, smem + t2 * STAGE + TL::kBytes);
    }
    const T *ob = (const T *)p.o.ptr + sq.b * p.o.sb + h * p.o.sh + (int64_t)qi0 * p.o.st;
#pragma unroll
    for (int j = 0; j < OCH; ++j) {
      const int r = tid / CPR + j * (NT / CPR), ch = tid % CPR;
      oreg[j] = make_uint4(0, 0, 0, 0);
      if (qi0 + r >= 0 && qi0 + r < sq.q_len && (!PAD || ch * 8 < p.D))
        oreg[j] = *reinterpret_cast<const uint4 *>(ob + (int64_t)r * p.o.st + ch * 8);
    }
    if (row_ok) {
      lse_raw = p.lse.ptr[sq.b * p.lse.sb + h * p.lse.sh + (int64_t)qi * p.lse.st];
      if (p.dlse.ptr) dlse_raw = p.dlse.ptr[sq.b * p.dlse.sb + h * p.dlse.sh + (int64_t)qi * p.dlse.st];
    }
  }

  // the two table rows: entries [e0, emid) are row 2u, [emid, e1) row 2u + 1 (consecutive rows
  // follow each other in the table); a row without queries of this sequence contributes nothing
  const int lh = lut_head(p.csr, h, p.Hq, p.Hkv);
  int e0 = 0, emid = 0, e1 = 0;
  {
    const int32_t *rp = p.csr.ptr + lh * p.csr.ptr_sh;
    if (ra < p.csr.num_rows) scalar_load2(rp + ra, rp + ra + 1, e0, emid);
    e1 = emid;
    if (ra + 1 < p.csr.num_rows) e1 = scalar_load(rp + ra + 2);
    if (ra < first_rb) e0 = emid;
    if (ra + 1 > last_rb) e1 = emid;
  }
  const int32_t *cols = p.csr.idx + lh * p.csr.idx_sh;
  const T *kbase = (const T *)p.k.ptr + sq.b * p.k.sb + kvh * p.k.sh;
  const T *vbase = (const T *)p.v.ptr + sq.b * p.v.sb + kvh * p.v.sh;

  TileLoader<D, NT, PAD> kload, vload;
  kload.init(tid, p.k.st, p.D);
  vload.init(tid, p.v.st, p.D);
  // blocks whose first key lies in [0, k_full_span) hold 64 keys of the sequence
  const uint32_t k_full_span = sq.k_len >= 64 ? (uint32_t)(sq.k_len - 64) + 1u : 0u;
  const uint32_t k_row_bytes = (uint32_t)p.k.st * 2u, v_row_bytes = (uint32_t)p.v.st * 2u;
  auto issue = [&](int col, int stage) {  // asynchronous copy of K/V block `col` into `stage`
    const int key0 = col * 64;
    char *ks = smem + stage * STAGE;
    if ((uint32_t)key0 < k_full_span) {  // main path (one scalar compare; a padding entry is negative)
      kload.issue_full(row_address(reinterpret_cast<const char *>(kbase), key0, k_row_bytes), ks);
      vload.issue_full(row_address(reinterpret_cast<const char *>(vbase), key0, v_row_bytes), ks + TL::kBytes);
      return;
    }
    const int valid = col < 0 ? 0 : sq.k_len - key0;
    kload.issue(reinterpret_cast<const char *>(kbase + (int64_t)key0 * p.k.st), 0, valid, ks);
    vload.issue(reinterpret_cast<const char *>(vbase + (int64_t)key0 * p.v.st), 0, valid, ks + TL::kBytes);
  };
  // operand read addresses for a tile at offset 0: row m of a 32-key half, chunk 2ks+g swizzled;
  // transpose-read pairs of d-tile dt.  Stage, key half and k-step offsets are immediates.
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

  floatx16 acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;

  // The union of the two rows in column order: head_a / head_b are the next unconsumed entries
  // (scalar), pend_a / pend_b the entries after them (vector loads, first used behind a tile
  // wait, so that no table read stalls the loop); flg_cur says which rows hold the current column.
  constexpr int kEnd = 0x7fffffff;
  int a_pos = e0, b_pos = emid, head_a = kEnd, head_b = kEnd, pend_a = 0, pend_b = 0;
  int hbits_a = 0, hbits_b = 0, pbits_a = 0, pbits_b = 0;  // SUB: the entries' masks, carried like the columns
  if (a_pos < emid) head_a = scalar_load(cols + a_pos * EW);
  if (b_pos < e1) head_b = scalar_load(cols + b_pos * EW);
  if (a_pos + 1 < emid) pend_a = cols[(a_pos + 1) * EW];
  if (b_pos + 1 < e1) pend_b = cols[(b_pos + 1) * EW];
  if constexpr (SUB) {
    if (a_pos < emid) hbits_a = scalar_load(cols + a_pos * EW + 1);
    if (b_pos < e1) hbits_b = scalar_load(cols + b_pos * EW + 1);
    if (a_pos + 1 < emid) pbits_a = cols[(a_pos + 1) * EW + 1];
    if (b_pos + 1 < e1) pbits_b = cols[(b_pos + 1) * EW + 1];
  }
  int col_cur = min(head_a, head_b);
  int flg_cur = (head_a == col_cur ? 1 : 0) | (head_b == col_cur ? 2 : 0);
  int bits_cur = ts ? hbits_b : hbits_a;  // mask of the current column in this wave's row (if it holds it)

  // Q and dO fragments, lse in the log2 domain, and delta = rowsum(O * dO) - dLSE, which this
  // kernel computes itself and also leaves in p.delta for the dK/dV pass that follows
  wait_tile_loads();
  __syncthreads();  // the Q and dO tiles are visible
  vec8 qf[KS], dof[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    qf[ks] = lds_read8<vec8>(smem + ts * STAGE + TL::off(rh * 32 + m, 2 * ks + g));
    dof[ks] = lds_read8<vec8>(smem + ts * STAGE + TL::kBytes + TL::off(rh * 32 + m, 2 * ks + g));
  }
#pragma unroll
  for (int j = 0; j < OCH; ++j) {
    const int r = tid / CPR + j * (NT / CPR), ch = tid % CPR;
    const uint4 dow = *reinterpret_cast<const uint4 *>(smem + (r >> 6) * STAGE + TL::kBytes + TL::off(r & 63, ch));
    float d = dot8<T>(oreg[j], dow, 0.f);
#pragma unroll
    for (int off = CPR / 2; off > 0; off >>= 1) d += __shfl_xor(d, off);
    if (ch == 0) delta_rows[r] = d;
  }
  __syncthreads();  // the row sums are there; every wave has its fragments: both stages are free
  if (col_cur != kEnd) issue(col_cur, 0);
  float lse2 = INFINITY, delta = 0.f;
  if (row_ok) {
    lse2 = lse_raw == -INFINITY ? INFINITY : lse_raw * kLog2e;
    delta = delta_rows[ts * 64 + rh * 32 + m] - dlse_raw;
    if (g == 0) p.delta[((int64_t)sq.b * p.Hq + h) * p.seqs.max_q_len + qi] = delta;
  }

  auto block_step = [&](auto stage_tag) {
    constexpr int stage = decltype(stage_tag)::value;
    const int col = col_cur;
    const int flg = flg_cur;
    const int bits = bits_cur;
    wait_tile_loads();
    __syncthreads();  // the tile is visible; every wave is done with the other stage
    if (flg & 1) {
      ++a_pos;
      head_a = a_pos < emid ? __builtin_amdgcn_readfirstlane(pend_a) : kEnd;
      if (a_pos + 1 < emid) pend_a = cols[(a_pos + 1) * EW];
      if constexpr (SUB) {
        hbits_a = __builtin_amdgcn_readfirstlane(pbits_a);
        if (a_pos + 1 < emid) pbits_a = cols[(a_pos + 1) * EW + 1];
      }
    }
    if (flg & 2) {
      ++b_pos;
      head_b = b_pos < e1 ? __builtin_amdgcn_readfirstlane(pend_b) : kEnd;
      if (b_pos + 1 < e1) pend_b = cols[(b_pos + 1) * EW];
      if constexpr (SUB) {
        hbits_b = __builtin_amdgcn_readfirstlane(pbits_b);
        if (b_pos + 1 < e1) pbits_b = cols[(b_pos + 1) * EW + 1];
      }
    }
    const int col_next = min(head_a, head_b);
    flg_cur = (head_a == col_next ? 1 : 0) | (head_b == col_next ? 2 : 0);
    if constexpr (SUB) bits_cur = ts ? hbits_b : hbits_a;
    if (col_next != kEnd) issue(col_next, stage ^ 1);
    col_cur = col_next;
    if (!((flg >> ts) & 1)) return;  // not in this wave's row
    if (col < 0) return;
    constexpr int ks_ = stage * STAGE, vs_ = ks_ + TL::kBytes;  // byte offsets of this stage's K and V tiles

#pragma unroll
    for (int kh = 0; kh < 2; ++kh) {  // the two 32-key halves of the block
      const int key0 = col * 64 + kh * 32;
      if (key0 >= sq.k_len || (p.causal && key0 > row0 + 31)) continue;  // nothing visible (wave-uniform)
      constexpr int kRow32 = 32 * TL::kRowBytes;
      floatx16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
      // batches of operand reads, then the multiplies (the scheduler barriers keep
      // the compiler from sinking each read next to its MFMA)
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        vec8 ka[KS / 2];
#pragma unroll
        for (int i = 0; i < KS / 2; ++i) ka[i] = lds_operand<vec8>(rd[half * (KS / 2) + i] + ks_ + kh * kRow32);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < KS / 2; ++i) s = M::mma(ka[i], qf[half * (KS / 2) + i], s);
      }
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        vec8 va[KS / 2];
#pragma unroll
        for (int i = 0; i < KS / 2; ++i) va[i] = lds_operand<vec8>(rd[half * (KS / 2) + i] + vs_ + kh * kRow32);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < KS / 2; ++i) dp = M::mma(va[i], dof[half * (KS / 2) + i], dp);
      }
      // K^T operands of the dQ product do not depend on dS: fetch them now
      vec8 kt[DT];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) kt[dt] = lds_operand_tr<vec8>(tr[dt][0] + ks_ + kh * kRow32, tr[dt][1] + ks_ + kh * kRow32);

      const bool need_mask = (key0 + 31 >= sq.k_len) || (p.causal && key0 + 31 > row0);
      const int lim = p.causal ? min(pos, sq.k_len - 1) : sq.k_len - 1;  // last visible key of this row
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = fast_exp2(fmaf(s[r], p.scale_log2, -lse2));
      if (need_mask) {  // wave-uniform: only the diagonal block and the last, partial one pay for masks
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = key0 + (r >> 2) * 8 + g * 4 + (r & 3);
          s[r] = key > lim ? 0.f : s[r];
        }
      }
      if constexpr (SUB) {
        // pattern blocks of the tile that this row does not attend: bit (row part) * f + (key part)
        const int lb = p.csr.sub_block == 16 ? 4 : 5, f = 64 >> lb;
        const int full = f == 4 ? 0xffff : 0xf;
        if ((bits & full) != full) {  // wave-uniform
          const int row_bits = bits >> (((rh * 32 + m) >> lb) * f);
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            // key kh 32 + 8 (r / 4) + 4 g + r % 4: the last two terms stay inside a part of >= 16 keys
            const int key_part = (kh * 32 + (r >> 2) * 8) >> lb;
            s[r] = ((row_bits >> key_part) & 1) ? s[r] : 0.f;
          }
        }
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] *= dp[r] - delta;  // dS^T without sm_scale (applied once at the end)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        float f[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = s[t * 8 + i];
        const vec8 dsb = M::pack(f);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          acc[dt] = M::mma(kt[dt], dsb, acc[dt]);
          if (t == 0)  // refill with the second k-step's operand as soon as the register is free
            kt[dt] = lds_operand_tr<vec8>(tr[dt][0] + ks_ + kh * kRow32 + 16 * TL::kRowBytes,
                                          tr[dt][1] + ks_ + kh * kRow32 + 16 * TL::kRowBytes);
        }
      }
    }
  };
  while (col_cur != kEnd) {
    block_step(IntConst<0>{});
    if (col_cur == kEnd) break;
    block_step(IntConst<1>{});
  }

  // every wave holds the finished dQ^T of its 32 rows
  __syncthreads();  // the K / V stages are free: each wave stages its tile in 32 rows of them
  {
    const int qi0 = row0 - sq.past;  // may be negative or beyond q_len: those rows are skipped
    T *dq_row0 = (T *)p.dq.ptr + sq.b * p.dq.sb + h * p.dq.sh + (int64_t)qi0 * p.dq.st;
    store_tile_rows<T, D, PAD>(smem + wave * 32 * TL::kRowBytes, acc, p.sm_scale, dq_row0, p.dq.st, lane, -qi0,
                               sq.q_len - qi0, p.D);
  }
}

// ---------------------------------------------------------------------------
// dK / dV pass
// ---------------------------------------------------------------------------
// One workgroup = one 64-key column block of one kv head, 4 waves, two workgroups per CU (the
// start-up and close-down of one column then overlap with the other workgroup's loop, and the
// two workgroups' barriers are independent).  A listed q block is worked on in two steps of 32
// q rows; in each step the two 32 x 32 (q rows x keys) quadrants are each shared by a pair of
// waves:
//   the S wave:   S = Q K^T, P = exp(S - lse), dV^T += dO^T P     (K fragments and dV in registers)
//   the dP wave:  dP = dO V^T, dS = P (dP - delta), dK^T += Q^T dS (V fragments and dK in registers)
// so that each wave holds the accumulators of one matrix for 32 keys and fits in the 256
// registers of two waves per SIMD.  P goes from the S wave to the dP wave through LDS in fp32,
// exactly as computed.  The dP wave finishes a step one iteration late (after the next step's
// barrier has published P), so one barrier per step is enough: Q tiles and the lse / delta
// vectors live one iteration longer than dO tiles (rings of 4 and 3 stages of 32-row tiles), and
// tile loads run two steps ahead.
template <int D>
struct DkdvSmem {
  using TL = Tile<D>;
  static constexpr int kRows = 32;                            // q rows per step
  static constexpr int kTile = kRows * TL::kRowBytes;         // one 32-row tile
  static constexpr int kQStages = 4, kDoStages = 3, kAhead = 2;
  static constexpr int kQ = 0;                                // Q ring
  static constexpr int kDo = kQ + kQStages * kTile;           // dO ring
  static constexpr int kVec = kDo + kDoStages * kTile;        // per Q stage: lse[32], delta[32]
  static constexpr int kX = kVec + kQStages * 256;            // P exchange: [pair 2][buffer 2][16][64] floats
  static constexpr int kBytes = kX + 2 * 2 * 4096;
};

template <typename T, int D, bool PAD, bool SUB>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(D == 256 ? 1 : 2, D == 256 ? 1 : 2))) void mfma_dkdv_kernel(const BwdParams p, int head_split) {
  using M = Mma<T>;
  using vec8 = typename M::vec8;
  using TL = Tile<D>;
  using S = DkdvSmem<D>;
  constexpr int NT = 256;
  constexpr int KS = D / 16, DT = D / 32;
  using Loader = TileLoader<D, NT, PAD, S::kRows>;
  constexpr int LPT = 2 * Loader::kChunks + 1;  // load instructions per wave per step
  // SUB: table entries are (row block, bit mask over the pattern blocks inside the 64 x 64 tile)
  constexpr int EW = SUB ? 2 : 1;  // ints per table entry
  extern __shared__ __align__(16) char smem[];

  const SeqInfo sq = load_seq(p.seqs, blockIdx.z, p.causal);
  // head_split: one workgroup per q head instead of per kv head; p.dk / p.dv then describe
  // per-q-head partial buffers that a second kernel sums over each kv group
  const int ratio = __builtin_amdgcn_readfirstlane(p.Hq / p.Hkv);  // integer division runs on the VALU
  const int out_head = grid_head(p.csc);
  const int kvh = head_split ? __builtin_amdgcn_readfirstlane(out_head / ratio) : out_head;
  const int gq_first = head_split ? out_head - kvh * ratio : 0;
  const int gq_end = head_split ? gq_first + 1 : ratio;
  // Columns are handed out longest first when the table says in which order: the hardware deals
  // workgroups to its shader engines round-robin and in order, so long columns that recur with a
  // period pile up on a few engines otherwise.
  int cb = blockIdx.y;
  if (p.csc.order)  // (the grid then covers every column of the table)
    cb = scalar_load(p.csc.order + lut_head(p.csc, kvh * ratio + gq_first, p.Hq, p.Hkv) * p.csc.order_sh + blockIdx.y);
  if (cb * 64 >= sq.k_len) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nh = wave & 1;  // key half; also the index of the (S wave, dP wave) pair
  const bool dp_wave = wave >= 2;
  const int n = lane & 31, g = lane >> 5;
  const int key = cb * 64 + nh * 32 + n;
  const bool key_ok = key < sq.k_len;

  Loader qload, doload;
  qload.init(tid, p.q.st, p.D);
  doload.init(tid, p.dout.st, p.D);
  if constexpr (PAD) {  // the slots of the head dims beyond p.D stay zero in every stage
    zero_tiles<NT>(smem, S::kBytes, tid);
    __syncthreads();
  }
  // K fragments (S wave) or V fragments (dP wave): B operand of the first product.  Up to the
  // 128-wide tile the K and V tiles of the column come in by LDS DMA (whole cache lines; K into
  // the two Q stages that the first two steps do not use, V into the P exchange area) and the
  // waves take their fragments from there behind the first tile wait.  Loaded straight into the
  // fragment layout (lane = key), every load instruction touches 32 rows with 32 bytes each:
  // measured 8 % of the pass on columns of 16 blocks.  (At the 256-wide tile the V tile does not
  // fit the exchange area: direct loads.)
  constexpr bool kKvTiles = D <= 128;
  char *const k_tile = smem + S::kQ + 2 * S::kTile, *const v_tile = smem + S::kX;
  vec8 kvf[KS];
  if constexpr (kKvTiles) {
    static_assert(!kKvTiles || (2 * S::kTile == TL::kBytes && 2 * 2 * 4096 >= TL::kBytes), "a 64-row tile fits either place");
    TileLoader<D, NT, PAD> kload, vload;
    kload.init(tid, p.k.st, p.D);
    vload.init(tid, p.v.st, p.D);
    const T *kb = (const T *)p.k.ptr + sq.b * p.k.sb + kvh * p.k.sh + (int64_t)cb * 64 * p.k.st;
    const T *vb = (const T *)p.v.ptr + sq.b * p.v.sb + kvh * p.v.sh + (int64_t)cb * 64 * p.v.st;
    kload.issue(reinterpret_cast<const char *>(kb), 0, sq.k_len - cb * 64, k_tile);
    vload.issue(reinterpret_cast<const char *>(vb), 0, sq.k_len - cb * 64, v_tile);
  } else {
    const T *src = dp_wave ? (const T *)p.v.ptr + sq.b * p.v.sb + kvh * p.v.sh + (int64_t)key * p.v.st
                           : (const T *)p.k.ptr + sq.b * p.k.sb + kvh * p.k.sh + (int64_t)key * p.k.st;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 a = make_uint4(0, 0, 0, 0);
      if (key_ok && (!PAD || ks * 16 + g * 8 < p.D)) a = *reinterpret_cast<const uint4 *>(src + ks * 16 + g * 8);
      kvf[ks] = as_vec8<vec8>(a);
    }
    // The fragments pass through an empty asm statement: the compiler then waits for their
    // loads here, once.  Left to itself it waits at their first use inside the loop, in every
    // iteration, with vmcnt(0) -- which also waits for the tile copies in flight (issued from
    // inline assembly, so unknown to its counter bookkeeping) and undoes the prefetch.
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(kvf[ks]));
  }
  floatx16 acc[DT];  // dV^T (S wave) or dK^T (dP wave): d x keys, summed over every q row of the column
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;

  int rd[KS], tr[DT][2];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) rd[ks] = TL::off(n, 2 * ks + g);
  transposed_offsets<D>(lane, tr);
  float *xbuf = reinterpret_cast<float *>(smem + S::kX) + nh * 2 * 1024;  // this pair's two P buffers

  // tiles whose first query index lies in [0, full_span) hold 32 queries
  const uint32_t full_span = sq.q_len >= S::kRows ? (uint32_t)(sq.q_len - S::kRows) + 1u : 0u;
  const uint32_t q_row_bytes = (uint32_t)p.q.st * 2u, do_row_bytes = (uint32_t)p.dout.st * 2u;
  // (the body is instantiated twice: the first head also takes the K / V fragments out of LDS,
  // unconditionally - guarded by a run-time test on gq the fragments and accumulators spill)
  auto head_body = [&](int gq, auto first_tag) {
    const int h = kvh * ratio + gq;
    const int lh = lut_head(p.csc, h, p.Hq, p.Hkv);
    int e0 = 0, e1 = 0;
    if (cb < p.csc.num_rows)
      scalar_load2(p.csc.ptr + lh * p.csc.ptr_sh + cb, p.csc.ptr + lh * p.csc.ptr_sh + cb + 1, e0, e1);
    const int nstep = 2 * (e1 - e0);  // two steps of 32 q rows per listed block
    const int32_t *rows = p.csc.idx + lh * p.csc.idx_sh + e0 * EW;
    const T *qbase = (const T *)p.q.ptr + sq.b * p.q.sb + h * p.q.sh;
    const T *dobase = (const T *)p.dout.ptr + sq.b * p.dout.sb + h * p.dout.sh;
    const float *lsebase = p.lse.ptr + sq.b * p.lse.sb + h * p.lse.sh;
    const float *deltabase = p.delta + ((int64_t)sq.b * p.Hq + h) * p.seqs.max_q_len;

    // asynchronous copy of half `half` of q block rbq: Q and dO tiles and the 32 lse / 32 delta
    // values of its rows (lanes 0..31 copy lse, lanes 32..63 delta; every wave copies the same
    // values, so that every wave issues the same number of load instructions).  Returns false
    // when rows had to be zero-filled, i.e. when the per-wave load count is not LPT.
    auto issue = [&](int rbq, int half, int qstage, int dostage) -> bool {
      const int qi0 = rbq * 64 + half * 32 - sq.past;  // query index of the tile's first row
      const int row = lane & 31;
      const bool is_delta = lane >= 32;
      char *dst = smem + S::kVec + qstage * 256;
      // main path: a listed block whose 32 rows all are queries (one scalar compare: a padding
      // entry, rbq < 0, gives a negative qi0)
      if (D <= 128 && (uint32_t)qi0 < full_span) {
        qload.issue_full(row_address(reinterpret_cast<const char *>(qbase), qi0, q_row_bytes),
                         smem + S::kQ + qstage * S::kTile);
        doload.issue_full(row_address(reinterpret_cast<const char *>(dobase), qi0, do_row_bytes),
                          smem + S::kDo + dostage * S::kTile);
        const float *src = is_delta ? deltabase + qi0 + row : lsebase + (int64_t)(qi0 + row) * p.lse.st;
        lds_dma4_lane(src, lds_address(dst));
        return true;
      }
      // rows before the first query (qi < 0, when k is longer than q) and beyond the last are zero-filled
      const int lo = rbq < 0 ? S::kRows : -qi0, hi = sq.q_len - qi0;
      const bool full = qload.issue(reinterpret_cast<const char *>(qbase + (int64_t)qi0 * p.q.st), lo, hi,
                                    smem + S::kQ + qstage * S::kTile);
      doload.issue(reinterpret_cast<const char *>(dobase + (int64_t)qi0 * p.dout.st), lo, hi,
                   smem + S::kDo + dostage * S::kTile);
      if (full) {
        const float *src = is_delta ? deltabase + qi0 + row : lsebase + (int64_t)(qi0 + row) * p.lse.st;
        lds_dma4_lane(src, lds_address(dst));
      } else if (wave == 0) {
        // rows outside the sequence: lse = +inf makes their probabilities 0
        const int qi = qi0 + row;
        float x = is_delta ? 0.f : INFINITY;
        if (row >= lo && row < hi) x = is_delta ? deltabase[qi] : lsebase[(int64_t)qi * p.lse.st];
        reinterpret_cast<float *>(dst)[lane] = x;
      }
      return full;
    };

    // second half of the dP wave's work on step u (whose P the S wave published before the
    // last barrier): dS = P (dP - delta), dK^T += Q^T dS
    auto finish_dk = [&](int u, int qstage, const floatx16 &dp) {
      const char *qs_ = smem + S::kQ + qstage * S::kTile;
      const float *delta_s = reinterpret_cast<const float *>(smem + S::kVec + qstage * 256) + 32;
      const float *x = xbuf + (u & 1) * 1024;
      float ds[16];
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const float4 p4 = *reinterpret_cast<const float4 *>(x + (r4 * 64 + lane) * 4);
        const float4 d4 = *reinterpret_cast<const float4 *>(delta_s + r4 * 8 + g * 4);
        ds[r4 * 4 + 0] = p4.x * (dp[r4 * 4 + 0] - d4.x);  // without sm_scale
        ds[r4 * 4 + 1] = p4.y * (dp[r4 * 4 + 1] - d4.y);
        ds[r4 * 4 + 2] = p4.z * (dp[r4 * 4 + 2] - d4.z);
        ds[r4 * 4 + 3] = p4.w * (dp[r4 * 4 + 3] - d4.w);
      }
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        const vec8 dsb = M::pack(ds + t2 * 8);
        const int rowoff = t2 * 16 * TL::kRowBytes;
        vec8 qt[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) qt[dt] = lds_read_tr8<vec8>(qs_ + rowoff + tr[dt][0], qs_ + rowoff + tr[dt][1]);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[dt] = M::mma(qt[dt], dsb, acc[dt]);
      }
    };

    // The loop is instantiated once per role (not branched inside), so that the accumulators
    // are not merged through a join every iteration.
    auto run_head = [&](auto role_tag) {
    constexpr bool kDp = decltype(role_tag)::value;
    int issued = 0, iq = 0, ido = 0;  // next step to request and its ring positions
    bool exact = true;                // every wave has issued exactly LPT load instructions per outstanding step
    static_assert(S::kAhead == 2, "the first block's two steps are requested together");
    int rb_next = 0;                  // q block of the next step to request (steps 2k and 2k + 1 share block k)
    if (nstep > 0) {
      rb_next = scalar_load(rows);
      for (int i = 0; i < S::kAhead; ++i, ++issued) {
        exact = issue(rb_next, i, iq, ido) && exact;
        iq = iq + 1 == S::kQStages ? 0 : iq + 1;
        ido = ido + 1 == S::kDoStages ? 0 : ido + 1;
      }
    }
    if constexpr (kKvTiles) {
      if constexpr (decltype(first_tag)::value) {
        // the K / V tiles are older than the requests above: everything has landed behind this wait
        wait_tile_loads();
        __syncthreads();
        const char *src = dp_wave ? v_tile : k_tile;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) kvf[ks] = lds_read8<vec8>(src + TL::off(nh * 32 + n, 2 * ks + g));
        // (the loop's first barrier comes before anything is copied over the two tiles: step 2's Q
        // tile is requested behind it, and the S waves write P behind it)
      }
    }
    floatx16 dp_prev;
    int cq = 0, cdo = 0, pq = 0;  // ring positions of step t (Q, dO) and of step t - 1 (Q)
    int rbq = 0, bits = 0;        // S wave: q block (and its mask) of the current step
    for (int t = 0; t < nstep; ++t) {
      const int half = t & 1;
      wait_tiles_ahead<LPT>(exact ? issued - t - 1 : 0);
      __syncthreads();  // step t is visible, so is P of step t - 1; the stages of step t - 2 are free
      if (issued < nstep) {
        if ((issued & 1) == 0) rb_next = scalar_load(rows + (issued >> 1) * EW);
        exact = issue(rb_next, issued & 1, iq, ido) && exact;
        iq = iq + 1 == S::kQStages ? 0 : iq + 1;
        ido = ido + 1 == S::kDoStages ? 0 : ido + 1;
        ++issued;
      }
      const char *qs_ = smem + S::kQ + cq * S::kTile, *dos_ = smem + S::kDo + cdo * S::kTile;
      if constexpr (!kDp) {
        if (half == 0) {
          if constexpr (SUB)
            scalar_load2(rows + (t >> 1) * EW, rows + (t >> 1) * EW + 1, rbq, bits);
          else
            rbq = scalar_load(rows + (t >> 1));
        }
        const int pos0 = rbq * 64 + half * 32;  // first q position of this step
        const float *lse_s = reinterpret_cast<const float *>(smem + S::kVec + cq * 256);
        // S = Q K^T : rows = 32 q positions, cols = 32 keys
        floatx16 sc;
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = 0.f;
        {
          vec8 qa[KS];
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) qa[ks] = lds_read8<vec8>(qs_ + rd[ks]);
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) sc = M::mma(qa[ks], kvf[ks], sc);
        }
        // first dO^T operands do not depend on P
        vec8 dot[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) dot[dt] = lds_read_tr8<vec8>(dos_ + tr[dt][0], dos_ + tr[dt][1]);
        // P = exp2(S scale - lse log2e).  Rows outside the sequence arrive with lse = +inf
        // (P = 0).  A row that saw no key has lse = -inf, but then every one of its entries
        // here is masked by causality and the select below discards the infinite value, so no
        // conversion is needed.  Masks are applied only in steps that need them (the diagonal
        // block and the last, partial column block): wave-uniform choice between two loops.
        const bool edge = (p.causal && (cb * 64 + nh * 32 + 31 > pos0)) || cb * 64 + 63 >= sq.k_len;
        // last visible q-row offset test: key is visible to row pos iff key <= pos
        const int kcmp = key_ok ? (p.causal ? key - pos0 : INT_MIN) : INT_MAX;  // masked iff kcmp > row offset
        float *x = xbuf + (t & 1) * 1024;
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          // registers 4*r4 .. +3 are q rows 8*r4 + 4g + {0..3} of the step
          const float4 l4 = *reinterpret_cast<const float4 *>(lse_s + r4 * 8 + g * 4);
          const float lr[4] = {l4.x, l4.y, l4.z, l4.w};
#pragma unroll
          for (int i = 0; i < 4; ++i)
            sc[r4 * 4 + i] = fast_exp2(fmaf(sc[r4 * 4 + i], p.scale_log2, -lr[i] * kLog2e));
        }
        if (edge) {
#pragma unroll
          for (int r = 0; r < 16; ++r) sc[r] = kcmp > (r >> 2) * 8 + g * 4 + (r & 3) ? 0.f : sc[r];
        }
        if constexpr (SUB) {
          // pattern blocks of the tile that are not attended: bit (row part) * f + (key part); this
          // lane's key is nh 32 + n, register r is q row half 32 + 8 (r / 4) + 4 g + r % 4
          const int lb = p.csc.sub_block == 16 ? 4 : 5, f = 64 >> lb;
          const int full = f == 4 ? 0xffff : 0xf;
          if ((bits & full) != full) {  // wave-uniform
            const int key_bits = bits >> ((nh * 32 + n) >> lb);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int row_part = (half * 32 + (r >> 2) * 8) >> lb;
              sc[r] = ((key_bits >> (row_part * f)) & 1) ? sc[r] : 0.f;
            }
          }
        }
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4)
          *reinterpret_cast<float4 *>(x + (r4 * 64 + lane) * 4) =
              make_float4(sc[r4 * 4], sc[r4 * 4 + 1], sc[r4 * 4 + 2], sc[r4 * 4 + 3]);
        // dV^T += dO^T P
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
          float pf[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) pf[i] = sc[t2 * 8 + i];
          const vec8 pb = M::pack(pf);
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            acc[dt] = M::mma(dot[dt], pb, acc[dt]);
            if (t2 == 0) {
              const int rowoff = 16 * TL::kRowBytes;
              dot[dt] = lds_read_tr8<vec8>(dos_ + rowoff + tr[dt][0], dos_ + rowoff + tr[dt][1]);
            }
          }
        }
      } else {
        // second half of step t - 1 first: it frees dp_prev for this step's dP
        if (t > 0) finish_dk(t - 1, pq, dp_prev);
        // dP = dO V^T
#pragma unroll
        for (int r = 0; r < 16; ++r) dp_prev[r] = 0.f;
        {
          vec8 da[KS];
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) da[ks] = lds_read8<vec8>(dos_ + rd[ks]);
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) dp_prev = M::mma(da[ks], kvf[ks], dp_prev);
        }
      }
      pq = cq;
      cq = cq + 1 == S::kQStages ? 0 : cq + 1;
      cdo = cdo + 1 == S::kDoStages ? 0 : cdo + 1;
    }
    __syncthreads();  // P of the last step is visible
    if constexpr (kDp) {
      if (nstep > 0) finish_dk(nstep - 1, pq, dp_prev);
    }
    };
    if (dp_wave)
      run_head(BoolConst<true>{});
    else
      run_head(BoolConst<false>{});
    if (gq + 1 < gq_end) __syncthreads();  // every wave is done with every stage before the next head reuses them
  };
  head_body(gq_first, BoolConst<true>{});
  for (int gq = gq_first + 1; gq < gq_end; ++gq) head_body(gq, BoolConst<false>{});

  // every wave holds the finished dV^T (S wave) or dK^T (dP wave) of its 32 keys
  const float out_scale = dp_wave ? p.sm_scale : 1.f;
  const TensorView &outv = dp_wave ? p.dk : p.dv;
  if (head_split) {  // fp32 partial of this q head
    if (!key_ok) return;
    float *outp = (float *)outv.ptr + sq.b * outv.sb + out_head * outv.sh + (int64_t)key * outv.st;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        float4 o4;
        o4.x = acc[dt][r4 * 4 + 0] * out_scale;
        o4.y = acc[dt][r4 * 4 + 1] * out_scale;
        o4.z = acc[dt][r4 * 4 + 2] * out_scale;
        o4.w = acc[dt][r4 * 4 + 3] * out_scale;
        if (!PAD || dt * 32 + r4 * 8 + g * 4 < p.D) *reinterpret_cast<float4 *>(outp + dt * 32 + r4 * 8 + g * 4) = o4;
      }
    return;
  }
  if constexpr (D >= 128) {
    // each wave stages its 32 keys x D in one stage of the Q ring and writes whole rows (as in
    // the dQ pass: from the 128-wide tile on)
    __syncthreads();  // the dP waves have finished their last step (it reads the Q ring)
    const int key0 = cb * 64 + nh * 32;
    T *out_row0 = (T *)outv.ptr + sq.b * outv.sb + out_head * outv.sh + (int64_t)key0 * outv.st;
    store_tile_rows<T, D, PAD>(smem + S::kQ + wave * S::kTile, acc, out_scale, out_row0, outv.st, lane, 0, sq.k_len - key0, p.D);
  } else {
    if (!key_ok) return;
    T *outp = (T *)outv.ptr + sq.b * outv.sb + out_head * outv.sh + (int64_t)key * outv.st;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        if (!PAD || dt * 32 + r4 * 8 + g * 4 < p.D)
          *reinterpret_cast<uint2 *>(outp + dt * 32 + r4 * 8 + g * 4) =
              pack4<T>(acc[dt][r4 * 4] * out_scale, acc[dt][r4 * 4 + 1] * out_scale, acc[dt][r4 * 4 + 2] * out_scale,
                       acc[dt][r4 * 4 + 3] * out_scale);
      }
  }
}

// Explicit instantiations: with only the implicit ones the fp16 host stubs of
// these kernels are not emitted by this compiler version.
// (256-wide tiles: the zero-padding instantiations only; they also take head_dim 256 itself)
template __global__ void mfma_dq_kernel<bf16_t, 256, true, false>(const BwdParams, int);
template __global__ void mfma_dq_kernel<bf16_t, 256, true, true>(const BwdParams, int);
template __global__ void mfma_dq_kernel<f16_t, 256, true, false>(const BwdParams, int);
template __global__ void mfma_dq_kernel<f16_t, 256, true, true>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<bf16_t, 256, true, false>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<bf16_t, 256, true, true>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<f16_t, 256, true, false>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<f16_t, 256, true, true>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<bf16_t, 128, false, false>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<bf16_t, 128, true, false>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<bf16_t, 128, false, true>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<bf16_t, 128, true, true>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<bf16_t, 64, false, false>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<bf16_t, 64, true, false>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<bf16_t, 64, false, true>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<bf16_t, 64, true, true>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<f16_t, 128, false, false>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<f16_t, 128, true, false>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<f16_t, 128, false, true>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<f16_t, 128, true, true>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<f16_t, 64, false, false>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<f16_t, 64, true, false>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<f16_t, 64, false, true>(const BwdParams, int);
template __global__ void mfma_dq_pair_kernel<f16_t, 64, true, true>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<bf16_t, 128, false, false>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<bf16_t, 128, true, false>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<bf16_t, 128, false, true>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<bf16_t, 128, true, true>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<bf16_t, 64, false, false>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<bf16_t, 64, true, false>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<bf16_t, 64, false, true>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<bf16_t, 64, true, true>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<f16_t, 128, false, false>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<f16_t, 128, true, false>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<f16_t, 128, false, true>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<f16_t, 128, true, true>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<f16_t, 64, false, false>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<f16_t, 64, true, false>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<f16_t, 64, false, true>(const BwdParams, int);
template __global__ void mfma_dkdv_kernel<f16_t, 64, true, true>(const BwdParams, int);

// Sum of the per-q-head dK / dV partials over each kv group (head_split mode).  One thread
// per 8 head dims of one (batch, kv head, key): blockIdx.y = 0 sums dK, 1 sums dV.
// part: fp32 [batch][Hq][keys][D] contiguous.
template <typename T>
__global__ __launch_bounds__(256) void dkdv_group_sum_kernel(const float *part_k, const float *part_v, TensorView dk,
                                                             TensorView dv, int batch, int Hq, int Hkv, int keys,
                                                             int D) {
  const int cpr = D / 8;
  const int64_t total = (int64_t)batch * Hkv * keys * cpr;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int ch = (int)(i % cpr);
  const int key = (int)((i / cpr) % keys);
  const int kvh = (int)((i / ((int64_t)cpr * keys)) % Hkv);
  const int b = (int)(i / ((int64_t)cpr * keys * Hkv));
  const int ratio = Hq / Hkv;
  const float *part = blockIdx.y ? part_v : part_k;
  const TensorView &out = blockIdx.y ? dv : dk;
  float4 lo = make_float4(0.f, 0.f, 0.f, 0.f), hi = lo;
  const float *src = part + (((int64_t)b * Hq + kvh * ratio) * keys + key) * D + ch * 8;
  for (int gq = 0; gq < ratio; ++gq) {
    const float4 a = *reinterpret_cast<const float4 *>(src + (int64_t)gq * keys * D);
    const float4 c = *reinterpret_cast<const float4 *>(src + (int64_t)gq * keys * D + 4);
    lo.x += a.x, lo.y += a.y, lo.z += a.z, lo.w += a.w;
    hi.x += c.x, hi.y += c.y, hi.z += c.z, hi.w += c.w;
  }
  T o8[8] = {from_float<T>(lo.x), from_float<T>(lo.y), from_float<T>(lo.z), from_float<T>(lo.w),
             from_float<T>(hi.x), from_float<T>(hi.y), from_float<T>(hi.z), from_float<T>(hi.w)};
  *reinterpret_cast<uint4 *>((T *)out.ptr + b * out.sb + kvh * out.sh + (int64_t)key * out.st + ch * 8) =
      *reinterpret_cast<const uint4 *>(o8);
}

// Scratch for the head-split dK/dV pass: fp32 per-q-head partials of dK and dV (16-bit partials
// would round each head's share before the sum).  Zero when the pass would not be split (one
// q head per kv head).
size_t mfma_bwd_workspace_bytes(const BwdParams &p) {
  if (p.Hq == p.Hkv) return 0;
  const size_t need = 2 * (size_t)p.seqs.batch * p.Hq * p.seqs.max_k_len * p.D * sizeof(float);
  // beyond 4 GiB of partials (large batches) the pass keeps its in-workgroup loop over the group:
  // there are enough columns to balance then, and the scratch would rival the tensors themselves
  return need <= ((size_t)4 << 30) ? need : 0;
}

bool mfma_bwd_supported(const BwdParams &p, int dtype) {
  return (dtype == DK_BF16 || dtype == DK_F16) && mfma_head_dim_ok(p.D) && p.csr.block_rows == 64 &&
         p.csr.block_cols == 64 && p.csr.sub_block == p.csc.sub_block &&
         (p.csr.sub_block != 0 || (p.csr.entry_width == 1 && p.csc.entry_width == 1)) &&
         p.csc.block_rows == 64 && p.csc.block_cols == 64 &&
         p.vec_ok && mfma_row_bytes_ok(p.q) && mfma_row_bytes_ok(p.k) && mfma_row_bytes_ok(p.v) &&
         mfma_row_bytes_ok(p.dout);
}

template <typename T, int D, bool PAD, bool SUB>
static int launch_bwd_td(const BwdParams &p, void *workspace, size_t workspace_bytes, hipStream_t stream) {
  const SeqView &s = p.seqs;
  constexpr int smem_dq = 2 * 2 * Tile<D>::kBytes;
  constexpr int smem_dkdv = DkdvSmem<D>::kBytes;
  DK_ALLOW_DYNAMIC_LDS((mfma_dkdv_kernel<T, D, PAD, SUB>), smem_dkdv);
  const int past = p.causal ? s.max_k_len - s.max_q_len : 0;
  const int tiles = (past + s.max_q_len - 1) / 64 - past / 64 + 1;
  DK_REQUIRE(tiles <= 65535 && cdiv(s.max_k_len, 64) <= 65535 && p.csc.num_rows <= 65535 &&
                 (!(p.csr.order || p.csr.pair_order) || p.csr.num_rows <= 65535),
             "sequence too long for one launch");
  // dQ first: it also writes delta, which the dK/dV pass reads
  if constexpr (D <= 128) {  // two table rows per workgroup
    int pairs = (((past + s.max_q_len - 1) / 64) >> 1) - ((past / 64) >> 1) + 1;
    DK_ALLOW_DYNAMIC_LDS((mfma_dq_pair_kernel<T, D, PAD, SUB>), smem_dq);
    if (p.csr.pair_order) pairs = (p.csr.num_rows + 1) / 2;  // handed out in the table's order: all of them
    BwdParams pq = p;
    pq.csr.rot = head_rotation(p.csr, p.Hq, pairs);  // (uneven heads: dealt to the queues in rotation)
    DK_NOTE_KERNEL(pq.csr.rot ? "mfma_dq_pair_kernel, heads in rotation" : "mfma_dq_pair_kernel");
    hipLaunchKernelGGL((mfma_dq_pair_kernel<T, D, PAD, SUB>), dim3(p.Hq, pairs, s.batch), dim3(256), smem_dq, stream, pq, pairs);
  } else {
    DK_ALLOW_DYNAMIC_LDS((mfma_dq_kernel<T, D, PAD, SUB>), smem_dq);
    const int rows = p.csr.order ? p.csr.num_rows : tiles;  // handed out in the table's order: all of them
    BwdParams pq = p;
    pq.csr.rot = head_rotation(p.csr, p.Hq, rows);
    DK_NOTE_KERNEL(pq.csr.rot ? "mfma_dq_kernel, heads in rotation" : "mfma_dq_kernel");
    hipLaunchKernelGGL((mfma_dq_kernel<T, D, PAD, SUB>), dim3(p.Hq, rows, s.batch), dim3(256), smem_dq, stream, pq, rows);
  }
  DK_HIP_CHECK(hipGetLastError());
  // With several q heads per kv head a workgroup per kv head walks all of them, and the longest
  // column (a vertical one near the start: every later q block, times the group size) alone
  // outlasts the average CU's share of the whole pass.  Given scratch, the pass runs one
  // workgroup per q head into per-head partials and a bandwidth-bound kernel sums each group.
  const size_t need = mfma_bwd_workspace_bytes(p);
  const bool per_q_head = need > 0 && workspace && workspace_bytes >= need && ((uintptr_t)workspace % 16) == 0;
  // The table's longest-first order is taken unless the heads along grid.x are a multiple of the
  // 32 (XCD, shader engine) queues that the hardware deals workgroups to in turn: then every queue
  // serves whole heads, long columns and short ones alike, and the ascending order keeps
  // neighbouring columns - which share most of their Q / dO tiles - together in time (1.7 %
  // faster on the 32-head benchmark; with 8 or 16 heads the order is worth 20 - 40 %).
  BwdParams po = p;
  if (((per_q_head ? p.Hq : p.Hkv) % 32) == 0) po.csc.order = nullptr;
  // with a hand-out order the grid covers every column of the table (those beyond the keys exit at once)
  const int cblocks = po.csc.order ? p.csc.num_rows : cdiv(s.max_k_len, 64);
  po.csc.rot = head_rotation(p.csc, per_q_head ? p.Hq : p.Hkv, cblocks);
  if (per_q_head) {
    BwdParams pp = po;
    const int64_t keys = s.max_k_len;
    float *part_k = (float *)workspace, *part_v = part_k + (int64_t)s.batch * p.Hq * keys * p.D;
    pp.dk = TensorView{part_k, p.Hq * keys * p.D, keys * p.D, p.D};
    pp.dv = TensorView{part_v, p.Hq * keys * p.D, keys * p.D, p.D};
    DK_NOTE_KERNEL(pp.csc.rot ? "mfma_dkdv_kernel (one workgroup per q head), heads in rotation"
                              : "mfma_dkdv_kernel (one workgroup per q head)");
    hipLaunchKernelGGL((mfma_dkdv_kernel<T, D, PAD, SUB>), dim3(p.Hq, cblocks, s.batch), dim3(256), smem_dkdv, stream, pp, 1);
    DK_HIP_CHECK(hipGetLastError());
    const int64_t total = (int64_t)s.batch * p.Hkv * keys * (p.D / 8);
    DK_NOTE_KERNEL("dkdv_group_sum_kernel");
    hipLaunchKernelGGL((dkdv_group_sum_kernel<T>), dim3((unsigned)cdiv64(total, 256), 2), dim3(256), 0, stream, part_k,
                       part_v, p.dk, p.dv, s.batch, p.Hq, p.Hkv, (int)keys, p.D);
    DK_HIP_CHECK(hipGetLastError());
    return DK_OK;
  }
  DK_NOTE_KERNEL(po.csc.rot ? "mfma_dkdv_kernel, heads in rotation" : "mfma_dkdv_kernel");
  hipLaunchKernelGGL((mfma_dkdv_kernel<T, D, PAD, SUB>), dim3(p.Hkv, cblocks, s.batch), dim3(256), smem_dkdv, stream, po, 0);
  DK_HIP_CHECK(hipGetLastError());
  return DK_OK;
}

// head dims below the tile width (64 or 128) run the zero-padded instantiation
template <typename T>
static int launch_bwd_t(const BwdParams &p, void *ws, size_t ws_bytes, hipStream_t stream) {
  if (p.D > 128)  // 256-wide tiles, one wave per SIMD
    return p.csr.sub_block ? launch_bwd_td<T, 256, true, true>(p, ws, ws_bytes, stream)
                           : launch_bwd_td<T, 256, true, false>(p, ws, ws_bytes, stream);
  if (p.csr.sub_block) {  // entries carry a bit mask over the pattern's 16- or 32-token blocks
    if (p.D == 128) return launch_bwd_td<T, 128, false, true>(p, ws, ws_bytes, stream);
    if (p.D == 64) return launch_bwd_td<T, 64, false, true>(p, ws, ws_bytes, stream);
    return p.D > 64 ? launch_bwd_td<T, 128, true, true>(p, ws, ws_bytes, stream)
                    : launch_bwd_td<T, 64, true, true>(p, ws, ws_bytes, stream);
  }
  if (p.D == 128) return launch_bwd_td<T, 128, false, false>(p, ws, ws_bytes, stream);
  if (p.D == 64) return launch_bwd_td<T, 64, false, false>(p, ws, ws_bytes, stream);
  return p.D > 64 ? launch_bwd_td<T, 128, true, false>(p, ws, ws_bytes, stream)
                  : launch_bwd_td<T, 64, true, false>(p, ws, ws_bytes, stream);
}

int launch_mfma_bwd(const BwdParams &p, int dtype, void *workspace, size_t workspace_bytes, hipStream_t stream) {
  return dtype == DK_BF16 ? launch_bwd_t<bf16_t>(p, workspace, workspace_bytes, stream)
                          : launch_bwd_t<f16_t>(p, workspace, workspace_bytes, stream);
}

}  // namespace dk
