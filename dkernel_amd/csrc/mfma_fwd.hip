// MFMA forward kernel for gfx950: bf16 / fp16, head_dim 64 or 128, 64 x 64
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
#include <cstdlib>

#include "common.h"
#include "device_common.h"
#include "mfma_common.h"

namespace dk {

template <int D>
struct FwdSmem {  // one stage = K tile + V tile, swizzled row-major (mfma_common.h)
  static constexpr int kStage = 2 * Tile<D>::kBytes;
};

template <typename T, int D, int G>
__global__ __launch_bounds__(128 * G) __attribute__((amdgpu_waves_per_eu(G == 1 ? 1 : 2, 2))) void mfma_fwd_kernel(const FwdParams p, int tiles_y) {
  using M = Mma<T>;
  using vec8 = typename M::vec8;
  using S = FwdSmem<D>;
  constexpr int NT = 128 * G;   // threads
  constexpr int KS = D / 16;    // k-steps of the QK^T product
  constexpr int DT = D / 32;    // d-tiles of the output
  using TL = Tile<D>;
  extern __shared__ __align__(16) char smem[];

  SeqInfo sq;
  int tile;
  const int ty = p.seqs.packed ? blockIdx.y : tiles_y - 1 - (int)blockIdx.y;
  if (!resolve_tile(p.seqs, p.causal, 64, 1, ty, blockIdx.z, sq, tile)) return;
  const int rb = sq.past / 64 + tile;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int h = blockIdx.x * G + (wave >> 1);
  const int kvh = h / (p.Hq / p.Hkv);
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
      if (row_ok) w = *reinterpret_cast<const uint4 *>(qp + ks * 16 + g * 8);
      qf[ks] = as_vec8<vec8>(w);
    }
  }

  const int lh = lut_head(p.csr, blockIdx.x * G, p.Hq, p.Hkv);
  int e0 = 0, e1 = 0;
  if (rb < p.csr.num_rows) {
    e0 = p.csr.ptr[lh * p.csr.ptr_sh + rb];
    e1 = p.csr.ptr[lh * p.csr.ptr_sh + rb + 1];
  }
  const int32_t *cols = p.csr.idx + lh * p.csr.idx_sh;
  const T *kbase = (const T *)p.k.ptr + sq.b * p.k.sb + kvh * p.k.sh + (int64_t)sq.k_start * p.k.st;
  const T *vbase = (const T *)p.v.ptr + sq.b * p.v.sb + kvh * p.v.sh + (int64_t)sq.k_start * p.v.st;

  // ---- asynchronous HBM -> LDS copy of one K/V tile pair (no staging registers) ----
  TileLoader<D, NT> kload, vload;
  kload.init(tid, p.k.st);
  vload.init(tid, p.v.st);
  auto issue = [&](int e, int stage) {
    const int col = cols[e];
    const int key0 = col * 64;
    const int valid = col < 0 ? 0 : sq.k_len - key0;
    char *ks = smem + stage * S::kStage;
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
  int rd[KS], tr[DT][2];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) rd[ks] = TL::off(m, 2 * ks + g);
  transposed_offsets<D>(lane, tr);

  if (e0 < e1) issue(e0, 0);
  for (int e = e0; e < e1; ++e) {
    const int stage = (e - e0) & 1;
    const int col = cols[e];
    wait_tile_loads();
    __syncthreads();  // tile e is visible; every wave is done with the other stage
    if (e + 1 < e1) issue(e + 1, stage ^ 1);
    const int key0 = col * 64;
    if (col < 0 || key0 >= sq.k_len || (p.causal && key0 > row0 + 31)) continue;  // nothing visible (wave-uniform)
    const char *ks_ = smem + stage * S::kStage, *vs_ = ks_ + TL::kBytes;

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
    {
      vec8 ka[2][KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ka[0][ks] = lds_read8<vec8>(ks_ + rd[ks]);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ka[1][ks] = lds_read8<vec8>(ks_ + 32 * TL::kRowBytes + rd[ks]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) sacc[0] = M::mma(ka[0][ks], qf[ks], sacc[0]);
      // first V^T operands do not depend on the softmax: fetch them behind the multiplies
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) va[0][dt] = lds_read_tr8<vec8>(vs_ + tr[dt][0], vs_ + tr[dt][1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) sacc[1] = M::mma(ka[1][ks], qf[ks], sacc[1]);
      __builtin_amdgcn_sched_barrier(0);
    }

    // online softmax in the log2 domain.  Register r of tile nt is key
    // 32nt + 8(r/4) + 4g + r%4.  m_run is a reference maximum that is only
    // raised when a row's maximum grows by more than 2^8 (the accumulator
    // and the row sum stay consistent with it, so the result is exact).
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
    float mx = fmaxf(sacc[0][0], sacc[1][0]);
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = fmaxf(mx, fmaxf(sacc[0][r], sacc[1][r]));
    mx = fmaxf(mx, xor32(mx)) * p.scale_log2;  // scale > 0: max commutes with it
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
        const char *vrow = vs_ + ((step + 1) * 16) * TL::kRowBytes;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) va[(step + 1) & 1][dt] = lds_read_tr8<vec8>(vrow + tr[dt][0], vrow + tr[dt][1]);
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) oacc[dt] = M::mma(va[step & 1][dt], pb, oacc[dt]);
    }
  }

  // l_run holds this lane's share of the row sum (keys with this lane's g)
  l_run += xor32(l_run);

  // ---- epilogue: O = O^T / l, LSE = (m + log2 l) ln 2 ----
  if (!row_ok) return;
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  T *op = (T *)p.o.ptr + sq.b * p.o.sb + h * p.o.sh + (int64_t)(sq.q_start + qi) * p.o.st;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      // registers 4*r4 .. 4*r4+3 are dims 32dt + 8r4 + 4g + {0..3}
      T o4[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) o4[i] = from_float<T>(oacc[dt][r4 * 4 + i] * inv);
      *reinterpret_cast<uint2 *>(op + dt * 32 + r4 * 8 + g * 4) = *reinterpret_cast<const uint2 *>(o4);
    }
  if (p.lse.ptr && g == 0) {
    const float lse = l_run > 0.f ? (m_run + log2f(l_run)) * kLn2 : -INFINITY;
    p.lse.ptr[sq.b * p.lse.sb + h * p.lse.sh + (int64_t)(sq.q_start + qi) * p.lse.st] = lse;
  }
}

// Explicit instantiations: with only the implicit ones the fp16 host stubs of
// this kernel are not emitted by this compiler version.
#define DK_INSTANTIATE_FWD(T, D)                                                  \
  template __global__ void mfma_fwd_kernel<T, D, 1>(const FwdParams, int);       \
  template __global__ void mfma_fwd_kernel<T, D, 2>(const FwdParams, int);       \
  template __global__ void mfma_fwd_kernel<T, D, 4>(const FwdParams, int);
DK_INSTANTIATE_FWD(bf16_t, 128)
DK_INSTANTIATE_FWD(bf16_t, 64)
DK_INSTANTIATE_FWD(f16_t, 128)
DK_INSTANTIATE_FWD(f16_t, 64)
#undef DK_INSTANTIATE_FWD

// Largest G in {4, 2, 1} such that G consecutive q heads share the kv head and
// the look-up-table row.
static int fwd_group(const FwdParams &p) {
  const int ratio = p.Hq / p.Hkv;
  static const int max_group = getenv("DKERNEL_FWD_GROUP") ? atoi(getenv("DKERNEL_FWD_GROUP")) : 4;
  // a table with one row per q head may differ inside a kv group
  const int same_lut = (p.csr.num_heads == p.Hq && p.Hq != p.Hkv) ? p.csr.group : ratio;
  for (int g = 4; g > 1; g >>= 1)
    if (g <= max_group && ratio % g == 0 && same_lut % g == 0) return g;
  return 1;
}

bool mfma_fwd_supported(const FwdParams &p, int dtype) {
  return (dtype == DK_BF16 || dtype == DK_F16) && (p.D == 128 || p.D == 64) && p.csr.block_rows == 64 &&
         p.csr.block_cols == 64 && p.csr.entry_width == 1 && p.vec_ok;
}

template <typename T, int D, int G>
static int launch_tdg(const FwdParams &p, dim3 grid, int tiles_y, hipStream_t stream) {
  constexpr int smem = 2 * FwdSmem<D>::kStage;
  static bool attr_set = false;  // raising the dynamic LDS limit is idempotent; a race only repeats it
  if (!attr_set) {
    DK_HIP_CHECK(hipFuncSetAttribute((const void *)mfma_fwd_kernel<T, D, G>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    attr_set = true;
  }
  grid.x = p.Hq / G;
  hipLaunchKernelGGL((mfma_fwd_kernel<T, D, G>), grid, dim3(128 * G), smem, stream, p, tiles_y);
  DK_HIP_CHECK(hipGetLastError());
  return DK_OK;
}

template <typename T, int D>
static int launch_td(const FwdParams &p, dim3 grid, int tiles_y, hipStream_t stream) {
  switch (fwd_group(p)) {
    case 4: return launch_tdg<T, D, 4>(p, grid, tiles_y, stream);
    case 2: return launch_tdg<T, D, 2>(p, grid, tiles_y, stream);
    default: return launch_tdg<T, D, 1>(p, grid, tiles_y, stream);
  }
}

int launch_mfma_fwd(const FwdParams &p, int dtype, hipStream_t stream) {
  const SeqView &s = p.seqs;
  int tiles;
  if (s.packed)
    tiles = cdiv(s.max_q_len, 64) + s.batch;
  else if (s.q_starts)
    tiles = cdiv(s.max_q_len, 64) + 1;
  else {
    const int past = p.causal ? s.max_k_len - s.max_q_len : 0;
    tiles = (past + s.max_q_len - 1) / 64 - past / 64 + 1;
  }
  DK_REQUIRE(tiles <= 65535, "too many q tiles for one launch (%d)", tiles);
  dim3 grid(1, tiles, s.packed ? 1 : s.batch);
  if (dtype == DK_BF16)
    return p.D == 128 ? launch_td<bf16_t, 128>(p, grid, tiles, stream) : launch_td<bf16_t, 64>(p, grid, tiles, stream);
  return p.D == 128 ? launch_td<f16_t, 128>(p, grid, tiles, stream) : launch_td<f16_t, 64>(p, grid, tiles, stream);
}

}  // namespace dk
