// Generic forward kernel: any of bf16 / fp16 / fp32, head_dim <= 256, any
// power-of-two tile sizes (including merged-Q look-up tables), fixed, padded,
// packed and single-token (decode) sequences.  fp32 FMA arithmetic, K/V chunks
// staged in LDS.  It is the always-available path and the on-device
// cross-check for the MFMA kernels; the headline shapes are served by
// mfma_fwd.hip.
//
// Work split: a thread owns 32 head dims of one query row, DPAD/32 adjacent
// lanes share a row (dot products are finished with lane shuffles), a
// workgroup of 256 threads covers 256/(DPAD/32) rows.
#include "common.h"
#include "device_common.h"
#include "generic_io.h"

namespace dk {

template <typename T, int DPAD>
__global__ __launch_bounds__(256) void generic_fwd_kernel(const FwdParams p) {
  constexpr int TPR = DPAD / 32;
  constexpr int R = 256 / TPR;
  constexpr int KC = (sizeof(T) == 4 && DPAD == 256) ? 16 : 32;
  constexpr int CH = DPAD / 8;  // 8-element chunks per row
  __shared__ __align__(16) T sK[KC * DPAD];
  __shared__ __align__(16) T sV[KC * DPAD];

  const int BM = p.csr.block_rows, BN = p.csr.block_cols;
  const int rows_wg = BM < R ? BM : R;
  const int tiles_per_block = BM / rows_wg;
  SeqInfo sq;
  int tile;
  const bool has_rows = resolve_tile(p.seqs, p.causal, BM, tiles_per_block, blockIdx.x, blockIdx.z, sq, tile);
  if (p.seqs.zero_outside)
    zero_rows_outside<T>(p.seqs, sq, blockIdx.x, gridDim.x, p.o, p.lse, blockIdx.y, 1, p.D, p.vec_ok, threadIdx.x, 256);
  if (!has_rows) return;
  const int h = blockIdx.y;
  const int kvh = h / (p.Hq / p.Hkv);
  const int rb = sq.past / BM + tile / tiles_per_block;
  const int tid = threadIdx.x, r = tid / TPR, j = tid % TPR;
  const int row_in_block = (tile % tiles_per_block) * rows_wg + r;
  const int pos = rb * BM + row_in_block;
  const int qi = pos - sq.past;
  const bool row_ok = (r < rows_wg) && qi >= 0 && qi < sq.q_len;
  const int D = p.D;

  float qf[32], acc[32];
#pragma unroll
  for (int i = 0; i < 32; ++i) acc[i] = 0.f;
  {
    const T *qp = (const T *)p.q.ptr + sq.b * p.q.sb + h * p.q.sh + (int64_t)(sq.q_start + qi) * p.q.st;
#pragma unroll
    for (int c = 0; c < 4; ++c) load8_guard<T>(qp, (c * TPR + j) * 8, D, row_ok, p.vec_ok, qf + c * 8);
  }
  float m_run = -INFINITY, l_run = 0.f;

  const int lh = lut_head(p.csr, h, p.Hq, p.Hkv);
  int e0 = 0, e1 = 0;
  if (rb < p.csr.num_rows) {
    e0 = p.csr.ptr[lh * p.csr.ptr_sh + rb];
    e1 = p.csr.ptr[lh * p.csr.ptr_sh + rb + 1];
  }
  const T *kbase = (const T *)p.k.ptr + sq.b * p.k.sb + kvh * p.k.sh + (int64_t)sq.k_start * p.k.st;
  const T *vbase = (const T *)p.v.ptr + sq.b * p.v.sb + kvh * p.v.sh + (int64_t)sq.k_start * p.v.st;
  const int kc_n = BN < KC ? BN : KC;
  const int wg_last_pos = rb * BM + (tile % tiles_per_block) * rows_wg + rows_wg - 1;

  for (int e = e0; e < e1; ++e) {
    const int32_t *ent = p.csr.idx + lh * p.csr.idx_sh + (int64_t)e * p.csr.entry_width;
    const int col = ent[0];
    const int micro = p.csr.entry_width == 2 ? ent[1] : BM;
    const int kb0 = col * BN;
    if (col < 0 || kb0 >= sq.k_len) continue;
    if (p.causal && kb0 > wg_last_pos) continue;
    for (int ch = 0; ch < BN / kc_n; ++ch) {
      const int key0 = kb0 + ch * kc_n;
      __syncthreads();
      for (int t = tid; t < kc_n * CH; t += 256) {
        const int n = t / CH, c8 = t % CH;
        const bool ok = key0 + n < sq.k_len;
        copy8_guard<T>(kbase + (int64_t)(key0 + n) * p.k.st, c8 * 8, D, ok, p.vec_ok, sK + n * DPAD + c8 * 8);
        copy8_guard<T>(vbase + (int64_t)(key0 + n) * p.v.st, c8 * 8, D, ok, p.vec_ok, sV + n * DPAD + c8 * 8);
      }
      __syncthreads();

      float s[KC];
#pragma unroll
      for (int n = 0; n < KC; ++n) {
        float a = 0.f;
        if (n < kc_n) {
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            float kf[8];
            lds_load8<T>(sK + n * DPAD + (c * TPR + j) * 8, kf);
#pragma unroll
            for (int i = 0; i < 8; ++i) a = fmaf(qf[c * 8 + i], kf[i], a);
          }
        }
        s[n] = a;
      }
#pragma unroll
      for (int n = 0; n < KC; ++n) {
#pragma unroll
        for (int off = 1; off < TPR; off <<= 1) s[n] += __shfl_xor(s[n], off);
      }
      float m_new = m_run;
#pragma unroll
      for (int n = 0; n < KC; ++n) {
        const int key = key0 + n;
        const bool vis = row_ok && n < kc_n && key < sq.k_len && (!p.causal || key <= pos) &&
                         row_in_block < micro;
        s[n] = vis ? s[n] * p.scale_log2 : -INFINITY;
        m_new = fmaxf(m_new, s[n]);
      }
      if (m_new > -INFINITY) {  // this row has seen at least one visible key
        const float alpha = exp2f(m_run - m_new);
        float psum = 0.f;
#pragma unroll
        for (int n = 0; n < KC; ++n) {
          s[n] = exp2f(s[n] - m_new);
          psum += s[n];
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int i = 0; i < 32; ++i) acc[i] *= alpha;
#pragma unroll
        for (int n = 0; n < KC; ++n) {
          if (n < kc_n) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
              float vf[8];
              lds_load8<T>(sV + n * DPAD + (c * TPR + j) * 8, vf);
#pragma unroll
              for (int i = 0; i < 8; ++i) acc[c * 8 + i] = fmaf(s[n], vf[i], acc[c * 8 + i]);
            }
          }
        }
      }
    }
  }

  if (!row_ok) return;
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  T *op = (T *)p.o.ptr + sq.b * p.o.sb + h * p.o.sh + (int64_t)(sq.q_start + qi) * p.o.st;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    float of[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) of[i] = acc[c * 8 + i] * inv;
    store8_guard<T>(op, (c * TPR + j) * 8, D, p.vec_ok, of);
  }
  if (p.lse.ptr && j == 0) {
    const float lse = l_run > 0.f ? (m_run + log2f(l_run)) * kLn2 : -INFINITY;
    p.lse.ptr[sq.b * p.lse.sb + h * p.lse.sh + (int64_t)(sq.q_start + qi) * p.lse.st] = lse;
  }
}

template <typename T>
static int launch_generic_fwd_t(const FwdParams &p, dim3 grid_for[3], hipStream_t stream) {
  const int dpad = p.D <= 64 ? 64 : (p.D <= 128 ? 128 : 256);
  DK_NOTE_KERNEL(dpad == 64 ? "generic_fwd_kernel<64>" : dpad == 128 ? "generic_fwd_kernel<128>" : "generic_fwd_kernel<256>");
  if (dpad == 64)
    hipLaunchKernelGGL((generic_fwd_kernel<T, 64>), grid_for[0], dim3(256), 0, stream, p);
  else if (dpad == 128)
    hipLaunchKernelGGL((generic_fwd_kernel<T, 128>), grid_for[1], dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((generic_fwd_kernel<T, 256>), grid_for[2], dim3(256), 0, stream, p);
  DK_HIP_CHECK(hipGetLastError());
  return DK_OK;
}

// Upper bound on the number of tiles along grid.x (workgroups beyond the real
// count exit at once).
static int fwd_tiles_x(const FwdParams &p, int rows_per_wg) {
  const int BM = p.csr.block_rows;
  const int rows_wg = BM < rows_per_wg ? BM : rows_per_wg;
  const int tpb = BM / rows_wg;
  const SeqView &s = p.seqs;
  int blocks;
  if (s.packed)
    // a sequence's queries touch at most ceil(q_len / BM) + 1 row blocks (they may start inside
    // one), and the ceilings add up to at most total / BM + batch
    blocks = cdiv(s.max_q_len, BM) + 2 * s.batch;
  else if (s.q_starts)
    blocks = cdiv(s.max_q_len, BM) + 1;
  else {
    const int past = p.causal ? s.max_k_len - s.max_q_len : 0;
    blocks = (past + s.max_q_len - 1) / BM - past / BM + 1;
  }
  return blocks * tpb;
}

int launch_generic_fwd(const FwdParams &p, int dtype, hipStream_t stream) {
  dim3 grids[3];
  const int rows[3] = {128, 64, 32};
  for (int i = 0; i < 3; ++i)
    grids[i] = dim3(fwd_tiles_x(p, rows[i]), p.Hq, p.seqs.packed ? 1 : p.seqs.batch);
  switch (dtype) {
    case DK_BF16: return launch_generic_fwd_t<bf16_t>(p, grids, stream);
    case DK_F16: return launch_generic_fwd_t<f16_t>(p, grids, stream);
    case DK_F32: return launch_generic_fwd_t<float>(p, grids, stream);
  }
  return fail(DK_ERR_UNSUPPORTED, "unknown dtype %d", dtype);
}

}  // namespace dk
