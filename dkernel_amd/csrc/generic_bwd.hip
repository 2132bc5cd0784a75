// Generic backward kernels (any dtype, head_dim <= 256, any power-of-two
// block size): delta = rowsum(O * dO) - dLSE, the dQ pass over CSR rows and
// the dK/dV pass over CSC columns (q heads of a GQA group summed inside the
// workgroup, so no atomics).  Same thread layout as generic_fwd.hip: a thread
// owns 32 head dims of one row, DPAD/32 lanes share a row.
#include "common.h"
#include "device_common.h"
#include "generic_io.h"

namespace dk {

template <typename T, int DPAD>
__global__ __launch_bounds__(256) void generic_delta_kernel(const BwdParams p) {
  constexpr int TPR = DPAD / 32;
  constexpr int R = 256 / TPR;
  const int tid = threadIdx.x, r = tid / TPR, j = tid % TPR;
  const int qi = blockIdx.x * R + r;
  const int h = blockIdx.y, b = blockIdx.z;
  const int Lq = p.seqs.max_q_len;
  const bool ok = qi < Lq;
  const T *op = (const T *)p.o.ptr + b * p.o.sb + h * p.o.sh + (int64_t)qi * p.o.st;
  const T *dp = (const T *)p.dout.ptr + b * p.dout.sb + h * p.dout.sh + (int64_t)qi * p.dout.st;
  float a = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    float x[8], y[8];
    load8_guard<T>(op, (c * TPR + j) * 8, p.D, ok, p.vec_ok, x);
    load8_guard<T>(dp, (c * TPR + j) * 8, p.D, ok, p.vec_ok, y);
#pragma unroll
    for (int i = 0; i < 8; ++i) a = fmaf(x[i], y[i], a);
  }
#pragma unroll
  for (int off = 1; off < TPR; off <<= 1) a += __shfl_xor(a, off);
  if (ok && j == 0) {
    if (p.dlse.ptr) a -= p.dlse.ptr[b * p.dlse.sb + h * p.dlse.sh + (int64_t)qi * p.dlse.st];
    p.delta[((int64_t)b * p.Hq + h) * Lq + qi] = a;
  }
}

template <typename T, int DPAD>
__global__ __launch_bounds__(256) void generic_dq_kernel(const BwdParams p) {
  constexpr int TPR = DPAD / 32;
  constexpr int R = 256 / TPR;
  constexpr int KC = (sizeof(T) == 4 && DPAD == 256) ? 16 : 32;
  constexpr int CH = DPAD / 8;
  __shared__ __align__(16) T sK[KC * DPAD];
  __shared__ __align__(16) T sV[KC * DPAD];

  const int BM = p.csr.block_rows, BN = p.csr.block_cols;
  const int rows_wg = BM < R ? BM : R;
  const int tiles_per_block = BM / rows_wg;
  const SeqInfo sq = load_seq(p.seqs, blockIdx.z, p.causal);
  const int tile = blockIdx.x;
  if (tile >= seq_row_blocks(sq, BM) * tiles_per_block) return;
  const int h = blockIdx.y;
  const int kvh = h / (p.Hq / p.Hkv);
  const int rb = sq.past / BM + tile / tiles_per_block;
  const int tid = threadIdx.x, r = tid / TPR, j = tid % TPR;
  const int row_in_block = (tile % tiles_per_block) * rows_wg + r;
  const int pos = rb * BM + row_in_block;
  const int qi = pos - sq.past;
  const bool row_ok = (r < rows_wg) && qi >= 0 && qi < sq.q_len;
  const int D = p.D;

  float qf[32], dof[32], acc[32];
  {
    const T *qp = (const T *)p.q.ptr + sq.b * p.q.sb + h * p.q.sh + (int64_t)qi * p.q.st;
    const T *dop = (const T *)p.dout.ptr + sq.b * p.dout.sb + h * p.dout.sh + (int64_t)qi * p.dout.st;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      load8_guard<T>(qp, (c * TPR + j) * 8, D, row_ok, p.vec_ok, qf + c * 8);
      load8_guard<T>(dop, (c * TPR + j) * 8, D, row_ok, p.vec_ok, dof + c * 8);
    }
  }
#pragma unroll
  for (int i = 0; i < 32; ++i) acc[i] = 0.f;
  float lse2 = 0.f, delta = 0.f;
  if (row_ok) {
    lse2 = p.lse.ptr[sq.b * p.lse.sb + h * p.lse.sh + (int64_t)qi * p.lse.st] * kLog2e;
    delta = p.delta[((int64_t)sq.b * p.Hq + h) * p.seqs.max_q_len + qi];
  }

  const int lh = lut_head(p.csr, h, p.Hq, p.Hkv);
  int e0 = 0, e1 = 0;
  if (rb < p.csr.num_rows) {
    e0 = p.csr.ptr[lh * p.csr.ptr_sh + rb];
    e1 = p.csr.ptr[lh * p.csr.ptr_sh + rb + 1];
  }
  const T *kbase = (const T *)p.k.ptr + sq.b * p.k.sb + kvh * p.k.sh;
  const T *vbase = (const T *)p.v.ptr + sq.b * p.v.sb + kvh * p.v.sh;
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

      float s[KC], dp[KC];
#pragma unroll
      for (int n = 0; n < KC; ++n) {
        float a = 0.f, b2 = 0.f;
        if (n < kc_n) {
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            float kf[8], vf[8];
            lds_load8<T>(sK + n * DPAD + (c * TPR + j) * 8, kf);
            lds_load8<T>(sV + n * DPAD + (c * TPR + j) * 8, vf);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              a = fmaf(qf[c * 8 + i], kf[i], a);
              b2 = fmaf(dof[c * 8 + i], vf[i], b2);
            }
          }
        }
        s[n] = a;
        dp[n] = b2;
      }
#pragma unroll
      for (int n = 0; n < KC; ++n) {
#pragma unroll
        for (int off = 1; off < TPR; off <<= 1) {
          s[n] += __shfl_xor(s[n], off);
          dp[n] += __shfl_xor(dp[n], off);
        }
      }
#pragma unroll
      for (int n = 0; n < KC; ++n) {
        const int key = key0 + n;
        const bool vis = row_ok && n < kc_n && key < sq.k_len && (!p.causal || key <= pos) &&
                         row_in_block < micro;
        const float pr = vis ? exp2f(s[n] * p.scale_log2 - lse2) : 0.f;
        s[n] = pr * (dp[n] - delta) * p.sm_scale;  // dS
      }
#pragma unroll
      for (int n = 0; n < KC; ++n) {
        if (n < kc_n) {
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            float kf[8];
            lds_load8<T>(sK + n * DPAD + (c * TPR + j) * 8, kf);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[c * 8 + i] = fmaf(s[n], kf[i], acc[c * 8 + i]);
          }
        }
      }
    }
  }
  if (!row_ok) return;
  T *dqp = (T *)p.dq.ptr + sq.b * p.dq.sb + h * p.dq.sh + (int64_t)qi * p.dq.st;
#pragma unroll
  for (int c = 0; c < 4; ++c) store8_guard<T>(dqp, (c * TPR + j) * 8, D, p.vec_ok, acc + c * 8);
}

template <typename T, int DPAD>
__global__ __launch_bounds__(256) void generic_dkdv_kernel(const BwdParams p) {
  constexpr int TPR = DPAD / 32;
  constexpr int R = 256 / TPR;
  constexpr int QC = (sizeof(T) == 4 && DPAD == 256) ? 16 : 32;
  constexpr int CH = DPAD / 8;
  __shared__ __align__(16) T sQ[QC * DPAD];
  __shared__ __align__(16) T sDO[QC * DPAD];
  __shared__ float sLse[QC], sDelta[QC];

  const int BN = p.csc.block_rows;  // keys per column block
  const int BM = p.csc.block_cols;  // query rows per listed entry
  const int keys_wg = BN < R ? BN : R;
  const int tiles_per_block = BN / keys_wg;
  const SeqInfo sq = load_seq(p.seqs, blockIdx.z, p.causal);
  const int tile = blockIdx.x;
  const int cb = tile / tiles_per_block;
  if (cb * BN >= sq.k_len) return;
  const int kvh = blockIdx.y;
  const int ratio = p.Hq / p.Hkv;
  const int tid = threadIdx.x, r = tid / TPR, j = tid % TPR;
  const int key = cb * BN + (tile % tiles_per_block) * keys_wg + r;
  const bool key_ok = (r < keys_wg) && key < sq.k_len;
  const int wg_first_key = cb * BN + (tile % tiles_per_block) * keys_wg;
  const int D = p.D;

  float kf[32], vf[32], dk[32], dv[32];
  {
    const T *kp = (const T *)p.k.ptr + sq.b * p.k.sb + kvh * p.k.sh + (int64_t)key * p.k.st;
    const T *vp = (const T *)p.v.ptr + sq.b * p.v.sb + kvh * p.v.sh + (int64_t)key * p.v.st;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      load8_guard<T>(kp, (c * TPR + j) * 8, D, key_ok, p.vec_ok, kf + c * 8);
      load8_guard<T>(vp, (c * TPR + j) * 8, D, key_ok, p.vec_ok, vf + c * 8);
    }
  }
#pragma unroll
  for (int i = 0; i < 32; ++i) dk[i] = dv[i] = 0.f;
  const int qc_n = BM < QC ? BM : QC;

  for (int g = 0; g < ratio; ++g) {
    const int h = kvh * ratio + g;
    const int lh = lut_head(p.csc, h, p.Hq, p.Hkv);
    int e0 = 0, e1 = 0;
    if (cb < p.csc.num_rows) {
      e0 = p.csc.ptr[lh * p.csc.ptr_sh + cb];
      e1 = p.csc.ptr[lh * p.csc.ptr_sh + cb + 1];
    }
    const T *qbase = (const T *)p.q.ptr + sq.b * p.q.sb + h * p.q.sh;
    const T *dobase = (const T *)p.dout.ptr + sq.b * p.dout.sb + h * p.dout.sh;
    const float *lsebase = p.lse.ptr + sq.b * p.lse.sb + h * p.lse.sh;
    const float *deltabase = p.delta + ((int64_t)sq.b * p.Hq + h) * p.seqs.max_q_len;
    for (int e = e0; e < e1; ++e) {
      const int rbq = p.csc.idx[lh * p.csc.idx_sh + e];
      const int pos0 = rbq * BM;
      if (rbq < 0 || pos0 >= sq.past + sq.q_len || pos0 + BM <= sq.past) continue;
      if (p.causal && pos0 + BM - 1 < wg_first_key) continue;
      for (int ch = 0; ch < BM / qc_n; ++ch) {
        const int p0 = pos0 + ch * qc_n;
        __syncthreads();
        for (int t = tid; t < qc_n * CH; t += 256) {
          const int m = t / CH, c8 = t % CH;
          const int qi = p0 + m - sq.past;
          const bool ok = qi >= 0 && qi < sq.q_len;
          copy8_guard<T>(qbase + (int64_t)qi * p.q.st, c8 * 8, D, ok, p.vec_ok, sQ + m * DPAD + c8 * 8);
          copy8_guard<T>(dobase + (int64_t)qi * p.dout.st, c8 * 8, D, ok, p.vec_ok, sDO + m * DPAD + c8 * 8);
        }
        if (tid < qc_n) {
          const int qi = p0 + tid - sq.past;
          const bool ok = qi >= 0 && qi < sq.q_len;
          sLse[tid] = ok ? lsebase[(int64_t)qi * p.lse.st] * kLog2e : 0.f;
          sDelta[tid] = ok ? deltabase[qi] : 0.f;
        }
        __syncthreads();

        float s[QC], dp[QC];
#pragma unroll
        for (int m = 0; m < QC; ++m) {
          float a = 0.f, b2 = 0.f;
          if (m < qc_n) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
              float qv[8], dov[8];
              lds_load8<T>(sQ + m * DPAD + (c * TPR + j) * 8, qv);
              lds_load8<T>(sDO + m * DPAD + (c * TPR + j) * 8, dov);
#pragma unroll
              for (int i = 0; i < 8; ++i) {
                a = fmaf(kf[c * 8 + i], qv[i], a);
                b2 = fmaf(vf[c * 8 + i], dov[i], b2);
              }
            }
          }
          s[m] = a;
          dp[m] = b2;
        }
#pragma unroll
        for (int m = 0; m < QC; ++m) {
#pragma unroll
          for (int off = 1; off < TPR; off <<= 1) {
            s[m] += __shfl_xor(s[m], off);
            dp[m] += __shfl_xor(dp[m], off);
          }
        }
#pragma unroll
        for (int m = 0; m < QC; ++m) {
          const int pos = p0 + m;
          const int qi = pos - sq.past;
          const bool vis = key_ok && m < qc_n && qi >= 0 && qi < sq.q_len && (!p.causal || key <= pos);
          const float lse2 = m < qc_n ? sLse[m] : 0.f;
          const float dl = m < qc_n ? sDelta[m] : 0.f;
          const float pr = vis ? exp2f(s[m] * p.scale_log2 - lse2) : 0.f;
          s[m] = pr;                                // P
          dp[m] = pr * (dp[m] - dl) * p.sm_scale;   // dS
        }
#pragma unroll
        for (int m = 0; m < QC; ++m) {
          if (m < qc_n) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
              float qv[8], dov[8];
              lds_load8<T>(sQ + m * DPAD + (c * TPR + j) * 8, qv);
              lds_load8<T>(sDO + m * DPAD + (c * TPR + j) * 8, dov);
#pragma unroll
              for (int i = 0; i < 8; ++i) {
                dv[c * 8 + i] = fmaf(s[m], dov[i], dv[c * 8 + i]);
                dk[c * 8 + i] = fmaf(dp[m], qv[i], dk[c * 8 + i]);
              }
            }
          }
        }
      }
    }
  }
  if (!key_ok) return;
  T *dkp = (T *)p.dk.ptr + sq.b * p.dk.sb + kvh * p.dk.sh + (int64_t)key * p.dk.st;
  T *dvp = (T *)p.dv.ptr + sq.b * p.dv.sb + kvh * p.dv.sh + (int64_t)key * p.dv.st;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    store8_guard<T>(dkp, (c * TPR + j) * 8, D, p.vec_ok, dk + c * 8);
    store8_guard<T>(dvp, (c * TPR + j) * 8, D, p.vec_ok, dv + c * 8);
  }
}

template <typename T, int DPAD>
static int launch_bwd_td(const BwdParams &p, hipStream_t stream) {
  constexpr int R = 256 / (DPAD / 32);
  const SeqView &s = p.seqs;
  DK_NOTE_KERNEL("generic_delta_kernel");
  hipLaunchKernelGGL((generic_delta_kernel<T, DPAD>), dim3(cdiv(s.max_q_len, R), p.Hq, s.batch), dim3(256), 0,
                     stream, p);
  DK_HIP_CHECK(hipGetLastError());
  {
    const int BM = p.csr.block_rows;
    const int rows_wg = BM < R ? BM : R;
    const int past = p.causal ? s.max_k_len - s.max_q_len : 0;
    const int blocks = (past + s.max_q_len - 1) / BM - past / BM + 1;
    DK_NOTE_KERNEL("generic_dq_kernel");
    hipLaunchKernelGGL((generic_dq_kernel<T, DPAD>), dim3(blocks * (BM / rows_wg), p.Hq, s.batch), dim3(256), 0,
                       stream, p);
    DK_HIP_CHECK(hipGetLastError());
  }
  {
    const int BN = p.csc.block_rows;
    const int keys_wg = BN < R ? BN : R;
    DK_NOTE_KERNEL("generic_dkdv_kernel");
    hipLaunchKernelGGL((generic_dkdv_kernel<T, DPAD>),
                       dim3(cdiv(s.max_k_len, BN) * (BN / keys_wg), p.Hkv, s.batch), dim3(256), 0, stream, p);
    DK_HIP_CHECK(hipGetLastError());
  }
  return DK_OK;
}

template <typename T>
static int launch_bwd_t(const BwdParams &p, hipStream_t stream) {
  if (p.D <= 64) return launch_bwd_td<T, 64>(p, stream);
  if (p.D <= 128) return launch_bwd_td<T, 128>(p, stream);
  return launch_bwd_td<T, 256>(p, stream);
}

int launch_generic_bwd(const BwdParams &p, int dtype, hipStream_t stream) {
  switch (dtype) {
    case DK_BF16: return launch_bwd_t<bf16_t>(p, stream);
    case DK_F16: return launch_bwd_t<f16_t>(p, stream);
    case DK_F32: return launch_bwd_t<float>(p, stream);
  }
  return fail(DK_ERR_UNSUPPORTED, "unknown dtype %d", dtype);
}

}  // namespace dk
