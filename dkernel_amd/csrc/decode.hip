// Split-KV decode kernel for gfx950: one new query token per sequence over
// padded (left or right) or unpadded 4-D K/V, bf16 / fp16, head_dim 128 or 64,
// 64 x 64 blocks, grouped-query attention with all q heads of a kv head
// sharing the look-up-table row.  The step is HBM-bound (every attended K/V
// byte is read exactly once, for all q heads of the group together), so the
// design goal is bytes in flight, not FLOPs:
//
//   workgroup = (sequence, kv head, split); its 4 waves each own whole K/V
//               blocks of the row (round-robin), so 4 x 32 KB of loads are in
//               flight per workgroup with no barrier between them;
//   wave      = loads its block with coalesced 16-byte accesses into a private
//               LDS tile, computes S^T = K Q^T (the q heads of the group are
//               the MFMA columns), softmax, O^T += V^T P^T with LDS transpose
//               reads, keeping a private running (max, sum, O);
//   epilogue  = the 4 waves are merged through LDS into one fp32 partial
//               (O unnormalised, max, sum) per (sequence, q head, split) in
//               the caller's workspace; a second small kernel merges the
//               splits, normalises and writes O and LSE.
#include "common.h"
#include "device_common.h"
#include "mfma_common.h"

namespace dk {

constexpr int kDecodeSplits = 4;
constexpr int kDecodeWaves = 4;

template <int D>
struct DecSmem {
  static constexpr int kKStride = D * 2 + 16;
  static constexpr int kVStride = D * 2 + 64;
  static constexpr int kKBytes = 64 * kKStride;
  static constexpr int kVBytes = 64 * kVStride;
  static constexpr int kWave = kKBytes + kVBytes;
};

// workspace layout: [batch][Hq][splits][D + 2] floats (O[D], max, sum)
template <typename T, int D>
__global__ __launch_bounds__(64 * kDecodeWaves) void decode_partial_kernel(const FwdParams p, float *ws) {
  using M = Mma<T>;
  using vec8 = typename M::vec8;
  using S = DecSmem<D>;
  constexpr int KS = D / 16, DT = D / 32, CPR = D / 8;
  constexpr int CHUNKS = 64 * CPR / 64;  // 16-byte chunks per lane per tile
  extern __shared__ __align__(16) char smem[];

  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const SeqInfo sq = load_seq(p.seqs, b, p.causal);
  const int ratio = p.Hq / p.Hkv;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 31, g = lane >> 5;  // m = q head inside the group (MFMA column)
  const bool active = sq.q_len > 0 && sq.k_len > 0;
  const int pos = sq.past;                 // absolute position of the single query token
  const int rb = pos / 64;
  const int h0 = kvh * ratio;

  vec8 qf[KS];
  {
    const T *qp = (const T *)p.q.ptr + sq.b * p.q.sb + (int64_t)(h0 + m) * p.q.sh + (int64_t)sq.q_start * p.q.st;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 w = make_uint4(0, 0, 0, 0);
      if (active && m < ratio) w = *reinterpret_cast<const uint4 *>(qp + ks * 16 + g * 8);
      qf[ks] = as_vec8<vec8>(w);
    }
  }
  const int lh = lut_head(p.csr, h0, p.Hq, p.Hkv);
  int e0 = 0, e1 = 0;
  if (active && rb < p.csr.num_rows) {
    e0 = p.csr.ptr[lh * p.csr.ptr_sh + rb];
    e1 = p.csr.ptr[lh * p.csr.ptr_sh + rb + 1];
  }
  const int32_t *cols = p.csr.idx + lh * p.csr.idx_sh;
  const T *kbase = (const T *)p.k.ptr + sq.b * p.k.sb + kvh * p.k.sh + (int64_t)sq.k_start * p.k.st;
  const T *vbase = (const T *)p.v.ptr + sq.b * p.v.sb + kvh * p.v.sh + (int64_t)sq.k_start * p.v.st;

  char *ks_ = smem + wave * S::kWave, *vs_ = ks_ + S::kKBytes;
  uint4 kreg[CHUNKS], vreg[CHUNKS];
  auto prefetch = [&](int e) {
    const int col = cols[e];
    const int key0 = col * 64;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int idx = lane + c * 64;
      const int r = idx / CPR, ch = idx % CPR;
      kreg[c] = vreg[c] = make_uint4(0, 0, 0, 0);
      if (col >= 0 && key0 + r < sq.k_len) {
        kreg[c] = *reinterpret_cast<const uint4 *>(kbase + (int64_t)(key0 + r) * p.k.st + ch * 8);
        vreg[c] = *reinterpret_cast<const uint4 *>(vbase + (int64_t)(key0 + r) * p.v.st + ch * 8);
      }
    }
  };

  floatx16 oacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  const int k_read = m * S::kKStride + g * 16;
  const int i16 = lane & 15, dgrp = (lane >> 4) & 1;
  const int v_read = (4 * g + (i16 >> 2)) * S::kVStride + (16 * dgrp + 4 * (i16 & 3)) * 2;
  constexpr int STEP = kDecodeSplits * kDecodeWaves;

  int e = e0 + split * kDecodeWaves + wave;
  if (e < e1) prefetch(e);
  for (; e < e1; e += STEP) {
    const int col = cols[e];
    const int key0 = col * 64;
    // this wave's private tile: the previous block's reads are complete
    // (program order within the wave), so it can be overwritten
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int idx = lane + c * 64;
      const int r = idx / CPR, ch = idx % CPR;
      *reinterpret_cast<uint4 *>(ks_ + r * S::kKStride + ch * 16) = kreg[c];
      *reinterpret_cast<uint4 *>(vs_ + r * S::kVStride + ch * 16) = vreg[c];
    }
    if (e + STEP < e1) prefetch(e + STEP);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (col < 0 || key0 >= sq.k_len || (p.causal && key0 > pos)) continue;

    floatx16 sacc[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[nt][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        vec8 a = lds_read8<vec8>(ks_ + k_read + nt * 32 * S::kKStride + ks * 32);
        sacc[nt] = M::mma(a, qf[ks], sacc[nt]);
      }
    }
    const bool need_mask = (key0 + 63 >= sq.k_len) || (p.causal && key0 + 63 > pos);
    float mx = -INFINITY;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float s = sacc[nt][r] * p.scale_log2;
        if (need_mask) {
          const int key = key0 + nt * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
          if (key >= sq.k_len || (p.causal && key > pos)) s = -INFINITY;
        }
        sacc[nt][r] = s;
        mx = fmaxf(mx, s);
      }
    mx = fmaxf(mx, xor32(mx));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_use);
    float psum = 0.f;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pv = fast_exp2(sacc[nt][r] - m_use);
        sacc[nt][r] = pv;
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
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        float pf[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) pf[i] = sacc[nt][t * 8 + i];
        const vec8 pb = M::pack(pf);
        const char *vrow = vs_ + v_read + (nt * 32 + t * 16) * S::kVStride;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          vec8 a = lds_read_tr8<vec8>(vrow + dt * 64, vrow + 8 * S::kVStride + dt * 64);
          oacc[dt] = M::mma(a, pb, oacc[dt]);
        }
      }
  }

  // ---- merge the 4 waves through LDS (tiles are dead now) ----
  __syncthreads();
  float *red_o = reinterpret_cast<float *>(smem);            // [wave][head][D]
  float *red_ml = red_o + kDecodeWaves * 32 * D;             // [wave][head][2]
  if (m < ratio) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        red_o[(wave * 32 + m) * D + dt * 32 + (r >> 2) * 8 + g * 4 + (r & 3)] = oacc[dt][r];
    if (g == 0) {
      red_ml[(wave * 32 + m) * 2 + 0] = m_run;
      red_ml[(wave * 32 + m) * 2 + 1] = l_run;
    }
  }
  __syncthreads();
  for (int idx = tid; idx < ratio * D; idx += 64 * kDecodeWaves) {
    const int hh = idx / D, d = idx % D;
    float mw[kDecodeWaves], mmax = -INFINITY;
#pragma unroll
    for (int w = 0; w < kDecodeWaves; ++w) {
      mw[w] = red_ml[(w * 32 + hh) * 2];
      mmax = fmaxf(mmax, mw[w]);
    }
    const float muse = mmax == -INFINITY ? 0.f : mmax;
    float o = 0.f, l = 0.f;
#pragma unroll
    for (int w = 0; w < kDecodeWaves; ++w) {
      const float sc = fast_exp2(mw[w] - muse);
      o += sc * red_o[(w * 32 + hh) * D + d];
      l += sc * red_ml[(w * 32 + hh) * 2 + 1];
    }
    float *dst = ws + (((int64_t)b * p.Hq + h0 + hh) * kDecodeSplits + split) * (D + 2);
    dst[d] = o;
    if (d == 0) {
      dst[D] = mmax;
      dst[D + 1] = l;
    }
  }
}

template <typename T, int D>
__global__ __launch_bounds__(D) void decode_combine_kernel(const FwdParams p, const float *ws) {
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  const SeqInfo sq = load_seq(p.seqs, b, p.causal);
  if (sq.q_len <= 0) return;
  const float *src = ws + ((int64_t)b * p.Hq + h) * kDecodeSplits * (D + 2);
  float mmax = -INFINITY;
#pragma unroll
  for (int s = 0; s < kDecodeSplits; ++s) mmax = fmaxf(mmax, src[s * (D + 2) + D]);
  const float muse = mmax == -INFINITY ? 0.f : mmax;
  float o = 0.f, l = 0.f;
#pragma unroll
  for (int s = 0; s < kDecodeSplits; ++s) {
    const float sc = fast_exp2(src[s * (D + 2) + D] - muse);
    o += sc * src[s * (D + 2) + d];
    l += sc * src[s * (D + 2) + D + 1];
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  T *op = (T *)p.o.ptr + sq.b * p.o.sb + h * p.o.sh + (int64_t)sq.q_start * p.o.st;
  op[d] = from_float<T>(o * inv);
  if (p.lse.ptr && d == 0)
    p.lse.ptr[sq.b * p.lse.sb + h * p.lse.sh + (int64_t)sq.q_start * p.lse.st] =
        l > 0.f ? (mmax + log2f(l)) * kLn2 : -INFINITY;
}

bool decode_supported(const FwdParams &p, int dtype) {
  const int ratio = p.Hq / p.Hkv;
  const bool shared_row = p.csr.num_heads == 1 || (p.csr.num_heads == p.Hkv && p.Hkv != p.Hq) || ratio == 1 ||
                          (p.csr.num_heads == p.Hq && p.csr.group % ratio == 0);
  return (dtype == DK_BF16 || dtype == DK_F16) && (p.D == 128 || p.D == 64) && p.csr.block_rows == 64 &&
         p.csr.block_cols == 64 && p.csr.entry_width == 1 && p.vec_ok && !p.seqs.packed &&
         p.seqs.max_q_len == 1 && ratio <= 32 && shared_row && p.causal;
}

size_t decode_workspace_bytes(const FwdParams &p) {
  return (size_t)p.seqs.batch * p.Hq * kDecodeSplits * (p.D + 2) * sizeof(float);
}

template <typename T, int D>
static int launch_decode_td(const FwdParams &p, float *ws, hipStream_t stream) {
  constexpr int tiles = kDecodeWaves * DecSmem<D>::kWave;
  constexpr int red = (kDecodeWaves * 32 * D + kDecodeWaves * 32 * 2) * 4;
  constexpr int smem = tiles > red ? tiles : red;
  static bool attr_set = false;
  if (!attr_set) {
    DK_HIP_CHECK(hipFuncSetAttribute((const void *)decode_partial_kernel<T, D>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    attr_set = true;
  }
  hipLaunchKernelGGL((decode_partial_kernel<T, D>), dim3(kDecodeSplits, p.Hkv, p.seqs.batch),
                     dim3(64 * kDecodeWaves), smem, stream, p, ws);
  DK_HIP_CHECK(hipGetLastError());
  hipLaunchKernelGGL((decode_combine_kernel<T, D>), dim3(p.Hq, p.seqs.batch), dim3(D), 0, stream, p, ws);
  DK_HIP_CHECK(hipGetLastError());
  return DK_OK;
}

int launch_decode(const FwdParams &p, int dtype, void *workspace, size_t workspace_bytes, hipStream_t stream) {
  DK_REQUIRE(workspace && workspace_bytes >= decode_workspace_bytes(p), "decode workspace too small");
  DK_REQUIRE(((uintptr_t)workspace % 16) == 0, "decode workspace must be 16-byte aligned");
  float *ws = (float *)workspace;
  if (dtype == DK_BF16)
    return p.D == 128 ? launch_decode_td<bf16_t, 128>(p, ws, stream) : launch_decode_td<bf16_t, 64>(p, ws, stream);
  return p.D == 128 ? launch_decode_td<f16_t, 128>(p, ws, stream) : launch_decode_td<f16_t, 64>(p, ws, stream);
}

}  // namespace dk
