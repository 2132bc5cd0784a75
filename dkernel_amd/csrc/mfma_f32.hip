// fp32 inputs on the matrix cores of gfx950: v_mfma_f32_32x32x2_f32, head dims up to 64 (multiples
// of 4, zero-padded to 64 on chip), 64 x 64 tiles with one int per table entry.  Forward (fixed,
// padded, packed and single-token sequences, LSE) and backward (dQ over CSR rows, dK/dV over CSC
// columns; delta = rowsum(O * dO) - dLSE by a small kernel ahead of them).  fp32 products with
// fp32 accumulation: results agree with the generic fp32-FMA kernels to rounding.
//
//   D(32x32) += A(32x2) * B(2x32):  A operand, lane l: row l%32, k = l/32 (one float)
//                                   B operand, lane l: col l%32, k = l/32
//                                   accumulator, lane l, register r: col l%32, row 8(r/4) + 4(l/32) + r%4
//
// The contraction index of a product may be walked in any order as long as A and B agree, so:
//  * products over head dims (S = K Q^T, dP = V dO^T, ...) give lane (x, g) the dims 32 g + s in
//    step s: a lane's operands of 32 steps are 32 consecutive floats (16-byte reads);
//  * products over keys or q rows (O^T += V^T P^T, dQ^T += K^T dS^T, dV^T += dO^T P, dK^T += Q^T dS)
//    take step (tile, r) = the pair of rows that accumulator register r of the two half-waves
//    stands for, 8(r/4) + r%4 and 8(r/4) + 4 + r%4: the second operand is then the lane's own
//    register r of the S / P / dS accumulator, with no exchange between lanes, and the first
//    one a 4-byte LDS read per lane, 32 consecutive floats of one tile row per half-wave.
// Tiles live in LDS as plain rows of 64 floats plus 4 floats of padding (16-byte row reads of 16
// consecutive rows then touch every bank once).  One stage per workgroup: with up to five small
// workgroups per CU, one loads while the others multiply.
#include "common.h"
#include "device_common.h"
#include "mfma_common.h"

namespace dk {

namespace f32 {

constexpr int kD = 64;        // tile width (head dims, zero-padded)
constexpr int kLd = kD + 4;   // floats per tile row in LDS

__device__ __forceinline__ floatx16 mma(float a, float b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// 64 rows x 64 floats from memory (row r at base + r * stride, rows outside [lo, hi) and head
// dims at or beyond d as zeros) into an LDS tile, by NT threads; 16-byte pieces, consecutive
// threads along a row.
template <int NT>
__device__ __forceinline__ void load_tile(const float *base, int64_t stride, int lo, int hi, int d, float *tile, int tid) {
#pragma unroll
  for (int i = 0; i < 64 * 16 / NT; ++i) {
    const int c = tid + i * NT, r = c >> 4, ch = c & 15;
    float4 w = make_float4(0.f, 0.f, 0.f, 0.f);
    if (r >= lo && r < hi && ch * 4 < d) w = *reinterpret_cast<const float4 *>(base + (int64_t)r * stride + ch * 4);
    *reinterpret_cast<float4 *>(tile + r * kLd + ch * 4) = w;
  }
}

// acc(32 x 32) += X Y^T over the 64 head dims: rows = the 32 rows of tile `xt` from row0, columns =
// the lanes' own rows of Y.  Lane (x, g) multiplies dims 32 g + s in step s; yf[s] is dim 32 g + s
// of the row of Y that is the lane's column.
__device__ __forceinline__ floatx16 dot_dims(const float *xt, int row0, const float (&yf)[32], int lane, floatx16 acc) {
  const float *src = xt + (row0 + (lane & 31)) * kLd + (lane >> 5) * 32;
#pragma unroll
  for (int s4 = 0; s4 < 8; ++s4) {
    const float4 x = *reinterpret_cast<const float4 *>(src + s4 * 4);
    acc = mma(x.x, yf[s4 * 4], acc);
    acc = mma(x.y, yf[s4 * 4 + 1], acc);
    acc = mma(x.z, yf[s4 * 4 + 2], acc);
    acc = mma(x.w, yf[s4 * 4 + 3], acc);
  }
  return acc;
}

// acc[dt](32 dims x 32 columns) += T^T(dims x rows) * W(rows x columns) over the 32 rows row0 .. row0 + 31 of
// tile `t`: step r takes rows 8(r/4) + r%4 (+4 in the upper half-wave), w[r] is the lane's own
// accumulator register r of W^T's product (column = lane % 32).
__device__ __forceinline__ void dot_rows(const float *t, int row0, const floatx16 &w, int lane, floatx16 (&acc)[2]) {
  const int g = lane >> 5, m = lane & 31;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float *row = t + (row0 + (r >> 2) * 8 + g * 4 + (r & 3)) * kLd + m;
    acc[0] = mma(row[0], w[r], acc[0]);
    acc[1] = mma(row[32], w[r], acc[1]);
  }
}

// 32 consecutive floats of a row (dims 32 g ..) as one lane's operands; zeros when !ok or beyond d
__device__ __forceinline__ void load_frag(const float *row, bool ok, int g, int d, float (&f)[32]) {
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    float4 w = make_float4(0.f, 0.f, 0.f, 0.f);
    if (ok && g * 32 + c * 4 < d) w = *reinterpret_cast<const float4 *>(row + g * 32 + c * 4);
    f[c * 4] = w.x, f[c * 4 + 1] = w.y, f[c * 4 + 2] = w.z, f[c * 4 + 3] = w.w;
  }
}

// the lane's 32 result values of a (dims x columns) accumulator pair: dims 32 dt + 8 r4 + 4 g + {0..3}
__device__ __forceinline__ void store_frag(float *row, const floatx16 (&acc)[2], float scale, int g, int d) {
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const int d0 = dt * 32 + r4 * 8 + g * 4;
      if (d0 < d)
        *reinterpret_cast<float4 *>(row + d0) = make_float4(acc[dt][r4 * 4] * scale, acc[dt][r4 * 4 + 1] * scale,
                                                            acc[dt][r4 * 4 + 2] * scale, acc[dt][r4 * 4 + 3] * scale);
    }
}

// ---------------------------------------------------------------------------
// forward: workgroup = 64 q rows of one head, 2 waves of 32 rows
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(128) void fwd_kernel(const FwdParams p, int tiles_y) {
  __shared__ __align__(16) float sK[64 * kLd];
  __shared__ __align__(16) float sV[64 * kLd];
  SeqInfo sq;
  int tile;
  bool has_rows;
  if (p.csr.order && !p.seqs.packed) {  // the table's own order, longest rows first (the grid covers every row of it)
    sq = load_seq(p.seqs, blockIdx.z, p.causal);
    tile = p.csr.order[lut_head(p.csr, grid_head(p.csr), p.Hq, p.Hkv) * p.csr.order_sh + blockIdx.y] - sq.past / 64;
    has_rows = tile >= 0 && tile < seq_row_blocks(sq, 64);
  } else {
    has_rows = resolve_tile(p.seqs, p.causal, 64, 1, tiles_y - 1 - (int)blockIdx.y, blockIdx.z, sq, tile);
  }
  if (p.seqs.zero_outside)
    zero_rows_outside<float>(p.seqs, sq, blockIdx.y, tiles_y, p.o, p.lse, grid_head(p.csr), 1, p.D, p.vec_ok, threadIdx.x, 128);
  if (!has_rows) return;
  const int rb = sq.past / 64 + tile;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int h = grid_head(p.csr), kvh = h / (p.Hq / p.Hkv);
  const int m = lane & 31, g = lane >> 5;
  const int row0 = rb * 64 + wave * 32;
  const int pos = row0 + m, qi = pos - sq.past;
  const bool row_ok = qi >= 0 && qi < sq.q_len;

  float qf[32];
  load_frag((const float *)p.q.ptr + sq.b * p.q.sb + h * p.q.sh + (int64_t)(sq.q_start + qi) * p.q.st, row_ok, g, p.D, qf);
  const int lh = lut_head(p.csr, h, p.Hq, p.Hkv);
  int e0 = 0, e1 = 0;
  if (rb < p.csr.num_rows) e0 = p.csr.ptr[lh * p.csr.ptr_sh + rb], e1 = p.csr.ptr[lh * p.csr.ptr_sh + rb + 1];
  const int32_t *cols = p.csr.idx + lh * p.csr.idx_sh;
  const float *kbase = (const float *)p.k.ptr + sq.b * p.k.sb + kvh * p.k.sh + (int64_t)sq.k_start * p.k.st;
  const float *vbase = (const float *)p.v.ptr + sq.b * p.v.sb + kvh * p.v.sh + (int64_t)sq.k_start * p.v.st;

  floatx16 oacc[2];
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;  // running maximum (log2 domain) and this lane's share of the row sum
  const int lim = p.causal ? min(pos, sq.k_len - 1) : sq.k_len - 1;  // last visible key of this row

  for (int e = e0; e < e1; ++e) {
    const int col = cols[e];
    const int key0 = col * 64;
    if (col < 0 || key0 >= sq.k_len || (p.causal && key0 > rb * 64 + 63)) continue;  // (workgroup-uniform)
    __syncthreads();  // every wave is done with the tiles of the block before
    load_tile<128>(kbase + (int64_t)key0 * p.k.st, p.k.st, 0, sq.k_len - key0, p.D, sK, tid);
    load_tile<128>(vbase + (int64_t)key0 * p.v.st, p.v.st, 0, sq.k_len - key0, p.D, sV, tid);
    __syncthreads();
    if (p.causal && key0 > row0 + 31) continue;  // nothing visible for this wave's rows (a barrier pair per block stays)
    // S^T = K Q^T: lane = q row, registers = keys 32 nt + 8(r/4) + 4g + r%4
    floatx16 s[2];
    float mx = -INFINITY;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[nt][r] = 0.f;
      s[nt] = dot_dims(sK, nt * 32, qf, lane, s[nt]);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = key0 + nt * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
        s[nt][r] = key > lim || !row_ok ? -INFINITY : s[nt][r] * p.scale_log2;
        mx = fmaxf(mx, s[nt][r]);
      }
    }
    mx = fmaxf(mx, xor32(mx));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_use);  // exp2(-inf) = 0 before the first visible key
    float psum = 0.f;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        s[nt][r] = fast_exp2(s[nt][r] - m_use);
        psum += s[nt][r];
      }
    l_run = l_run * alpha + psum;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
    // O^T += V^T P^T
    dot_rows(sV, 0, s[0], lane, oacc);
    dot_rows(sV, 32, s[1], lane, oacc);
  }
  l_run += xor32(l_run);
  if (!row_ok) return;
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  store_frag((float *)p.o.ptr + sq.b * p.o.sb + h * p.o.sh + (int64_t)(sq.q_start + qi) * p.o.st, oacc, inv, g, p.D);
  if (p.lse.ptr && g == 0)
    p.lse.ptr[sq.b * p.lse.sb + h * p.lse.sh + (int64_t)(sq.q_start + qi) * p.lse.st] =
        l_run > 0.f ? (m_run + log2f(l_run)) * kLn2 : -INFINITY;
}

// ---------------------------------------------------------------------------
// backward
// ---------------------------------------------------------------------------
// delta = rowsum(O * dO) - dLSE: one thread per 16-byte piece of a row, 16 pieces per row
__global__ __launch_bounds__(256) void delta_kernel(const BwdParams p) {
  const int r = threadIdx.x >> 4, ch = threadIdx.x & 15;
  const int qi = blockIdx.x * 16 + r, h = blockIdx.y, b = blockIdx.z;
  const bool ok = qi < p.seqs.max_q_len;
  float d = 0.f;
  if (ok && ch * 4 < p.D) {
    const float4 o = *reinterpret_cast<const float4 *>((const float *)p.o.ptr + b * p.o.sb + h * p.o.sh + (int64_t)qi * p.o.st + ch * 4);
    const float4 g = *reinterpret_cast<const float4 *>((const float *)p.dout.ptr + b * p.dout.sb + h * p.dout.sh + (int64_t)qi * p.dout.st + ch * 4);
    d = o.x * g.x + o.y * g.y + o.z * g.z + o.w * g.w;
  }
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) d += __shfl_xor(d, off);
  if (ok && ch == 0) {
    if (p.dlse.ptr) d -= p.dlse.ptr[b * p.dlse.sb + h * p.dlse.sh + (int64_t)qi * p.dlse.st];
    p.delta[((int64_t)b * p.Hq + h) * p.seqs.max_q_len + qi] = d;
  }
}

// dQ: workgroup = 64 q rows of one head, 2 waves of 32 rows; per listed block S^T = K Q^T,
// dP^T = V dO^T (lane = q row: lse and delta are per-lane scalars), dS^T = P^T (dP^T - delta),
// dQ^T += K^T dS^T.
__global__ __launch_bounds__(128) void dq_kernel(const BwdParams p, int tiles_y) {
  __shared__ __align__(16) float sK[64 * kLd];
  __shared__ __align__(16) float sV[64 * kLd];
  const SeqInfo sq = load_seq(p.seqs, blockIdx.z, p.causal);
  const int h = grid_head(p.csr), kvh = h / (p.Hq / p.Hkv);
  int tile = tiles_y - 1 - (int)blockIdx.y;
  if (p.csr.order) tile = p.csr.order[lut_head(p.csr, h, p.Hq, p.Hkv) * p.csr.order_sh + blockIdx.y] - sq.past / 64;
  if (tile < 0 || tile >= seq_row_blocks(sq, 64)) return;
  const int rb = sq.past / 64 + tile;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 31, g = lane >> 5;
  const int row0 = rb * 64 + wave * 32;
  const int pos = row0 + m, qi = pos - sq.past;
  const bool row_ok = qi >= 0 && qi < sq.q_len;

  float qf[32], dof[32];
  load_frag((const float *)p.q.ptr + sq.b * p.q.sb + h * p.q.sh + (int64_t)qi * p.q.st, row_ok, g, p.D, qf);
  load_frag((const float *)p.dout.ptr + sq.b * p.dout.sb + h * p.dout.sh + (int64_t)qi * p.dout.st, row_ok, g, p.D, dof);
  float lse2 = INFINITY, delta = 0.f;  // a row outside the sequence: P = exp2(. - inf) = 0
  if (row_ok) {
    const float lse = p.lse.ptr[sq.b * p.lse.sb + h * p.lse.sh + (int64_t)qi * p.lse.st];
    lse2 = lse == -INFINITY ? INFINITY : lse * kLog2e;
    delta = p.delta[((int64_t)sq.b * p.Hq + h) * p.seqs.max_q_len + qi];
  }
  const int lh = lut_head(p.csr, h, p.Hq, p.Hkv);
  int e0 = 0, e1 = 0;
  if (rb < p.csr.num_rows) e0 = p.csr.ptr[lh * p.csr.ptr_sh + rb], e1 = p.csr.ptr[lh * p.csr.ptr_sh + rb + 1];
  const int32_t *cols = p.csr.idx + lh * p.csr.idx_sh;
  const float *kbase = (const float *)p.k.ptr + sq.b * p.k.sb + kvh * p.k.sh;
  const float *vbase = (const float *)p.v.ptr + sq.b * p.v.sb + kvh * p.v.sh;
  floatx16 acc[2];
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
  const int lim = p.causal ? min(pos, sq.k_len - 1) : sq.k_len - 1;

  for (int e = e0; e < e1; ++e) {
    const int col = cols[e];
    const int key0 = col * 64;
    if (col < 0 || key0 >= sq.k_len || (p.causal && key0 > rb * 64 + 63)) continue;
    __syncthreads();
    load_tile<128>(kbase + (int64_t)key0 * p.k.st, p.k.st, 0, sq.k_len - key0, p.D, sK, tid);
    load_tile<128>(vbase + (int64_t)key0 * p.v.st, p.v.st, 0, sq.k_len - key0, p.D, sV, tid);
    __syncthreads();
    if (p.causal && key0 > row0 + 31) continue;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      floatx16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
      s = dot_dims(sK, nt * 32, qf, lane, s);
      dp = dot_dims(sV, nt * 32, dof, lane, dp);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = key0 + nt * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
        const float pr = key > lim ? 0.f : fast_exp2(fmaf(s[r], p.scale_log2, -lse2));
        s[r] = pr * (dp[r] - delta);  // dS^T without sm_scale (applied once at the end)
      }
      dot_rows(sK, nt * 32, s, lane, acc);
    }
  }
  if (!row_ok) return;
  store_frag((float *)p.dq.ptr + sq.b * p.dq.sb + h * p.dq.sh + (int64_t)qi * p.dq.st, acc, p.sm_scale, g, p.D);
}

// dK / dV: workgroup = 64 keys of one kv head (the q heads of its group one after the other), 2
// waves of 32 keys with their K and V rows in registers; per listed q block (64 rows in two halves)
// S = Q K^T, dP = dO V^T (lane = key, registers = q rows), P = exp(S - lse), dS = P (dP - delta),
// dV^T += dO^T P, dK^T += Q^T dS.  Every CSC entry is tested against the sequence length.
__global__ __launch_bounds__(128) void dkdv_kernel(const BwdParams p) {
  __shared__ __align__(16) float sQ[64 * kLd];
  __shared__ __align__(16) float sDo[64 * kLd];
  __shared__ float sLse[64], sDelta[64];
  const SeqInfo sq = load_seq(p.seqs, blockIdx.z, p.causal);
  const int kvh = grid_head(p.csc), ratio = p.Hq / p.Hkv;
  int cb = blockIdx.y;  // longest columns first when the table gives the order (as in the 16-bit pass)
  if (p.csc.order) cb = p.csc.order[lut_head(p.csc, kvh * ratio, p.Hq, p.Hkv) * p.csc.order_sh + blockIdx.y];
  if (cb * 64 >= sq.k_len) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, g = lane >> 5;
  const int key = cb * 64 + wave * 32 + n;
  const bool key_ok = key < sq.k_len;
  float kf[32], vf[32];
  load_frag((const float *)p.k.ptr + sq.b * p.k.sb + kvh * p.k.sh + (int64_t)key * p.k.st, key_ok, g, p.D, kf);
  load_frag((const float *)p.v.ptr + sq.b * p.v.sb + kvh * p.v.sh + (int64_t)key * p.v.st, key_ok, g, p.D, vf);
  floatx16 dk[2], dv[2];
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) dk[dt][r] = dv[dt][r] = 0.f;

  for (int gq = 0; gq < ratio; ++gq) {
    const int h = kvh * ratio + gq;
    const int lh = lut_head(p.csc, h, p.Hq, p.Hkv);
    int e0 = 0, e1 = 0;
    if (cb < p.csc.num_rows) e0 = p.csc.ptr[lh * p.csc.ptr_sh + cb], e1 = p.csc.ptr[lh * p.csc.ptr_sh + cb + 1];
    const int32_t *rows = p.csc.idx + lh * p.csc.idx_sh;
    const float *qbase = (const float *)p.q.ptr + sq.b * p.q.sb + h * p.q.sh;
    const float *dobase = (const float *)p.dout.ptr + sq.b * p.dout.sb + h * p.dout.sh;
    for (int e = e0; e < e1; ++e) {
      const int rbq = rows[e];
      const int qi0 = rbq * 64 - sq.past;  // query index of the block's first row
      if (rbq < 0 || qi0 >= sq.q_len || qi0 + 64 <= 0) continue;
      if (p.causal && cb * 64 > rbq * 64 + 63) continue;
      __syncthreads();
      load_tile<128>(qbase + (int64_t)qi0 * p.q.st, p.q.st, -qi0, sq.q_len - qi0, p.D, sQ, tid);
      load_tile<128>(dobase + (int64_t)qi0 * p.dout.st, p.dout.st, -qi0, sq.q_len - qi0, p.D, sDo, tid);
      if (tid < 64) {
        const int qi = qi0 + tid;
        const bool ok = qi >= 0 && qi < sq.q_len;
        const float lse = ok ? p.lse.ptr[sq.b * p.lse.sb + h * p.lse.sh + (int64_t)qi * p.lse.st] : 0.f;
        sLse[tid] = !ok || lse == -INFINITY ? INFINITY : lse * kLog2e;  // +inf: P = 0 for rows outside the sequence
        sDelta[tid] = ok ? p.delta[((int64_t)sq.b * p.Hq + h) * p.seqs.max_q_len + qi] : 0.f;
      }
      __syncthreads();
#pragma unroll
      for (int qt = 0; qt < 2; ++qt) {  // 32 q rows at a time
        const int pos0 = rbq * 64 + qt * 32;
        if (p.causal && cb * 64 + wave * 32 > pos0 + 31) continue;  // every key of this wave lies beyond these rows
        floatx16 s, dp;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
        s = dot_dims(sQ, qt * 32, kf, lane, s);     // rows = q (tile), columns = keys (registers)
        dp = dot_dims(sDo, qt * 32, vf, lane, dp);
        floatx16 ds;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int ql = qt * 32 + (r >> 2) * 8 + g * 4 + (r & 3);  // row of the block
          const bool vis = key_ok && (!p.causal || key <= rbq * 64 + ql);
          const float pr = vis ? fast_exp2(fmaf(s[r], p.scale_log2, -sLse[ql])) : 0.f;
          s[r] = pr;
          ds[r] = pr * (dp[r] - sDelta[ql]);
        }
        dot_rows(sDo, qt * 32, s, lane, dv);
        dot_rows(sQ, qt * 32, ds, lane, dk);
      }
    }
  }
  if (!key_ok) return;
  store_frag((float *)p.dk.ptr + sq.b * p.dk.sb + kvh * p.dk.sh + (int64_t)key * p.dk.st, dk, p.sm_scale, g, p.D);
  store_frag((float *)p.dv.ptr + sq.b * p.dv.sb + kvh * p.dv.sh + (int64_t)key * p.dv.st, dv, 1.f, g, p.D);
}

static bool lut_ok(const LutView &l) {
  return l.block_rows == 64 && l.block_cols == 64 && l.entry_width == 1 && l.sub_block == 0;
}

}  // namespace f32

bool mfma_f32_fwd_supported(const FwdParams &p, int dtype) {
  return dtype == DK_F32 && p.D >= 4 && p.D <= f32::kD && p.D % 4 == 0 && p.vec_ok && f32::lut_ok(p.csr);
}

bool mfma_f32_bwd_supported(const BwdParams &p, int dtype) {
  return dtype == DK_F32 && p.D >= 4 && p.D <= f32::kD && p.D % 4 == 0 && p.vec_ok && f32::lut_ok(p.csr) && f32::lut_ok(p.csc);
}

int launch_mfma_f32_fwd(const FwdParams &p, hipStream_t stream) {
  const SeqView &s = p.seqs;
  int tiles;
  if (s.packed)
    tiles = cdiv(s.max_q_len, 64) + 2 * s.batch;  // as for the 16-bit forward: an upper bound over all sequences
  else if (s.q_starts)
    tiles = cdiv(s.max_q_len, 64) + 1;
  else {
    const int past = p.causal ? s.max_k_len - s.max_q_len : 0;
    tiles = (past + s.max_q_len - 1) / 64 - past / 64 + 1;
  }
  if (p.csr.order && !s.packed) tiles = p.csr.num_rows;  // handed out in the table's order: all of them
  DK_REQUIRE(tiles <= 65535, "too many q tiles for one launch (%d)", tiles);
  FwdParams pr = p;
  pr.csr.rot = head_rotation(p.csr, p.Hq, tiles);  // (uneven heads: dealt to the queues in rotation)
  DK_NOTE_KERNEL(pr.csr.rot ? "f32::fwd_kernel, heads in rotation" : "f32::fwd_kernel");
  hipLaunchKernelGGL(f32::fwd_kernel, dim3(p.Hq, tiles, s.packed ? 1 : s.batch), dim3(128), 0, stream, pr, tiles);
  DK_HIP_CHECK(hipGetLastError());
  return DK_OK;
}

int launch_mfma_f32_bwd(const BwdParams &p, hipStream_t stream) {
  const SeqView &s = p.seqs;
  const int past = p.causal ? s.max_k_len - s.max_q_len : 0;
  const int tiles = (past + s.max_q_len - 1) / 64 - past / 64 + 1;
  const int cblocks = cdiv(s.max_k_len, 64);
  DK_REQUIRE(tiles <= 65535 && cblocks <= 65535, "sequence too long for one launch");
  DK_NOTE_KERNEL("f32::delta_kernel");
  hipLaunchKernelGGL(f32::delta_kernel, dim3(cdiv(s.max_q_len, 16), p.Hq, s.batch), dim3(256), 0, stream, p);
  DK_HIP_CHECK(hipGetLastError());
  DK_REQUIRE(!p.csr.order || p.csr.num_rows <= 65535, "sequence too long for one launch");
  const int rows = p.csr.order ? p.csr.num_rows : tiles;  // handed out in the table's order: all of them
  BwdParams pq = p;
  pq.csr.rot = head_rotation(p.csr, p.Hq, rows);
  DK_NOTE_KERNEL(pq.csr.rot ? "f32::dq_kernel, heads in rotation" : "f32::dq_kernel");
  hipLaunchKernelGGL(f32::dq_kernel, dim3(p.Hq, rows, s.batch), dim3(128), 0, stream, pq, rows);
  DK_HIP_CHECK(hipGetLastError());
  BwdParams po = p;  // the order only where heads do not line up with the hardware's 32 workgroup queues
  if (p.Hkv % 32 == 0) po.csc.order = nullptr;
  DK_REQUIRE(p.csc.num_rows <= 65535, "sequence too long for one launch");
  const int columns = po.csc.order ? p.csc.num_rows : cblocks;
  po.csc.rot = head_rotation(p.csc, p.Hkv, columns);
  DK_NOTE_KERNEL(po.csc.rot ? "f32::dkdv_kernel, heads in rotation" : "f32::dkdv_kernel");
  hipLaunchKernelGGL(f32::dkdv_kernel, dim3(p.Hkv, columns, s.batch), dim3(128), 0, stream, po);
  DK_HIP_CHECK(hipGetLastError());
  return DK_OK;
}

}  // namespace dk
