// Device-side helpers shared by the kernels: element types and conversions,
// the kernel parameter blocks, and the mapping from a workgroup to
// (sequence, row block) that needs no host synchronisation.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace dk {

struct bf16_t {
  uint16_t bits;
};
using f16_t = _Float16;

__device__ __forceinline__ float to_float(bf16_t x) { return __uint_as_float((uint32_t)x.bits << 16); }
__device__ __forceinline__ float to_float(f16_t x) { return (float)x; }
__device__ __forceinline__ float to_float(float x) { return x; }

template <typename T>
__device__ __forceinline__ T from_float(float x);
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float x) {
  uint32_t u = __float_as_uint(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return bf16_t{(uint16_t)((u >> 16) | 0x40)};  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);                                                   // round to nearest even
  return bf16_t{(uint16_t)(u >> 16)};
}
template <>
__device__ __forceinline__ f16_t from_float<f16_t>(float x) {
  return (f16_t)x;
}
template <>
__device__ __forceinline__ float from_float<float>(float x) {
  return x;
}

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct TensorView {
  void *ptr;
  int64_t sb, sh, st;
};
struct RowView {
  float *ptr;
  int64_t sb, sh, st;
};
struct LutView {
  const int32_t *ptr, *idx;
  int64_t ptr_sh, idx_sh;
  int32_t entry_width, num_heads, num_rows, block_rows, block_cols, group, max_row_entries, sub_block;
};
struct SeqView {
  int32_t batch, max_q_len, max_k_len, packed;
  const int32_t *q_starts, *q_ends, *k_starts, *k_ends;
};

// Paged K/V (decode only): k / v point at page pools, token t of sequence b lives in page
// table[b * table_sb + (t >> page_shift)] at in-page position t & (page_size - 1); inside a page
// tokens and heads use the tensors' own token / head strides.  table == nullptr: contiguous K/V.
struct PagedView {
  const int32_t *table;
  int64_t table_sb;
  int64_t k_page_stride, v_page_stride;  // elements
  int32_t page_shift;
  int32_t kv_fp8;    // pools hold OCP e4m3 bytes (k / v strides then count bytes); q / o keep their type
  float out_scale;   // V scale of an fp8 cache, applied to O (the K scale is folded into scale_log2)
};

struct FwdParams {
  TensorView q, k, v, o;
  RowView lse;
  LutView csr;
  SeqView seqs;
  PagedView paged;
  int32_t Hq, Hkv, D, causal;
  float scale_log2;  // sm_scale * log2(e)
  int32_t vec_ok;    // 16-byte vector loads / stores are legal for q, k, v, o
};

struct BwdParams {
  TensorView q, k, v, o, dout, dq, dk, dv;
  RowView lse, dlse;
  float *delta;      // (batch, Hq, max_q_len) contiguous
  LutView csr, csc;
  SeqView seqs;
  int32_t Hq, Hkv, D, causal;
  float sm_scale, scale_log2;
  int32_t vec_ok;
};

// Which LUT head serves q head h (h is the same for every lane of a wave).
__device__ __forceinline__ int lut_head(const LutView &l, int h, int Hq, int Hkv) {
  if (l.num_heads == 1) return 0;
  if (l.num_heads == Hq) return h;
  return __builtin_amdgcn_readfirstlane(h / (Hq / Hkv));  // integer division runs on the VALU
}

struct SeqInfo {
  int b;
  int q_start, q_len, k_start, k_len, past;
};

__device__ __forceinline__ SeqInfo load_seq(const SeqView &s, int b, int causal) {
  SeqInfo r;
  r.b = b;
  if (s.q_starts) {
    // ends beyond the token dimension are clamped, so a bad length can never
    // make a kernel read or write outside the tensors
    r.q_start = max(s.q_starts[b], 0);
    r.q_len = min(s.q_ends[b], s.max_q_len) - r.q_start;
    r.k_start = max(s.k_starts[b], 0);
    r.k_len = min(s.k_ends[b], s.max_k_len) - r.k_start;
  } else {
    r.q_start = r.k_start = 0;
    r.q_len = s.max_q_len;
    r.k_len = s.max_k_len;
  }
  if (r.q_len < 0) r.q_len = 0;
  if (r.k_len < 0) r.k_len = 0;
  r.past = causal ? r.k_len - r.q_len : 0;
  if (r.past < 0) r.past = 0;
  // b is the same for every lane of a wave, so the fields are too; saying so keeps the
  // addresses derived from them in scalar registers
  r.q_start = __builtin_amdgcn_readfirstlane(r.q_start);
  r.q_len = __builtin_amdgcn_readfirstlane(r.q_len);
  r.k_start = __builtin_amdgcn_readfirstlane(r.k_start);
  r.k_len = __builtin_amdgcn_readfirstlane(r.k_len);
  r.past = __builtin_amdgcn_readfirstlane(r.past);
  return r;
}

// Number of row blocks (of block_rows tokens, in absolute positions) that the
// queries of a sequence touch.
__device__ __forceinline__ int seq_row_blocks(const SeqInfo &s, int block_rows) {
  if (s.q_len <= 0) return 0;
  return (s.past + s.q_len - 1) / block_rows - s.past / block_rows + 1;
}

// Maps (blockIdx.x = tile index, blockIdx.z = batch) to a sequence and the
// index of the tile within it; tiles_per_block sub-tiles per row block.
// Returns false when the workgroup has nothing to do.  For packed inputs
// the sequences are scanned on the device (batch is small), so no tile map
// has to be built on the host.
__device__ __forceinline__ bool resolve_tile(const SeqView &s, int causal, int block_rows,
                                             int tiles_per_block, int tile_x, int bz, SeqInfo &info,
                                             int &tile_in_seq) {
  if (!s.packed) {
    info = load_seq(s, bz, causal);
    tile_in_seq = tile_x;
    return tile_x < seq_row_blocks(info, block_rows) * tiles_per_block;
  }
  int acc = 0;
  for (int b = 0; b < s.batch; ++b) {
    SeqInfo t = load_seq(s, b, causal);
    int n = seq_row_blocks(t, block_rows) * tiles_per_block;
    if (tile_x < acc + n) {
      info = t;
      tile_in_seq = tile_x - acc;
      return true;
    }
    acc += n;
  }
  return false;
}

}  // namespace dk
