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
  const int32_t *order = nullptr;  // optional: work item i of head h takes table row order[h * order_sh + i]
  const int32_t *pair_order = nullptr;  // optional: ... or the rows 2u, 2u + 1 with u = pair_order[h * order_sh + i]
  int64_t order_sh = 0;
  int32_t uneven = 0;  // the heads hold clearly different numbers of entries
  int32_t rot = 0;     // set per launch (head_rotation): 0, or 1 + shift of grid_head()
};

// Workgroups reach the chip's 32 queues (8 dies x 4 shader engines) by their linear id, in order.
// With x = head and a head count that is a multiple of 8, 16 or 32 every head stays on the same
// few queues, and heads of unequal density (dense heads beside sparse ones) leave most of the
// chip waiting for the busiest queue.  For such tables the head of a workgroup moves on by one
// with every step in y (every second step once that still takes each head around the queues
// eight times), so that every queue serves every head in quick succession.  Coarser steps keep
// more neighbours in y on one die, where they share their K/V (or Q/dO) tiles through its L2,
// but hand a queue many long workgroups in a row, and the in-order hand-out then stalls behind
// it: with 32 heads, steps of 4 and 8 measured up to 1.6 x slower, also when every other round
// ran backwards to even out the growth of the rows along y.  Tables with even heads keep
// x = head, which shares most (the rotation costs them 8 - 13 %).
inline int head_rotation(const LutView &l, int gx, int gy) {
  if (!l.uneven || gx < 2) return 0;
  return 1 + ((gy >> 3) >= gx ? 1 : 0);
}
// Head (or head group) of this workgroup in a grid of (heads, work items, batch).  For every y the
// map x -> head is a permutation, so each (head, item) pair is still taken exactly once.
__device__ __forceinline__ int grid_head(const LutView &l) {
  unsigned x = blockIdx.x;
  if (l.rot) x = (x + (blockIdx.y >> (l.rot - 1))) % gridDim.x;
  return __builtin_amdgcn_readfirstlane((int)x);
}

struct SeqView {
  int32_t batch, max_q_len, max_k_len, packed;
  const int32_t *q_starts, *q_ends, *k_starts, *k_ends;
  // packed inputs, optional: batch + 1 ints, entry b = work items (q tiles or pairs of q tiles) of
  // the sequences before b, written by a small kernel ahead of the one that reads it
  int32_t *item_offsets = nullptr;
  // padded inputs: the forward kernels also write the rows of o (zeros) and lse (-inf) that hold
  // no query of their sequence, so that the caller need not clear the outputs first
  int32_t zero_outside = 0;
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

// Geometry of sequence b as this lane sees it (b may differ between lanes).
__device__ __forceinline__ SeqInfo load_seq_lane(const SeqView &s, int b, int causal) {
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
  return r;
}

// The same for a b that every lane of the wave shares.
__device__ __forceinline__ SeqInfo load_seq(const SeqView &s, int b, int causal) {
  SeqInfo r = load_seq_lane(s, b, causal);
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

// Pairs of adjacent table rows (2u, 2u + 1) that hold queries of a sequence.
__device__ __forceinline__ int seq_row_pairs(const SeqInfo &s) {
  if (s.q_len <= 0) return 0;
  const int first = s.past / 64, last = (s.past + s.q_len - 1) / 64;
  return (last >> 1) - (first >> 1) + 1;
}

// Packed inputs: the sequences share one token dimension and work items (q tiles, pairs of q
// tiles) are numbered through all of them, count(sequence) items each.  Finds the sequence that
// holds `item` and the item's index inside it; returns -1 beyond the last item.  The search runs
// on the device (no host copy of the lengths), a wave at a time with every lane active and the
// same `item`: each lane adds up the counts of batch / 64 consecutive sequences, a prefix sum over
// the lanes names the lane whose chunk holds the item, and its sequences are searched the same
// way, 64 at a time -- a few dependent loads whatever the batch size.
template <typename Count>
__device__ __forceinline__ int find_packed_sequence(const SeqView &s, int causal, int item, Count count,
                                                    int &index_in_seq) {
  if (s.item_offsets) {
    // the running item counts are there: bisect (wave-uniform addresses; zero-item sequences
    // share their successor's offset and are never the answer)
    const int32_t *off = s.item_offsets;
    if (item >= __builtin_amdgcn_readfirstlane(off[s.batch])) return -1;
    int lo = 0, hi = s.batch;  // off[lo] <= item < off[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (__builtin_amdgcn_readfirstlane(off[mid]) <= item)
        lo = mid;
      else
        hi = mid;
    }
    index_in_seq = item - __builtin_amdgcn_readfirstlane(off[lo]);
    return lo;
  }
  const int lane = threadIdx.x & 63;
  const int per_lane = (s.batch + 63) / 64;
  int mine = 0;
  // (indices clamped instead of branched around, eight at a time: the loads of a group are
  // independent and leave together)
  for (int i0 = 0; i0 < per_lane; i0 += 8) {
    int n[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int b = lane * per_lane + i0 + i;
      const bool real = i0 + i < per_lane && b < s.batch;
      n[i] = count(load_seq_lane(s, real ? b : 0, causal));
      if (!real) n[i] = 0;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) mine += n[i];
  }
  auto prefix = [&](int v) {  // inclusive sum over the lanes
    for (int off = 1; off < 64; off <<= 1) {
      const int t = __shfl_up(v, off);
      if (lane >= off) v += t;
    }
    return v;
  };
  const int upto = prefix(mine);
  const unsigned long long holders = __ballot(item < upto);
  if (holders == 0) return -1;
  const int owner = __ffsll(holders) - 1;                     // first lane whose chunk reaches past the item
  int before = __shfl(upto - mine, owner);                    // items of the chunks before it
  if (per_lane == 1) {
    index_in_seq = __builtin_amdgcn_readfirstlane(item - before);
    return __builtin_amdgcn_readfirstlane(owner);
  }
  for (int j0 = 0; j0 < per_lane; j0 += 64) {
    const int j = j0 + lane, b = owner * per_lane + j;
    const int n = (j < per_lane && b < s.batch) ? count(load_seq_lane(s, b, causal)) : 0;
    const int upto2 = prefix(n);
    const unsigned long long hit = __ballot(item < before + upto2);
    if (hit != 0) {
      const int l2 = __ffsll(hit) - 1;
      index_in_seq = __builtin_amdgcn_readfirstlane(item - before - __shfl(upto2 - n, l2));
      return __builtin_amdgcn_readfirstlane(owner * per_lane + j0 + l2);
    }
    before += __shfl(upto2, 63);
  }
  return -1;  // not reached: the owner's chunk holds the item
}

// Fills SeqView::item_offsets: one workgroup of 1024 threads; count(sequence) as in
// find_packed_sequence.  Thread t adds up batch / 1024 consecutive sequences, the partial sums
// are scanned in LDS, and each thread writes the running counts of its sequences.
template <typename Count>
__device__ __forceinline__ void write_item_offsets(const SeqView &s, int causal, Count count, int32_t *out) {
  __shared__ int part[1024];
  const int t = threadIdx.x;
  const int per = (s.batch + 1023) / 1024;
  int sum = 0;
  for (int i = 0; i < per; ++i) {
    const int b = t * per + i;
    if (b < s.batch) sum += count(load_seq_lane(s, b, causal));
  }
  part[t] = sum;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {
    const int v = t >= off ? part[t - off] : 0;
    __syncthreads();
    part[t] += v;
    __syncthreads();
  }
  int run = part[t] - sum;
  for (int i = 0; i < per; ++i) {
    const int b = t * per + i;
    if (b < s.batch) {
      out[b] = run;
      run += count(load_seq_lane(s, b, causal));
    }
  }
  if (t == 1023) out[s.batch] = part[1023];
}

// Padded inputs with SeqView::zero_outside: work item `item` of the `items` that a launch has along
// the q tiles of one batch entry clears its share of the token rows that hold no query of the
// sequence (positions outside [q_start, q_start + q_len) of the token dimension), for heads
// [h0, h0 + nh): o = 0, lse = -inf.  Every item takes part, those without queries too, so the
// rows are covered whatever the sequence's length.  `vec`: 16-byte stores are legal.
template <typename T>
__device__ __forceinline__ void zero_rows_outside(const SeqView &s, const SeqInfo &sq, int item, int items,
                                                  const TensorView &o, const RowView &lse, int h0, int nh, int D,
                                                  bool vec, int tid, int nthreads) {
  const int q_len = sq.q_len > 0 ? sq.q_len : 0;
  const int outside = s.max_q_len - q_len;
  if (outside <= 0) return;
  const int share = (outside + items - 1) / items;
  const int lo = item * share, hi = min(outside, lo + share);
  if (lo >= hi) return;
  auto token = [&](int i) { return i < sq.q_start ? i : i + q_len; };  // i-th row outside the queries
  // A thread keeps one (head, piece of the row) and walks the rows: the index arithmetic is done
  // once per thread, not once per store.
  const bool vec16 = vec && (D * (int)sizeof(T)) % 16 == 0;
  const int pieces = vec16 ? D * (int)sizeof(T) / 16 : D;  // 16-byte chunks, or elements, per head row
  const int per_row = nh * pieces;
  const int groups = nthreads >= per_row ? nthreads / per_row : 1;  // token rows cleared side by side
  T *ob = (T *)o.ptr + sq.b * o.sb;
  for (int j = tid; j < per_row * groups; j += nthreads) {
    const int grp = j / per_row, col = j - grp * per_row;
    const int hh = col / pieces, c = col - hh * pieces;
    T *dst = ob + (h0 + hh) * o.sh + (vec16 ? c * (16 / (int)sizeof(T)) : c);
    for (int i = lo + grp; i < hi; i += groups) {
      if (vec16)
        *reinterpret_cast<uint4 *>(dst + (int64_t)token(i) * o.st) = make_uint4(0, 0, 0, 0);
      else
        dst[(int64_t)token(i) * o.st] = from_float<T>(0.f);
    }
  }
  if (lse.ptr) {
    for (int idx = tid; idx < (hi - lo) * nh; idx += nthreads) {
      const int hh = idx % nh, i = lo + idx / nh;
      lse.ptr[sq.b * lse.sb + (h0 + hh) * lse.sh + (int64_t)token(i) * lse.st] = -INFINITY;
    }
  }
}

// Maps (tile_x = tile index, bz = batch index) to a sequence and the index of the tile within
// it; tiles_per_block sub-tiles per row block.  Returns false when the workgroup has nothing to
// do.  Packed inputs: tile_x counts through all sequences (every lane of the wave must call).
__device__ __forceinline__ bool resolve_tile(const SeqView &s, int causal, int block_rows,
                                             int tiles_per_block, int tile_x, int bz, SeqInfo &info,
                                             int &tile_in_seq) {
  if (!s.packed) {
    info = load_seq(s, bz, causal);
    tile_in_seq = tile_x;
    return tile_x < seq_row_blocks(info, block_rows) * tiles_per_block;
  }
  const int b = find_packed_sequence(
      s, causal, tile_x, [&](const SeqInfo &t) { return seq_row_blocks(t, block_rows) * tiles_per_block; },
      tile_in_seq);
  if (b < 0) return false;
  info = load_seq(s, b, causal);
  return true;
}

}  // namespace dk
