/*
 * dkernel_hip.h -- C ABI of libdkernel_hip.so, the gfx950 (MI355X) block-sparse
 * attention engine.  Plain pointers, sizes and element strides only; the
 * library never allocates, frees or keeps caller memory, never synchronises
 * the device, and launches on the hipStream_t handed in.
 *
 * Every function returns 0 (DK_OK) or a negative code; dk_last_error() gives
 * the message of the calling thread's last failure.
 *
 * Each entry point names the interface of the reference (linxihui/dkernel)
 * that it replaces.
 */
#ifndef DKERNEL_HIP_H
#define DKERNEL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DK_OK 0
#define DK_ERR_INVALID (-1)     /* argument check failed (the reference's Python asserts) */
#define DK_ERR_UNSUPPORTED (-2) /* shape / dtype without a kernel */
#define DK_ERR_HIP (-3)         /* a HIP runtime call failed */

enum dk_dtype { DK_BF16 = 0, DK_F16 = 1, DK_F32 = 2,
                DK_FP8_E4M3 = 3 /* OCP e4m3 bytes; K/V pools of dk_fwd_paged only */ };
enum dk_impl { DK_IMPL_AUTO = 0, DK_IMPL_GENERIC = 1, DK_IMPL_MFMA = 2 };

int dk_version(void);              /* 10000*major + 100*minor + patch */
const char *dk_last_error(void);   /* thread-local, never NULL */
/* Kernels that the latest dk_fwd / dk_fwd_paged / dk_fwd_noalloc / dk_bwd call on this thread
 * launched, "name [template arguments]; " each, in launch order (thread-local, never NULL).  No
 * counterpart in the reference; tests and bench.py use it to tell which path a call took. */
const char *dk_last_kernels(void);

/* --------------------------------------------------------------------------
 * Host side: layout / look-up-table builder (runs on the CPU, no GPU needed)
 * -------------------------------------------------------------------------- */

/* Block mask of the local + vertical-stride pattern, out[num_heads][nb_q][nb_k]
 * (uint8, 1 = attend).  Replaces the mask arithmetic of get_sparse_attn_mask,
 * dkernel/utils.py:157-215.  num_heads is the number of pattern heads (1 for
 * homo_head); kv head of pattern head h is h / (num_heads / num_kv_heads);
 * the LAST num_dense_heads kv heads are dense.  relative != 0 selects the
 * 'relative' vertical positions of utils.py:197-211. */
int dk_local_stride_mask(int32_t num_heads, int32_t num_kv_heads, int32_t nb_q, int32_t nb_k,
                         int32_t local_left, int32_t local_right, int32_t vert_stride,
                         int32_t num_dense_heads, int32_t head_sliding_step,
                         int32_t head_sliding_offset, int32_t q_start_block,
                         int32_t kv_start_block, int32_t causal, int32_t relative, uint8_t *out);

/* CSR of an int32 pattern[H][M][N] given by element strides (pass the strides
 * of the transpose for CSC).  Pass 1 fills ptr[H][M+1] and *max_nnz; pass 2
 * fills idx[H][width] (right-padded with -1) and, if val != NULL,
 * val[H][width] (padded with 0).  Replaces to_csr / dense_to_crow_col /
 * dense_to_ccol_row, dkernel/utils.py:19-24, :27-65, :91-95. */
int dk_csr_count(const int32_t *pattern, int32_t H, int32_t M, int32_t N, int64_t stride_h,
                 int64_t stride_m, int64_t stride_n, int32_t *ptr, int32_t *max_nnz);
int dk_csr_fill(const int32_t *pattern, int32_t H, int32_t M, int32_t N, int64_t stride_h,
                int64_t stride_m, int64_t stride_n, int32_t width, int32_t *idx, int32_t *val);

/* Pattern at kernel-tile granularity (split to block_m x block_n sub-blocks,
 * sub-blocks wholly above the token diagonal dropped when prune_above_diagonal,
 * then groups of block_m / block_size row blocks merged with value
 * micro_M = (last non-empty sub-row + 1) * block_size).  Replaces the dense
 * stage of merge_split_fwd_kernel_blocks, dkernel/utils.py:286-307.
 * dk_tile_pattern_shape gives the output shape and whether values (merged
 * rows) are meaningful. */
int dk_tile_pattern_shape(int32_t M, int32_t N, int32_t block_size, int32_t block_m,
                          int32_t block_n, int32_t *out_m, int32_t *out_n, int32_t *merged);
int dk_tile_pattern(const uint8_t *pattern, int32_t H, int32_t M, int32_t N, int32_t block_size,
                    int32_t block_m, int32_t block_n, int32_t prune_above_diagonal,
                    int32_t *out /* [H][out_m][out_n] */);

/* 1 if the pattern is KV-cache friendly, 0 if not, <0 on error.  Replaces
 * is_kv_cache_efficient, dkernel/utils.py:232-245. */
int dk_kv_cache_efficient(const uint8_t *pattern, int32_t H, int32_t M, int32_t N,
                          int32_t block_m, int32_t block_n);

/* --------------------------------------------------------------------------
 * Device side
 * -------------------------------------------------------------------------- */

/* A (batch, head, token, dim) view: element strides for batch / head / token,
 * dim stride must be 1.  Packed variable-length tensors use stride_b = 0. */
typedef struct dk_tensor {
  void *ptr;
  int64_t stride_b, stride_h, stride_t;
} dk_tensor;

/* A per-row fp32 quantity (LSE, dLSE): element strides batch / head / token. */
typedef struct dk_rowvec {
  float *ptr;
  int64_t stride_b, stride_h, stride_t;
} dk_rowvec;

/* CSR (or CSC) look-up table in device memory.  ptr[h][r], ptr[h][r+1] bound
 * the entries of row block r; entry e is idx[h][e * entry_width] (and the
 * micro_M value at +1 when entry_width == 2).  num_heads is 1 (shared), the
 * number of kv heads, or the number of q heads.  Mirrors the tuples
 * (layout_crow, layout_col, block_m, block_n) of dkernel/interface.py:207-208. */
typedef struct dk_lut {
  const int32_t *ptr;
  const int32_t *idx;
  int64_t ptr_stride_h, idx_stride_h;
  int32_t entry_width;
  int32_t num_heads;
  int32_t num_rows;    /* row blocks (ptr has num_rows + 1 entries per head) */
  int32_t block_rows;  /* tokens per row block of this table */
  int32_t block_cols;  /* tokens per listed entry */
  int32_t group;       /* consecutive table heads known to hold identical rows (1 if unknown);
                          lets heads of a GQA group share K/V tiles inside a workgroup */
  int32_t max_row_entries; /* largest number of entries in one row (0 if unknown: the number of
                              row blocks is assumed); sizes the split-KV decode grid and
                              workspace.  A row that holds more entries than this is still
                              computed in full, inside the same grid and workspace: its work
                              units only get larger shares */
  int32_t sub_block;   /* 0, or 16 / 32 with entry_width 2 and 64 x 64 tiles: the pattern's own block
                          size.  The second int of an entry is then a bit mask over the tile's
                          f x f pattern blocks, f = 64 / sub_block: bit i * f + j set = rows
                          [i, i+1) * sub_block x columns [j, j+1) * sub_block are attended.  Taken
                          by the matrix-core kernels only. */
  const int32_t *row_order; /* optional (NULL: ascending): row_order[h * row_order_stride_h + i] is
                               the table row that the i-th work item of head h takes, a
                               permutation of 0 .. num_rows-1 with the longest rows first.  Read
                               by the dK/dV pass for its column table, and by the forward and dQ
                               kernels for their row table (see pair_order): workgroups are handed to
                               the shader engines round-robin and in order, so long columns that
                               recur with a period (vertical strides) otherwise pile up on a few
                               of them while the rest wait behind a full queue. */
  int64_t row_order_stride_h;
  int32_t uneven_heads; /* nonzero: the heads of the table hold clearly different numbers of entries
                           (dense heads beside sparse ones).  The matrix-core prefill and backward
                           kernels then deal the heads to the workgroup queues in rotation instead
                           of one head per queue, so that no part of the chip is left with the
                           dense heads alone; with even heads (0) a fixed head per queue shares more
                           tiles through the caches.  Results do not depend on it. */
  int32_t reserved;     /* 0 */
  const int32_t *pair_order; /* optional, with row_order on the row table of dk_fwd / dk_bwd (same head
                                stride): pair_order[h * row_order_stride_h + i] is the pair u of table
                                rows (2u, 2u + 1) that the i-th work item of head h takes in the kernels
                                that work on two rows at a time, a permutation of
                                0 .. (num_rows + 1) / 2 - 1 by descending length of the pair.  Without
                                the two orders the forward and dQ kernels start from the last row, which
                                is the longest of a causal pattern; a pattern whose long rows come
                                first (global rows of a non-causal pattern) would start them last,
                                with the rest of the chip idle while they finish.  Not read for packed
                                inputs. */
} dk_lut;

/* Sequence geometry.  With all four pointers NULL every sequence has
 * q_len = max_q_len and k_len = max_k_len starting at token 0.  Otherwise the
 * arrays (device memory, int32, `batch` entries) give the first token and the
 * end (exclusive) of each sequence's queries and keys inside the token
 * dimension; query tokens are the LAST q_len positions of the sequence when
 * causal (past_len = k_len - q_len), positions counted from the first real
 * token.  Mirrors q/k_batch_starts/ends of
 * dkernel/ops/sparse_attn_inference.py:431-434,503-507. */
typedef struct dk_seqs {
  int32_t batch;
  int32_t max_q_len; /* extent of the q token dimension (total tokens when packed) */
  int32_t max_k_len;
  int32_t packed;    /* bit 0: sequences share one token dimension (3-D inputs);
                        bit 1 (with bit 0): the caller guarantees exactly one query token per
                        sequence, which lets dk_fwd take the split-KV decode path;
                        bit 2 (without bit 0, with the arrays below): dk_fwd also writes the rows
                        of o (zeros) and lse (-inf) that hold no query of their sequence, so a
                        padded output need not be cleared first (the reference clears it with
                        torch.zeros, dkernel/ops/sparse_attn_inference.py:67) */
  const int32_t *q_starts, *q_ends, *k_starts, *k_ends;
} dk_seqs;

/* Forward: O = softmax(mask(Q K^T * sm_scale)) V over the K/V blocks listed in
 * the CSR table, token-causal when `causal`.  lse.ptr may be NULL.  Rows with
 * no visible key give O = 0, LSE = -inf.  Tokens outside [q_start, q_end) are
 * not written.  Replaces the launches of _sparse_fwd_kernel
 * (dkernel/ops/sparse_attn_fwd.py:519-546) and _fwd_kernel_batch_inference
 * (dkernel/ops/sparse_attn_inference.py:113-145, :245-285). */
typedef struct dk_fwd_args {
  dk_tensor q, k, v, o;
  dk_rowvec lse; /* natural log */
  dk_lut csr;
  dk_seqs seqs;
  int32_t num_q_heads, num_kv_heads, head_dim;
  int32_t dtype;  /* enum dk_dtype, of q/k/v/o */
  int32_t causal;
  int32_t impl;   /* enum dk_impl */
  float sm_scale;
  void *workspace;        /* optional device scratch (16-byte aligned): split-KV decode partials,
                             or the running tile counts of packed sequences; may be NULL */
  size_t workspace_bytes;
  void *stream;           /* hipStream_t */
} dk_fwd_args;

int dk_fwd(const dk_fwd_args *args);
/* Scratch that dk_fwd can use for these arguments (0 = none needed): single-token decode runs
 * the split-KV kernels only with it; packed prefill runs without it too, but then every
 * workgroup scans the sequence lengths to find its own, which costs with hundreds of sequences. */
size_t dk_fwd_workspace_bytes(const dk_fwd_args *args);

/* dk_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): the same kernels and results as dk_fwd, with
 * the scratch (split-KV decode partials, running tile counts of packed sequences) taken from a
 * device array that is part of the library image instead of args->workspace, which is ignored.
 * Calls no allocating routine.  Arguments that need more than DK_NOALLOC_SCRATCH_BYTES of
 * scratch are refused with DK_ERR_INVALID (dk_fwd_workspace_bytes tells how much a call needs).
 * Each GPU holds one such array for the life of the process and every call on that GPU uses it:
 * calls that overlap on one GPU (two streams, two threads) race on it -- serialise them or use
 * dk_fwd with separate workspaces.  The device that owns args->stream must be the current one.
 * Before a call is recorded into a HIP graph, make one ordinary call with the same kind of
 * arguments on that device: the first call looks up the array's address and raises the kernels'
 * LDS limits, which a capturing stream does not allow.  No counterpart in the reference, whose launchers allocate
 * with torch on every call (dkernel/ops/sparse_attn_inference.py:67,230). */
#define DK_NOALLOC_SCRATCH_BYTES (8u << 20)
int dk_fwd_noalloc(const dk_fwd_args *args);

/* Paged K/V cache for single-token decode (serving).  args->k / args->v point at
 * page pools: token t of sequence b lives in page block_table[b][t / page_size]
 * at in-page position t % page_size; a page starts page_stride_k / _v elements
 * after the previous one, tokens and heads inside a page use args->k / v
 * stride_t / stride_h (stride_b is ignored).  page_size is a power of two >= 16.
 * Table entries past a sequence's last token are never read; entries before it
 * must name pages of the pools (the library cannot check their upper bound; a
 * negative one is read as page 0).  args->seqs
 * gives the lengths as for padded decode (q one token per sequence, k_starts 0,
 * k_ends the context lengths, max_k_len the table's capacity in tokens) and
 * args->workspace must hold dk_fwd_workspace_bytes(args).  No counterpart in
 * the reference, which lists per-sequence cache sizes and FP8 as future work
 * (README.md:257-260). */
typedef struct dk_paged_kv {
  const int32_t *block_table; /* device, (batch, pages per sequence) */
  int64_t table_stride_b;
  int64_t page_stride_k, page_stride_v;
  int32_t page_size;
  int32_t kv_dtype;     /* args->dtype (pools hold q's type), or DK_FP8_E4M3: the pools hold bytes,
                           value = byte as e4m3 * k_scale / v_scale, and all K/V strides count
                           bytes; head_dim 64 or 128, pattern blocks >= 64 */
  float k_scale, v_scale; /* used with DK_FP8_E4M3 */
} dk_paged_kv;

int dk_fwd_paged(const dk_fwd_args *args, const dk_paged_kv *pages);

/* Backward of dk_fwd for equal-length, unpadded sequences (seqs pointers
 * NULL).  delta is caller scratch of batch * num_q_heads * max_q_len floats.
 * dlse.ptr may be NULL.  dk/dv are written for every kv head (sum over the q
 * heads of the group).  workspace is optional device scratch (16-byte
 * aligned, dk_bwd_workspace_bytes): with it and several q heads per kv head
 * the dK/dV pass runs one workgroup per q head and sums the groups afterwards,
 * which balances much better; without it the result is the same, only
 * slower.  Replaces _bwd_preprocess and _sparse_bwd_kernel launches,
 * dkernel/ops/sparse_attn_bwd.py:781-788, :811-850. */
typedef struct dk_bwd_args {
  dk_tensor q, k, v, o, dout, dq, dk, dv;
  dk_rowvec lse, dlse;
  float *delta;
  dk_lut csr, csc;
  dk_seqs seqs;
  int32_t num_q_heads, num_kv_heads, head_dim;
  int32_t dtype;
  int32_t causal;
  int32_t impl;
  float sm_scale;
  void *workspace;        /* optional device scratch, may be NULL */
  size_t workspace_bytes;
  void *stream;
} dk_bwd_args;

int dk_bwd(const dk_bwd_args *args);
/* Scratch that dk_bwd can use for these arguments (0 = none useful; never more than 4 GiB). */
size_t dk_bwd_workspace_bytes(const dk_bwd_args *args);

/* Merge of attention results computed over disjoint K/V partitions, per row:
 *     out = sum_p softmax_p(lse_p) * out_p
 * in fp32, rounded once to the outputs' type.  A partition in which a row saw no key
 * (lse = -inf) gets weight 0; a row that saw none in any partition gives 0.  Every tensor is
 * addressed as rows (i0, i1, i2) of head_dim contiguous elements through the three element
 * strides of its view (named b / h / t in dk_tensor and dk_rowvec), so outputs in (batch,
 * heads, tokens, dim), (batch, tokens, heads, dim) or packed (tokens, heads, dim) order and
 * log-sum-exps in (batch, heads, tokens) or (heads, tokens) order all fit; the caller lines
 * the dims up.  Replaces the torch expression of combine_attn_partitions,
 * dkernel/interface.py:303-324.
 *
 * dk_combine_bwd is its backward: given dout it writes dparts[p] = w_p * dout and (where
 * dlses[p].ptr is not NULL) dlses[p] = w_p * (<dout, out_p> - <dout, out>).  The reference gets
 * these from autograd through the same torch expression. */
#define DK_MAX_PARTITIONS 8
typedef struct dk_combine_args {
  int32_t num_partitions; /* 2 .. DK_MAX_PARTITIONS */
  int32_t dtype;          /* enum dk_dtype of out, dout, parts, dparts */
  int32_t n0, n1, n2;     /* row extents; i2 runs fastest over the launch */
  int32_t head_dim;
  dk_tensor out;                        /* dk_combine: result */
  dk_tensor dout;                       /* dk_combine_bwd: gradient of the result */
  dk_tensor parts[DK_MAX_PARTITIONS];   /* out_p */
  dk_rowvec lses[DK_MAX_PARTITIONS];    /* lse_p, natural log */
  dk_tensor dparts[DK_MAX_PARTITIONS];  /* dk_combine_bwd: gradients of out_p */
  dk_rowvec dlses[DK_MAX_PARTITIONS];   /* dk_combine_bwd: gradients of lse_p (ptr may be NULL) */
  void *stream;                         /* hipStream_t */
} dk_combine_args;

int dk_combine(const dk_combine_args *args);
int dk_combine_bwd(const dk_combine_args *args);

#ifdef __cplusplus
}
#endif
#endif /* DKERNEL_HIP_H */
