// C-ABI entry points for the device side: argument checks (the reference's
// Python asserts, done before any launch so that a bad shape can never reach a
// kernel), parameter-block construction and dispatch between the MFMA kernels
// (bf16 / fp16, head_dim 128 or 64, 64x64 blocks) and the generic kernels.
#include <hip/hip_runtime.h>

#include "common.h"
#include "device_common.h"

namespace dk {

int launch_generic_fwd(const FwdParams &p, int dtype, hipStream_t stream);
int launch_generic_bwd(const BwdParams &p, int dtype, hipStream_t stream);
bool mfma_fwd_supported(const FwdParams &p, int dtype);
int launch_mfma_fwd(const FwdParams &p, int dtype, void *workspace, size_t workspace_bytes, hipStream_t stream);
size_t mfma_fwd_workspace_bytes(const FwdParams &p);
bool mfma_bwd_supported(const BwdParams &p, int dtype);
int launch_mfma_bwd(const BwdParams &p, int dtype, void *workspace, size_t workspace_bytes, hipStream_t stream);
size_t mfma_bwd_workspace_bytes(const BwdParams &p);
bool mfma_f32_fwd_supported(const FwdParams &p, int dtype);
bool mfma_f32_bwd_supported(const BwdParams &p, int dtype);
int launch_mfma_f32_fwd(const FwdParams &p, hipStream_t stream);
int launch_mfma_f32_bwd(const BwdParams &p, hipStream_t stream);
bool decode_supported(const FwdParams &p, int dtype);
size_t decode_workspace_bytes(const FwdParams &p);
int launch_decode(const FwdParams &p, int dtype, void *workspace, size_t workspace_bytes, hipStream_t stream);

static size_t elem_size(int dtype) { return dtype == DK_F32 ? 4 : 2; }

static TensorView view(const dk_tensor &t) { return TensorView{t.ptr, t.stride_b, t.stride_h, t.stride_t}; }
static RowView view(const dk_rowvec &t) { return RowView{t.ptr, t.stride_b, t.stride_h, t.stride_t}; }
static LutView view(const dk_lut &l) {
  LutView v{l.ptr, l.idx, l.ptr_stride_h, l.idx_stride_h, l.entry_width, l.num_heads,
            l.num_rows, l.block_rows, l.block_cols, l.group < 1 ? 1 : l.group,
            l.max_row_entries, l.sub_block};
  v.order = l.row_order, v.pair_order = l.pair_order, v.order_sh = l.row_order_stride_h;
  v.uneven = l.uneven_heads != 0;
  return v;
}
static SeqView view(const dk_seqs &s) {
  SeqView v{s.batch, s.max_q_len, s.max_k_len, s.packed & 3, s.q_starts, s.q_ends, s.k_starts, s.k_ends};
  v.zero_outside = (s.packed & 4) && !(s.packed & 1) && s.q_starts ? 1 : 0;  // (without lengths every row holds a query)
  return v;
}

static bool vec_aligned(const dk_tensor &t, size_t es) {
  return ((uintptr_t)t.ptr % 16 == 0) && ((t.stride_b * es) % 16 == 0) && ((t.stride_h * es) % 16 == 0) &&
         ((t.stride_t * es) % 16 == 0);
}

static int check_lut(const dk_lut &l, const char *name, int Hq, int Hkv) {
  DK_REQUIRE(l.ptr && l.idx, "%s look-up table is NULL", name);
  DK_REQUIRE(l.num_heads == 1 || l.num_heads == Hkv || l.num_heads == Hq,
             "Input (q, k) have (%d, %d) heads but the number of heads in the sparse pattern is %d", Hq, Hkv,
             l.num_heads);
  DK_REQUIRE(is_pow2(l.block_rows) && is_pow2(l.block_cols) && l.block_rows >= 16 && l.block_cols >= 16 &&
                 l.block_rows <= 1024 && l.block_cols <= 1024,
             "%s tile sizes must be powers of 2 in [16, 1024], got (%d, %d)", name, l.block_rows, l.block_cols);
  DK_REQUIRE(l.entry_width == 1 || l.entry_width == 2, "%s entry_width must be 1 or 2", name);
  DK_REQUIRE(l.num_rows >= 0, "%s num_rows negative", name);
  DK_REQUIRE(l.sub_block == 0 || ((l.sub_block == 16 || l.sub_block == 32) && l.entry_width == 2 &&
                                  l.block_rows == 64 && l.block_cols == 64),
             "%s sub_block must be 0, or 16 / 32 with entry_width 2 and 64 x 64 tiles", name);
  return DK_OK;
}

static int check_common(const dk_seqs &s, int Hq, int Hkv, int D, int dtype, int causal) {
  DK_REQUIRE(Hq >= 1 && Hkv >= 1 && Hq % Hkv == 0, "num_q_heads (%d) must be a multiple of num_kv_heads (%d)", Hq,
             Hkv);
  DK_REQUIRE(D >= 1 && D <= 256, "head_dim %d not in [1, 256]", D);
  DK_REQUIRE(dtype == DK_BF16 || dtype == DK_F16 || dtype == DK_F32, "unknown dtype %d", dtype);
  DK_REQUIRE(s.batch >= 0 && s.max_q_len >= 0 && s.max_k_len >= 0, "negative sizes");
  DK_REQUIRE(Hq <= 65535 && s.batch <= 65535, "too many heads or sequences for one launch");
  const bool all = s.q_starts && s.q_ends && s.k_starts && s.k_ends;
  const bool none = !s.q_starts && !s.q_ends && !s.k_starts && !s.k_ends;
  DK_REQUIRE(all || none, "q/k starts/ends must be given together");
  DK_REQUIRE(!s.packed || all, "packed inputs need sequence offsets");
  if (none && causal)
    DK_REQUIRE(s.max_k_len >= s.max_q_len, "causal attention needs k length (%d) >= q length (%d)", s.max_k_len,
               s.max_q_len);
  return DK_OK;
}

static int make_fwd_params(const dk_fwd_args *a, FwdParams &p) {
  DK_REQUIRE(a != nullptr, "args is NULL");
  int rc = check_common(a->seqs, a->num_q_heads, a->num_kv_heads, a->head_dim, a->dtype, a->causal);
  if (rc) return rc;
  rc = check_lut(a->csr, "csr", a->num_q_heads, a->num_kv_heads);
  if (rc) return rc;
  DK_REQUIRE((int64_t)a->csr.num_rows * a->csr.block_rows >= a->seqs.max_k_len || a->seqs.packed,
             "Input length %d is larger than the maximum length allowed (%lld)", a->seqs.max_k_len,
             (long long)a->csr.num_rows * a->csr.block_rows);
  const bool empty = a->seqs.batch == 0 || a->seqs.max_q_len == 0;
  DK_REQUIRE(empty || (a->q.ptr && a->k.ptr && a->v.ptr && a->o.ptr) || a->seqs.max_k_len == 0, "q/k/v/o is NULL");
  p.q = view(a->q);
  p.k = view(a->k);
  p.v = view(a->v);
  p.o = view(a->o);
  p.lse = view(a->lse);
  p.csr = view(a->csr);
  p.seqs = view(a->seqs);
  p.Hq = a->num_q_heads;
  p.Hkv = a->num_kv_heads;
  p.D = a->head_dim;
  p.causal = a->causal ? 1 : 0;
  p.scale_log2 = a->sm_scale * kLog2e;
  const size_t es = elem_size(a->dtype);
  p.vec_ok = vec_aligned(a->q, es) && vec_aligned(a->k, es) && vec_aligned(a->v, es) && vec_aligned(a->o, es);
  p.paged = PagedView{nullptr, 0, 0, 0, 0};
  return DK_OK;
}

// Checks the backward arguments and fills the kernel parameter block.  `empty` is set when
// there is nothing to compute (no pointers are looked at then).
static int make_bwd_params(const dk_bwd_args *a, BwdParams &p, bool &empty) {
  empty = false;
  DK_REQUIRE(a != nullptr, "args is NULL");
  int rc = check_common(a->seqs, a->num_q_heads, a->num_kv_heads, a->head_dim, a->dtype, a->causal);
  if (rc) return rc;
  DK_REQUIRE(!a->seqs.q_starts && !a->seqs.packed,
             "Currently does not support paddings or variable length inputs in backward.");
  rc = check_lut(a->csr, "csr", a->num_q_heads, a->num_kv_heads);
  if (rc) return rc;
  rc = check_lut(a->csc, "csc", a->num_q_heads, a->num_kv_heads);
  if (rc) return rc;
  DK_REQUIRE(a->csc.entry_width == 1 || a->csc.sub_block != 0, "csc table cannot carry values other than sub-block masks");
  DK_REQUIRE((int64_t)a->csr.num_rows * a->csr.block_rows >= a->seqs.max_k_len,
             "Input length %d is larger than the maximum length allowed", a->seqs.max_k_len);
  if (a->seqs.batch == 0 || a->seqs.max_q_len == 0) {
    empty = true;
    return DK_OK;
  }
  DK_REQUIRE(a->q.ptr && a->k.ptr && a->v.ptr && a->o.ptr && a->dout.ptr && a->dq.ptr && a->dk.ptr && a->dv.ptr,
             "a tensor pointer is NULL");
  DK_REQUIRE(a->lse.ptr && a->delta, "lse / delta is NULL");
  p.q = view(a->q);
  p.k = view(a->k);
  p.v = view(a->v);
  p.o = view(a->o);
  p.dout = view(a->dout);
  p.dq = view(a->dq);
  p.dk = view(a->dk);
  p.dv = view(a->dv);
  p.lse = view(a->lse);
  p.dlse = view(a->dlse);
  p.delta = a->delta;
  p.csr = view(a->csr);
  p.csc = view(a->csc);
  p.seqs = view(a->seqs);
  p.Hq = a->num_q_heads;
  p.Hkv = a->num_kv_heads;
  p.D = a->head_dim;
  p.causal = a->causal ? 1 : 0;
  p.sm_scale = a->sm_scale;
  p.scale_log2 = a->sm_scale * kLog2e;
  const size_t es = elem_size(a->dtype);
  p.vec_ok = vec_aligned(a->q, es) && vec_aligned(a->k, es) && vec_aligned(a->v, es) && vec_aligned(a->o, es) &&
             vec_aligned(a->dout, es) && vec_aligned(a->dq, es) && vec_aligned(a->dk, es) && vec_aligned(a->dv, es);
  return DK_OK;
}

// ---------------------------------------------------------------------------
// Scratch of dk_fwd_noalloc: a file-scope device array, so that callers that may not allocate
// (HIP graph capture, serving loops) need no workspace of their own.  Every GPU the library runs
// on holds its own copy at its own address; the array's name is only a host-side handle, so the
// device address is looked up once per device and that pointer is what kernels receive.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[DK_NOALLOC_SCRATCH_BYTES];

static int static_scratch(hipStream_t stream, void **out) {
  constexpr int kMaxDevices = 64;
  static std::atomic<void *> per_device[kMaxDevices];  // zero-initialised
  int dev = 0;
  DK_HIP_CHECK(hipGetDevice(&dev));
  DK_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal %d beyond %d", dev, kMaxDevices);
  if (stream) {  // the array of the current device is the one the kernels of this stream can reach
    hipDevice_t sdev = 0;
    DK_HIP_CHECK(hipStreamGetDevice(stream, &sdev));
    DK_REQUIRE((int)sdev == dev, "the stream belongs to device %d but device %d is current", (int)sdev, dev);
  }
  void *ptr = per_device[dev].load(std::memory_order_acquire);
  if (!ptr) {  // first call on this device (a race between threads only repeats the lookup)
    DK_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    DK_REQUIRE(ptr != nullptr, "no device address for the static scratch");
    per_device[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return DK_OK;
}

}  // namespace dk

using namespace dk;

extern "C" {

int dk_fwd_noalloc(const dk_fwd_args *a) {
  clear_error();
  DK_REQUIRE(a != nullptr, "args is NULL");
  dk_fwd_args b = *a;
  b.workspace = nullptr;
  b.workspace_bytes = 0;
  // (argument errors are reported by dk_fwd below; the query returns 0 for them)
  const size_t need = dk_fwd_workspace_bytes(&b);
  DK_REQUIRE(need <= (size_t)DK_NOALLOC_SCRATCH_BYTES,
             "these arguments need %zu bytes of scratch, dk_fwd_noalloc holds %zu: use dk_fwd with a workspace", need,
             (size_t)DK_NOALLOC_SCRATCH_BYTES);
  if (need > 0) {
    void *ptr = nullptr;
    if (int rc = static_scratch((hipStream_t)a->stream, &ptr)) return rc;
    b.workspace = ptr;
    b.workspace_bytes = (size_t)DK_NOALLOC_SCRATCH_BYTES;
  }
  return dk_fwd(&b);
}

size_t dk_fwd_workspace_bytes(const dk_fwd_args *a) {
  FwdParams p;
  if (make_fwd_params(a, p) != DK_OK) return 0;
  if (a->impl != DK_IMPL_GENERIC && decode_supported(p, a->dtype)) return decode_workspace_bytes(p);
  if (a->impl != DK_IMPL_GENERIC && mfma_fwd_supported(p, a->dtype)) return mfma_fwd_workspace_bytes(p);
  return 0;
}

int dk_fwd(const dk_fwd_args *a) {
  clear_error();
  clear_kernels();
  FwdParams p;
  int rc = make_fwd_params(a, p);
  if (rc) return rc;
  if (p.seqs.batch == 0 || p.seqs.max_q_len == 0) return DK_OK;
  hipStream_t stream = (hipStream_t)a->stream;
  if (a->impl != DK_IMPL_GENERIC) {
    if (decode_supported(p, a->dtype) && a->workspace &&
        a->workspace_bytes >= decode_workspace_bytes(p))
      return launch_decode(p, a->dtype, a->workspace, a->workspace_bytes, stream);
    if (mfma_fwd_supported(p, a->dtype))
      return launch_mfma_fwd(p, a->dtype, a->workspace, a->workspace_bytes, stream);
    if (mfma_f32_fwd_supported(p, a->dtype)) return launch_mfma_f32_fwd(p, stream);
    if (a->impl == DK_IMPL_MFMA)
      return fail(DK_ERR_UNSUPPORTED, "no MFMA forward kernel for dtype %d, head_dim %d, tiles (%d, %d)", a->dtype,
                  p.D, p.csr.block_rows, p.csr.block_cols);
  }
  if (p.csr.sub_block)
    return fail(DK_ERR_UNSUPPORTED, "tables with sub-block masks need the matrix-core kernels (dtype %d, head_dim %d)",
                a->dtype, p.D);
  return launch_generic_fwd(p, a->dtype, stream);
}

size_t dk_bwd_workspace_bytes(const dk_bwd_args *a) {
  BwdParams p;
  bool empty;
  if (make_bwd_params(a, p, empty) != DK_OK || empty) return 0;
  if (a->impl != DK_IMPL_GENERIC && mfma_bwd_supported(p, a->dtype)) return mfma_bwd_workspace_bytes(p);
  return 0;
}

int dk_fwd_paged(const dk_fwd_args *a, const dk_paged_kv *pg) {
  clear_error();
  clear_kernels();
  DK_REQUIRE(pg != nullptr && pg->block_table != nullptr, "page table is NULL");
  DK_REQUIRE(pg->page_size >= 16 && is_pow2(pg->page_size), "page_size must be a power of two >= 16, got %d",
             pg->page_size);
  FwdParams p;
  int rc = make_fwd_params(a, p);
  if (rc) return rc;
  if (p.seqs.batch == 0 || p.seqs.max_q_len == 0) return DK_OK;
  DK_REQUIRE(!p.seqs.packed && p.seqs.q_starts, "paged decode takes per-sequence lengths (dk_seqs arrays)");
  DK_REQUIRE(pg->kv_dtype == DK_FP8_E4M3 || ((pg->page_stride_k * (int64_t)elem_size(a->dtype)) % 16 == 0 &&
                                              (pg->page_stride_v * (int64_t)elem_size(a->dtype)) % 16 == 0),
             "page strides must keep rows 16-byte aligned");
  int shift = 0;
  while ((1 << shift) < pg->page_size) ++shift;
  const bool fp8 = pg->kv_dtype == DK_FP8_E4M3;
  DK_REQUIRE(fp8 || pg->kv_dtype == a->dtype, "kv_dtype must be the q dtype or DK_FP8_E4M3, got %d", pg->kv_dtype);
  DK_REQUIRE(!fp8 || (pg->k_scale > 0.f && pg->v_scale > 0.f), "fp8 K/V scales must be positive");
  const int64_t kv_es = fp8 ? 1 : (int64_t)elem_size(a->dtype);
  DK_REQUIRE((pg->page_stride_k * kv_es) % 8 == 0 && (pg->page_stride_v * kv_es) % 8 == 0 &&
                 (!fp8 || (a->k.stride_h % 8 == 0 && a->k.stride_t % 8 == 0 && a->v.stride_h % 8 == 0 &&
                           a->v.stride_t % 8 == 0 && ((uintptr_t)a->k.ptr % 8) == 0 && ((uintptr_t)a->v.ptr % 8) == 0)),
             "fp8 K/V rows must be 8-byte aligned");
  p.paged = PagedView{pg->block_table, pg->table_stride_b, pg->page_stride_k, pg->page_stride_v, shift,
                      fp8 ? 1 : 0, fp8 ? pg->v_scale : 1.f};
  if (fp8) p.scale_log2 *= pg->k_scale;  // S = (q . k8) k_scale sm_scale
  if (a->impl == DK_IMPL_GENERIC || !decode_supported(p, a->dtype))
    return fail(DK_ERR_UNSUPPORTED,
                "paged K/V is served by the split-KV decode kernels only (one query token per sequence, 16-bit "
                "floats, head_dim a multiple of 8 up to 256, 64 x 64 tiles, causal)");
  DK_REQUIRE(a->workspace && a->workspace_bytes >= decode_workspace_bytes(p), "decode workspace too small");
  return launch_decode(p, a->dtype, a->workspace, a->workspace_bytes, (hipStream_t)a->stream);
}

int dk_bwd(const dk_bwd_args *a) {
  clear_error();
  clear_kernels();
  BwdParams p;
  bool empty;
  const int rc = make_bwd_params(a, p, empty);
  if (rc || empty) return rc;
  hipStream_t stream = (hipStream_t)a->stream;
  if (a->impl != DK_IMPL_GENERIC) {
    if (mfma_bwd_supported(p, a->dtype)) {
      return launch_mfma_bwd(p, a->dtype, a->workspace, a->workspace_bytes, stream);
    }
    if (mfma_f32_bwd_supported(p, a->dtype)) return launch_mfma_f32_bwd(p, stream);
    if (a->impl == DK_IMPL_MFMA)
      return fail(DK_ERR_UNSUPPORTED, "no MFMA backward kernel for dtype %d, head_dim %d, tiles (%d, %d)",
                  a->dtype, p.D, p.csr.block_rows, p.csr.block_cols);
  }
  if (p.csr.sub_block || p.csc.sub_block)
    return fail(DK_ERR_UNSUPPORTED, "tables with sub-block masks need the matrix-core kernels (dtype %d, head_dim %d)",
                a->dtype, p.D);
  return launch_generic_bwd(p, a->dtype, stream);
}

}  // extern "C"
