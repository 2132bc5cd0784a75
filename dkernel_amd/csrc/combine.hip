// Merge of attention results over disjoint K/V partitions and its backward (dk_combine,
// dk_combine_bwd).  Per (n0, n1, n2) row:
//     w_p  = softmax_p(lse_p)                 (a partition whose lse is -inf gets 0; all -inf: all 0)
//     out  = sum_p w_p * out_p                (fp32, rounded once to the outputs' type)
//     dout_p = w_p * dout,   dlse_p = w_p * (<dout, out_p> - <dout, out>)
// Both kernels stream every tensor once: bound by HBM bandwidth.
//
// Work split: a row of D elements is covered by L lanes (the power of two >= D / 8 chunks of
// 16 bytes, at most 64), a wave holds 64 / L rows; rows are numbered with dim 2 fastest, so a
// wave reads consecutive rows of a contiguous tensor as one run of bytes.  Rows whose D or
// strides do not allow 16-byte accesses take the same kernels with one element per chunk.
#include <hip/hip_runtime.h>

#include "common.h"
#include "device_common.h"

namespace dk {

struct CombineParams {
  int num_parts;
  int n1, n2, D;
  int64_t rows;                         // rows of one i0: n1 * n2
  TensorView out;                       // forward: the result; backward: unused
  TensorView dout;                      // backward only
  TensorView parts[DK_MAX_PARTITIONS];  // out_p
  RowView lses[DK_MAX_PARTITIONS];      // lse_p
  TensorView dparts[DK_MAX_PARTITIONS]; // backward: dout_p
  RowView dlses[DK_MAX_PARTITIONS];     // backward: dlse_p
};

template <typename T, int CH>
struct Chunk {  // CH elements of T as floats
  float v[CH];
  __device__ __forceinline__ void load(const T *p) {
    if constexpr (CH == 1) {
      v[0] = to_float(*p);
    } else {
      typedef uint32_t u32xN __attribute__((ext_vector_type(4)));
      const u32xN w = __builtin_nontemporal_load(reinterpret_cast<const u32xN *>(p));
      const T *e = reinterpret_cast<const T *>(&w);
#pragma unroll
      for (int i = 0; i < CH; ++i) v[i] = to_float(e[i]);
    }
  }
  __device__ __forceinline__ void store(T *p) const {
    if constexpr (CH == 1) {
      *p = from_float<T>(v[0]);
    } else {
      typedef uint32_t u32xN __attribute__((ext_vector_type(4)));
      u32xN w;
      T *e = reinterpret_cast<T *>(&w);
#pragma unroll
      for (int i = 0; i < CH; ++i) e[i] = from_float<T>(v[i]);
      __builtin_nontemporal_store(w, reinterpret_cast<u32xN *>(p));
    }
  }
};

// softmax weights of one row over the partitions; returns false when no partition saw a key
template <int P>
__device__ __forceinline__ bool row_weights(const CombineParams &p, int64_t i0, int i1, int i2, float (&w)[P]) {
  float mx = -INFINITY;
#pragma unroll
  for (int q = 0; q < P; ++q) {
    w[q] = p.lses[q].ptr[i0 * p.lses[q].sb + i1 * p.lses[q].sh + (int64_t)i2 * p.lses[q].st];
    mx = fmaxf(mx, w[q]);
  }
  if (!(mx > -INFINITY)) {  // nothing attended anywhere (or NaN input): weights 0, as the reference's NaN -> 0 rule
#pragma unroll
    for (int q = 0; q < P; ++q) w[q] = 0.f;
    return false;
  }
  float sum = 0.f;
#pragma unroll
  for (int q = 0; q < P; ++q) {
    w[q] = __expf(w[q] - mx);
    sum += w[q];
  }
  const float inv = sum == sum ? 1.f / sum : 0.f;  // a NaN among the inputs: weights 0, like the all -inf row
#pragma unroll
  for (int q = 0; q < P; ++q) w[q] = sum == sum ? w[q] * inv : 0.f;
  return true;
}

// P, the number of partitions, is a template argument: with a run-time count every partition's
// load sits behind its own branch and the loads of a row go out one after the other (4.2 against
// 5.9 TB/s with two partitions).  U rows per lane group (all their loads issued before the first
// result is formed) is kept at 1: two rows measured like one.
template <typename T, int CH, bool BWD, int P>
__global__ __launch_bounds__(256) void combine_kernel(const CombineParams p, int lanes_per_row) {
  constexpr int U = 1;
  const int lane = threadIdx.x & 63;
  const int L = lanes_per_row;  // power of two, <= 64
  const int rows_per_wave = 64 / L;
  const int64_t wave_id = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int l = lane & (L - 1);
  const int chunks = p.D / CH;
  bool active[U];
  int64_t i0[U];
  int i1[U], i2[U];
  float w[U][P];
  // rows are numbered inside one i0 (blockIdx.y): 32-bit index arithmetic, one division per lane
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t row = (uint32_t)((wave_id * U + u) * rows_per_wave + lane / L);
    active[u] = row < (uint32_t)p.rows;
    const uint32_t r = active[u] ? row : 0u;
    i1[u] = (int)(r / (uint32_t)p.n2);
    i2[u] = (int)(r - (uint32_t)i1[u] * (uint32_t)p.n2);
    i0[u] = blockIdx.y;
  }
#pragma unroll
  for (int u = 0; u < U; ++u) row_weights(p, i0[u], i1[u], i2[u], w[u]);
  auto part_ptr = [&](const TensorView &t, int u) {
    return (T *)t.ptr + i0[u] * t.sb + i1[u] * t.sh + (int64_t)i2[u] * t.st;
  };
  if constexpr (!BWD) {
    for (int c = l; c < chunks; c += L) {
      Chunk<T, CH> x[U][P];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int q = 0; q < P; ++q)
          if (active[u]) x[u][q].load(part_ptr(p.parts[q], u) + c * CH);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (!active[u]) continue;
        Chunk<T, CH> acc;
#pragma unroll
        for (int i = 0; i < CH; ++i) acc.v[i] = 0.f;
#pragma unroll
        for (int q = 0; q < P; ++q)
          {
#pragma unroll
            for (int i = 0; i < CH; ++i) acc.v[i] = fmaf(w[u][q], x[u][q].v[i], acc.v[i]);
          }
        acc.store(part_ptr(p.out, u) + c * CH);
      }
    }
  } else {
    // <dout, out_p> of the row: partial sums over this lane's chunks, then across the row's lanes
    float dot[U][P];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int q = 0; q < P; ++q) dot[u][q] = 0.f;
    for (int c = l; c < chunks; c += L) {
      Chunk<T, CH> d[U], x[U][P];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (!active[u]) continue;
        d[u].load(part_ptr(p.dout, u) + c * CH);
#pragma unroll
        for (int q = 0; q < P; ++q)
          x[u][q].load(part_ptr(p.parts[q], u) + c * CH);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (!active[u]) continue;
#pragma unroll
        for (int q = 0; q < P; ++q)
          {
            Chunk<T, CH> y;
#pragma unroll
            for (int i = 0; i < CH; ++i) {
              dot[u][q] = fmaf(d[u].v[i], x[u][q].v[i], dot[u][q]);
              y.v[i] = w[u][q] * d[u].v[i];
            }
            y.store(part_ptr(p.dparts[q], u) + c * CH);
          }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float dot_out = 0.f;
#pragma unroll
      for (int q = 0; q < P; ++q) {
        for (int off = 1; off < L; off <<= 1) dot[u][q] += __shfl_xor(dot[u][q], off);
        dot_out = fmaf(w[u][q], dot[u][q], dot_out);
      }
      if (active[u] && l == 0) {
#pragma unroll
        for (int q = 0; q < P; ++q)
          if (p.dlses[q].ptr)
            p.dlses[q].ptr[i0[u] * p.dlses[q].sb + i1[u] * p.dlses[q].sh + (int64_t)i2[u] * p.dlses[q].st] =
                w[u][q] * (dot[u][q] - dot_out);
      }
    }
  }
}

static TensorView view_of(const dk_tensor &t) {
  TensorView v;
  v.ptr = t.ptr, v.sb = t.stride_b, v.sh = t.stride_h, v.st = t.stride_t;
  return v;
}
static RowView row_of(const dk_rowvec &t) {
  RowView v;
  v.ptr = t.ptr, v.sb = t.stride_b, v.sh = t.stride_h, v.st = t.stride_t;
  return v;
}

static bool chunk_ok(const dk_tensor &t, int elem) {  // 16-byte accesses at every row start
  const int per = 16 / elem;
  return ((uintptr_t)t.ptr % 16) == 0 && t.stride_b % per == 0 && t.stride_h % per == 0 && t.stride_t % per == 0;
}

template <typename T, bool BWD>
static int launch_combine_t(const CombineParams &p, int n0, bool vec, hipStream_t stream) {
  constexpr int CH = 16 / (int)sizeof(T);
  const int chunks = vec ? p.D / CH : p.D;
  int L = 1;
  while (L < chunks && L < 64) L <<= 1;
  const int64_t rows_per_wg = 4 * (64 / L);
  const int64_t wgs = cdiv64(p.rows, rows_per_wg);
  DK_REQUIRE(wgs <= 0x7fffffff, "too many rows for one launch");
  DK_NOTE_KERNEL(BWD ? "combine_bwd_kernel" : "combine_kernel");
  const dim3 grid((unsigned)wgs, n0);
#define DK_COMBINE_CASE(P)                                                                                   \
  case P:                                                                                                    \
    if (vec)                                                                                                 \
      hipLaunchKernelGGL((combine_kernel<T, CH, BWD, P>), grid, dim3(256), 0, stream, p, L);                 \
    else                                                                                                     \
      hipLaunchKernelGGL((combine_kernel<T, 1, BWD, P>), grid, dim3(256), 0, stream, p, L);                  \
    break;
  switch (p.num_parts) {
    DK_COMBINE_CASE(2)
    DK_COMBINE_CASE(3)
    DK_COMBINE_CASE(4)
    DK_COMBINE_CASE(5)
    DK_COMBINE_CASE(6)
    DK_COMBINE_CASE(7)
    DK_COMBINE_CASE(8)
  }
#undef DK_COMBINE_CASE
  DK_HIP_CHECK(hipGetLastError());
  return DK_OK;
}

static int run_combine(const dk_combine_args *a, bool bwd) {
  clear_error();
  clear_kernels();
  DK_REQUIRE(a != nullptr, "args is NULL");
  DK_REQUIRE(a->num_partitions >= 2 && a->num_partitions <= DK_MAX_PARTITIONS, "2 to %d partitions, got %d",
             DK_MAX_PARTITIONS, a->num_partitions);
  DK_REQUIRE(a->n0 >= 0 && a->n1 >= 0 && a->n2 >= 0 && a->head_dim > 0, "negative extent");
  DK_REQUIRE(a->dtype == DK_BF16 || a->dtype == DK_F16 || a->dtype == DK_F32, "unknown dtype %d", a->dtype);
  CombineParams p{};
  p.num_parts = a->num_partitions;
  p.n1 = a->n1, p.n2 = a->n2, p.D = a->head_dim;
  p.rows = (int64_t)a->n1 * a->n2;
  if (p.rows == 0 || a->n0 == 0) return DK_OK;
  DK_REQUIRE(p.rows < (1ll << 31) && a->n0 <= 65535, "extents beyond one launch: n0 %d, n1 * n2 %lld", a->n0, (long long)p.rows);
  const int n0 = a->n0;
  const int elem = a->dtype == DK_F32 ? 4 : 2;
  bool vec = p.D % (16 / elem) == 0;
  for (int q = 0; q < p.num_parts; ++q) {
    DK_REQUIRE(a->parts[q].ptr && a->lses[q].ptr, "partition %d: NULL pointer", q);
    p.parts[q] = view_of(a->parts[q]);
    p.lses[q] = row_of(a->lses[q]);
    vec = vec && chunk_ok(a->parts[q], elem);
    if (bwd) {
      DK_REQUIRE(a->dparts[q].ptr, "partition %d: NULL gradient pointer", q);
      p.dparts[q] = view_of(a->dparts[q]);
      p.dlses[q] = row_of(a->dlses[q]);  // ptr may be NULL: that gradient is not wanted
      vec = vec && chunk_ok(a->dparts[q], elem);
    }
  }
  if (bwd) {
    DK_REQUIRE(a->dout.ptr, "dout is NULL");
    p.dout = view_of(a->dout);
    vec = vec && chunk_ok(a->dout, elem);
  } else {
    DK_REQUIRE(a->out.ptr, "out is NULL");
    p.out = view_of(a->out);
    vec = vec && chunk_ok(a->out, elem);
  }
  hipStream_t stream = (hipStream_t)a->stream;
  switch (a->dtype) {
    case DK_BF16: return bwd ? launch_combine_t<bf16_t, true>(p, n0, vec, stream) : launch_combine_t<bf16_t, false>(p, n0, vec, stream);
    case DK_F16: return bwd ? launch_combine_t<f16_t, true>(p, n0, vec, stream) : launch_combine_t<f16_t, false>(p, n0, vec, stream);
    default: return bwd ? launch_combine_t<float, true>(p, n0, vec, stream) : launch_combine_t<float, false>(p, n0, vec, stream);
  }
}

}  // namespace dk

extern "C" {
int dk_combine(const dk_combine_args *a) { return dk::run_combine(a, false); }
int dk_combine_bwd(const dk_combine_args *a) { return dk::run_combine(a, true); }
}
