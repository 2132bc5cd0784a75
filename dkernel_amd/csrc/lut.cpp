// Host-side layout builder: block mask of the local + vertical-stride pattern,
// CSR / CSC look-up tables with -1 padding, kernel-tile merge / split, and the
// KV-cache-efficiency check.  Integer work on the CPU, one pass per table; it
// replaces the per-head Python loops of dkernel/utils.py.
#include <cstring>
#include <vector>

#include "common.h"

namespace dk {

static thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}
void clear_error() { g_err[0] = 0; }

static thread_local char g_kernels[1024] = "";

void clear_kernels() { g_kernels[0] = 0; }
void note_kernel(const char *kernel, const char *launcher_signature) {
  // "... launcher(args) [T = dk::bf16_t, D = 128, ...]" -> "kernel [T = dk::bf16_t, D = 128, ...]; "
  const char *args = launcher_signature ? strrchr(launcher_signature, '[') : nullptr;
  const size_t used = strlen(g_kernels);
  snprintf(g_kernels + used, sizeof(g_kernels) - used, "%s%s%s; ", kernel, args ? " " : "", args ? args : "");
}

}  // namespace dk

using dk::fail;

extern "C" {

int dk_version(void) { return 500; /* 0.5.0 */ }
const char *dk_last_error(void) { return dk::g_err; }
const char *dk_last_kernels(void) { return dk::g_kernels; }

// dkernel/utils.py:157-215.  Head h of the pattern belongs to kv head
// h / (num_heads / num_kv_heads); kv heads >= num_kv_heads - num_dense_heads
// are dense.  Absolute positions: a column is vertical when
// (kv_start_block + j + kvh * step + offset) % vert_stride == 0; relative
// positions: when (distance beyond the local window) % vert_stride == 0.
int dk_local_stride_mask(int32_t num_heads, int32_t num_kv_heads, int32_t nb_q, int32_t nb_k,
                         int32_t local_left, int32_t local_right, int32_t vert_stride,
                         int32_t num_dense_heads, int32_t head_sliding_step,
                         int32_t head_sliding_offset, int32_t q_start_block,
                         int32_t kv_start_block, int32_t causal, int32_t relative, uint8_t *out) {
  dk::clear_error();
  DK_REQUIRE(out != nullptr, "out is NULL");
  DK_REQUIRE(num_heads >= 1 && num_kv_heads >= 1 && num_heads % num_kv_heads == 0,
             "num_heads (%d) must be a positive multiple of num_kv_heads (%d)", num_heads, num_kv_heads);
  DK_REQUIRE(nb_q >= 0 && nb_k >= 0, "negative block counts");
  DK_REQUIRE(vert_stride >= 1, "vert_stride must be >= 1, got %d", vert_stride);
  DK_REQUIRE(num_dense_heads >= 0 && num_dense_heads <= num_kv_heads, "num_dense_heads out of range");
  const int q_per_kv = num_heads / num_kv_heads;
  const int num_sparse = num_kv_heads - num_dense_heads;
  for (int h = 0; h < num_heads; ++h) {
    const int kvh = h / q_per_kv;
    const bool dense = kvh >= num_sparse;
    uint8_t *o = out + (size_t)h * nb_q * nb_k;
    for (int i = 0; i < nb_q; ++i) {
      const int64_t q = (int64_t)q_start_block + i;
      for (int j = 0; j < nb_k; ++j) {
        const int64_t k = (int64_t)kv_start_block + j;
        bool on;
        if (!relative) {
          const bool local = (q - k < local_left) && (k - q < local_right);
          const bool vert =
              dense || ((k + (int64_t)kvh * head_sliding_step + head_sliding_offset) % vert_stride == 0);
          on = local || vert;
        } else {
          int64_t l = (q - k) - local_left + 1;
          if (l < 0) l = 0;
          int64_t r = (k - q) - local_right + 1;
          if (r < 0) r = 0;
          on = dense || ((l + r) % vert_stride == 0);
        }
        if (causal && q < k) on = false;
        o[(size_t)i * nb_k + j] = on ? 1 : 0;
      }
    }
  }
  return DK_OK;
}

int dk_csr_count(const int32_t *pattern, int32_t H, int32_t M, int32_t N, int64_t sh, int64_t sm,
                 int64_t sn, int32_t *ptr, int32_t *max_nnz) {
  dk::clear_error();
  DK_REQUIRE(pattern && ptr && max_nnz, "NULL argument");
  DK_REQUIRE(H >= 1 && M >= 0 && N >= 0, "bad shape (%d, %d, %d)", H, M, N);
  int32_t mx = 0;
  // The transpose of a row-major matrix (CSC) is walked in memory order, columns of the output
  // outermost: along its rows every step would touch another cache line (2.5 s for 8 heads of
  // 2048 x 2048 blocks against 0.2 s).
  const bool by_memory = sm < sn;
  for (int h = 0; h < H; ++h) {
    int32_t *p = ptr + (size_t)h * (M + 1);
    p[0] = 0;
    if (by_memory) {
      for (int i = 0; i < M; ++i) p[i + 1] = 0;
      for (int j = 0; j < N; ++j) {
        const int32_t *col = pattern + h * sh + j * sn;
        for (int i = 0; i < M; ++i) p[i + 1] += col[i * sm] != 0;
      }
      for (int i = 0; i < M; ++i) p[i + 1] += p[i];
    } else {
      for (int i = 0; i < M; ++i) {
        const int32_t *row = pattern + h * sh + i * sm;
        int32_t c = 0;
        for (int j = 0; j < N; ++j) c += row[j * sn] != 0;
        p[i + 1] = p[i] + c;
      }
    }
    if (p[M] > mx) mx = p[M];
  }
  *max_nnz = mx;
  return DK_OK;
}

int dk_csr_fill(const int32_t *pattern, int32_t H, int32_t M, int32_t N, int64_t sh, int64_t sm,
                int64_t sn, int32_t width, int32_t *idx, int32_t *val) {
  dk::clear_error();
  DK_REQUIRE(pattern && (idx || width == 0), "NULL argument");
  DK_REQUIRE(H >= 1 && M >= 0 && N >= 0 && width >= 0, "bad shape");
  const bool by_memory = sm < sn;  // as in dk_csr_count
  std::vector<int32_t> cursor;
  for (int h = 0; h < H; ++h) {
    int32_t *o = idx + (size_t)h * width;
    int32_t *ov = val ? val + (size_t)h * width : nullptr;
    int32_t e = 0;
    if (by_memory) {
      // first entry of every output row, then one sweep in memory order: column indices reach
      // each row's list in ascending order
      cursor.assign((size_t)M + 1, 0);
      for (int j = 0; j < N; ++j) {
        const int32_t *col = pattern + h * sh + j * sn;
        for (int i = 0; i < M; ++i) cursor[i + 1] += col[i * sm] != 0;
      }
      for (int i = 0; i < M; ++i) cursor[i + 1] += cursor[i];
      e = cursor[M];
      if (e > width) return fail(DK_ERR_INVALID, "width %d too small for head %d", width, h);
      for (int j = 0; j < N; ++j) {
        const int32_t *col = pattern + h * sh + j * sn;
        for (int i = 0; i < M; ++i) {
          const int32_t x = col[i * sm];
          if (x != 0) {
            const int32_t at = cursor[i]++;
            o[at] = j;
            if (ov) ov[at] = x;
          }
        }
      }
    } else {
      for (int i = 0; i < M; ++i) {
        const int32_t *row = pattern + h * sh + i * sm;
        for (int j = 0; j < N; ++j) {
          const int32_t x = row[j * sn];
          if (x != 0) {
            if (e >= width) return fail(DK_ERR_INVALID, "width %d too small for head %d", width, h);
            o[e] = j;
            if (ov) ov[e] = x;
            ++e;
          }
        }
      }
    }
    for (; e < width; ++e) {
      o[e] = -1;
      if (ov) ov[e] = 0;
    }
  }
  return DK_OK;
}

// dkernel/utils.py:280-307 without the final CSR conversion.
int dk_tile_pattern_shape(int32_t M, int32_t N, int32_t block_size, int32_t block_m,
                          int32_t block_n, int32_t *out_m, int32_t *out_n, int32_t *merged) {
  dk::clear_error();
  DK_REQUIRE(out_m && out_n && merged, "NULL argument");
  DK_REQUIRE(block_size > 0 && block_m > 0 && block_n > 0, "non-positive block size");
  DK_REQUIRE((block_m % block_size == 0) || (block_size % block_n == 0),
             "block_m must be mutliple or a factor of sparse block size for merging on Q blocks");
  DK_REQUIRE(block_size % block_n == 0,
             "block_n must be a factor of sparse block size for splitting on K blocks");
  const int split_m = block_size > block_m ? block_size / block_m : 1;
  const int split_n = block_size / block_n;
  int m = M * split_m, n = N * split_n;
  *merged = 0;
  if (block_size < block_m) {
    const int mm = block_m / block_size;
    DK_REQUIRE(m % mm == 0, "M=%d, m_mult=%d", m, mm);
    m /= mm;
    *merged = 1;
  }
  *out_m = m;
  *out_n = n;
  return DK_OK;
}

int dk_tile_pattern(const uint8_t *pattern, int32_t H, int32_t M, int32_t N, int32_t block_size,
                    int32_t block_m, int32_t block_n, int32_t prune, int32_t *out) {
  int32_t om, on, merged;
  int rc = dk_tile_pattern_shape(M, N, block_size, block_m, block_n, &om, &on, &merged);
  if (rc) return rc;
  DK_REQUIRE(pattern && out, "NULL argument");
  const int split_m = block_size > block_m ? block_size / block_m : 1;
  const int split_n = block_size / block_n;
  const int sub_m = block_size / split_m, sub_n = block_size / split_n;  // tokens per sub-block
  const int Ms = M * split_m, Ns = N * split_n;
  const bool do_prune = prune && (split_m * split_n > 1);
  std::vector<uint8_t> split((size_t)Ms * Ns);
  for (int h = 0; h < H; ++h) {
    const uint8_t *p = pattern + (size_t)h * M * N;
    for (int i = 0; i < Ms; ++i)
      for (int j = 0; j < Ns; ++j) {
        uint8_t x = p[(size_t)(i / split_m) * N + j / split_n];
        if (do_prune && !((int64_t)(i + 1) * sub_m > (int64_t)j * sub_n)) x = 0;
        split[(size_t)i * Ns + j] = x;
      }
    int32_t *o = out + (size_t)h * om * on;
    if (!merged) {
      for (size_t t = 0; t < (size_t)Ms * Ns; ++t) o[t] = split[t];
    } else {
      const int mm = block_m / block_size;
      for (int i = 0; i < om; ++i)
        for (int j = 0; j < Ns; ++j) {
          int last = 0;  // (index of last non-zero sub-row) + 1
          for (int s = 0; s < mm; ++s)
            if (split[(size_t)(i * mm + s) * Ns + j]) last = s + 1;
          o[(size_t)i * on + j] = last * block_size;
        }
    }
  }
  return DK_OK;
}

int dk_kv_cache_efficient(const uint8_t *pattern, int32_t H, int32_t M, int32_t N, int32_t block_m,
                          int32_t block_n) {
  dk::clear_error();
  DK_REQUIRE(pattern != nullptr, "NULL argument");
  for (int h = 0; h < H; ++h) {
    const uint8_t *p = pattern + (size_t)h * M * N;
    for (int i = 1; i < M; ++i)
      for (int j = 0; j < N; ++j) {
        const bool below_diag = (int64_t)i * block_m >= (int64_t)(j + 1) * block_n;
        if (below_diag && (p[(size_t)i * N + j] != 0) > (p[(size_t)(i - 1) * N + j] != 0)) return 0;
      }
  }
  return 1;
}

}  // extern "C"
