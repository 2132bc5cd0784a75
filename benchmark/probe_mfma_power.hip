// Stand-alone probe (no part of the library): what rate of v_mfma_f32_32x32x16_bf16 the whole
// MI355X sustains, as a function of the operand data and of the work issued next to the
// multiplies.  No global memory traffic inside the timed loops, no barriers, 8 waves per CU (two per
// SIMD) on every CU unless said otherwise, 32 multiplies per loop iteration in 2 + 4 accumulator
// chains like a wave of the forward kernel per (32 rows x 64 keys) block at head dim 128.
//
//   zeros / random    operands all zero, or random bf16 values (sign, exponent around 1 and
//                     mantissa bits random): the same instruction stream;
//   lds N             a fresh 1 KB operand from LDS (16-byte reads) for one multiply in N;
//   valu N            N dependent fp32 FMAs per multiply next to them;
//   forward mix       per 32 multiplies what the forward kernel issues for a block: 16 16-byte LDS
//                     operand reads, 32 transpose reads (ds_read_b64_tr_b16), 32 exponentials,
//                     32 FMAs, 32 adds, 16 three-way maxima, 16 conversions to packed bf16.
//
//   hipcc --offload-arch=gfx950 -O3 -Xclang -target-feature -Xclang -packed-fp32-ops \
//       -o /tmp/probe_mfma_power benchmark/probe_mfma_power.hip && /tmp/probe_mfma_power
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#define CHECK(x)                                     \
  do {                                               \
    hipError_t e_ = (x);                             \
    if (e_ != hipSuccess) {                          \
      printf("%s: %s\n", #x, hipGetErrorString(e_)); \
      exit(1);                                       \
    }                                                \
  } while (0)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(4))) short shortx4;
typedef __attribute__((ext_vector_type(8))) short shortx8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

constexpr int kIters = 3000;
constexpr int kMfmaPerIter = 32;

__device__ __forceinline__ floatx16 mma(bf16x8 a, bf16x8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ float drain(const floatx16 *acc, int n) {
  float s = 0.f;
  for (int c = 0; c < n; ++c)
    for (int r = 0; r < 16; ++r) s += acc[c][r];
  return s;
}

// LDS_EVERY = 0: operands stay in registers; N > 0: one multiply in N takes a fresh LDS operand.
// VALU: dependent FMAs per multiply.
template <int LDS_EVERY, int VALU>
__global__ __launch_bounds__(512) void mfma_loop(const uint4 *in, float *out, int iters) {
  __shared__ uint4 lds[4096];  // 64 KB of operand data
  for (int i = threadIdx.x; i < 4096; i += 512) lds[i] = in[i];
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  bf16x8 a = __builtin_bit_cast(bf16x8, in[threadIdx.x]);
  const bf16x8 b = __builtin_bit_cast(bf16x8, in[512 + threadIdx.x]);
  floatx16 acc[4];
  for (int c = 0; c < 4; ++c)
    for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
  float x = lane * 1e-9f, y = 0.f;
  for (int i = 0; i < iters; ++i) {
    const uint4 *base = lds + lane + ((i + wave) & 3) * 1024;
#pragma unroll
    for (int j = 0; j < kMfmaPerIter; ++j) {
      if (LDS_EVERY > 0 && j % LDS_EVERY == 0) a = __builtin_bit_cast(bf16x8, base[(j * 32) & 1023]);
      acc[j & 3] = mma(a, b, acc[j & 3]);
#pragma unroll
      for (int v = 0; v < VALU; v += 2) {
        y = fmaf(x, y, 1.0f + v);
        x = fmaf(y, 0.5f, x);
      }
    }
  }
  out[blockIdx.x * 512 + threadIdx.x] = drain(acc, 4) + x + y;
}

// The instruction mix of the forward kernel for one (32 rows x 64 keys) block at head dim 128:
// S (2 chains of 8 multiplies, operands by 16-byte LDS reads), softmax of the 32 S values per lane,
// O (4 chains of 4 multiplies, operands by transpose reads, second operand = the packed
// probabilities).
__global__ __launch_bounds__(512) void forward_mix(const uint4 *in, float *out, int iters, float scale) {
  __shared__ uint4 lds[4096];
  for (int i = threadIdx.x; i < 4096; i += 512) lds[i] = in[i];
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  bf16x8 q[8];
  for (int k = 0; k < 8; ++k) q[k] = __builtin_bit_cast(bf16x8, in[512 + k * 512 + threadIdx.x]);
  floatx16 o[4];
  for (int c = 0; c < 4; ++c)
    for (int r = 0; r < 16; ++r) o[c][r] = 0.f;
  float l = 0.f, m = 0.f;
  typedef shortx4 __attribute__((address_space(3))) * lds_tr_ptr;
  for (int i = 0; i < iters; ++i) {
    const uint4 *base = lds + lane + ((i + wave) & 3) * 1024;
    floatx16 s[2];
    for (int c = 0; c < 2; ++c)
      for (int r = 0; r < 16; ++r) s[c][r] = 0.f;
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int k = 0; k < 8; ++k) s[c] = mma(__builtin_bit_cast(bf16x8, base[(c * 8 + k) * 64 & 1023]), q[k], s[c]);
    float mx = fmaxf(s[0][0], s[1][0]);
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = fmaxf(fmaxf(mx, s[0][r]), s[1][r]);
    m = fmaxf(m, mx * scale);
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        s[c][r] = __builtin_amdgcn_exp2f(fmaf(s[c][r], scale, -m));
        sum += s[c][r];
      }
    l += sum;
#pragma unroll
    for (int step = 0; step < 4; ++step) {
      bf16x8 p;
#pragma unroll
      for (int e = 0; e < 8; ++e) p[e] = (__bf16)s[step >> 1][(step & 1) * 8 + e];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const char *ad = reinterpret_cast<const char *>(base) + ((step * 4 + c) * 1024 & 8191);
        const shortx4 t0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(uintptr_t)(uint32_t)(uintptr_t)ad);
        const shortx4 t1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(uintptr_t)(uint32_t)(uintptr_t)(ad + 512));
        const shortx8 t = __builtin_shufflevector(t0, t1, 0, 1, 2, 3, 4, 5, 6, 7);
        o[c] = mma(__builtin_bit_cast(bf16x8, t), p, o[c]);
      }
    }
  }
  out[blockIdx.x * 512 + threadIdx.x] = drain(o, 4) + l + m;
}

static std::vector<unsigned short> random_bf16(size_t n) {
  std::vector<unsigned short> h(n);
  for (auto &v : h) v = (unsigned short)(0x3f00 ^ (rand() & 0x80ff) ^ ((rand() & 1) << 8));  // +-[0.5, 2)
  return h;
}

template <typename F>
static void timed(const char *name, int wgs, F launch) {
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  float best = 1e30f;
  for (int rep = 0; rep < 3; ++rep) {
    CHECK(hipEventRecord(e0));
    launch();
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    if (rep && ms < best) best = ms;
  }
  const double flop = (double)wgs * 8 * kIters * kMfmaPerIter * 32768.0;
  printf("%-58s %4d workgroups: %6.3f ms  %5.0f TFLOP/s = %4.1f %% of 2500\n", name, wgs, best, flop / best / 1e9,
         flop / best / 1e9 / 25.0);
}

int main() {
  const size_t n16 = 8192;  // uint4 elements of operand data
  uint4 *in;
  float *out;
  CHECK(hipMalloc(&in, n16 * 16));
  CHECK(hipMalloc(&out, 256 * 512 * 4));
  for (int pass = 0; pass < 2; ++pass) {
    const char *data = pass ? "random" : "zeros";
    if (pass) {
      auto h = random_bf16(n16 * 8);
      CHECK(hipMemcpy(in, h.data(), n16 * 16, hipMemcpyHostToDevice));
    } else {
      CHECK(hipMemset(in, 0, n16 * 16));
    }
    char name[96];
    for (int wgs : {256, 128}) {
      snprintf(name, sizeof name, "%s, multiplies only", data);
      timed(name, wgs, [&] { hipLaunchKernelGGL((mfma_loop<0, 0>), dim3(wgs), dim3(512), 0, 0, in, out, kIters); });
    }
    snprintf(name, sizeof name, "%s, lds 4 (one LDS operand per 4 multiplies)", data);
    timed(name, 256, [&] { hipLaunchKernelGGL((mfma_loop<4, 0>), dim3(256), dim3(512), 0, 0, in, out, kIters); });
    snprintf(name, sizeof name, "%s, lds 2", data);
    timed(name, 256, [&] { hipLaunchKernelGGL((mfma_loop<2, 0>), dim3(256), dim3(512), 0, 0, in, out, kIters); });
    snprintf(name, sizeof name, "%s, lds 1 (every multiply)", data);
    timed(name, 256, [&] { hipLaunchKernelGGL((mfma_loop<1, 0>), dim3(256), dim3(512), 0, 0, in, out, kIters); });
    snprintf(name, sizeof name, "%s, valu 4", data);
    timed(name, 256, [&] { hipLaunchKernelGGL((mfma_loop<0, 4>), dim3(256), dim3(512), 0, 0, in, out, kIters); });
    snprintf(name, sizeof name, "%s, valu 6", data);
    timed(name, 256, [&] { hipLaunchKernelGGL((mfma_loop<0, 6>), dim3(256), dim3(512), 0, 0, in, out, kIters); });
    snprintf(name, sizeof name, "%s, lds 1 + valu 6", data);
    timed(name, 256, [&] { hipLaunchKernelGGL((mfma_loop<1, 6>), dim3(256), dim3(512), 0, 0, in, out, kIters); });
    for (int wgs : {256, 128}) {
      snprintf(name, sizeof name, "%s, forward mix", data);
      timed(name, wgs, [&] { hipLaunchKernelGGL(forward_mix, dim3(wgs), dim3(512), 0, 0, in, out, kIters, 0.01f); });
    }
    snprintf(name, sizeof name, "%s, multiplies only (again, after the others)", data);
    timed(name, 256, [&] { hipLaunchKernelGGL((mfma_loop<0, 0>), dim3(256), dim3(512), 0, 0, in, out, kIters); });
  }
  return 0;
}
