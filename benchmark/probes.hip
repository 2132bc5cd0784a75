// Two stand-alone probes of the MI355X memory system behind design decisions of the kernels
// (no part of the library; results in profiles/probe_atomic_add_and_cu_stream.md):
//
//   atomic   fp32 global atomic adds in the access pattern of a one-pass backward that would add a
//            32 x 128 fp32 tile of dQ partials per listed (q block, column) pair: 87 008 blocks of the
//            benchmark pattern, 2.85 GB of atomic traffic per backward, next to plain and
//            non-temporal stores of the same bytes.
//   stream   how fast one workgroup can stream HBM as a function of waves per workgroup, 16 KB
//            pieces in flight per wave and the number of workgroups active on the chip (the
//            access pattern of a decode wave without the arithmetic).
//
//   hipcc --offload-arch=gfx950 -O3 -munsafe-fp-atomics -o probes benchmark/probes.hip && ./probes
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#define CHECK(x)                                                  \
  do {                                                            \
    hipError_t e_ = (x);                                          \
    if (e_ != hipSuccess) {                                       \
      printf("%s: %s\n", #x, hipGetErrorString(e_));              \
      exit(1);                                                    \
    }                                                             \
  } while (0)

// ---------------------------------------------------------------------------
// atomic: every column workgroup (4 waves) adds 32 x 128 fp32 tiles for its listed q blocks
// ---------------------------------------------------------------------------
namespace atomic_probe {

constexpr int L = 8192, H = 32, D = 128, NB = L / 64, LOCAL = 16, VERT = 8;

// MODE 0: device-scope atomic add, 1: workgroup-scope atomic add, 2: non-temporal store, 3: plain store
template <int MODE, bool HEAD_FAST>
__global__ __launch_bounds__(256) void pattern(float *dq) {
  const int h = HEAD_FAST ? blockIdx.x : blockIdx.y;
  const int c = HEAD_FAST ? blockIdx.y : blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const bool vert = (c + h) % VERT == 0;
  float *base = dq + (size_t)h * L * D + 32 * wave + (lane & 31);
  for (int rb = c; rb < NB; ++rb) {
    if (rb >= c + LOCAL && !vert) break;
    for (int step = 0; step < 2; ++step) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = rb * 64 + step * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        float *p = base + (size_t)row * D;
        if (MODE == 0) unsafeAtomicAdd(p, 1.0f);
        else if (MODE == 1) __hip_atomic_fetch_add(p, 1.0f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        else if (MODE == 2) __builtin_nontemporal_store(1.0f, p);
        else *p = 1.0f;
      }
    }
  }
}

template <int MODE, bool HEAD_FAST>
static void run(const char *name, float *dq) {
  hipEvent_t a, b;
  CHECK(hipEventCreate(&a));
  CHECK(hipEventCreate(&b));
  const dim3 grid = HEAD_FAST ? dim3(H, NB) : dim3(NB, H);
  for (int i = 0; i < 3; ++i) hipLaunchKernelGGL((pattern<MODE, HEAD_FAST>), grid, dim3(256), 0, 0, dq);
  CHECK(hipDeviceSynchronize());
  CHECK(hipMemset(dq, 0, (size_t)H * L * D * 4));
  CHECK(hipEventRecord(a));
  const int n = 10;
  for (int i = 0; i < n; ++i) hipLaunchKernelGGL((pattern<MODE, HEAD_FAST>), grid, dim3(256), 0, 0, dq);
  CHECK(hipEventRecord(b));
  CHECK(hipDeviceSynchronize());
  float ms;
  CHECK(hipEventElapsedTime(&ms, a, b));
  long blocks = 0;
  for (int h = 0; h < H; ++h)
    for (int c = 0; c < NB; ++c)
      for (int rb = c; rb < NB; ++rb) {
        if (rb >= c + LOCAL && (c + h) % VERT) break;
        ++blocks;
      }
  const double bytes = (double)blocks * 64 * D * 4;
  printf("atomic  %-36s %8.1f us per launch, %5.2f GB -> %7.1f GB/s (%ld blocks)\n", name, ms / n * 1e3, bytes / 1e9,
         bytes / (ms / n * 1e-3) / 1e9, blocks);
  if (MODE <= 1) {  // every element must hold n x (columns that attend its row block)
    std::vector<float> host((size_t)L * D);
    CHECK(hipMemcpy(host.data(), dq + (size_t)3 * L * D, host.size() * 4, hipMemcpyDeviceToHost));
    long bad = 0;
    for (int rb = 0; rb < NB; ++rb) {
      int cnt = 0;
      for (int c = 0; c <= rb; ++c)
        if (rb < c + LOCAL || (c + 3) % VERT == 0) ++cnt;
      for (int i = 0; i < 64 * D; ++i)
        if (host[(size_t)rb * 64 * D + i] != (float)(cnt * n)) ++bad;
    }
    printf("        check of head 3: %ld wrong elements\n", bad);
  }
  fflush(stdout);
}

static void all() {
  float *dq;
  CHECK(hipMalloc(&dq, (size_t)H * L * D * 4));
  run<3, true>("plain stores, heads fastest in the grid", dq);
  run<2, true>("non-temporal stores, heads fastest", dq);
  run<0, true>("atomic add (device), heads fastest", dq);
  run<0, false>("atomic add (device), columns fastest", dq);
  run<1, true>("atomic add (workgroup), heads fastest", dq);
  CHECK(hipFree(dq));
}

}  // namespace atomic_probe

// ---------------------------------------------------------------------------
// stream: every wave reads `pieces` pieces of 16 KB (64 lanes x 16 loads x 16 B), one piece ahead
// ---------------------------------------------------------------------------
namespace stream_probe {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(512) void stream(const u32x4 *src, uint32_t *sink, int pieces, size_t wg_stride16) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const u32x4 *base = src + (size_t)blockIdx.x * wg_stride16 + lane;
  u32x4 buf[16];
  uint32_t acc = 0;
  auto piece = [&](int i) { return base + ((size_t)i * nw + wave) * 1024; };  // 1024 x 16 B
#pragma unroll
  for (int c = 0; c < 16; ++c) buf[c] = __builtin_nontemporal_load(piece(0) + c * 64);
  for (int i = 0; i < pieces; ++i) {
    u32x4 cur[16];
#pragma unroll
    for (int c = 0; c < 16; ++c) cur[c] = buf[c];
    if (i + 1 < pieces) {
#pragma unroll
      for (int c = 0; c < 16; ++c) buf[c] = __builtin_nontemporal_load(piece(i + 1) + c * 64);
    }
#pragma unroll
    for (int c = 0; c < 16; ++c) acc += cur[c][0] ^ cur[c][3];
  }
  if (acc == 0x12345678u) sink[0] = acc;
}

static void run(const u32x4 *src, uint32_t *sink, int wgs, int waves, size_t wg_bytes, size_t total_bytes) {
  const int pieces = (int)(wg_bytes / waves / 16384);
  const size_t per_wg = (size_t)waves * pieces * 16384;
  if (per_wg * wgs > total_bytes) return;
  hipEvent_t a, b;
  CHECK(hipEventCreate(&a));
  CHECK(hipEventCreate(&b));
  for (int i = 0; i < 2; ++i) hipLaunchKernelGGL(stream, dim3(wgs), dim3(64 * waves), 0, 0, src, sink, pieces, per_wg / 16);
  CHECK(hipDeviceSynchronize());
  CHECK(hipEventRecord(a));
  const int n = 5;
  for (int i = 0; i < n; ++i) hipLaunchKernelGGL(stream, dim3(wgs), dim3(64 * waves), 0, 0, src, sink, pieces, per_wg / 16);
  CHECK(hipEventRecord(b));
  CHECK(hipDeviceSynchronize());
  float ms;
  CHECK(hipEventElapsedTime(&ms, a, b));
  const double us = ms / n * 1e3;
  printf("stream  %4d workgroups x %d waves, %5.0f KB each: %8.1f us  %6.1f GB/s per workgroup  %7.1f GB/s in all\n", wgs, waves,
         per_wg / 1024.0, us, per_wg / us / 1e3, per_wg * wgs / us / 1e3);
  fflush(stdout);
}

static void all() {
  const size_t total = (size_t)3 << 30;
  u32x4 *src;
  uint32_t *sink;
  CHECK(hipMalloc(&src, total));
  CHECK(hipMalloc(&sink, 4));
  CHECK(hipMemset(src, 1, total));
  for (int wgs : {1, 16, 64, 128, 256, 512})
    for (int waves : {4, 8}) run(src, sink, wgs, waves, (size_t)4 << 20, total);
  CHECK(hipFree(src));
  CHECK(hipFree(sink));
}

}  // namespace stream_probe

int main() {
  atomic_probe::all();
  stream_probe::all();
  return 0;
}
