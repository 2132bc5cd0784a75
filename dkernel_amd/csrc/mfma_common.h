// MFMA building blocks for gfx950 (CDNA4), 64-lane wavefronts.
//
// v_mfma_f32_32x32x16_{bf16,f16}: D(32x32) += A(32x16) * B(16x32).
//   A operand, lane l: row l%32, k = 8*(l/32) .. +7      (8 x 16-bit, one 16-byte word)
//   B operand, lane l: col l%32, k = 8*(l/32) .. +7
//   accumulator, lane l, register r (0..15): col l%32, row 8*(r/4) + 4*(l/32) + r%4
// (layouts verified on hardware with an integer-valued GEMM.)
//
// ds_read_tr16_b64 (LDS transpose read): inside each group of 16 lanes, lane i
// supplies the address of four consecutive 16-bit values S[i][0..3] and
// receives S[4j + (i>>2)][i&3] for j = 0..3.  Pointing lane i at
// M[n0 + (i>>2)][d0 + 4*(i&3)] of a row-major matrix therefore returns
// M[n0 .. n0+3][d0 + i]: a column slice, i.e. the k-contiguous MFMA operand of
// the transposed matrix, without ever storing the transpose.
#pragma once

#include <hip/hip_runtime.h>

#include "device_common.h"

namespace dk {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef short shortx8 __attribute__((ext_vector_type(8)));

template <typename T>
struct Mma;  // 16-bit element type -> operand vector, MFMA, conversion

template <>
struct Mma<bf16_t> {
  using vec8 = bf16x8;
  static __device__ __forceinline__ floatx16 mma(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ vec8 pack(const float *x) {
    vec8 r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = (__bf16)x[i];
    return r;
  }
};

template <>
struct Mma<f16_t> {
  using vec8 = f16x8;
  static __device__ __forceinline__ floatx16 mma(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ vec8 pack(const float *x) {
    vec8 r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = (_Float16)x[i];
    return r;
  }
};

template <typename V>
__device__ __forceinline__ V as_vec8(uint4 w) {
  return __builtin_bit_cast(V, w);
}

// 16-byte LDS read of 8 consecutive 16-bit values.
template <typename V>
__device__ __forceinline__ V lds_read8(const char *p) {
  return as_vec8<V>(*reinterpret_cast<const uint4 *>(p));
}

// Two transpose reads -> the 8 k-values of one operand lane.
template <typename V>
__device__ __forceinline__ V lds_read_tr8(const char *p0, const char *p1) {
  typedef shortx4 __attribute__((address_space(3))) * lds_ptr;
  shortx4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0));
  shortx4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p1));
  shortx8 r = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(V, r);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Exchange with the lane 32 away (the other half-wave that holds the rest of
// an accumulator row).
__device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32); }

}  // namespace dk
