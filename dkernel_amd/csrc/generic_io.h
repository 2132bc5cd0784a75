// Guarded 8-element loads / stores for the generic kernels: 16-byte vector
// accesses when the host has verified alignment (vec_ok) and the chunk lies
// inside the head dim, scalar accesses with zero fill otherwise.
#pragma once

#include "device_common.h"

namespace dk {

template <typename T>
struct Pack8 {  // 8 elements of T as 16-byte words
  static constexpr int kWords = sizeof(T) * 8 / 16;
  uint4 w[kWords];
};

template <typename T>
__device__ __forceinline__ void unpack8(const Pack8<T> &pk, float *out) {
  const T *e = reinterpret_cast<const T *>(&pk);
#pragma unroll
  for (int i = 0; i < 8; ++i) out[i] = to_float(e[i]);
}

template <typename T>
__device__ __forceinline__ Pack8<T> gather8(const T *row, int d0, int D, bool ok, int vec_ok) {
  Pack8<T> pk;
#pragma unroll
  for (int w = 0; w < Pack8<T>::kWords; ++w) pk.w[w] = make_uint4(0, 0, 0, 0);
  if (ok && d0 < D) {
    if (vec_ok && d0 + 8 <= D) {
      const uint4 *src = reinterpret_cast<const uint4 *>(row + d0);
#pragma unroll
      for (int w = 0; w < Pack8<T>::kWords; ++w) pk.w[w] = src[w];
    } else {
      T *e = reinterpret_cast<T *>(&pk);
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (d0 + i < D) e[i] = row[d0 + i];
    }
  }
  return pk;
}

template <typename T>
__device__ __forceinline__ void load8_guard(const T *row, int d0, int D, bool ok, int vec_ok, float *out) {
  unpack8<T>(gather8<T>(row, d0, D, ok, vec_ok), out);
}

template <typename T>
__device__ __forceinline__ void copy8_guard(const T *row, int d0, int D, bool ok, int vec_ok, T *dst) {
  *reinterpret_cast<Pack8<T> *>(dst) = gather8<T>(row, d0, D, ok, vec_ok);
}

template <typename T>
__device__ __forceinline__ void lds_load8(const T *src, float *out) {
  unpack8<T>(*reinterpret_cast<const Pack8<T> *>(src), out);
}

template <typename T>
__device__ __forceinline__ void store8_guard(T *row, int d0, int D, int vec_ok, const float *in) {
  if (d0 >= D) return;
  Pack8<T> pk;
  T *e = reinterpret_cast<T *>(&pk);
#pragma unroll
  for (int i = 0; i < 8; ++i) e[i] = from_float<T>(in[i]);
  if (vec_ok && d0 + 8 <= D) {
    uint4 *dst = reinterpret_cast<uint4 *>(row + d0);
#pragma unroll
    for (int w = 0; w < Pack8<T>::kWords; ++w) dst[w] = pk.w[w];
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (d0 + i < D) row[d0 + i] = e[i];
  }
}

}  // namespace dk
