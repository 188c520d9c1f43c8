// Row body of the per-row dynamic int8 quantisation (shared by the stand-alone kernel and by the
// launch that also sorts the assignments): one 256-thread block quantises row r.
#pragma once
#include "common.h"

namespace {

template <int DT>
struct Elem;
template <>
struct Elem<OMNI_DT_BF16> {
  typedef uint16_t T;
  static __device__ __forceinline__ float cvt(uint16_t v) { return bf16_to_f32(v); }
};
template <>
struct Elem<OMNI_DT_F16> {
  typedef uint16_t T;
  static __device__ __forceinline__ float cvt(uint16_t v) { return f16_to_f32(v); }
};
template <>
struct Elem<OMNI_DT_F32> {
  typedef float T;
  static __device__ __forceinline__ float cvt(float v) { return v; }
};

__device__ __forceinline__ float block_allmax(float v, float* red) {
  v = wave_allmax_f(v);
  const int w = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1);
  if (lane == 0) red[w] = v;
  __syncthreads();
  float m = red[0];
  for (int i = 1; i < (int)(blockDim.x / WAVE); ++i) m = fmaxf(m, red[i]);
  return m;
}

// vectorised path: cols % 8 == 0, row base 16-byte aligned (8-byte for 4-byte elements handled by VEC)
template <int DT, int MAXV>
__device__ __forceinline__ void quant_row_vec_body(const void* __restrict__ xv, int64_t r, int cols, int64_t ld,
                                                   int8_t* __restrict__ q, float* __restrict__ scale, float* red) {
  typedef typename Elem<DT>::T ET;
  const ET* x = (const ET*)xv + r * ld;
  const int nvec = cols / 8;
  float v[MAXV][8];
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    int vi = threadIdx.x + i * 256;
    if (vi < nvec) {
      if constexpr (sizeof(ET) == 2) {
        v4i raw = __builtin_nontemporal_load((const v4i*)(x + (size_t)vi * 8));  // the row is read once here
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t u = (uint32_t)raw[j];
          v[i][2 * j] = Elem<DT>::cvt((uint16_t)(u & 0xffffu));
          v[i][2 * j + 1] = Elem<DT>::cvt((uint16_t)(u >> 16));
        }
      } else {
        v4f a = __builtin_nontemporal_load((const v4f*)(x + (size_t)vi * 8));
        v4f b = __builtin_nontemporal_load((const v4f*)(x + (size_t)vi * 8 + 4));
#pragma unroll
        for (int j = 0; j < 4; ++j) { v[i][j] = a[j]; v[i][4 + j] = b[j]; }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[i][j]));
    }
  }
  amax = block_allmax(amax, red);
  const float s = amax / 127.0f;
  if (threadIdx.x == 0) scale[r] = s;
  int8_t* qr = q + r * (int64_t)cols;
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    int vi = threadIdx.x + i * 256;
    if (vi < nvec) {
      uint32_t w0 = 0, w1 = 0;
      if (s > 0.0f) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          w0 |= ((uint32_t)(quant_i8(v[i][j], s) & 0xff)) << (8 * j);
          w1 |= ((uint32_t)(quant_i8(v[i][4 + j], s) & 0xff)) << (8 * j);
        }
      }
      v2i o = {(int)w0, (int)w1};
      *(v2i*)(qr + (size_t)vi * 8) = o;
    }
  }
}

}  // namespace
