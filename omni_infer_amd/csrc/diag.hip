// Diagnostics that put a number on what the hardware delivers, for reading the GEMM kernels' figures against:
// the sustained rate of the int8 matrix instruction on given operand bits, with nothing else in the loop.
#include "common.h"

namespace {

typedef int v16i __attribute__((ext_vector_type(16)));

// Every wavefront keeps 8 independent 32x32 accumulators going with operands that stay in registers: no
// memory access, no LDS, no dependency stall (8 instructions of 32 cycles are in flight per wavefront, two
// wavefronts per SIMD).  What the operands hold decides how much of the datapath toggles, and with it the
// clock the chip sustains.
__global__ __launch_bounds__(512, 2) void mfma_i8_rate_kernel(const int8_t* __restrict__ operands, int iters,
                                                              int32_t* __restrict__ sink) {
#if defined(__HIP_DEVICE_COMPILE__)
  const int lane = threadIdx.x & (WAVE - 1);
  const int wv = threadIdx.x / WAVE;
  const v4i* p = (const v4i*)operands + ((blockIdx.x * 8 + wv) % 32) * 2 * WAVE + lane;
  v4i a = p[0], b = p[WAVE];
  v16i acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[j][i] = 0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[j], 0, 0, 0);
  }
  int32_t s = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[j][i];
  if (s == 0x7fffffff) sink[0] = s;  // keeps the loop alive; practically never true
#endif
}

// The matrix instruction on the operand pattern of the tile kernel: a 128 x 64 piece per wavefront, 128 accumulator
// registers, and from one instruction to the next another pair of operands (four row operands x two channel
// operands per half k-step for 32x32x32, eight x four per k-step for 16x16x64).  Same products, same registers;
// what differs is how many accumulators an instruction touches per product.
__global__ __launch_bounds__(512, 2) void mfma_tile32_kernel(const int8_t* __restrict__ operands, int iters, int32_t* __restrict__ sink) {
#if defined(__HIP_DEVICE_COMPILE__)
  const int lane = threadIdx.x & (WAVE - 1);
  const int wv = threadIdx.x / WAVE;
  const v4i* p = (const v4i*)operands + ((blockIdx.x * 8 + wv) % 4) * 16 * WAVE + lane;
  v4i a[2][4], b[2][2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int i = 0; i < 4; ++i) a[h][i] = p[(h * 6 + i) * WAVE];
#pragma unroll
    for (int i = 0; i < 2; ++i) b[h][i] = p[(h * 6 + 4 + i) * WAVE];
  }
  v16i acc[4][2];
#pragma unroll
  for (int m = 0; m < 4; ++m)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[m][t][i] = 0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int t = 0; t < 2; ++t) acc[m][t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[h][m], b[h][t], acc[m][t], 0, 0, 0);
  }
  int32_t s = 0;
#pragma unroll
  for (int m = 0; m < 4; ++m)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) s += acc[m][t][i];
  if (s == 0x7fffffff) sink[0] = s;
#endif
}
__global__ __launch_bounds__(512, 2) void mfma_tile16_kernel(const int8_t* __restrict__ operands, int iters, int32_t* __restrict__ sink) {
#if defined(__HIP_DEVICE_COMPILE__)
  const int lane = threadIdx.x & (WAVE - 1);
  const int wv = threadIdx.x / WAVE;
  const v4i* p = (const v4i*)operands + ((blockIdx.x * 8 + wv) % 4) * 16 * WAVE + lane;
  v4i a[8], b[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = p[i * WAVE];
#pragma unroll
  for (int i = 0; i < 4; ++i) b[i] = p[(8 + i) * WAVE];
  v4i acc[8][4];
#pragma unroll
  for (int m = 0; m < 8; ++m)
#pragma unroll
    for (int n = 0; n < 4; ++n) acc[m][n] = (v4i){0, 0, 0, 0};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int m = 0; m < 8; ++m) acc[m][n] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[m], b[n], acc[m][n], 0, 0, 0);
  }
  int32_t s = 0;
#pragma unroll
  for (int m = 0; m < 8; ++m)
#pragma unroll
    for (int n = 0; n < 4; ++n) s += acc[m][n][0] + acc[m][n][1] + acc[m][n][2] + acc[m][n][3];
  if (s == 0x7fffffff) sink[0] = s;
#endif
}

// Streaming read of a buffer, nothing else: every lane asks for 16 bytes at a time, `DEPTH` requests of a lane in
// flight, blocks walk the buffer with a grid stride; what arrives is folded into one word so that the loads stay.
// This is what the memory system delivers to a kernel that only reads: the ceiling of the weight-streaming GEMMs.
template <int DEPTH>
__global__ __launch_bounds__(256) void hbm_read_rate_kernel(const v4i* __restrict__ p, size_t n16, int32_t* __restrict__ sink) {
  const size_t stride = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  int32_t s = 0;
  for (; i + (DEPTH - 1) * stride < n16; i += DEPTH * stride) {
    v4i v[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) v[d] = __builtin_nontemporal_load(p + i + d * stride);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) s ^= v[d][0] ^ v[d][1] ^ v[d][2] ^ v[d][3];
  }
  for (; i < n16; i += stride) {
    const v4i v = __builtin_nontemporal_load(p + i);
    s ^= v[0] ^ v[1] ^ v[2] ^ v[3];
  }
  if (s == 0x5a5a5a5a) sink[0] = s;  // keeps the loads alive; practically never true
}

}  // namespace

extern "C" int omni_diag_hbm_read_rate(const void* buf, size_t bytes, int blocks, int32_t* sink, void* stream) {
  if (!buf || !sink || blocks <= 0 || bytes < 16) OMNI_FAIL(OMNI_E_INVALID, "diag_hbm_read_rate: bad arguments");
  if ((uintptr_t)buf % 16) OMNI_FAIL(OMNI_E_INVALID, "diag_hbm_read_rate: buffer must be 16-byte aligned");
  hipLaunchKernelGGL(hbm_read_rate_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const v4i*)buf,
                     bytes / 16, sink);
  OMNI_CHECK_LAUNCH("diag_hbm_read_rate");
  return OMNI_OK;
}

extern "C" int omni_diag_mfma_i8_tile_rate(const int8_t* operands, size_t operand_bytes, int form, int iters, int blocks,
                                           int32_t* sink, void* stream) {
  if (!operands || !sink || iters <= 0 || blocks <= 0) OMNI_FAIL(OMNI_E_INVALID, "diag_mfma_i8_tile_rate: bad arguments");
  if (form != 16 && form != 32) OMNI_FAIL(OMNI_E_INVALID, "diag_mfma_i8_tile_rate: form %d (16: 16x16x64, 32: 32x32x32)", form);
  if (operand_bytes < (size_t)4 * 16 * WAVE * 16) OMNI_FAIL(OMNI_E_INVALID, "diag_mfma_i8_tile_rate: operand buffer below 64 KiB");
  if ((uintptr_t)operands % 16) OMNI_FAIL(OMNI_E_INVALID, "diag_mfma_i8_tile_rate: operands must be 16-byte aligned");
  if (form == 32) hipLaunchKernelGGL(mfma_tile32_kernel, dim3((unsigned)blocks), dim3(512), 0, (hipStream_t)stream, operands, iters, sink);
  else hipLaunchKernelGGL(mfma_tile16_kernel, dim3((unsigned)blocks), dim3(512), 0, (hipStream_t)stream, operands, iters, sink);
  OMNI_CHECK_LAUNCH("diag_mfma_i8_tile_rate");
  return OMNI_OK;
}

extern "C" int omni_diag_mfma_i8_rate(const int8_t* operands, size_t operand_bytes, int iters, int blocks, int32_t* sink,
                                      void* stream) {
  if (!operands || !sink || iters <= 0 || blocks <= 0) OMNI_FAIL(OMNI_E_INVALID, "diag_mfma_i8_rate: bad arguments");
  if (operand_bytes < (size_t)32 * 2 * WAVE * 16) OMNI_FAIL(OMNI_E_INVALID, "diag_mfma_i8_rate: operand buffer below 64 KiB");
  if ((uintptr_t)operands % 16) OMNI_FAIL(OMNI_E_INVALID, "diag_mfma_i8_rate: operands must be 16-byte aligned");
  hipLaunchKernelGGL(mfma_i8_rate_kernel, dim3((unsigned)blocks), dim3(512), 0, (hipStream_t)stream, operands, iters, sink);
  OMNI_CHECK_LAUNCH("diag_mfma_i8_rate");
  return OMNI_OK;
}
