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

}  // namespace

extern "C" int omni_diag_mfma_i8_rate(const int8_t* operands, size_t operand_bytes, int iters, int blocks, int32_t* sink,
                                      void* stream) {
  if (!operands || !sink || iters <= 0 || blocks <= 0) OMNI_FAIL(OMNI_E_INVALID, "diag_mfma_i8_rate: bad arguments");
  if (operand_bytes < (size_t)32 * 2 * WAVE * 16) OMNI_FAIL(OMNI_E_INVALID, "diag_mfma_i8_rate: operand buffer below 64 KiB");
  if ((uintptr_t)operands % 16) OMNI_FAIL(OMNI_E_INVALID, "diag_mfma_i8_rate: operands must be 16-byte aligned");
  hipLaunchKernelGGL(mfma_i8_rate_kernel, dim3((unsigned)blocks), dim3(512), 0, (hipStream_t)stream, operands, iters, sink);
  OMNI_CHECK_LAUNCH("diag_mfma_i8_rate");
  return OMNI_OK;
}
