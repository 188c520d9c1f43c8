// Per-row dynamic int8 quantisation: scale = max|x| / 127, q = rint(x / scale).
//
// One 256-thread block per row.  Each thread keeps up to 4 eight-element vectors of its row in
// registers between the absmax pass and the quantise pass, so a row of up to 8192 elements is
// read from memory once; longer or unaligned rows are read twice.  The absmax is reduced inside
// each wavefront with DPP/bpermute steps and across the four wavefronts through LDS.
#include "common.h"
#include "quant_rows.h"

namespace {

// vectorised path: cols % 8 == 0, row base 16-byte aligned
template <int DT, int MAXV>
__global__ __launch_bounds__(256) void quant_rows_vec(const void* __restrict__ xv, int64_t rows, int cols, int64_t ld,
                                                      int8_t* __restrict__ q, float* __restrict__ scale) {
  __shared__ float red[4];
  quant_row_vec_body<DT, MAXV>(xv, (int64_t)blockIdx.x, cols, ld, q, scale, red);
}

// general path: any cols / stride, two passes over the row
template <int DT>
__global__ __launch_bounds__(256) void quant_rows_any(const void* __restrict__ xv, int64_t rows, int cols, int64_t ld,
                                                      int8_t* __restrict__ q, float* __restrict__ scale) {
  typedef typename Elem<DT>::T ET;
  __shared__ float red[4];
  const int64_t r = blockIdx.x;
  const ET* x = (const ET*)xv + r * ld;
  float amax = 0.0f;
  for (int c = threadIdx.x; c < cols; c += 256) amax = fmaxf(amax, fabsf(Elem<DT>::cvt(x[c])));
  amax = block_allmax(amax, red);
  const float s = amax / 127.0f;
  if (threadIdx.x == 0) scale[r] = s;
  int8_t* qr = q + r * (int64_t)cols;
  for (int c = threadIdx.x; c < cols; c += 256) qr[c] = (s > 0.0f) ? (int8_t)quant_i8(Elem<DT>::cvt(x[c]), s) : (int8_t)0;
}

template <int DT>
int launch_quant(const void* x, int64_t rows, int cols, int64_t ld, int8_t* q, float* scale, hipStream_t st) {
  const size_t esz = sizeof(typename Elem<DT>::T);
  const bool aligned = (cols % 8 == 0) && (((uintptr_t)x) % 16 == 0) && ((ld * esz) % 16 == 0) && (((uintptr_t)q) % 8 == 0);
  dim3 grid((unsigned)rows), block(256);
  if (aligned && cols <= 8 * 256 * 1) hipLaunchKernelGGL((quant_rows_vec<DT, 1>), grid, block, 0, st, x, rows, cols, ld, q, scale);
  else if (aligned && cols <= 8 * 256 * 2) hipLaunchKernelGGL((quant_rows_vec<DT, 2>), grid, block, 0, st, x, rows, cols, ld, q, scale);
  else if (aligned && cols <= 8 * 256 * 4) hipLaunchKernelGGL((quant_rows_vec<DT, 4>), grid, block, 0, st, x, rows, cols, ld, q, scale);
  else hipLaunchKernelGGL((quant_rows_any<DT>), grid, block, 0, st, x, rows, cols, ld, q, scale);
  OMNI_CHECK_LAUNCH("dynamic_quant");
  return OMNI_OK;
}

}  // namespace

extern "C" int omni_dynamic_quant(const void* x, int in_dtype, int64_t rows, int cols, int64_t ld, int8_t* q,
                                  float* scale, void* stream) {
  if (rows < 0 || cols <= 0 || ld < cols) OMNI_FAIL(OMNI_E_INVALID, "dynamic_quant: bad shape rows=%lld cols=%d ld=%lld", (long long)rows, cols, (long long)ld);
  if (rows == 0) return OMNI_OK;
  if (!x || !q || !scale) OMNI_FAIL(OMNI_E_INVALID, "dynamic_quant: null pointer");
  if (rows > 0x7fffffffLL) OMNI_FAIL(OMNI_E_UNSUPPORTED, "dynamic_quant: too many rows");
  hipStream_t st = (hipStream_t)stream;
  switch (in_dtype) {
    case OMNI_DT_BF16: return launch_quant<OMNI_DT_BF16>(x, rows, cols, ld, q, scale, st);
    case OMNI_DT_F16: return launch_quant<OMNI_DT_F16>(x, rows, cols, ld, q, scale, st);
    case OMNI_DT_F32: return launch_quant<OMNI_DT_F32>(x, rows, cols, ld, q, scale, st);
    default: OMNI_FAIL(OMNI_E_INVALID, "dynamic_quant: unknown dtype %d", in_dtype);
  }
}
