// Residual add + RMSNorm + per-token dynamic int8 quantisation in one pass over the row.
//
// One 256-thread block per row; a thread keeps up to 4 vectors of 8 elements of its row in
// registers, so the row is read once (x and residual) and written once per requested output.
// Arithmetic, every step one fp32 rounding:
//   s   = float(x) + float(residual)                      (residual_out = bf16(s))
//   ss  = sum of s*s over the row in a fixed order: thread t owns vectors t, t+256, ... and adds
//         their elements in index order; the 64 threads of a wavefront are combined by the butterfly
//         (partner distance 1, 2, 4, 8, 16, 32), the four wavefronts as ((w0 + w1) + w2) + w3
//   r   = 1 / sqrt(ss / H + eps)
//   y   = bf16((s * r) * float(weight))
//   scale = max|y| / 127,  q = rint(y / scale)            (on the bf16-rounded y)
#include "common.h"

namespace {

constexpr int NORM_MAXV = 4;  // rows up to 8 * 256 * 4 = 8192 elements

struct NormArgs {
  const uint16_t* x;
  const uint16_t* residual;  // nullable: plain RMSNorm of x
  const uint16_t* weight;
  int64_t rows;
  int H;
  float eps;
  uint16_t* residual_out;  // nullable
  uint16_t* y;             // nullable
  int8_t* q;               // nullable (with scale)
  float* scale;
};

__device__ __forceinline__ void unpack8(v4i raw, float* v) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint32_t u = (uint32_t)raw[j];
    v[2 * j] = bf16_to_f32((uint16_t)(u & 0xffffu));
    v[2 * j + 1] = bf16_to_f32((uint16_t)(u >> 16));
  }
}
__device__ __forceinline__ v4i pack8(const float* v) {
  v4i o;
#pragma unroll
  for (int j = 0; j < 4; ++j)
    o[j] = (int)((uint32_t)f32_to_bf16(v[2 * j]) | ((uint32_t)f32_to_bf16(v[2 * j + 1]) << 16));
  return o;
}

__global__ __launch_bounds__(256) void add_rms_norm_quant_kernel(NormArgs a) {
  __shared__ float red_sum[4], red_max[4];
  const int64_t r = blockIdx.x;
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  const int nvec = a.H / 8;
  const uint16_t* xr = a.x + r * a.H;
  const uint16_t* rr = a.residual ? a.residual + r * a.H : nullptr;
  float s[NORM_MAXV][8];
  float ss = 0.0f;
#pragma unroll
  for (int i = 0; i < NORM_MAXV; ++i) {
    const int vi = threadIdx.x + i * 256;
    if (vi < nvec) {
      unpack8(__builtin_nontemporal_load((const v4i*)(xr + (size_t)vi * 8)), s[i]);  // read once
      if (rr) {
        float t[8];
        unpack8(__builtin_nontemporal_load((const v4i*)(rr + (size_t)vi * 8)), t);
#pragma unroll
        for (int j = 0; j < 8; ++j) s[i][j] = s[i][j] + t[j];
        if (a.residual_out)  // next read: the following layer's norm, long after it left the caches
          __builtin_nontemporal_store(pack8(s[i]), (v4i*)(a.residual_out + r * a.H + (size_t)vi * 8));
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float sq = s[i][j] * s[i][j];
        ss = ss + sq;
      }
    }
  }
  ss = wave_allsum_f(ss);
  if (lane == 0) red_sum[w] = ss;
  __syncthreads();
  const float total = ((red_sum[0] + red_sum[1]) + red_sum[2]) + red_sum[3];
  const float mean = total / (float)a.H;
  const float rstd = 1.0f / sqrtf(mean + a.eps);
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < NORM_MAXV; ++i) {
    const int vi = threadIdx.x + i * 256;
    if (vi < nvec) {
      float g[8];
      unpack8(*(const v4i*)(a.weight + (size_t)vi * 8), g);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float y = (s[i][j] * rstd) * g[j];
        s[i][j] = round_bf16(y);
        amax = fmaxf(amax, fabsf(s[i][j]));
      }
      if (a.y) *(v4i*)(a.y + r * a.H + (size_t)vi * 8) = pack8(s[i]);
    }
  }
  if (a.q == nullptr) return;
  amax = wave_allmax_f(amax);
  if (lane == 0) red_max[w] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red_max[0], red_max[1]), fmaxf(red_max[2], red_max[3]));
  const float sc = amax / 127.0f;
  if (threadIdx.x == 0) a.scale[r] = sc;
  int8_t* qr = a.q + r * (int64_t)a.H;
#pragma unroll
  for (int i = 0; i < NORM_MAXV; ++i) {
    const int vi = threadIdx.x + i * 256;
    if (vi < nvec) {
      uint32_t w0 = 0, w1 = 0;
      if (sc > 0.0f) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          w0 |= ((uint32_t)(quant_i8(s[i][j], sc) & 0xff)) << (8 * j);
          w1 |= ((uint32_t)(quant_i8(s[i][4 + j], sc) & 0xff)) << (8 * j);
        }
      }
      v2i o = {(int)w0, (int)w1};
      *(v2i*)(qr + (size_t)vi * 8) = o;
    }
  }
}

}  // namespace

extern "C" int omni_add_rms_norm_quant(const void* x_bf16, const void* residual_bf16, const void* weight_bf16,
                                       int64_t rows, int H, float eps, void* residual_out_bf16, void* y_bf16,
                                       int8_t* q, float* scale, void* stream) {
  if (rows < 0 || H <= 0) OMNI_FAIL(OMNI_E_INVALID, "add_rms_norm_quant: bad shape rows=%lld H=%d", (long long)rows, H);
  if (rows == 0) return OMNI_OK;
  if (!x_bf16 || !weight_bf16) OMNI_FAIL(OMNI_E_INVALID, "add_rms_norm_quant: null pointer");
  if ((q == nullptr) != (scale == nullptr)) OMNI_FAIL(OMNI_E_INVALID, "add_rms_norm_quant: q and scale go together");
  if (!y_bf16 && !q && !residual_out_bf16) OMNI_FAIL(OMNI_E_INVALID, "add_rms_norm_quant: no output requested");
  if (residual_out_bf16 && !residual_bf16) OMNI_FAIL(OMNI_E_INVALID, "add_rms_norm_quant: residual_out without residual");
  if (H % 8 != 0 || H > 8 * 256 * NORM_MAXV) OMNI_FAIL(OMNI_E_UNSUPPORTED, "add_rms_norm_quant: H=%d must be a multiple of 8, at most %d", H, 8 * 256 * NORM_MAXV);
  if (rows > 0x7fffffffLL) OMNI_FAIL(OMNI_E_UNSUPPORTED, "add_rms_norm_quant: too many rows");
  if (((uintptr_t)x_bf16 % 16) || ((uintptr_t)residual_bf16 % 16) || ((uintptr_t)weight_bf16 % 16) ||
      ((uintptr_t)residual_out_bf16 % 16) || ((uintptr_t)y_bf16 % 16) || ((uintptr_t)q % 8))
    OMNI_FAIL(OMNI_E_INVALID, "add_rms_norm_quant: misaligned pointer");
  NormArgs a{(const uint16_t*)x_bf16, (const uint16_t*)residual_bf16, (const uint16_t*)weight_bf16, rows, H, eps,
             (uint16_t*)residual_out_bf16, (uint16_t*)y_bf16, q, scale};
  hipLaunchKernelGGL(add_rms_norm_quant_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, a);
  OMNI_CHECK_LAUNCH("add_rms_norm_quant");
  return OMNI_OK;
}
