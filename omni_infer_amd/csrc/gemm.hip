// Grouped int8 x int8 -> int32 GEMMs on the gfx950 int8 MFMAs with fused epilogues.
//
// Operand layouts
//   B (weights) is in the frag16 format: tiles of 16 output channels x 64 reduction elements,
//   1 KiB each, in exactly the order v_mfma_i32_16x16x64_i8 wants them in registers (lane l owns
//   bytes [16 l, 16 l + 16) of a tile).  A 16-channel strip is contiguous along k, so a wavefront
//   that walks k streams one contiguous region per strip with 16-byte loads.  Two neighbouring
//   strips hold the operands of v_mfma_i32_32x32x32_i8 as 256-byte runs.
//   A (int8 activations) is row major in memory.  It is staged through LDS in the same fragment
//   order: one wavefront load instruction fetches a 16 row x 64 byte fragment (lane l: row l%16,
//   bytes 16*(l/16)..+16) and stores it linearly, so LDS writes and the later ds_read_b128
//   fragment reads are both conflict free.  The gather by sorted slot (the permutation of the
//   MoE) happens in this load: no sorted copy of the activations is ever made.
//   C of a 16x16 tile: lane l holds rows 4*(l/16)..+4 of column l%16; of a 32x32 tile: column
//   l%32, rows 8*(i/4) + 4*(l/32) + i%4 for i = 0..15.
//
// Two kernels share the epilogue arithmetic:
//   gemm_stream  few rows per group (decode): weight streaming on the 16x16x64 MFMA.  Each
//                wavefront owns whole 16-channel strips of B and loads them straight from global
//                memory into MFMA registers through a ring of D outstanding k-steps (each weight
//                byte is used by exactly one wavefront, so LDS staging would only add traffic); A
//                is small and shared by the four wavefronts of a block through LDS.
//   gemm_pipe    many rows per group (prefill): 256 x 256 (or 256 x 128) block tiles, A and B both
//                loaded straight into LDS (global_load_lds) through a three-stage ring, each
//                wavefront a 128 x 64 sub-tile: on the 16x16x64 MFMA in the line layout (the default
//                wherever it applies), on the 32x32x32 MFMA in the fragment layout.
//
// GEMM1 pairs gate channel n with up channel I + n in the same lane so SwiGLU needs no exchange.
// Its epilogue writes y = silu(gate) * up in fp32 to a scratch matrix; a row kernel
// (quant_rows_y) then takes max|y| of each row and quantises it.  With several k shares or when
// the raw accumulators are asked for, gemm_stream stores int32 partial sums instead and
// swiglu_quant_rows finishes them.
#include "common.h"
#include <type_traits>

#include "gemm_stream.h"

namespace {

// =====================================================================================
// Row kernel after the split-k GEMM1: one 256-thread block per sorted row.  Adds the S partial
// accumulators (exact in int32), dequantises, applies SwiGLU, reduces max|y| over the row and
// quantises.  Each thread keeps its y values in registers between the two passes (PMAX pairs,
// I <= 256*PMAX); nothing but the int8 row and its scale is written.
// =====================================================================================
// NTH threads per row (a multiple of 64, at most 1024); a thread owns PMAX channel pairs
template <int PMAX, int NTH>
__global__ __launch_bounds__(NTH) void swiglu_quant_rows(GemmArgs a, int8_t* __restrict__ hq, float* __restrict__ hs) {
  __shared__ float red[NTH / WAVE];
  __shared__ int s_group, s_first;
  const int64_t m = blockIdx.x;  // < M_cap: the row's partial sums exist (unused rows hold anything)
  const int I = a.N / 2;
  // everything that does not depend on the row's group is requested first: the partial sums and
  // the row's source assignment; the group lookup (one thread per group) overlaps with them
  const size_t plane = (size_t)a.M_cap * a.N;
  const int32_t* prow = a.part + (size_t)m * a.N;
  int ag[PMAX], au[PMAX];
#pragma unroll
  for (int i = 0; i < PMAX; ++i) {
    const int n = threadIdx.x + i * NTH;
    ag[i] = 0;
    au[i] = 0;
    if (n < I) {
      for (int sp = 0; sp < a.S; ++sp) {
        ag[i] += prow[sp * plane + n];
        au[i] += prow[sp * plane + I + n];
      }
    }
  }
  int src = 0;
  if (a.sorted_src != nullptr && m < (int64_t)a.T * a.K) src = a.sorted_src[m];
  if (threadIdx.x == 0) s_group = -1;
  __syncthreads();
  for (int g = threadIdx.x; g <= a.G; g += NTH) {
    const int64_t lo = a.offsets[g];
    const int64_t hi = (g < a.G) ? (int64_t)a.offsets[g + 1] : lo + a.extra_rows;
    if (m >= lo && m < hi) {
      s_group = g;
      s_first = (int)lo;
    }
  }
  __syncthreads();
  if (s_group < 0) return;  // past the last row
  const int g = s_group;
  const float* wsc = (g < a.G) ? a.w_scale + (size_t)g * a.N : a.w_extra_scale;
  int token;  // row of the activation matrix this row came from (what source_row<1> computes)
  if (g >= a.G) token = (int)m - s_first;
  else if (a.sorted_src == nullptr) token = (int)m;
  else token = (a.idx_mode == OMNI_IDX_TOKEN_MAJOR) ? src / a.K : src % a.T;
  const float ts = a.a_scale[token];
  const bool bf = a.flags & OMNI_GEMM1_BF16_INTERMEDIATE;
  float y[PMAX];
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < PMAX; ++i) {
    const int n = threadIdx.x + i * NTH;
    y[i] = 0.0f;
    if (n < I) {
      if (a.acc_dbg) {
        a.acc_dbg[(size_t)m * a.N + n] = ag[i];
        a.acc_dbg[(size_t)m * a.N + I + n] = au[i];
      }
      float dg = ((float)ag[i] * wsc[n]) * ts;
      float du = ((float)au[i] * wsc[I + n]) * ts;
      if (bf) { dg = round_bf16(dg); du = round_bf16(du); }
      float yv = silu_spec(dg) * du;
      if (bf) yv = round_bf16(yv);
      if (a.smooth != nullptr && g < a.G) yv = yv * a.smooth[(size_t)g * I + n];
      y[i] = yv;
      amax = fmaxf(amax, fabsf(yv));
    }
  }
  amax = wave_allmax_f(amax);
  if ((threadIdx.x & (WAVE - 1)) == 0) red[threadIdx.x / WAVE] = amax;
  __syncthreads();
  amax = red[0];
#pragma unroll
  for (int i = 1; i < NTH / WAVE; ++i) amax = fmaxf(amax, red[i]);
  const float sc = amax / 127.0f;
  if (threadIdx.x == 0) hs[m] = sc;
  int8_t* qr = hq + (size_t)m * I;
#pragma unroll
  for (int i = 0; i < PMAX; ++i) {
    const int n = threadIdx.x + i * NTH;
    if (n < I) qr[n] = (sc > 0.0f) ? (int8_t)quant_i8(y[i], sc) : (int8_t)0;
  }
}

// =====================================================================================
// gemm_pipe: large row counts.  Block tile 256 rows x 128 channels (GEMM1: 64 gate + 64 up),
// four wavefronts as 2 (rows) x 2 (channels), each a 128 x 64 sub-tile held as 4 x 2 accumulator
// tiles of v_mfma_i32_32x32x32_i8 (a single wavefront issues the 32x32x32 form at nearly the
// full MFMA rate, the 16x16x64 form at about half of it; with the two wavefronts per SIMD of this
// kernel both forms issue at the full rate, and the line-layout loop further down uses 16x16x64).
//   Operands go from global memory straight into LDS (global_load_lds, 16 bytes per lane, no
//   register staging) through a three-stage ring: while stage s is multiplied, stages s+1 and s+2
//   are in flight.  A wavefront's load instruction moves one 1 KiB fragment of 16 rows (or 16
//   channels) x 64 k, lane l -> bytes [16 l, 16 l + 16).  The 32x32x32 operand of lane l (row
//   l%32, k-quarter 2*half + l/32 of the k-step) is then bytes
//       fragment[(l%32)/16][ (l%16) + 16*(2*half + l/32) ]
//   of two neighbouring fragments: groups of 16 lanes read 256 contiguous bytes.
//   The stage buffers are separate __shared__ objects and the step function takes them as
//   __restrict__ pointers: that is what lets the compiler see that the LDS reads of one stage do
//   not alias the asynchronous writes into another, so it keeps the explicit
//   "s_waitcnt vmcnt(loads of one stage)" and does not drain the ring before every LDS read.
// =====================================================================================
#define OMNI_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
typedef int v16i __attribute__((ext_vector_type(16)));

template <int WN>
struct PipeCtx {
  static constexpr int NWAVES = 2 * WN;          // 2 wavefronts along the rows x WN along the channels
  static constexpr int A_PER_WAVE = 16 / NWAVES; // A fragments (of 16) a wavefront loads per stage
  static constexpr int LPS = A_PER_WAVE + 2;     // loads per stage per wavefront (2 B fragments each)
  const int8_t* asrc[A_PER_WAVE];
  const int8_t* bsrc[2];
  int w, lane, wm, wn;
  int mt_count;  // 32-row tiles of this wavefront that hold rows of the block (0..4)
  int a_off;     // v4i index of this lane's A operand inside the wavefront's first 32-row pair, half 0
  int b_off[2];  // same for the two 32-channel tiles of the wavefront
};

template <int WN>
__device__ __forceinline__ void pipe_load(const PipeCtx<WN>& c, int k, v4i* __restrict__ dst_a, v4i* __restrict__ dst_b) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub
  constexpr int AP = PipeCtx<WN>::A_PER_WAVE;
#pragma unroll
  for (int i = 0; i < AP; ++i)
    __builtin_amdgcn_global_load_lds(c.asrc[i] + (size_t)k * 64, OMNI_LDS_PTR(dst_a + (AP * c.w + i) * WAVE), 16, 0, 0);
#pragma unroll
  for (int i = 0; i < 2; ++i)
    __builtin_amdgcn_global_load_lds(c.bsrc[i] + (size_t)k * 1024, OMNI_LDS_PTR(dst_b + (2 * c.w + i) * WAVE), 16, 0, 0);
#endif
}

// PARTIAL: the wavefront owns fewer than four 32-row tiles with rows in them (the last row block of a
// group): it reads and multiplies only those, and a wavefront without rows only takes part in the
// loads and the barriers.  Full wavefronts run the variant without any of the tests.
template <int WN, bool PARTIAL>
__device__ __forceinline__ void pipe_step(const PipeCtx<WN>& c, int kload, v4i* __restrict__ dst_a,
                                          v4i* __restrict__ dst_b, const v4i* __restrict__ src_a,
                                          const v4i* __restrict__ src_b, v16i (&acc)[4][2]) {
#if defined(__HIP_DEVICE_COMPILE__)
  pipe_load<WN>(c, kload, dst_a, dst_b);
  if (PARTIAL && c.mt_count == 0) return;
  // operands of both halves: the second half is requested before the first half's MFMAs are issued,
  // so its LDS latency hides behind them
  v4i bf[2][2], af[2][4];
#pragma unroll
  for (int t = 0; t < 2; ++t) bf[0][t] = src_b[c.b_off[t]];
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
    if (!PARTIAL || mt < c.mt_count) af[0][mt] = src_a[c.a_off + mt * 2 * WAVE];
#pragma unroll
  for (int t = 0; t < 2; ++t) bf[1][t] = src_b[c.b_off[t] + 32];
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
    if (!PARTIAL || mt < c.mt_count) af[1][mt] = src_a[c.a_off + mt * 2 * WAVE + 32];
#pragma unroll
  for (int half = 0; half < 2; ++half)
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
      if (!PARTIAL || mt < c.mt_count) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
          acc[mt][t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[half][mt], bf[half][t], acc[mt][t], 0, 0, 0);
      }
#endif
}

// wait until at most one stage of this wavefront's loads is still in flight, then meet the block
template <int WN>
__device__ __forceinline__ void pipe_sync() {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int N = PipeCtx<WN>::LPS;
  __builtin_amdgcn_s_waitcnt((N & 0xF) | (0x7 << 4) | (0xF << 8));  // vmcnt(N), other counters untouched
  __builtin_amdgcn_s_barrier();
#endif
}

// the k loop of one tile: a ring of three stages, two k-steps in flight while one is multiplied; the first
// two k-steps are already on their way into stages 0 and 1
template <int WN, bool PARTIAL>
__device__ __forceinline__ void pipe_k_loop(const PipeCtx<WN>& c, int nk64, v4i* __restrict__ sa0, v4i* __restrict__ sa1,
                                            v4i* __restrict__ sa2, v4i* __restrict__ sb0, v4i* __restrict__ sb1,
                                            v4i* __restrict__ sb2, v16i (&acc)[4][2]) {
  const int last = nk64 - 1;
  int ks = 0;
  for (; ks + 3 <= nk64; ks += 3) {
    pipe_sync<WN>();
    pipe_step<WN, PARTIAL>(c, min(ks + 2, last), sa2, sb2, sa0, sb0, acc);
    pipe_sync<WN>();
    pipe_step<WN, PARTIAL>(c, min(ks + 3, last), sa0, sb0, sa1, sb1, acc);
    pipe_sync<WN>();
    pipe_step<WN, PARTIAL>(c, min(ks + 4, last), sa1, sb1, sa2, sb2, acc);
  }
  if (ks < nk64) {  // one or two k-steps left; the ring is back at stage 0
    pipe_sync<WN>();
    pipe_step<WN, PARTIAL>(c, last, sa2, sb2, sa0, sb0, acc);
    if (ks + 1 < nk64) {
      pipe_sync<WN>();
      pipe_step<WN, PARTIAL>(c, last, sa0, sb0, sa1, sb1, acc);
    }
  }
}

// =====================================================================================
// Line layout of the activation operand (256 x 256 tiles, reduction length a multiple of 128).
//   What bounds the tile kernel is the vector memory path of the CU (address unit and L1 busy all the time,
//   the address unit held up by the L1 half of it), and a 16 row x 64 byte fragment is sixteen half cache
//   lines: every line of an activation row was asked for twice, one k-step apart.  Here a load instruction
//   fetches 8 rows x 128 bytes (whole lines; lane l: row l/8, one 16-byte piece) and an A stage holds two
//   k-steps ("super-step"): 256 rows x 128 bytes = 32 KiB, three of them, next to the three 16 KiB B stages.
//   global_load_lds stores a wavefront's 64 pieces linearly, so the bank swizzle is applied on the global
//   side: slot q of row r holds piece q ^ f(r), f(r) = (r >> 1) & 7.  The 16 lanes of a quarter wavefront
//   read one piece number of 16 consecutive rows: addresses 128 r + 16 (p ^ f(r)), which fall into 16
//   different 16-byte bank groups.
//   The instruction order of every half k-step is pinned: operands are read from LDS half a k-step before they
//   are multiplied, into the registers the half step before has just released, and the reads and the loads
//   that refill the ring are issued in the shadow of the running MFMAs.  The block barrier of a k-step sits
//   between its halves.  sched_group_barrier masks: 0x008 MFMA, 0x020 vector memory read, 0x100 LDS read.
// =====================================================================================
struct LineCtx {
  const int8_t* asrc[2][2];  // [k-step parity][i]: this lane's piece of its row, super-step 0
  const int8_t* bsrc[2];
  int w, lane;
  int a_off[2][2];  // [k-step parity][half]: v4i index of the lane's A operand in a super-stage, row tile 0
  int b_off[2];     // same for the two 32-channel tiles of the wavefront, half 0
  // the 16x16x64 form: [k-step parity][upper 16 rows of the 32-row tile] and the four strips of the wavefront
  int a16_off[2][2];
  int b16_off[4];
};
[[maybe_unused]] constexpr int LINE_LPS = 4;  // loads per k-step per wavefront: 2 A instructions (8 rows each), 2 B fragments

// the A loads of parity E fill rows [128 E, 128 E + 128) of a super-stage
template <int E>
__device__ __forceinline__ void line_load_a(const LineCtx& c, int ss, v4i* __restrict__ dst_a) {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
  for (int i = 0; i < 2; ++i)
    __builtin_amdgcn_global_load_lds(c.asrc[E][i] + (size_t)ss * 128, OMNI_LDS_PTR(dst_a + (E * 16 + 2 * c.w + i) * WAVE), 16, 0, 0);
#endif
}
__device__ __forceinline__ void line_load_b(const LineCtx& c, int k, v4i* __restrict__ dst_b) {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
  for (int i = 0; i < 2; ++i)
    __builtin_amdgcn_global_load_lds(c.bsrc[i] + (size_t)k * 1024, OMNI_LDS_PTR(dst_b + (2 * c.w + i) * WAVE), 16, 0, 0);
#endif
}

// operands of one half k-step of a wavefront that multiplies MTC row tiles of 32
template <int MTC>
struct LineOps { v4i a[MTC > 0 ? MTC : 1]; v4i b[2]; };

template <int MTC, int E, int HALF>
__device__ __forceinline__ void line_read(const LineCtx& c, const v4i* __restrict__ src_a, const v4i* __restrict__ src_b,
                                          LineOps<MTC>& o) {
#pragma unroll
  for (int t = 0; t < 2; ++t) o.b[t] = src_b[c.b_off[t] + 32 * HALF];
#pragma unroll
  for (int mt = 0; mt < MTC; ++mt) o.a[mt] = src_a[c.a_off[E][HALF] + mt * 256];
}

template <int MTC>
__device__ __forceinline__ void line_mfma(const LineOps<MTC>& o, v16i (&acc)[4][2]) {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
  for (int mt = 0; mt < MTC; ++mt)
#pragma unroll
    for (int t = 0; t < 2; ++t) acc[mt][t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.a[mt], o.b[t], acc[mt][t], 0, 0, 0);
#endif
}

// pins the order of what is left of a half step: LDS reads two at a time, then the loads one at a time, each
// group followed by one MFMA while there are MFMAs left, then the remaining MFMAs
template <int D, int M, int V>
__device__ __forceinline__ void line_pin() {
#if defined(__HIP_DEVICE_COMPILE__)
  if constexpr (D > 0) {
    constexpr int n = D >= 2 ? 2 : 1;
    __builtin_amdgcn_sched_group_barrier(0x100, n, 0);
    if constexpr (M > 0) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    line_pin<D - n, (M > 0 ? M - 1 : 0), V>();
  } else if constexpr (V > 0) {
    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    if constexpr (M > 0) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    line_pin<0, (M > 0 ? M - 1 : 0), V - 1>();
  } else if constexpr (M > 0) {
    __builtin_amdgcn_sched_group_barrier(0x008, M, 0);
  }
#endif
}

// One k-step of parity E.  X holds the first-half operands of this k-step on entry and those of the next one
// on exit.  After the barrier the B stage just read is refilled with k-step kb and this wavefront's share of
// rows [128 E, 128 E + 128) of super-step ssa goes into `fill_a` (the super-stage read two super-steps ago).
template <int MTC, int E>
__device__ __forceinline__ void line_step(const LineCtx& c, int kb, int ssa, const v4i* __restrict__ cur_a,
                                          v4i* __restrict__ cur_b, v4i* __restrict__ fill_a, const v4i* __restrict__ nxt_a,
                                          const v4i* __restrict__ nxt_b, LineOps<MTC>& X, LineOps<MTC>& Y, v16i (&acc)[4][2]) {
#if defined(__HIP_DEVICE_COMPILE__)
  if constexpr (MTC > 0) {
    line_read<MTC, E, 1>(c, cur_a, cur_b, Y);
    line_mfma<MTC>(X, acc);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    line_pin<2 + MTC, 2 * MTC - 1, 0>();
    __builtin_amdgcn_sched_barrier(0);
  }
  // the next stage has landed (at most this wavefront's last k-step of loads is still in flight) and the
  // wavefront has received everything it reads from the current one
  __builtin_amdgcn_s_waitcnt((LINE_LPS & 0xF) | (0x7 << 4) | (0x0 << 8));
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  line_load_b(c, kb, cur_b);
  line_load_a<E>(c, ssa, fill_a);
  if constexpr (MTC > 0) {
    line_read<MTC, 1 - E, 0>(c, nxt_a, nxt_b, X);
    line_mfma<MTC>(Y, acc);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    line_pin<2 + MTC, 2 * MTC - 1, LINE_LPS>();
  }
  __builtin_amdgcn_sched_barrier(0);
#endif
}

// the k loop: nk64 (even) k-steps; on entry super-steps 0 and 1 and k-steps 0 and 1 of B are on their way
template <int MTC>
__device__ __forceinline__ void line_k_loop(const LineCtx& c, int nk64, v4i* __restrict__ sa0, v4i* __restrict__ sa1,
                                            v4i* __restrict__ sa2, v4i* __restrict__ sb0, v4i* __restrict__ sb1,
                                            v4i* __restrict__ sb2, v16i (&acc)[4][2]) {
#if defined(__HIP_DEVICE_COMPILE__)
  const int last = nk64 - 1, last_ss = nk64 / 2 - 1;
  LineOps<MTC> X, Y;
  // super-step 0 and k-step 0 of B have landed: all loads but the last 6 (k-step 1 of B, super-step 1)
  __builtin_amdgcn_s_waitcnt((6 & 0xF) | (0x7 << 4) | (0xF << 8));
  __builtin_amdgcn_s_barrier();
  line_load_b(c, min(2, last), sb2);
  if constexpr (MTC > 0) line_read<MTC, 0, 0>(c, sa0, sb0, X);
  __builtin_amdgcn_sched_barrier(0);
  int k = 0;
  for (; k + 6 <= nk64; k += 6) {
    const int ss = k >> 1;
    line_step<MTC, 0>(c, min(k + 3, last), min(ss + 2, last_ss), sa0, sb0, sa2, sa0, sb1, X, Y, acc);
    line_step<MTC, 1>(c, min(k + 4, last), min(ss + 2, last_ss), sa0, sb1, sa2, sa1, sb2, X, Y, acc);
    line_step<MTC, 0>(c, min(k + 5, last), min(ss + 3, last_ss), sa1, sb2, sa0, sa1, sb0, X, Y, acc);
    line_step<MTC, 1>(c, min(k + 6, last), min(ss + 3, last_ss), sa1, sb0, sa0, sa2, sb1, X, Y, acc);
    line_step<MTC, 0>(c, min(k + 7, last), min(ss + 4, last_ss), sa2, sb1, sa1, sa2, sb2, X, Y, acc);
    line_step<MTC, 1>(c, min(k + 8, last), min(ss + 4, last_ss), sa2, sb2, sa1, sa0, sb0, X, Y, acc);
  }
  if (k < nk64) {  // two or four k-steps left; the rings are back at their first stages
    line_step<MTC, 0>(c, last, last_ss, sa0, sb0, sa2, sa0, sb1, X, Y, acc);
    line_step<MTC, 1>(c, last, last_ss, sa0, sb1, sa2, sa1, sb2, X, Y, acc);
    if (k + 2 < nk64) {
      line_step<MTC, 0>(c, last, last_ss, sa1, sb2, sa0, sa1, sb0, X, Y, acc);
      line_step<MTC, 1>(c, last, last_ss, sa1, sb0, sa0, sa2, sb1, X, Y, acc);
    }
  }
#endif
}

// =====================================================================================
// The same loop on v_mfma_i32_16x16x64_i8.  The chip lowers its clock with the switching activity of the matrix
// datapath, and an instruction that folds 64 products into each of 256 accumulators switches less per product than
// one that folds 32 into each of 1024: on the operand pattern of this kernel the 16x16x64 form sustains 4.1-4.3
// POPS where the 32x32x32 form sustains 3.1-3.2.  The wavefront's piece, its 128 accumulator registers and the
// bytes it reads from LDS are the same.  An instruction takes a whole k-step of 16 rows and 16 channels, so a
// half step is now the lower or the upper 16 rows of every 32-row tile against all four strips of the wavefront:
// the A operands of the two halves alternate between X and Y as before, the four B operands serve both halves
// and are replaced one by one, each after the last instruction of the k-step that uses it.
// Accumulators: acc[mt][t] (16 registers) holds four 16 x 16 results: registers 8 h + 4 s + i belong to rows
// 16 h + 4 (lane / 16) + i of the tile and channel 16 s + lane % 16 of the pair of strips t.
// =====================================================================================
template <int MTC>
struct Line16A { v4i a[MTC > 0 ? MTC : 1]; };

template <int MTC, int E, int H>
__device__ __forceinline__ void line16_read_a(const LineCtx& c, const v4i* __restrict__ src_a, Line16A<MTC>& o) {
#pragma unroll
  for (int mt = 0; mt < MTC; ++mt) o.a[mt] = src_a[c.a16_off[E][H] + mt * 256];
}

// the instructions of half H that use strip N of the wavefront
template <int MTC, int H, int N>
__device__ __forceinline__ void line16_mfma_n(const Line16A<MTC>& o, const v4i (&b)[4], v4i (&acc)[4][2][4]) {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
  for (int mt = 0; mt < MTC; ++mt)
    acc[mt][N >> 1][2 * H + (N & 1)] = __builtin_amdgcn_mfma_i32_16x16x64_i8(o.a[mt], b[N], acc[mt][N >> 1][2 * H + (N & 1)], 0, 0, 0);
#endif
}

// after the first MFMA: every LDS read, then every load, followed by one MFMA each while there are MFMAs left
template <int D, int M, int V>
__device__ __forceinline__ void line16_pin() {
#if defined(__HIP_DEVICE_COMPILE__)
  if constexpr (D > 0) {
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    if constexpr (M > 0) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    line16_pin<D - 1, (M > 0 ? M - 1 : 0), V>();
  } else if constexpr (V > 0) {
    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    if constexpr (M > 0) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    line16_pin<0, (M > 0 ? M - 1 : 0), V - 1>();
  } else if constexpr (M > 0) {
    __builtin_amdgcn_sched_group_barrier(0x008, M, 0);
  }
#endif
}

// One k-step of parity E.  X holds the lower-half A operands and B the strips of this k-step on entry, those of
// the next k-step on exit.  Stage roles as in line_step.
template <int MTC, int E>
__device__ __forceinline__ void line16_step(const LineCtx& c, int kb, int ssa, const v4i* __restrict__ cur_a,
                                            v4i* __restrict__ cur_b, v4i* __restrict__ fill_a, const v4i* __restrict__ nxt_a,
                                            const v4i* __restrict__ nxt_b, Line16A<MTC>& X, Line16A<MTC>& Y, v4i (&B)[4],
                                            v4i (&acc)[4][2][4]) {
#if defined(__HIP_DEVICE_COMPILE__)
  // The instructions of a strip stay together (scheduling fences between the strips).  The compiler waits for all
  // LDS reads at once, so no read may be issued shortly before a wait: strips 0 and 1 of the next k-step are read
  // in the second half of this one, each after its last use here and two strips before the half ends; strips 2
  // and 3 are read at the head of the first half of their own k-step, two strips before they are needed.
  if constexpr (MTC > 0) {
    B[2] = cur_b[c.b16_off[2]];
    B[3] = cur_b[c.b16_off[3]];
    line16_read_a<MTC, E, 1>(c, cur_a, Y);
    line16_mfma_n<MTC, 0, 0>(X, B, acc);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    line_pin<2 + MTC, MTC - 1, 0>();   // the reads two at a time behind the first instructions
    __builtin_amdgcn_sched_barrier(0);
    line16_mfma_n<MTC, 0, 1>(X, B, acc);
    __builtin_amdgcn_sched_barrier(0);
    line16_mfma_n<MTC, 0, 2>(X, B, acc);
    __builtin_amdgcn_sched_barrier(0);
    line16_mfma_n<MTC, 0, 3>(X, B, acc);
    __builtin_amdgcn_sched_barrier(0);
  }
  __builtin_amdgcn_s_waitcnt((LINE_LPS & 0xF) | (0x7 << 4) | (0x0 << 8));
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (MTC > 0) {
    line16_read_a<MTC, 1 - E, 0>(c, nxt_a, X);
    line16_mfma_n<MTC, 1, 0>(Y, B, acc);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    line16_pin<MTC, MTC - 1, 0>();
    __builtin_amdgcn_sched_barrier(0);
  }
  line_load_b(c, kb, cur_b);
  line_load_a<E>(c, ssa, fill_a);
  if constexpr (MTC > 0) {
    B[0] = nxt_b[c.b16_off[0]];
    line16_mfma_n<MTC, 1, 1>(Y, B, acc);
    line16_pin<0, MTC, LINE_LPS>();
    __builtin_amdgcn_sched_barrier(0);
    B[1] = nxt_b[c.b16_off[1]];
    line16_mfma_n<MTC, 1, 2>(Y, B, acc);
    __builtin_amdgcn_sched_barrier(0);
    line16_mfma_n<MTC, 1, 3>(Y, B, acc);
  }
  __builtin_amdgcn_sched_barrier(0);
#endif
}

template <int MTC>
__device__ __forceinline__ void line16_k_loop(const LineCtx& c, int nk64, v4i* __restrict__ sa0, v4i* __restrict__ sa1,
                                              v4i* __restrict__ sa2, v4i* __restrict__ sb0, v4i* __restrict__ sb1,
                                              v4i* __restrict__ sb2, v4i (&acc)[4][2][4]) {
#if defined(__HIP_DEVICE_COMPILE__)
  const int last = nk64 - 1, last_ss = nk64 / 2 - 1;
  Line16A<MTC> X, Y;
  v4i B[4];
  __builtin_amdgcn_s_waitcnt((6 & 0xF) | (0x7 << 4) | (0xF << 8));
  __builtin_amdgcn_s_barrier();
  line_load_b(c, min(2, last), sb2);
  if constexpr (MTC > 0) {
    line16_read_a<MTC, 0, 0>(c, sa0, X);
    B[0] = sb0[c.b16_off[0]];
    B[1] = sb0[c.b16_off[1]];
  }
  __builtin_amdgcn_sched_barrier(0);
  int k = 0;
  for (; k + 6 <= nk64; k += 6) {
    const int ss = k >> 1;
    line16_step<MTC, 0>(c, min(k + 3, last), min(ss + 2, last_ss), sa0, sb0, sa2, sa0, sb1, X, Y, B, acc);
    line16_step<MTC, 1>(c, min(k + 4, last), min(ss + 2, last_ss), sa0, sb1, sa2, sa1, sb2, X, Y, B, acc);
    line16_step<MTC, 0>(c, min(k + 5, last), min(ss + 3, last_ss), sa1, sb2, sa0, sa1, sb0, X, Y, B, acc);
    line16_step<MTC, 1>(c, min(k + 6, last), min(ss + 3, last_ss), sa1, sb0, sa0, sa2, sb1, X, Y, B, acc);
    line16_step<MTC, 0>(c, min(k + 7, last), min(ss + 4, last_ss), sa2, sb1, sa1, sa2, sb2, X, Y, B, acc);
    line16_step<MTC, 1>(c, min(k + 8, last), min(ss + 4, last_ss), sa2, sb2, sa1, sa0, sb0, X, Y, B, acc);
  }
  if (k < nk64) {
    line16_step<MTC, 0>(c, last, last_ss, sa0, sb0, sa2, sa0, sb1, X, Y, B, acc);
    line16_step<MTC, 1>(c, last, last_ss, sa0, sb1, sa2, sa1, sb2, X, Y, B, acc);
    if (k + 2 < nk64) {
      line16_step<MTC, 0>(c, last, last_ss, sa1, sb2, sa0, sa1, sb0, X, Y, B, acc);
      line16_step<MTC, 1>(c, last, last_ss, sa1, sb0, sa0, sa2, sb1, X, Y, B, acc);
    }
  }
#endif
}

// From the accumulator layout of the 16x16x64 loop to that of the 32x32x32 loop, in place: registers 8 h + i and
// 8 h + 4 + i of a 32 x 32 tile (the two strips of a pair, same rows) exchange 16-lane rows.  After the two swaps
// lane l holds channel l % 32 and rows 8 (r / 4) + 4 (l / 32) + r % 4 in register r, which is what the epilogues
// and the split-tile hand-over are written for.
__device__ __forceinline__ void acc16_to_acc32(const v4i (&a16)[4][2][4], v16i (&acc)[4][2]) {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const auto p = __builtin_amdgcn_permlane16_swap((unsigned)a16[mt][t][2 * h][i], (unsigned)a16[mt][t][2 * h + 1][i], false, false);
          const auto q = __builtin_amdgcn_permlane32_swap(p[0], p[1], false, false);
          acc[mt][t][8 * h + i] = (int)q[0];
          acc[mt][t][8 * h + 4 + i] = (int)q[1];
        }
#endif
}

// 32x32 accumulator tile: lane l holds column l%32, rows 8*(i/4) + 4*(l/32) + i%4 for i = 0..15
__device__ __forceinline__ int tile32_row(int lane, int i) { return 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3); }

// Epilogue of one 256 x (64*WN) tile, shared by the tile kernels: a wavefront holds a 128 x 64 piece as
// 4 x 2 accumulator tiles of 32 x 32.  GEMM1: dequantise, SwiGLU, y (fp32) with streaming stores.
// GEMM2: fp32 rows, or bf16 rows transposed through LDS (stage32: a private 32 x 64 piece per
// wavefront, rows padded to 192 bytes = 48 dwords, so that the two rows a half-wavefront writes at
// once fall into disjoint banks) and stored as whole 128-byte lines.
constexpr int TILE_OUT_PITCH_DW = 48;
#define TILE_STAGE_DWORDS (32 * TILE_OUT_PITCH_DW)  // staging dwords of one wavefront
template <int KIND, int WN, bool BF>
__device__ __forceinline__ void tile_epilogue(const GemmArgs& a, v16i (&acc)[4][2], const float* row_scale,
                                              uint32_t* stage32, int lane, int wave_row0, int mt_count, int wn, int bx,
                                              int row0, int nrows, const float* __restrict__ wsc, int I,
                                              int bf16_shift, const float* __restrict__ smooth_g) {
  constexpr int NBS = 4 * WN;
  constexpr int GS = 2 * WN;
  // ---- epilogue, one 32-row tile at a time
  const int c32 = lane & 31;
  constexpr int OUT_PITCH_DW = TILE_OUT_PITCH_DW;
  // bf16_shift >= 0: bf16 rows of the extra group inside an fp32 row buffer (GemmArgs::extra_rows_bf16)
  const bool bf16_out = (KIND == 2) && (a.out_dtype == OMNI_DT_BF16 || bf16_shift >= 0);
  const int out_row0 = row0 + (bf16_shift >= 0 ? bf16_shift : 0);  // first row of the block in bf16 rows
  constexpr bool bf = BF;
  float wsc_g[2];
  int ncol[2];
  if constexpr (KIND == 1) {
    ncol[0] = (bx * GS + 2 * wn) * 16 + c32;
    ncol[1] = I + ncol[0];
  } else {
    ncol[0] = (bx * NBS + 4 * wn) * 16 + c32;
    ncol[1] = ncol[0] + 32;
  }
  wsc_g[0] = wsc[ncol[0]];
  wsc_g[1] = wsc[ncol[1]];
  // GEMM1: the smoothing factor of the lane's channel (the group's row of GemmArgs::smooth), 1 without
  float sm_g = 1.0f;
  if constexpr (KIND == 1) {
    if (smooth_g != nullptr) sm_g = smooth_g[ncol[0]];
  }
  if (bf16_out) {
    if constexpr (KIND == 2) {
      const int odd = c32 & 1;
      // byte selector of v_perm_b32 over {theirs (bytes 4-7), mine (bytes 0-3)}: even lanes keep
      // their low half and take the neighbour's low half on top, odd lanes take the neighbour's
      // high half below their own high half
      const uint32_t sel = odd ? 0x03020706u : 0x05040100u;
      uint32_t* const stage_lane = stage32 + (4 * (lane >> 5) + odd) * OUT_PITCH_DW + (c32 >> 1);
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) {
        const int tile_r0 = wave_row0 + mt * 32;
        if (mt < mt_count) {
          // accumulator entries i, i+1 (i even) are rows r, r+1 of the same channel; neighbouring
          // lanes hold neighbouring channels.  One pack, one lane exchange and one byte permute give
          // every lane a dword of two neighbouring channels: even lanes for row r, odd lanes for row r+1.
          const float* ts_lane = row_scale + tile_r0 + 4 * (lane >> 5);
#pragma unroll
          for (int i = 0; i < 16; i += 2) {
            const int rr = 8 * (i >> 2) + (i & 3);  // row below the lane's first row of the tile
            const float ts0 = ts_lane[rr], ts1 = ts_lane[rr + 1];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
              const float o0 = ((float)acc[mt][t][i] * wsc_g[t]) * ts0;
              const float o1 = ((float)acc[mt][t][i + 1] * wsc_g[t]) * ts1;
              const uint32_t mine = f32x2_to_bf16x2(o0, o1);
              const uint32_t theirs = (uint32_t)xchg_i<1>((int)mine);
              stage_lane[rr * OUT_PITCH_DW + t * 16] = __builtin_amdgcn_perm(theirs, mine, sel);
            }
          }
          // the wavefront wrote its 32 x 64 piece; now 8 lanes per row store 16 bytes each
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int r = j * 8 + (lane >> 3);
            const int rr = tile_r0 + r;
            v4i v = *(const v4i*)(stage32 + r * OUT_PITCH_DW + (lane & 7) * 4);
            if (rr < nrows)  // read once, by the combine
              __builtin_nontemporal_store(v, (v4i*)((uint16_t*)a.rows_out + (size_t)(out_row0 + rr) * a.N + (ncol[0] - c32) + (lane & 7) * 8));
          }
          __builtin_amdgcn_wave_barrier();
        }
      }
    }
  } else {
    // one 32-row tile: FULL (all 32 rows exist, the common case) carries no per-row test, so the 16
    // entries of a lane form one straight run of independent arithmetic chains
    auto rows32 = [&](int mt, int tile_r0, auto full) {
      constexpr bool FULL = decltype(full)::value;
      // the lane's 16 rows are 4 runs of 4 consecutive rows: their scales come as 4 vector reads
      const v4f* ts4 = (const v4f*)(row_scale + tile_r0 + 4 * (lane >> 5));
      v4f ts[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) ts[q] = ts4[2 * q];
      const int lane_r0 = tile_r0 + 4 * (lane >> 5);  // the lane's first row of this tile
      float* ytile = nullptr;    // GEMM1: y element of the lane's first row
      float* otile = nullptr;    // GEMM2: fp32 output row element of the lane's first row, first tile
      if constexpr (KIND == 1) ytile = a.y + (size_t)(row0 + lane_r0) * I + ncol[0];
      else otile = (float*)a.rows_out + (size_t)(row0 + lane_r0) * (size_t)a.N + ncol[0];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int below = 8 * (i >> 2) + (i & 3);  // entry i is this many rows below the lane's first row
        if (FULL || lane_r0 + below < nrows) {
          const float tsv = ts[i >> 2][i & 3];
          if constexpr (KIND == 1) {
            float dg = ((float)acc[mt][0][i] * wsc_g[0]) * tsv;
            float du = ((float)acc[mt][1][i] * wsc_g[1]) * tsv;
            if (bf) { dg = round_bf16(dg); du = round_bf16(du); }
            float yv = silu_spec(dg) * du;
            if (bf) yv = round_bf16(yv);
            if (smooth_g != nullptr) yv = yv * sm_g;
            __builtin_nontemporal_store(yv, ytile + (size_t)below * I);  // read once, by the row quantiser
          } else {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
              float o = ((float)acc[mt][t][i] * wsc_g[t]) * tsv;
              __builtin_nontemporal_store(o, otile + (size_t)below * (size_t)a.N + 32 * t);
            }
          }
        }
      }
    };
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
      const int tile_r0 = wave_row0 + mt * 32;
      if (mt >= mt_count) continue;
      if (tile_r0 + 32 <= nrows) rows32(mt, tile_r0, std::true_type{});
      else rows32(mt, tile_r0, std::false_type{});
    }
  }
  // raw accumulators for the parity tests, kept out of the loops above so that none of their
  // address arithmetic is ever part of them
  if (a.acc_dbg) {
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int rr = wave_row0 + mt * 32 + tile32_row(lane, i);
        if (mt < mt_count && rr < nrows) {
#pragma unroll
          for (int t = 0; t < 2; ++t) a.acc_dbg[(size_t)(row0 + rr) * (size_t)a.N + ncol[t]] = acc[mt][t][i];
        }
      }
  }
}

// ---- which tile a block id names: omni_host::tile_count / tile_select (host_logic.h)
using omni_host::TileCount;
using omni_host::TileGeom;
using omni_host::TileSel;
using omni_host::TILE_LIGHT_MAX;

// Hand-over between the shares of a split tile (their blocks may run on different XCDs, each with its own
// L2).  Every wavefront stores its partial sums, all wavefronts meet at the block barrier, then one
// thread counts in with a device-scope acquire-release add: the release half makes every store
// that happened before it (the barrier orders the other wavefronts' stores before it) visible to
// the device before the counter moves, and whoever reads the final count has, through the acquire
// half and the chain of adds on the same counter, all other shares' stores visible to its block
// after the second barrier.  No share ever waits for another.  True for the share that arrived last: its
// accumulators then hold the sums of all shares.
template <int WN>
__device__ __forceinline__ bool tile_tail_handover(const GemmArgs& a, v16i (&acc)[4][2], int mt_count, int tail_tile,
                                                   int split, int share, int w, int lane, int* s_last) {
  constexpr int WAVE_INTS = 8 * 16 * WAVE;           // accumulator words of one wavefront
  constexpr int TILE_INTS = 2 * WN * WAVE_INTS;
  int32_t* mine = a.tail_part + ((size_t)tail_tile * split + share) * TILE_INTS + (size_t)w * WAVE_INTS + lane;
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
    if (mt < mt_count) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) mine[((mt * 2 + t) * 16 + i) * WAVE] = acc[mt][t][i];
    }
  __builtin_amdgcn_s_waitcnt(0);  // this wavefront's stores are acknowledged before it meets the block
  __syncthreads();
  if (threadIdx.x == 0)
    *s_last = (__hip_atomic_fetch_add(a.tail_cnt + tail_tile, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == split - 1);
  __syncthreads();
  if (!*s_last) return false;
  for (int s2 = 0; s2 < split; ++s2) {
    if (s2 == share) continue;
    const int32_t* theirs = a.tail_part + ((size_t)tail_tile * split + s2) * TILE_INTS + (size_t)w * WAVE_INTS + lane;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
      if (mt < mt_count) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[mt][t][i] += theirs[((mt * 2 + t) * 16 + i) * WAVE];
      }
  }
  return true;
}

// WN = 2: 256 threads, tile 256 x 128, two blocks per CU.  WN = 4: 512 threads, tile 256 x 256, one block
// per CU (a third fewer operand bytes through the vector memory path per MFMA).
// BF (GEMM1 only): round gate, up and their product to bf16 (the numerics of the reference's
// unfused bf16 path); a template parameter so that the fp32 path carries none of that arithmetic.
// LINES (WN = 4, reduction length a multiple of 128): the line layout of the activation operand and the
// pinned k loop above; otherwise fragments of 16 rows x 64 bytes and the loop the compiler schedules.
template <int KIND, int WN, bool BF, bool LINES, bool M16 = false>
__global__ __launch_bounds__(128 * WN, 2) void gemm_pipe(GemmArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub
  constexpr int BM = 256;
  constexpr int NBS = 4 * WN;             // B strips per stage
  constexpr int GS = 2 * WN;              // KIND 1: gate strips per block
  constexpr int AP = PipeCtx<WN>::A_PER_WAVE;
  static_assert(!LINES || WN == 4, "the line layout is written for the 256 x 256 tile");
  constexpr int A_STAGE = LINES ? 32 * WAVE : 16 * WAVE;  // v4i per A stage: 256 rows x 128 or x 64 bytes
  __shared__ v4i sa0[A_STAGE], sa1[A_STAGE], sa2[A_STAGE];
  __shared__ v4i sb0[NBS * WAVE], sb1[NBS * WAVE], sb2[NBS * WAVE];
  __shared__ __attribute__((aligned(16))) float row_scale[BM];  // activation scale of every row of the block

  PipeCtx<WN> c;
  c.lane = threadIdx.x & (WAVE - 1);
  c.w = threadIdx.x / WAVE;
  c.wm = c.w / WN;
  c.wn = c.w % WN;
  const int lane = c.lane, w = c.w, wm = c.wm, wn = c.wn;
  // ---- which tile, and which share of its reduction
  // A block's time is set by the wavefronts of its first 128 rows, so a row block costs the same from 97
  // rows on ("heavy"); only the last blocks of groups with at most 96 rows left are cheaper ("light").
  // Real tiles (row blocks that exist x column tiles) get the ids [0, n_real): first the tiles of the heavy
  // row blocks, then those of the light ones, each set in three runs:
  //   A: whole patches of TILE_PR row blocks x tile_pc column tiles, in rounds of 8 dealt to the 8 XCDs
  //      (workgroups go to the XCDs, each with its own L2 and its own dispatcher, round-robin by their
  //      linear id, so the tiles an XCD runs together share their row panels and, inside an expert,
  //      their weight panels in that L2);
  //   B: the whole patches that do not fill a round of 8, one after the other;
  //   C: the row blocks past the last whole patch row, row by row.
  // Every XCD works through its own ids in order and nothing moves work between XCDs, so the heavy tiles,
  // which all cost the same, are dealt out evenly by count and the cheap tiles fill in at the end (with
  // light blocks scattered among the heavy ones the XCDs finished 8 % apart at 8192 tokens).
  // With n_real tiles on `tile_slots` block slots the last n_real % tile_slots tiles would run alone
  // on a nearly idle chip.  When they are at most half a round, each of them is split S ways along the
  // reduction: the tile's own block takes the first share, helper blocks with ids past n_real the
  // others.  Every share stores its int32 partial accumulators; whoever arrives last at the tile's
  // counter adds the others' to its own (integer sums: the order cannot matter) and runs the
  // epilogue.  Nobody waits for anybody.
  constexpr int LIGHT_MAX = TILE_LIGHT_MAX;
  const RowBlockKinds scan = row_block_kinds_scan(a.offsets, a.G, a.extra_rows, BM, LIGHT_MAX);
  const int nk_all = a.Kdim / 64;
  const TileGeom geom{a.tile_gx, a.tile_pc, a.tile_slots, a.tile_split_max, a.tail_part != nullptr};
  const TileCount tc = omni_host::tile_count(geom, scan.total_h, scan.total_l, LINES ? nk_all / 2 : nk_all);
  TileSel sel;
  if (!omni_host::tile_select(geom, tc, scan.total_h, scan.total_l, (int)blockIdx.x, sel)) return;
  const int bx = sel.bx, by = sel.by, split = tc.split, share = sel.share, tail_tile = sel.tail_tile;
  const bool light = sel.light;
  RowBlock rb;
  row_block_kinds_find(scan, a.offsets, a.G, a.extra_rows, BM, LIGHT_MAX, light, by, rb);
  // this block's k-steps [k_first, k_first + nk64)
  // (shares of the line layout begin and end on whole super-steps of 128)
  constexpr int KU = LINES ? 2 : 1;
  int k_first = 0, k_end = nk_all;
  if (tail_tile >= 0) omni_host::tile_share_k_range(nk_all, KU, split, share, k_first, k_end);
  const int g = rb.group, row0 = rb.row0, nrows = rb.nrows;
  const int nk64 = k_end - k_first;
  const int I = (KIND == 1) ? a.N / 2 : 0;
  const int8_t* wbase = (g < a.G) ? a.w + (size_t)g * a.Kdim * a.N : a.w_extra;
  const float* wsc = (g < a.G) ? a.w_scale + (size_t)g * a.N : a.w_extra_scale;

  // block-level strips j = 0..NBS-1: KIND 1: gate strips GS*bx.. then the matching up strips;
  // KIND 2: strips NBS*bx...  A 32-channel tile is a pair of neighbouring strips.
  auto strip_of = [&](int j) -> int {
    if constexpr (KIND == 1) return (j < GS) ? bx * GS + j : I / 16 + bx * GS + (j - GS);
    else return bx * NBS + j;
  };
  const int last = nk64 - 1;
  // operand addressing of the 32x32x32 form (see the header comment): B, and A in the fragment layout
  const int in_pair = ((lane & 31) >> 4) * WAVE + (lane & 15) + 16 * (lane >> 5);
  // wavefront column wn: KIND 1: gate tile = strips {2wn, 2wn+1}, up tile = strips {GS+2wn, GS+2wn+1};
  //                      KIND 2: tiles = strips {4wn, 4wn+1} and {4wn+2, 4wn+3}
  int tile_strip0[2];
  if constexpr (KIND == 1) { tile_strip0[0] = 2 * wn; tile_strip0[1] = GS + 2 * wn; }
  else { tile_strip0[0] = 4 * wn; tile_strip0[1] = 4 * wn + 2; }
  // 32-row tiles of this wavefront that hold rows of the block
  // The two wavefront rows of the block share its rows: in the 16x16x64 loop the second one starts at the first
  // multiple of 32 past half the rows the block has (128 in a full block), so a block of 144 rows is 3 + 2
  // row tiles of 32 and not 4 + 1: every k-step ends at a block barrier and takes as long as the wavefront with
  // the most row tiles.  The other loops keep the fixed halves of 128.
  const int half_rows = (LINES && M16) ? min(128, ((nrows + 1) / 2 + 31) / 32 * 32) : 128;
  const int wave_row0 = wm * half_rows;
  c.mt_count = (wm == 0) ? min(half_rows / 32, (nrows + 31) / 32) : min(4, max(0, (nrows - half_rows + 31) / 32));
  LineCtx lc;
  if constexpr (LINES) {
    lc.w = w;
    lc.lane = lane;
#pragma unroll
    for (int e = 0; e < 2; ++e)
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int r_tile = (e * 16 + 2 * w + i) * 8 + (lane >> 3);  // the row of the tile this lane fetches a piece of
        int rr = r_tile;
        if (rr >= nrows) rr = 0;  // rows past the end alias the first row; their results are not stored
        const int piece = (lane & 7) ^ ((r_tile >> 1) & 7);
        lc.asrc[e][i] = a.a_q + (size_t)source_row<KIND>(a, g, row0 + rr) * a.Kdim + (size_t)k_first * 64 + piece * 16;
      }
#pragma unroll
    for (int i = 0; i < 2; ++i)
      lc.bsrc[i] = wbase + ((size_t)strip_of(2 * w + i) * nk_all + k_first) * 1024 + lane * 16;
    // the first two super-steps of A and k-steps of B are requested as soon as their addresses exist (in the
    // order the first barrier of the k loop counts on); everything else the block sets up overlaps with them
    const int last_ss = nk64 / 2 - 1;
    line_load_a<0>(lc, 0, sa0);
    line_load_a<1>(lc, 0, sa0);
    line_load_b(lc, 0, sb0);
    line_load_b(lc, min(1, last), sb1);
    line_load_a<0>(lc, min(1, last_ss), sa1);
    line_load_a<1>(lc, min(1, last_ss), sa1);
    const int r32 = lane & 31;
    const int gx = (lane >> 5) ^ ((r32 >> 1) & 7);
#pragma unroll
    for (int e = 0; e < 2; ++e)
#pragma unroll
      for (int h = 0; h < 2; ++h) lc.a_off[e][h] = (wm * 128 + r32) * 8 + ((4 * e + 2 * h) ^ gx);
#pragma unroll
    for (int t = 0; t < 2; ++t) lc.b_off[t] = tile_strip0[t] * WAVE + in_pair;
    if constexpr (M16) {
      const int r16 = lane & 15, swz = (r16 >> 1) & 7;
#pragma unroll
      for (int e = 0; e < 2; ++e)
#pragma unroll
        for (int h = 0; h < 2; ++h) lc.a16_off[e][h] = (wave_row0 + h * 16 + r16) * 8 + ((4 * e + (lane >> 4)) ^ swz);
#pragma unroll
      for (int n = 0; n < 4; ++n) lc.b16_off[n] = (tile_strip0[n >> 1] + (n & 1)) * WAVE + lane;
    }
  } else {
#pragma unroll
    for (int i = 0; i < AP; ++i) {
      int rr = (AP * w + i) * 16 + (lane & 15);
      if (rr >= nrows) rr = 0;  // rows past the end alias the first row; their results are not stored
      c.asrc[i] = a.a_q + (size_t)source_row<KIND>(a, g, row0 + rr) * a.Kdim + (size_t)k_first * 64 + (lane >> 4) * 16;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
      c.bsrc[i] = wbase + ((size_t)strip_of(2 * w + i) * nk_all + k_first) * 1024 + lane * 16;
    // the first two k-steps are requested as soon as their addresses exist; everything else the block
    // has to set up overlaps with their flight
    pipe_load<WN>(c, 0, sa0, sb0);
    pipe_load<WN>(c, min(1, last), sa1, sb1);
    c.a_off = (wm * 8) * WAVE + in_pair;
#pragma unroll
    for (int t = 0; t < 2; ++t) c.b_off[t] = tile_strip0[t] * WAVE + in_pair;
  }
  // per-row activation scales go to LDS once (read back in the epilogue, after many barriers)
  for (int r = threadIdx.x; r < BM; r += 128 * WN) {
    row_scale[r] = (r < nrows) ? a.a_scale[source_row<KIND>(a, g, row0 + r)] : 0.0f;
  }

  v16i acc[4][2];
  if constexpr (!(LINES && M16)) {
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][t][i] = 0;
  }

  if constexpr (LINES) {
    // one instantiation of the pinned loop per number of row tiles; a wavefront without rows only takes
    // part in the loads and the barriers
    if constexpr (M16) {
      v4i a16[4][2][4];
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int ch = 0; ch < 4; ++ch) a16[mt][t][ch] = (v4i){0, 0, 0, 0};
      switch (c.mt_count) {
        case 4: line16_k_loop<4>(lc, nk64, sa0, sa1, sa2, sb0, sb1, sb2, a16); break;
        case 3: line16_k_loop<3>(lc, nk64, sa0, sa1, sa2, sb0, sb1, sb2, a16); break;
        case 2: line16_k_loop<2>(lc, nk64, sa0, sa1, sa2, sb0, sb1, sb2, a16); break;
        case 1: line16_k_loop<1>(lc, nk64, sa0, sa1, sa2, sb0, sb1, sb2, a16); break;
        default: line16_k_loop<0>(lc, nk64, sa0, sa1, sa2, sb0, sb1, sb2, a16); break;
      }
      acc16_to_acc32(a16, acc);
    } else {
      switch (c.mt_count) {
        case 4: line_k_loop<4>(lc, nk64, sa0, sa1, sa2, sb0, sb1, sb2, acc); break;
        case 3: line_k_loop<3>(lc, nk64, sa0, sa1, sa2, sb0, sb1, sb2, acc); break;
        case 2: line_k_loop<2>(lc, nk64, sa0, sa1, sa2, sb0, sb1, sb2, acc); break;
        case 1: line_k_loop<1>(lc, nk64, sa0, sa1, sa2, sb0, sb1, sb2, acc); break;
        default: line_k_loop<0>(lc, nk64, sa0, sa1, sa2, sb0, sb1, sb2, acc); break;
      }
    }
  } else {
    // wavefronts whose 128 rows all exist take the loop without tests
    if (c.mt_count == 4) pipe_k_loop<WN, false>(c, nk64, sa0, sa1, sa2, sb0, sb1, sb2, acc);
    else pipe_k_loop<WN, true>(c, nk64, sa0, sa1, sa2, sb0, sb1, sb2, acc);
  }
  // no LDS traffic may still be in flight when the block's LDS is handed to the next block
  __builtin_amdgcn_s_waitcnt((0x7 << 4) | (0xF << 8));  // vmcnt(0)

  // ---- epilogue (the stage buffers are free now: the bf16 rows of GEMM2 are staged there, two
  // wavefronts per buffer)
  __syncthreads();  // every wavefront is done reading the last stage; the row scales written at the start are visible
  if (tail_tile >= 0) {
    // one share of a split tile: publish the partial sums, count in, and only the last one goes on
    __shared__ int s_last;
    if (!tile_tail_handover<WN>(a, acc, c.mt_count, tail_tile, split, share, w, lane, &s_last)) return;
  }
  uint32_t* stage32 = (uint32_t*)(w < 2 ? sa0 : (w < 4 ? sa1 : (w < 6 ? sa2 : sb0))) + (w & 1) * TILE_STAGE_DWORDS;
  int bf16_shift = -1;
  if constexpr (KIND == 2) {
    if (a.extra_rows_bf16 && a.out_dtype == OMNI_DT_F32 && g >= a.G) bf16_shift = a.offsets[a.G];
  }
  const float* smooth_g = nullptr;
  if constexpr (KIND == 1) {
    if (a.smooth != nullptr && g < a.G) smooth_g = a.smooth + (size_t)g * I;
  }
  tile_epilogue<KIND, WN, BF>(a, acc, row_scale, stage32, lane, wave_row0, c.mt_count, wn, bx, row0, nrows, wsc, I,
                              bf16_shift, smooth_g);
#endif
}

// =====================================================================================
// row quantisation of y = silu(gate) * up (fp32, written by gemm_pipe): one wavefront per row keeps
// up to 256*NV values in registers between the max|y| reduction and the rounding, so the row is read
// once; NV == 0 reads it twice
// =====================================================================================
template <int NV>
__global__ __launch_bounds__(256) void quant_rows_y(const float* __restrict__ y, const int32_t* __restrict__ offsets,
                                                    int G, int extra_rows, int I, int64_t M_cap,
                                                    int8_t* __restrict__ hq, float* __restrict__ hs) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int64_t m = (int64_t)blockIdx.x * 4 + threadIdx.x / WAVE;
  const int64_t total = (int64_t)offsets[G] + extra_rows;
  if (m >= total || m >= M_cap) return;
  quant_row_y_wave<NV>(y + m * I, I, hq + m * I, hs + m, lane);
}

// ---------------------------------------------------------------- weight packing
__global__ __launch_bounds__(256) void pack_weight_kernel(const int8_t* __restrict__ w, int src_layout, int Kdim, int N,
                                                          int8_t* __restrict__ out) {
  // one thread per 16-byte fragment piece
  const int nk64 = Kdim / 64;
  const size_t per_mat = (size_t)Kdim * N;
  const size_t piece = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t npieces = per_mat / 16;
  if (piece >= npieces) return;
  const int g = blockIdx.y;
  const int l = (int)(piece % 64);
  const size_t tile = piece / 64;
  const int k64 = (int)(tile % nk64);
  const int n16 = (int)(tile / nk64);
  const int n = n16 * 16 + (l & 15);
  const int k0 = k64 * 64 + (l >> 4) * 16;
  const int8_t* src = w + (size_t)g * per_mat;
  int8_t v[16];
  if (src_layout == 1) {
#pragma unroll
    for (int j = 0; j < 16; ++j) v[j] = src[(size_t)n * Kdim + k0 + j];
  } else {
#pragma unroll
    for (int j = 0; j < 16; ++j) v[j] = src[(size_t)(k0 + j) * N + n];
  }
  int8_t* dst = out + (size_t)g * per_mat + piece * 16;
#pragma unroll
  for (int j = 0; j < 16; ++j) dst[j] = v[j];
}

// ---------------------------------------------------------------- host side dispatch
// kernel choice (make_plan), tuning variables, workspace sizes: host_logic.h
using omni_host::Plan;
using omni_host::Tuning;
using omni_host::tuning;
using omni_host::tile_lines;
using omni_host::tile_wn;
using omni_host::TILE_TAIL_BYTES;
using omni_host::TILE_TAIL_CNT_BYTES;
using omni_host::TILE_TAIL_CNT_WORDS;
using omni_host::TILE_TAIL_PART_BYTES;
using omni_host::gemm1_ws_bytes;
template <int KIND>
Plan make_plan(int T, int K, int G, int extra_rows, int Kdim, int N, int64_t M_cap) {
  (void)M_cap;
  return omni_host::make_plan(KIND, T, K, G, extra_rows, Kdim, N);
}

// compute units of the current device (asked once per device)
int device_cu_count() {
  static int cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
    cached[dev] = n > 0 ? n : -1;
  }
  return cached[dev] > 0 ? cached[dev] : 0;
}

template <int KIND, int MT, int NT, int D>
void launch_stream(const GemmArgs& a0, int64_t M_cap, int units, hipStream_t st) {
  GemmArgs a = a0;
  const int BM = 16 * MT;
  const int Gt = a.G + (a.extra_rows > 0 ? 1 : 0);
  int64_t mblocks = (M_cap + BM - 1) / BM + Gt;
  // GEMM1 (every block resident at once, long streams) gains from equal progress; GEMM2 (three rounds of short
  // blocks, where the older round should finish first and make room) loses by it: measured 84.4 -> 87.6 us
  a.equal_progress = (KIND == 1 && a.S == 1) ? (tuning().equal_progress & 1) : (tuning().equal_progress >> 1);
  const int cb = units / (4 * NT);
  a.bal_cus = 0;
  if (a.bal_cnt != nullptr && a.bal_part != nullptr && a.S == 1 && (KIND == 2 || a.y != nullptr) && tuning().stream_balance) {
    // balanced numbering: needs the blocks a compute unit holds at once (asked once per variant)
    static int resident = 0;
    if (resident == 0) {
      int n = 0;
      if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gemm_stream<KIND, MT, NT, D>, 256, 0) != hipSuccess || n <= 0) n = -1;
      resident = n;
    }
    const int cus = device_cu_count();
    if (resident > 0 && cus > 0) {
      constexpr size_t SHARE_BYTES = (size_t)4 * MT * ((KIND == 1) ? 2 * NT : NT) * 4 * WAVE * sizeof(int32_t);
      const size_t cap = a.bal_part_bytes / SHARE_BYTES;
      a.bal_cus = cus;
      a.bal_resident = resident;
      a.bal_cb = cb;
      a.bal_share_cap = cap > 4096 ? 4096 : (int)cap;
    }
  }
  if (a.bal_cus > 0) {
    const int64_t nblocks = (int64_t)cb * mblocks + omni_host::stream_balance_max_helpers(a.bal_cus);
    hipLaunchKernelGGL((gemm_stream<KIND, MT, NT, D>), dim3((unsigned)nblocks), dim3(256), 0, st, a);
    return;
  }
  dim3 grid((unsigned)cb, (unsigned)mblocks, (unsigned)a.S), block(256);
  hipLaunchKernelGGL((gemm_stream<KIND, MT, NT, D>), grid, block, 0, st, a);
}

__global__ void zero_words_kernel(int32_t* p, int n) {
  for (int i = threadIdx.x; i < n; i += blockDim.x) p[i] = 0;
}

template <int KIND>
void launch_tile(const GemmArgs& a0, int64_t M_cap, int units, void* tail_ws, size_t tail_bytes, bool counters_clean,
                 hipStream_t st) {
  const int BM = 256;
  GemmArgs a = a0;
  const int Gt = a.G + (a.extra_rows > 0 ? 1 : 0);
  const int wn = tile_wn(KIND, units);
  a.tile_gx = units / ((KIND == 1) ? 2 * wn : 4 * wn);
  a.tile_gy = (int)((M_cap + BM - 1) / BM + Gt);
  a.tile_pc = 1;
  for (int c = 1; c <= 8; ++c)
    if (a.tile_gx % c == 0) a.tile_pc = c;
  // one block per real tile (the kernel numbers them from the row counts in device memory; ids past
  // the real tiles leave at once) plus, when the last partial round is split, up to one round of helpers
  int64_t nblocks = (int64_t)a.tile_gy * a.tile_gx;
  a.tile_slots = 0;
  a.tail_cnt = nullptr;
  a.tail_part = nullptr;
  const int cus = device_cu_count();
  if (tail_ws && tail_bytes >= TILE_TAIL_BYTES && cus > 0 && tuning().tile_tail) {
    const size_t slot_bytes = (size_t)2 * wn * 8 * 16 * WAVE * sizeof(int32_t);
    const int blocks_per_cu = (wn == 4) ? 1 : 2;
    int slots = cus * blocks_per_cu;
    if ((size_t)slots * slot_bytes > TILE_TAIL_PART_BYTES) slots = (int)(TILE_TAIL_PART_BYTES / slot_bytes);
    if (slots > TILE_TAIL_CNT_WORDS) slots = TILE_TAIL_CNT_WORDS;
    a.tile_slots = slots;
    a.tile_split_max = tuning().tile_split;
    a.tail_cnt = (int32_t*)tail_ws + (KIND - 1) * TILE_TAIL_CNT_WORDS;
    a.tail_part = (int32_t*)((char*)tail_ws + TILE_TAIL_CNT_BYTES);
    if (!counters_clean) hipLaunchKernelGGL(zero_words_kernel, dim3(1), dim3(256), 0, st, a.tail_cnt, slots);
    nblocks += slots;
  }
  dim3 grid((unsigned)nblocks), block(128 * wn);
  const bool bfi = KIND == 1 && (a.flags & OMNI_GEMM1_BF16_INTERMEDIATE);
  if (wn == 4 && tile_lines(a.Kdim)) {
    const bool m16 = tuning().tile_mfma16 != 0;
    if (bfi && m16) hipLaunchKernelGGL((gemm_pipe<KIND, 4, KIND == 1, true, true>), grid, block, 0, st, a);
    else if (bfi) hipLaunchKernelGGL((gemm_pipe<KIND, 4, KIND == 1, true>), grid, block, 0, st, a);
    else if (m16) hipLaunchKernelGGL((gemm_pipe<KIND, 4, false, true, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((gemm_pipe<KIND, 4, false, true>), grid, block, 0, st, a);
  } else if (wn == 4) {
    if (bfi) hipLaunchKernelGGL((gemm_pipe<KIND, 4, KIND == 1, false>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((gemm_pipe<KIND, 4, false, false>), grid, block, 0, st, a);
  } else {
    if (bfi) hipLaunchKernelGGL((gemm_pipe<KIND, 2, KIND == 1, false>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((gemm_pipe<KIND, 2, false, false>), grid, block, 0, st, a);
  }
}

template <int KIND>
int dispatch_gemm(const GemmArgs& a, const Plan& p, int64_t M_cap, void* tail_ws, size_t tail_bytes, bool counters_clean,
                  hipStream_t st, const char* what) {
  const int units = (KIND == 1) ? a.N / 32 : a.N / 16;
  if (p.tile) {
    launch_tile<KIND>(a, M_cap, units, tail_ws, tail_bytes, counters_clean, st);
  } else {
    const int mt = p.mt, nt = p.nt, d = p.d;
    if (units % (4 * nt) != 0) OMNI_FAIL(OMNI_E_UNSUPPORTED, "%s: %d output strips not divisible by %d", what, units, 4 * nt);
    if (a.Kdim % 256 != 0) OMNI_FAIL(OMNI_E_UNSUPPORTED, "%s: reduction length %d must be a multiple of 256", what, a.Kdim);
    // the stream kernel addresses its activation operand with 32-bit byte offsets
    const int64_t a_rows = (KIND == 1) ? (int64_t)a.T : M_cap;
    if (a_rows * a.Kdim >= ((int64_t)1 << 32))
      OMNI_FAIL(OMNI_E_UNSUPPORTED, "%s: %lld rows of %d bytes are too many for the small-batch kernel", what, (long long)a_rows, a.Kdim);
    bool ok = false;
#define TRY(K_, MT_, NT_, D_)                                                  \
  if (!ok && KIND == K_ && mt == MT_ && nt == NT_ && d == D_) {                \
    if constexpr (KIND == K_) launch_stream<K_, MT_, NT_, D_>(a, M_cap, units, st); \
    ok = true;                                                                 \
  }
    OMNI_STREAM_VARIANTS(TRY)
#undef TRY
    if (!ok) OMNI_FAIL(OMNI_E_UNSUPPORTED, "%s: no stream kernel variant mt=%d nt=%d d=%d", what, mt, nt, d);
  }
  OMNI_CHECK_LAUNCH(what);
  return OMNI_OK;
}

void launch_quant_rows_y(const float* y, const int32_t* offsets, int G, int extra_rows, int I, int64_t M_cap,
                         int8_t* h_q, float* h_scale, hipStream_t st) {
  dim3 qgrid((unsigned)((M_cap + 3) / 4)), qblock(256);
  if (I <= 256 * 4) hipLaunchKernelGGL(quant_rows_y<4>, qgrid, qblock, 0, st, y, offsets, G, extra_rows, I, M_cap, h_q, h_scale);
  else if (I <= 256 * 8) hipLaunchKernelGGL(quant_rows_y<8>, qgrid, qblock, 0, st, y, offsets, G, extra_rows, I, M_cap, h_q, h_scale);
  else if (I <= 256 * 16) hipLaunchKernelGGL(quant_rows_y<16>, qgrid, qblock, 0, st, y, offsets, G, extra_rows, I, M_cap, h_q, h_scale);
  else hipLaunchKernelGGL(quant_rows_y<0>, qgrid, qblock, 0, st, y, offsets, G, extra_rows, I, M_cap, h_q, h_scale);
}

int check_group_args(const char* what, const int32_t* offsets, int G, int H, int I, int64_t M_cap, int extra_rows,
                     const void* w_extra, const void* w_extra_scale) {
  if (G < 0 || H <= 0 || I <= 0 || M_cap < 0 || extra_rows < 0) OMNI_FAIL(OMNI_E_INVALID, "%s: bad sizes G=%d H=%d I=%d M_cap=%lld", what, G, H, I, (long long)M_cap);
  if (!offsets) OMNI_FAIL(OMNI_E_INVALID, "%s: offsets is null", what);
  if (H % 64 != 0 || I % 64 != 0) OMNI_FAIL(OMNI_E_UNSUPPORTED, "%s: H=%d and I=%d must be multiples of 64", what, H, I);
  if (extra_rows > 0 && (!w_extra || !w_extra_scale)) OMNI_FAIL(OMNI_E_INVALID, "%s: extra group without weights", what);
  if (M_cap > 0x7fffffffLL) OMNI_FAIL(OMNI_E_UNSUPPORTED, "%s: M_cap too large", what);
  return OMNI_OK;
}

}  // namespace

extern "C" size_t omni_moe_gemm1_workspace_bytes(int T, int K, int G, int extra_rows, int64_t M_cap, int H, int I) {
  return omni_host::gemm1_workspace_bytes(T, K, G, extra_rows, M_cap, H, I);
}

extern "C" int omni_moe_gemm1_swiglu_quant(const int8_t* x_q, const float* x_scale, const int32_t* sorted_src,
                                           int idx_mode, int T, int K, const int8_t* w13_packed,
                                           const float* w13_scale, const int8_t* w13_extra,
                                           const float* w13_extra_scale, int extra_rows, const int32_t* offsets, int G,
                                           int H, int I, int64_t M_cap, int flags, const float* quant_scale,
                                           int8_t* h_q, float* h_scale, int32_t* acc_dbg, void* workspace,
                                           size_t ws_bytes, void* stream) {
  // the promise of OMNI_GEMM1_WS_ZEROED is about the counters of the streaming kernel, which leaves them at zero; the
  // tile kernel's are cleared in front of every launch
  const bool zeroed = (flags & OMNI_GEMM1_WS_ZEROED) && T > 0 && K > 0 && G >= 0 && H > 0 && I > 0 &&
                      !make_plan<1>(T, K, G, extra_rows, H, 2 * I, M_cap).tile;
  return omni_gemm1_swiglu_quant_impl(x_q, x_scale, sorted_src, idx_mode, T, K, w13_packed, w13_scale, w13_extra,
                                      w13_extra_scale, extra_rows, offsets, G, H, I, M_cap, flags, quant_scale, h_q,
                                      h_scale, acc_dbg, workspace, ws_bytes, zeroed, stream);
}

void* omni_tile_tail_area(int T, int K, int G, int extra_rows, int64_t M_cap, int H, int I, void* gemm1_ws,
                          size_t gemm1_ws_bytes, int* counter_words, size_t* tail_bytes) {
  if (T <= 0 || K <= 0 || G < 0 || M_cap <= 0 || !gemm1_ws) return nullptr;
  const Plan p1 = make_plan<1>(T, K, G, extra_rows, H, 2 * I, M_cap);
  const Plan p2 = make_plan<2>((int)M_cap, 1, G, extra_rows, I, H, M_cap);
  if (!p1.tile || !p2.tile) return nullptr;
  const size_t at = align256((size_t)M_cap * I * sizeof(float) + 256);
  if (gemm1_ws_bytes < at + TILE_TAIL_BYTES) return nullptr;
  *counter_words = 2 * TILE_TAIL_CNT_WORDS;
  *tail_bytes = TILE_TAIL_BYTES;
  return (char*)gemm1_ws + at;
}

int omni_gemm1_swiglu_quant_impl(const int8_t* x_q, const float* x_scale, const int32_t* sorted_src, int idx_mode, int T,
                                 int K, const int8_t* w13_packed, const float* w13_scale, const int8_t* w13_extra,
                                 const float* w13_extra_scale, int extra_rows, const int32_t* offsets, int G, int H, int I,
                                 int64_t M_cap, int flags, const float* quant_scale, int8_t* h_q, float* h_scale,
                                 int32_t* acc_dbg, void* workspace, size_t ws_bytes, bool counters_clean, void* stream) {
  int rc = check_group_args("gemm1", offsets, G, H, I, M_cap, extra_rows, w13_extra, w13_extra_scale);
  if (rc) return rc;
  if (M_cap == 0) return OMNI_OK;
  if (!x_q || !x_scale || !h_q || !h_scale || (G > 0 && (!w13_packed || !w13_scale))) OMNI_FAIL(OMNI_E_INVALID, "gemm1: null pointer");
  if (T <= 0 || K <= 0) OMNI_FAIL(OMNI_E_INVALID, "gemm1: bad T=%d K=%d", T, K);
  Plan p = make_plan<1>(T, K, G, extra_rows, H, 2 * I, M_cap);
  const size_t need = gemm1_ws_bytes(p, M_cap, I);
  if (ws_bytes < need || !workspace) OMNI_FAIL(OMNI_E_WORKSPACE, "gemm1: workspace %zu < %zu", ws_bytes, need);
  if (((uintptr_t)x_q % 16) || ((uintptr_t)w13_packed % 16) || ((uintptr_t)w13_extra % 16) || ((uintptr_t)workspace % 16) || ((uintptr_t)h_q % 4))
    OMNI_FAIL(OMNI_E_INVALID, "gemm1: pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  GemmArgs a{};
  a.a_q = x_q; a.a_scale = x_scale; a.sorted_src = sorted_src; a.idx_mode = idx_mode; a.T = T; a.K = K;
  a.w = w13_packed; a.w_scale = w13_scale; a.w_extra = w13_extra; a.w_extra_scale = w13_extra_scale;
  a.extra_rows = extra_rows; a.offsets = offsets; a.G = G; a.Kdim = H; a.N = 2 * I; a.flags = flags;
  a.acc_dbg = acc_dbg; a.S = p.S; a.M_cap = M_cap;
  a.smooth = quant_scale;
  if (quant_scale && (flags & OMNI_GEMM1_BF16_INTERMEDIATE))
    OMNI_FAIL(OMNI_E_INVALID, "gemm1: quant_scale belongs to the fp32 epilogue (npu_dequant_swiglu_quant), not to the bf16 one");
  if (p.tile) {
    // fused epilogue: y = silu(gate)*up to scratch, then the row quantiser
    float* y = (float*)workspace;
    a.y = y;
    void* tail_ws = (char*)workspace + align256((size_t)M_cap * I * sizeof(float) + 256);
    rc = dispatch_gemm<1>(a, p, M_cap, tail_ws, TILE_TAIL_BYTES, counters_clean, st, "gemm1");
    if (rc) return rc;
    if (flags & OMNI_GEMM1_NO_REQUANT) return OMNI_OK;
    launch_quant_rows_y(y, offsets, G, extra_rows, I, M_cap, h_q, h_scale, st);
    OMNI_CHECK_LAUNCH("gemm1 quant");
    return OMNI_OK;
  }
  if (p.S == 1 && acc_dbg == nullptr) {
    // one k share: the stream kernel finishes y = silu(gate)*up itself (the workspace holds it, half
    // the bytes of the raw sums), then the row quantiser of the tile path
    a.y = (float*)workspace;
    // overflow blocks of a launch that is resident at once are split along k: their counters and the scratch for
    // the shares' partial sums end the workspace
    const size_t bal_at = omni_host::gemm1_stream_bal_at(p, M_cap, I);
    if (bal_at != 0 && tuning().stream_balance) {
      a.bal_cnt = (int32_t*)((char*)workspace + bal_at);
      a.bal_part = (int32_t*)((char*)workspace + bal_at + omni_host::STREAM_BAL_CNT_BYTES);
      a.bal_part_bytes = omni_host::STREAM_BAL_PART_BYTES;
      if (!counters_clean) hipLaunchKernelGGL(zero_words_kernel, dim3(1), dim3(256), 0, st, a.bal_cnt, omni_host::STREAM_BAL_CNT_WORDS);
    }
    rc = dispatch_gemm<1>(a, p, M_cap, nullptr, 0, false, st, "gemm1");
    if (rc) return rc;
    if (flags & OMNI_GEMM1_NO_REQUANT) return OMNI_OK;
    launch_quant_rows_y(a.y, offsets, G, extra_rows, I, M_cap, h_q, h_scale, st);
    OMNI_CHECK_LAUNCH("gemm1 quant");
    return OMNI_OK;
  }
  // split-k stream kernel: raw int32 partial sums, then one row kernel does the whole epilogue
  if (I > 256 * 16) OMNI_FAIL(OMNI_E_UNSUPPORTED, "gemm1: intermediate size %d > 4096 in the small-batch path", I);
  a.part = (int32_t*)workspace;
  rc = dispatch_gemm<1>(a, p, M_cap, nullptr, 0, false, st, "gemm1");
  if (rc) return rc;
  if (flags & OMNI_GEMM1_NO_REQUANT) return OMNI_OK;
  // few rows (decode): more threads per row shorten the per-thread chain of exp / divide sequences
  const int rq = tuning().rowq ? tuning().rowq : (M_cap <= 2048 ? 512 : 256);  // measured at 576 rows: 512 threads best
  if (I > 256 * 8) hipLaunchKernelGGL((swiglu_quant_rows<16, 256>), dim3((unsigned)M_cap), dim3(256), 0, st, a, h_q, h_scale);
  else if (rq == 1024 && I <= 1024 * 2) hipLaunchKernelGGL((swiglu_quant_rows<2, 1024>), dim3((unsigned)M_cap), dim3(1024), 0, st, a, h_q, h_scale);
  else if (rq >= 512 && I <= 512 * 4) hipLaunchKernelGGL((swiglu_quant_rows<4, 512>), dim3((unsigned)M_cap), dim3(512), 0, st, a, h_q, h_scale);
  else hipLaunchKernelGGL((swiglu_quant_rows<8, 256>), dim3((unsigned)M_cap), dim3(256), 0, st, a, h_q, h_scale);
  OMNI_CHECK_LAUNCH("gemm1 row epilogue");
  return OMNI_OK;
}

extern "C" int omni_moe_gemm2_dequant(const int8_t* h_q, const float* h_scale, const int8_t* w2_packed,
                                      const float* w2_scale, const int8_t* w2_extra, const float* w2_extra_scale,
                                      int extra_rows, const int32_t* offsets, int G, int H, int I, int64_t M_cap,
                                      int out_dtype, void* rows_out, int32_t* acc_dbg, void* workspace, size_t ws_bytes,
                                      void* stream) {
  return omni_gemm2_dequant_impl(h_q, h_scale, w2_packed, w2_scale, w2_extra, w2_extra_scale, extra_rows, offsets, G, H, I,
                                 M_cap, out_dtype, rows_out, acc_dbg, workspace, ws_bytes, false, false, stream);
}

int omni_gemm2_dequant_impl(const int8_t* h_q, const float* h_scale, const int8_t* w2_packed, const float* w2_scale,
                            const int8_t* w2_extra, const float* w2_extra_scale, int extra_rows, const int32_t* offsets,
                            int G, int H, int I, int64_t M_cap, int out_dtype, void* rows_out, int32_t* acc_dbg,
                            void* workspace, size_t ws_bytes, bool counters_clean, bool extra_rows_bf16, void* stream) {
  int rc = check_group_args("gemm2", offsets, G, H, I, M_cap, extra_rows, w2_extra, w2_extra_scale);
  if (rc) return rc;
  if (M_cap == 0) return OMNI_OK;
  if (!h_q || !h_scale || !rows_out || (G > 0 && (!w2_packed || !w2_scale))) OMNI_FAIL(OMNI_E_INVALID, "gemm2: null pointer");
  if (out_dtype != OMNI_DT_BF16 && out_dtype != OMNI_DT_F32) OMNI_FAIL(OMNI_E_INVALID, "gemm2: out_dtype %d", out_dtype);
  if (((uintptr_t)h_q % 16) || ((uintptr_t)w2_packed % 16) || ((uintptr_t)w2_extra % 16)) OMNI_FAIL(OMNI_E_INVALID, "gemm2: pointers must be 16-byte aligned");
  GemmArgs a{};
  a.a_q = h_q; a.a_scale = h_scale; a.sorted_src = nullptr; a.idx_mode = 0;
  // T and K only steer the kernel choice here: rows per group ~ M_cap / groups
  a.T = (int)M_cap; a.K = 1;
  a.w = w2_packed; a.w_scale = w2_scale; a.w_extra = w2_extra; a.w_extra_scale = w2_extra_scale;
  a.extra_rows = extra_rows; a.offsets = offsets; a.G = G; a.Kdim = I; a.N = H; a.flags = 0;
  a.rows_out = rows_out; a.out_dtype = out_dtype; a.acc_dbg = acc_dbg; a.S = 1; a.M_cap = M_cap;
  Plan p = make_plan<2>(a.T, a.K, G, extra_rows, I, H, M_cap);
  if (extra_rows_bf16 && !(p.tile && out_dtype == OMNI_DT_F32 && extra_rows > 0))
    OMNI_FAIL(OMNI_E_INVALID, "gemm2: packed bf16 rows of the extra group are written by the tile kernel into fp32 rows only");
  a.extra_rows_bf16 = extra_rows_bf16 ? 1 : 0;
  if (workspace && ((uintptr_t)workspace % 256)) OMNI_FAIL(OMNI_E_INVALID, "gemm2: workspace must be 256-byte aligned");
  return dispatch_gemm<2>(a, p, M_cap, workspace, workspace ? ws_bytes : 0, counters_clean, (hipStream_t)stream, "gemm2");
}

extern "C" size_t omni_moe_gemm2_workspace_bytes(int G, int extra_rows, int64_t M_cap, int H, int I) {
  return omni_host::gemm2_workspace_bytes(G, extra_rows, M_cap, H, I);
}

extern "C" void omni_moe_reload_tuning(void) { omni_host::tuning_store() = omni_host::read_tuning(); }

extern "C" int omni_moe_gemm_kernel_name(int kind, int T, int K, int G, int extra_rows, int64_t M_cap, int H, int I,
                                         char* buf, size_t buf_bytes) {
  if ((kind != 1 && kind != 2) || !buf || buf_bytes == 0) OMNI_FAIL(OMNI_E_INVALID, "gemm_kernel_name: bad arguments");
  if (M_cap < 0 || I <= 0 || H <= 0 || G < 0 || (kind == 1 && (T <= 0 || K <= 0))) OMNI_FAIL(OMNI_E_INVALID, "gemm_kernel_name: bad sizes");
  const Plan p = (kind == 1) ? make_plan<1>(T, K, G, extra_rows, H, 2 * I, M_cap)
                             : make_plan<2>((int)M_cap, 1, G, extra_rows, I, H, M_cap);
  if (p.tile) {
    const int wn = tile_wn(kind, kind == 1 ? 2 * I / 32 : H / 16);
    snprintf(buf, buf_bytes, "gemm_pipe<%d,%d,%s>", kind, wn, (wn == 4 && tile_lines(kind == 1 ? H : I)) ? "lines" : "frags");
  }
  else snprintf(buf, buf_bytes, "gemm_stream<%d,%d,%d,%d>", kind, p.mt, p.nt, p.d);
  return OMNI_OK;
}

extern "C" int omni_moe_pack_weight(const int8_t* w, int src_layout, int G, int Kdim, int N, int8_t* packed,
                                    void* stream) {
  if (G <= 0 || Kdim <= 0 || N <= 0) OMNI_FAIL(OMNI_E_INVALID, "pack_weight: bad sizes");
  if (!w || !packed) OMNI_FAIL(OMNI_E_INVALID, "pack_weight: null pointer");
  if (Kdim % 64 != 0 || N % 16 != 0) OMNI_FAIL(OMNI_E_UNSUPPORTED, "pack_weight: Kdim=%d must be a multiple of 64 and N=%d of 16", Kdim, N);
  if (src_layout != 0 && src_layout != 1) OMNI_FAIL(OMNI_E_INVALID, "pack_weight: src_layout %d", src_layout);
  size_t npieces = (size_t)Kdim * N / 16;
  dim3 grid((unsigned)((npieces + 255) / 256), (unsigned)G), block(256);
  hipLaunchKernelGGL(pack_weight_kernel, grid, block, 0, (hipStream_t)stream, w, src_layout, Kdim, N, packed);
  OMNI_CHECK_LAUNCH("pack_weight");
  return OMNI_OK;
}
