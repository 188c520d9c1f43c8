// The weight-streaming grouped int8 GEMM block (decode-sized batches) and what it shares with the other
// GEMM kernels: the argument record, the source-row lookup and the GEMM2 row epilogue.
#pragma once
#include "common.h"
#include <type_traits>

namespace {

struct GemmArgs {
  const int8_t* a_q;        // GEMM1: [T, Kdim] source rows; GEMM2: [M_cap, Kdim] sorted rows
  const float* a_scale;     // per source row (GEMM1) / per sorted row (GEMM2)
  const int32_t* sorted_src;  // GEMM1 only, nullable
  int idx_mode, T, K;
  const int8_t* w;
  const float* w_scale;
  const int8_t* w_extra;
  const float* w_extra_scale;
  int extra_rows;
  const int32_t* offsets;
  int G;
  int Kdim;  // reduction length
  int N;     // output channels of the GEMM: 2I (GEMM1) or H (GEMM2)
  int flags;
  // GEMM1: the quant_scale of npu_dequant_swiglu_quant, [G][I] fp32, nullable: y is multiplied by it before the row
  // is quantised (regular groups only; the extra group has none)
  const float* smooth;
  float* y;            // GEMM1: [M_cap, I]
  void* rows_out;      // GEMM2: [M_cap, N]
  int out_dtype;
  // Tile kernel, GEMM2 with fp32 rows: the extra group's rows are written as bf16 all the same, H bf16 values
  // each, packed from where that group's fp32 rows would begin (the whole-layer entry asks for this: the weighted
  // sum rounds the shared expert's rows to bf16 before it adds them, so the bits are the same and half the bytes move)
  int extra_rows_bf16;
  int32_t* acc_dbg;    // [M_cap, N], nullable
  int tile_gx, tile_gy, tile_pc;  // tile kernel: column tiles, row blocks (worst case), columns of a patch
  int tile_slots;                 // tile kernel: blocks the chip runs at once
  int tile_split_max;             // tile kernel: most shares a tile of the last partial round is split into
  int32_t* tail_cnt;              // tile kernel: arrival counters of the split tiles (zero at launch), or null
  int32_t* tail_part;             // tile kernel: partial accumulators of the split tiles
  int32_t* part;       // GEMM1 stream kernel: [S, M_cap, N] partial accumulators (split-k)
  int S;               // number of k splits (grid.z)
  int equal_progress;  // stream kernel: a wavefront lowers its issue priority as it advances through k
  // stream kernel, balanced numbering (omni_host::stream_balance): compute units (0: the plain 3-d grid), blocks a
  // unit holds at once, column blocks, shares the partial-sum scratch holds, the overflow blocks' arrival
  // counters (zero at launch) and the scratch
  int bal_cus, bal_resident, bal_cb, bal_share_cap;
  int32_t* bal_cnt;
  int32_t* bal_part;
  size_t bal_part_bytes;  // host side only: bal_share_cap follows from it and the variant's block size
  int64_t M_cap;
};

// source row of sorted row r of group g
template <int KIND>
__device__ __forceinline__ int source_row(const GemmArgs& a, int g, int r) {
  if constexpr (KIND == 2) {
    return r;
  } else {
    if (g >= a.G) return r - a.offsets[a.G];
    if (a.sorted_src == nullptr) return r;
    int s = a.sorted_src[r];
    return (a.idx_mode == OMNI_IDX_TOKEN_MAJOR) ? s / a.K : s % a.T;
  }
}

// GEMM2 rows of one accumulator tile of a lane: rows rbase .. rbase + 3 of the block, channel n.  The output type is
// a template parameter and the address of a row follows from the one above it, so that a row costs one add, one
// compare and one store.
// fp32 rows are written through (a device-scope store): the combine reads them under every L2, and the launch
// does not end on the write-back of 16 MB of dirty lines (measured: 1.3 us off the decode layer).
template <bool F32>
__device__ __forceinline__ void epilogue_gemm2(const GemmArgs& a, const float ws, int n, int row0, int rbase,
                                               int nrows, const float* ts, v4i acc) {
  using Out = typename std::conditional<F32, float, uint16_t>::type;
  Out* p = (Out*)a.rows_out + (size_t)(row0 + rbase) * (size_t)a.N + n;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (rbase + i < nrows) {
      const float o = ((float)acc[i] * ws) * ts[i];
      if constexpr (F32) __hip_atomic_store(p, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else *p = f32_to_bf16(o);
    }
    p += a.N;
  }
}
// raw accumulators for the parity tests, kept out of the epilogue so that none of their address arithmetic is
// ever part of it
__device__ __forceinline__ void dump_acc_gemm2(const GemmArgs& a, int n, int row0, int rbase, int nrows, v4i acc) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (rbase + i < nrows) a.acc_dbg[(size_t)(row0 + rbase + i) * (size_t)a.N + n] = acc[i];
}

// =====================================================================================
// gemm_stream
//   KIND 1: a wavefront owns NT (gate, up) strip pairs; KIND 2: NT strips.
//   MT: 16-row tiles per block (block covers up to 16*MT rows of one group).
//   D : k-steps of B kept in flight per wavefront (multiple of 4).
//   Requires Kdim % (64*D) == 0 (checked on the host).
//
// The k loop is free of data-dependent branches: rows past the end of a group read the group's
// first row (their accumulators are never stored), every tile of the body is multiplied (a 64-row
// kernel picks its two-, three- or four-tile body by the block's row count before the loop), and
// the loop is split into a part that refills the ring and a drain part, so the compiler can
// count outstanding loads exactly and never waits for more than the oldest k-step.
// =====================================================================================
// Occupancy asked of the compiler: the variants with one strip (pair) per wavefront are held to 5
// wavefronts per SIMD (96 registers) so that a launch of about 34 row blocks x 32 channel blocks is
// resident all at once: a second, nearly empty round of blocks would stream at a fraction of the bandwidth.
template <int KIND, int MT, int NT, int D>
constexpr int stream_min_waves() { return (NT == 1 && D == 4) ? 5 : 1; }
// Blocks of 64 rows keep nothing in LDS but the two activation buffers (32 KiB: five blocks fill the 160 KiB of a
// compute unit exactly, and 64-row launches of 100-220 tokens are then resident at once); their row scales wait in
// a register per thread and take over the first buffer after the k loop, and the hand-over flag sits behind them.
template <int MT>
constexpr bool stream_lds_overlay() { return MT >= 4; }

// Hand-over between the k shares of an overflow block (their blocks run on different compute units, possibly under
// different L2s).  The partial sums are stored and loaded with device-scope accesses, word by word (written
// through to where every L2 sees them, read past the caches), so that no bulk write-back or invalidation of
// an L2 is needed in the middle of a launch that streams through it: every wavefront stores its sums and waits until
// the stores are acknowledged, all wavefronts meet, one thread counts in at the block's counter.  True for the
// share that arrived last: its accumulators then hold the sums of all shares.  Nobody waits for anybody.
// STRIDE_MT: the tiles the kernel's largest body has; the scratch of a share is sized for that body whatever body
// the block runs, so that the shares of different blocks never overlap.
template <int MT, int NBF, int STRIDE_MT>
__device__ __forceinline__ bool stream_handover(const GemmArgs& a, v4i (&acc)[MT][NBF], int over, int split, int share,
                                                int w, int lane, int* s_last) {
  constexpr int WAVE_INTS = MT * NBF * 4 * WAVE;
  constexpr int BLOCK_INTS = 4 * STRIDE_MT * NBF * 4 * WAVE;
  int32_t* mine = a.bal_part + ((size_t)over * split + share) * BLOCK_INTS + (size_t)w * WAVE_INTS + lane;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NBF; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        __hip_atomic_store(mine + ((mt * NBF + j) * 4 + i) * WAVE, acc[mt][j][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_s_waitcnt(0);  // every store of this wavefront has been acknowledged
  __syncthreads();
  if (threadIdx.x == 0) {
    const bool last = __hip_atomic_fetch_add(a.bal_cnt + over, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == split - 1;
    // nobody else touches the word any more in this launch: it is left at zero for the next one
    if (last) __hip_atomic_store(a.bal_cnt + over, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *s_last = last;
  }
  __syncthreads();
  if (!*s_last) return false;
  for (int s2 = 0; s2 < split; ++s2) {
    if (s2 == share) continue;
    const int32_t* theirs = a.bal_part + ((size_t)over * split + s2) * BLOCK_INTS + (size_t)w * WAVE_INTS + lane;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < NBF; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[mt][j][i] += __hip_atomic_load(theirs + ((mt * NBF + j) * 4 + i) * WAVE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  return true;
}

// One block's work: the rows of row block `rb` times the channels of column block `bx` (4 wavefronts x NT
// strips, or strip pairs), k share `bz` of `nz`; over >= 0: the block is one share of overflow block `over` and
// hands its sums over.  `before_a()` runs after the first D k-steps of B have been requested and before anything
// of A is touched: a caller whose A is still being produced waits there, with its weight loads already in
// flight.  All four wavefronts of the block must call this together (block barriers inside); when it returns
// nobody reads the LDS buffers any more.
// OVERLAY: the row scales live on the first activation buffer after the k loop (stream_lds_overlay of the kernel).
template <int KIND, int MT, int NT, int D, bool OVERLAY, int STRIDE_MT, typename BeforeA>
__device__ __forceinline__ void stream_block(const GemmArgs& a, const RowBlock& rb, int bx, int bz, int nz, int over,
                                             int* s_last, v4i (*lds_a)[MT * 4 * WAVE], float* lds_ts, BeforeA before_a) {
  constexpr int NBF = (KIND == 1) ? 2 * NT : NT;  // B fragments per k-step
  constexpr int DC = D / 4;                       // chunks (4 k-steps) of B in flight
  static_assert(D % 4 == 0, "D counts whole chunks");

  const int lane = threadIdx.x & (WAVE - 1);
  // the wavefront's index as a scalar: its strips and their base addresses then live in scalar registers, and a
  // weight load is a scalar base plus one lane offset that all strips share
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
  const int g = rb.group, row0 = rb.row0, nrows = rb.nrows;
  const int mt_cnt = (nrows + 15) / 16;
  const int nk64_all = a.Kdim / 64;          // k-steps of the whole reduction
  const int nk64 = nk64_all / nz;            // k-steps of this block's share
  const int k64_0 = bz * nk64;
  const int nchunks = nk64 / 4;
  const int I = (KIND == 1) ? a.N / 2 : 0;

  const int8_t* wbase = (g < a.G) ? a.w + (size_t)g * a.Kdim * a.N : a.w_extra;
  const float* wsc = (g < a.G) ? a.w_scale + (size_t)g * a.N : a.w_extra_scale;

  // strips of this wavefront
  int strip[NBF];
  const int8_t* bp[NBF];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    int q = (bx * 4 + w) * NT + t;
    if constexpr (KIND == 1) {
      strip[2 * t] = q;
      strip[2 * t + 1] = I / 16 + q;
    } else {
      strip[t] = q;
    }
  }
#pragma unroll
  for (int j = 0; j < NBF; ++j) bp[j] = wbase + ((size_t)strip[j] * nk64_all + k64_0) * 1024;
  const uint32_t lane16 = lane * 16;

  // the first D k-steps of B are requested as soon as their addresses exist (they come from HBM and
  // take the longest); the A row lookup below overlaps with their flight
  v4i ring[D][NBF];
#pragma unroll
  for (int s = 0; s < D; ++s)
#pragma unroll
    for (int j = 0; j < NBF; ++j) ring[s][j] = __builtin_nontemporal_load((const v4i*)(bp[j] + (size_t)s * 1024 + lane16));
  __builtin_amdgcn_sched_barrier(0);
  before_a();
  // the activation scale of every row of the block goes to LDS now (one or two dependent loads per row, whose
  // way is then covered by the k loop instead of standing in front of the epilogue)
  float my_ts = 0.0f;
  if (threadIdx.x < 16 * MT) {
    my_ts = ((int)threadIdx.x < nrows) ? a.a_scale[source_row<KIND>(a, g, row0 + threadIdx.x)] : 0.0f;
    if constexpr (!OVERLAY) lds_ts[threadIdx.x] = my_ts;
  }

  // the weight scales of this lane's output channels are requested here as well: asked for in the epilogue they
  // would cost one more round trip through a saturated memory system at the end of every block's life
  float wsv[NBF];
#pragma unroll
  for (int j = 0; j < NBF; ++j) wsv[j] = wsc[strip[j] * 16 + (lane & 15)];

  // A staging.  A chunk of a 16-row tile is 16 rows x 256 bytes (4 k-steps); each wavefront fetches a quarter of
  // it, one 16-byte piece per lane, and stores it where the MFMA operand reads expect it: k-step kk, lane slot
  // 16 q + r for row r and k-quarter q.  GEMM1 (long rows, every block of a group re-reads the group's token rows
  // from the L2): a wavefront takes 4 whole rows, i.e. 8 whole cache lines per load instruction (measured
  // 1.8 us of the decode launch against the other split).  GEMM2: a wavefront takes one k-step of all 16 rows,
  // 16 half lines, and its LDS stores are conflict free (measured 0.5 us better there).
  // Rows past the end of the group alias the group's first row.
  constexpr bool WHOLE_ROWS = (KIND == 1);
  // byte offsets of the lane's pieces from a.a_q (the operand of a stream launch is far below 4 GiB: checked on the host)
  uint32_t arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int rr = mt * 16 + (WHOLE_ROWS ? 4 * w + (lane >> 4) : (lane & 15));
    if (rr >= nrows) rr = 0;
    arow[mt] = (uint32_t)source_row<KIND>(a, g, row0 + rr) * (uint32_t)a.Kdim + (uint32_t)k64_0 * 64 +
               (WHOLE_ROWS ? (lane & 15) * 16 : (lane >> 4) * 16 + w * 64);
  }
  const int a_slot = WHOLE_ROWS ? ((lane & 15) >> 2) * WAVE + (lane & 3) * 16 + 4 * w + (lane >> 4) : w * WAVE + lane;

  v4i acc[MT][NBF];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NBF; ++j) acc[mt][j] = (v4i){0, 0, 0, 0};

  // ---- prologue: A chunk 0 -> LDS
  // Blocks of four 16-row tiles stage the activation chunk in two halves (tiles 0-1 behind the first two k-steps
  // of a chunk, tiles 2-3 behind the last two) through two registers' worth of loads instead of four: part of
  // what lets the 64-row variants keep five wavefronts per SIMD.
  constexpr int AH = (MT == 4) ? 2 : MT;   // tiles staged at a time
  constexpr int APH = MT / AH;             // halves of a chunk's staging
  v4i areg[AH];
#pragma unroll
  for (int h = 0; h < APH; ++h) {
#pragma unroll
    for (int m = 0; m < AH; ++m) areg[m] = *(const v4i*)(a.a_q + arow[h * AH + m]);
#pragma unroll
    for (int m = 0; m < AH; ++m) lds_a[0][(h * AH + m) * 4 * WAVE + a_slot] = areg[m];
  }
  __syncthreads();

  // one chunk = 4 k-steps on ring slots [4*cc, 4*cc+4)
  auto chunk = [&](const int c, const int cc, const bool refill) {
    const int cnext = (c + 1 < nchunks) ? c + 1 : c;
    const v4i* la = lds_a[c & 1];
    v4i* ln = lds_a[(c + 1) & 1];
#pragma unroll
    for (int h = 0; h < APH; ++h) {
#pragma unroll
      for (int m = 0; m < AH; ++m) areg[m] = *(const v4i*)(a.a_q + (arow[h * AH + m] + (uint32_t)cnext * 256));
      // keep these loads ahead of the ring refills below: they are waited for at the end of their half of the
      // chunk, and loads complete in order, so a later position would drain the whole ring
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kk = h * (4 / APH); kk < (h + 1) * (4 / APH); ++kk) {
        const int s = cc * 4 + kk;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          v4i af = la[(mt * 4 + kk) * WAVE + lane];
#pragma unroll
          for (int j = 0; j < NBF; ++j) acc[mt][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, ring[s][j], acc[mt][j], 0, 0, 0);
        }
        // the slot is free once its MFMAs are issued: refill it with the k-step D ahead
        if (refill) {
#pragma unroll
          for (int j = 0; j < NBF; ++j)
            ring[s][j] = __builtin_nontemporal_load((const v4i*)(bp[j] + (size_t)(c * 4 + kk + D) * 1024 + lane16));
        }
        __builtin_amdgcn_sched_barrier(0);  // one k-step at a time: refills stay spread over the chunk
      }
      // the other buffer was last read a chunk ago, before the barrier that ended that chunk
#pragma unroll
      for (int m = 0; m < AH; ++m) ln[(h * AH + m) * 4 * WAVE + a_slot] = areg[m];
    }
    __syncthreads();
  };

  int c0 = 0;
  // Wavefronts of one SIMD are served oldest first, so without help the blocks of a launch that is resident
  // all at once finish in the order they started and the last ones stream alone, with too few loads in
  // flight to fill the memory system.  With a.equal_progress a wavefront lowers its issue priority by one level
  // per quarter of its reduction: wavefronts that are behind overtake those ahead, all of them finish
  // together, and the thin tail is gone (GEMM1 of the decode call: 162.7 -> 159.1 us).
  const bool equal_progress = a.equal_progress;
  for (; c0 < nchunks - DC; c0 += DC) {
    if (equal_progress) {
      const int q = (c0 * 4) / nchunks;
      if (q == 0) __builtin_amdgcn_s_setprio(3);
      else if (q == 1) __builtin_amdgcn_s_setprio(2);
      else if (q == 2) __builtin_amdgcn_s_setprio(1);
      else __builtin_amdgcn_s_setprio(0);
    }
#pragma unroll
    for (int cc = 0; cc < DC; ++cc) chunk(c0 + cc, cc, true);
  }
#pragma unroll
  for (int cc = 0; cc < DC; ++cc) chunk(c0 + cc, cc, false);

  if constexpr (OVERLAY) {
    // the last chunk ended at a block barrier: nobody reads the activation buffers any more
    if (threadIdx.x < 16 * MT) lds_ts[threadIdx.x] = my_ts;
    __syncthreads();
  }
  if (over >= 0) {
    if (!stream_handover<MT, NBF, STRIDE_MT>(a, acc, over, nz, bz, w, lane, s_last)) return;
  }
  // ---- epilogue
  const int col = lane & 15;
  if constexpr (KIND == 1) {
    if (a.y != nullptr) {
      // a single k share: the wavefront holds the gate and the up sums of its channels, so it
      // dequantises and applies SwiGLU here; the row quantiser is left with the maximum and the rounding
      const bool bf = a.flags & OMNI_GEMM1_BF16_INTERMEDIATE;
      // the smoothing factors of the lane's channels (rare: asked for here, not carried through the k loop)
      float smv[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t)
        smv[t] = (a.smooth != nullptr && g < a.G) ? a.smooth[(size_t)g * I + strip[2 * t] * 16 + col] : 1.0f;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt < mt_cnt) {
          const int rbase = mt * 16 + 4 * (lane >> 4);
          float ts[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) ts[i] = lds_ts[rbase + i];
#pragma unroll
          for (int t = 0; t < NT; ++t) {
            const int n = strip[2 * t] * 16 + col;
            const float wg = wsv[2 * t], wu = wsv[2 * t + 1];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              if (rbase + i < nrows) {
                float dg = ((float)acc[mt][2 * t][i] * wg) * ts[i];
                float du = ((float)acc[mt][2 * t + 1][i] * wu) * ts[i];
                if (bf) { dg = round_bf16(dg); du = round_bf16(du); }
                float yv = silu_spec(dg) * du;
                if (bf) yv = round_bf16(yv);
                if (a.smooth != nullptr) yv = yv * smv[t];
                a.y[(size_t)(row0 + rbase + i) * I + n] = yv;
              }
            }
          }
        }
      }
      return;
    }
    // raw int32 partial sums of this k share; the row kernel adds the shares and finishes
    int32_t* part = a.part + (size_t)bz * a.M_cap * a.N;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if (mt < mt_cnt) {
        const int rbase = mt * 16 + 4 * (lane >> 4);
#pragma unroll
        for (int j = 0; j < NBF; ++j) {
          const int n = strip[j] * 16 + col;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (rbase + i < nrows) part[(size_t)(row0 + rbase + i) * a.N + n] = acc[mt][j][i];
        }
      }
    }
  } else {
    const bool f32_rows = a.out_dtype == OMNI_DT_F32;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if (mt < mt_cnt) {
        const int rbase = mt * 16 + 4 * (lane >> 4);
        float ts[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) ts[i] = lds_ts[rbase + i];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          if (f32_rows) epilogue_gemm2<true>(a, wsv[t], strip[t] * 16 + col, row0, rbase, nrows, ts, acc[mt][t]);
          else epilogue_gemm2<false>(a, wsv[t], strip[t] * 16 + col, row0, rbase, nrows, ts, acc[mt][t]);
          if (a.acc_dbg) dump_acc_gemm2(a, strip[t] * 16 + col, row0, rbase, nrows, acc[mt][t]);
        }
      }
    }
  }
}

template <int KIND, int MT, int NT, int D>
__global__ __launch_bounds__(256, (stream_min_waves<KIND, MT, NT, D>())) void gemm_stream(GemmArgs a) {
  __shared__ v4i lds_a[2][MT * 4 * WAVE];
  float* lds_ts;
  int* s_last;
  if constexpr (stream_lds_overlay<MT>()) {
    lds_ts = (float*)&lds_a[0][0];
    s_last = (int*)(lds_ts + 16 * MT);
  } else {
    __shared__ float ts_own[16 * MT];
    __shared__ int last_own;
    lds_ts = ts_own;
    s_last = &last_own;
  }
  RowBlock rb;
  int bx = blockIdx.x, bz = blockIdx.z, nz = a.S, over = -1;
  if (a.bal_cus > 0) {
    // 1-d grid, balanced numbering: whole blocks, the overflow blocks' first shares, the helper shares
    const RowBlockScan sc = row_blocks_scan(a.offsets, a.G, a.extra_rows, 16 * MT);
    const int n_real = sc.total * a.bal_cb;
    const omni_host::StreamBalance bal =
        omni_host::stream_balance(n_real, a.bal_cus, a.bal_resident, a.Kdim / 256, D / 4, a.bal_share_cap,
                                  ((KIND == 1) ? 2 * NT : NT) * a.Kdim / 16);
    omni_host::StreamSel sel;
    if (!omni_host::stream_select(bal, n_real, (int)blockIdx.x, sel)) return;
    if (!row_blocks_find(sc, a.offsets, a.G, a.extra_rows, 16 * MT, sel.task / a.bal_cb, rb)) return;
    bx = sel.task % a.bal_cb;
    bz = sel.share;
    nz = sel.over >= 0 ? bal.split : 1;
    over = sel.over;
  } else if (!find_row_block(a.offsets, a.G, a.extra_rows, 16 * MT, blockIdx.y, rb)) {
    return;
  }
  constexpr bool OVL = stream_lds_overlay<MT>();
  if constexpr (MT == 4) {
    // a 64-row block with at most 32 rows runs the two-tile body: half the activation loads, LDS reads and MFMAs
    // (measured on the 64-row GEMM1: the two empty tiles cost a seventh of the launch)
    if (rb.nrows <= 32) {
      stream_block<KIND, 2, NT, D, OVL, MT>(a, rb, bx, bz, nz, over, s_last, (v4i(*)[2 * 4 * WAVE])lds_a, lds_ts, [] {});
      return;
    }
    if (rb.nrows <= 48) {
      stream_block<KIND, 3, NT, D, OVL, MT>(a, rb, bx, bz, nz, over, s_last, (v4i(*)[3 * 4 * WAVE])lds_a, lds_ts, [] {});
      return;
    }
  }
  stream_block<KIND, MT, NT, D, OVL, MT>(a, rb, bx, bz, nz, over, s_last, lds_a, lds_ts, [] {});
}

// Row quantisation of y = silu(gate) * up (fp32) by one wavefront: scale = max|y| / 127, q = rint(y / scale).
// Up to 256*NV values are kept in registers between the maximum and the rounding, so the row is read
// once; NV == 0 reads it twice.  The two halves are separate so that a caller can have the loads of
// several rows in flight before it reduces the first.
template <int NV>
__device__ __forceinline__ void load_row_y(const float* __restrict__ yr, int I, int lane, v4f (&v)[NV]) {
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = (i * WAVE + lane) * 4;
    v[i] = (c < I) ? __builtin_nontemporal_load((const v4f*)(yr + c)) : (v4f){0.0f, 0.0f, 0.0f, 0.0f};
  }
}
template <int NV>
__device__ __forceinline__ void quant_loaded_row(const v4f (&v)[NV], int I, int8_t* __restrict__ qr,
                                                 float* __restrict__ hs_m, int lane) {
  float mx = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) mx = fmaxf(mx, fabsf(v[i][j]));
  mx = wave_allmax_f(mx);
  const float s = mx / 127.0f;
  if (lane == 0) *hs_m = s;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = (i * WAVE + lane) * 4;
    if (c < I) {
      uint32_t o = 0;
      if (s > 0.0f) {
#pragma unroll
        for (int j = 0; j < 4; ++j) o |= ((uint32_t)(quant_i8(v[i][j], s) & 0xff)) << (8 * j);
      }
      *(uint32_t*)(qr + c) = o;
    }
  }
}
template <int NV>
__device__ __forceinline__ void quant_row_y_wave(const float* __restrict__ yr, int I, int8_t* __restrict__ qr,
                                                 float* __restrict__ hs_m, int lane) {
  if constexpr (NV > 0) {
    v4f v[NV];
    load_row_y<NV>(yr, I, lane, v);
    quant_loaded_row<NV>(v, I, qr, hs_m, lane);
  } else {
    float mx = 0.0f;
    for (int c = lane * 4; c < I; c += WAVE * 4) {
      v4f v = *(const v4f*)(yr + c);
#pragma unroll
      for (int j = 0; j < 4; ++j) mx = fmaxf(mx, fabsf(v[j]));
    }
    mx = wave_allmax_f(mx);
    const float s = mx / 127.0f;
    if (lane == 0) *hs_m = s;
    for (int c = lane * 4; c < I; c += WAVE * 4) {
      v4f v = *(const v4f*)(yr + c);
      uint32_t o = 0;
      if (s > 0.0f) {
#pragma unroll
        for (int j = 0; j < 4; ++j) o |= ((uint32_t)(quant_i8(v[j], s) & 0xff)) << (8 * j);
      }
      *(uint32_t*)(qr + c) = o;
    }
  }
}

}  // namespace
