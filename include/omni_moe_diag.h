/*
 * omni_moe_diag.h -- measurement helpers of libomni_moe_hip.so.  None of these is an operator of
 * the MoE path and none has a counterpart in the reference: they name kernels for profiles, time
 * the hardware alone (the calibration the layer's figures are read against) and re-read the
 * tuning variables.  The operator ABI is omni_moe_hip.h.
 */
#ifndef OMNI_MOE_DIAG_H
#define OMNI_MOE_DIAG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Which GEMM kernel omni_moe_gemm1_swiglu_quant (kind 1, with that call's arguments) or omni_moe_gemm2_dequant
 * (kind 2, T and K unused) launches for a call of these sizes, written to buf as the kernel's
 * template name, e.g. "gemm_stream<1,2,1,4>" or "gemm_pipe<2,4,lines>" (256 x 64*4 tile, line layout of the
 * activation operand; "frags": fragment layout).  A diagnostic for benchmarks and profiles
 * (no counterpart in the reference, whose kernels are chosen inside the closed operators).
 */
int omni_moe_gemm_kernel_name(int kind, int T, int K, int G, int extra_rows, int64_t M_cap, int H, int I, char* buf,
                              size_t buf_bytes);

/*
 * The OMNI_MOE_* tuning variables (kernel choice, tile shape, split tiles ...) are read from the environment
 * once, at the first GEMM call of the process.  This reads them again: for tests and tuning runs that change
 * them inside one process.  Not to be called while another thread launches GEMMs.  No counterpart in the
 * reference.
 */
void omni_moe_reload_tuning(void);

/*
 * Diagnostic (no counterpart in the reference): the sustained rate of v_mfma_i32_32x32x32_i8 on given operand
 * bits with nothing else in the loop.  `blocks` blocks of 8 wavefronts each issue 8 * iters instructions per
 * wavefront (65 536 op each) on operands taken from `operands` (>= 64 KiB; zeros and random bits give different
 * rates because the chip lowers its clock with the switching activity).  The caller times the launch.
 */
int omni_diag_mfma_i8_rate(const int8_t* operands, size_t operand_bytes, int iters, int blocks, int32_t* sink,
                           void* stream);
/*
 * Diagnostic (no counterpart in the reference): the int8 matrix instruction on the operand pattern of the tile
 * kernel (a 128 x 64 piece per wavefront, 128 accumulator registers, another operand pair from one instruction
 * to the next), as v_mfma_i32_32x32x32_i8 (form 32) or v_mfma_i32_16x16x64_i8 (form 16).  One pass of the loop is
 * 2 x 128 x 64 x 64 op per wavefront either way; `blocks` blocks of 8 wavefronts make `iters` passes.  The caller
 * times the launch: the two forms sustain different rates on the same operands.
 */
int omni_diag_mfma_i8_tile_rate(const int8_t* operands, size_t operand_bytes, int form, int iters, int blocks,
                                int32_t* sink, void* stream);
/*
 * Diagnostic (no counterpart in the reference): `blocks` blocks of 256 threads read `bytes` of `buf` once, 16
 * bytes per lane and request, eight requests of a lane in flight, and do nothing else.  The caller times the
 * launch: bytes / time is what the memory system delivers to a kernel that only streams, the practical ceiling
 * of the weight-streaming GEMMs.
 */
int omni_diag_hbm_read_rate(const void* buf, size_t bytes, int blocks, int32_t* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* OMNI_MOE_DIAG_H */
