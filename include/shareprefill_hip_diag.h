/*
 * shareprefill_hip_diag.h -- measurement and test aids of libshareprefill_hip.so.
 *
 * NOT part of the drop-in boundary: nothing here has a counterpart in the reference and nothing in the product path
 * (the shareprefill_amd package's attention function, selection and patch) calls it.  The benchmark uses these entry
 * points to report the shader clock under load and the sustained matrix-core rate of the chip beside its own
 * figures, one test uses the pairing read-out to check how work items were formed.  Unlike every entry point of
 * shareprefill_hip.h, the two read-outs synchronise the stream and copy to host memory.
 */
#ifndef SHAREPREFILL_HIP_DIAG_H
#define SHAREPREFILL_HIP_DIAG_H

#include "shareprefill_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Measurement aid (no counterpart in the reference): runs `iters` x 4 back-to-back bf16 32x32x16 MFMAs per wave on
 * every CU (8 waves per CU).  random_operands 0: one constant in every operand element; 1: random values per lane,
 * the same registers for every instruction (operand inputs never toggle); 2: four different random operand pairs in
 * rotation, so both operands change with every instruction as in a real product.  The caller times it; flops =
 * sp_diag_mfma_flops(iters).  Used to calibrate the sustained matrix-core rate under the board's power limit, which
 * depends on how much the operand bits toggle.  out: 512 floats of device scratch. */
int sp_diag_mfma_bf16(int32_t iters, int32_t random_operands, float* out, sp_stream_t stream);
double sp_diag_mfma_flops(int32_t iters);

/* Measurement aid (no counterpart in the reference): shader-clock cycles and 100 MHz wall ticks that workgroup 0
 * of the LAST sp_block_sparse_attn_fwd_bf16 launch on this workspace spent in the kernel; cycles / (ticks / 100)
 * is the average shader clock in MHz under that load.  Copies two int64 to host memory after synchronising the
 * stream. */
int sp_attn_last_launch_clocks(const void* workspace, int64_t n, int32_t hkv, int32_t d, int32_t bs,
                               int64_t* cycles_and_ticks, sp_stream_t stream);
/* Test / measurement aid (no counterpart in the reference): how the LAST sp_block_sparse_attn_fwd_bf16 launch on
 * this workspace paired query blocks into work items, one byte per two adjacent heads (2i, 2i+1): 0 = rows 2p and
 * 2p+1 of each head share an item, 1 = the same row of the two heads does (chosen when it makes the unions of the
 * paired masks smaller; only inside a kv group).  Copies (hq + 1) / 2 bytes to host memory after synchronising the
 * stream.  The pairing changes how the work is scheduled, never the result. */
int sp_attn_last_launch_pairing(const void* workspace, int64_t n, int32_t hq, int32_t hkv, int32_t d, int32_t bs,
                                uint8_t* by_heads, sp_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SHAREPREFILL_HIP_DIAG_H */
