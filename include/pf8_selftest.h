/*
 * pf8_selftest.h -- measurement and self-test hooks of libpf8.so.  They are exported next to the
 * operator entry points of pf8.h but replace nothing in the reference: the GPU tests sweep the device
 * codec, the fast-division path and the device SiLU through them, and the benchmark launches the copy
 * as the kernel of known traffic that hardware counters are scaled by.  Same conventions as pf8.h.
 */
#ifndef PF8_SELFTEST_H
#define PF8_SELFTEST_H

#include "pf8.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Measurement hook: a plain device-to-device copy of nbytes (multiple of 16).  bench.py launches it
 * so that hardware traffic counters (FETCH_SIZE / WRITE_SIZE) can be scaled by a kernel whose
 * traffic is known. */
int pf8_debug_copy(const void* src, void* dst, int64_t nbytes, pf8_stream_t stream);
/* Self-test hook used by the GPU tests: converts n floats to e4m3 with the same device routine the
 * quantizers use (hardware OCP convert), so the codec can be swept exhaustively. */
int pf8_debug_encode(const float* v, int64_t n, uint8_t* out, pf8_stream_t stream);
/* Self-test hook: q[i] = e4m3(x[i] / s[i]) through the quantizers' fast-division path. */
int pf8_debug_div_encode(const float* x, const float* s, int64_t n, uint8_t* out, pf8_stream_t stream);
/* Self-test hook: out[i] = silu(x[i]) with the device restatement of the oracle's expf. */
int pf8_debug_silu(const float* x, int64_t n, float* out, pf8_stream_t stream);
/* Self-test hook: the two quotients of the SwiGLU backward, out_silu[i] = x / (1 + exp(-x)) and out_sigmoid[i] = 1 / (1 + exp(-x)),
 * as the kernel forms them (one hardware reciprocal, exact residuals). */
int pf8_debug_silu_sigmoid(const float* x, int64_t n, float* out_silu, float* out_sigmoid, pf8_stream_t stream);

/* Measurement hook: pf8_grouped_gemm_nt_contiguous_fm (sa_layout 1) from an instantiation that reads the shader clock
 * at four points of every K block.  cycles int64 [workgroups][8], workgroups >= the launch's grid (at most one per
 * compute unit): per workgroup, wavefront 0's sums over all its K blocks of {MFMAs 0..23 with their copies and fragment
 * reads, the counted wait for the next block's data, the barrier, MFMAs 24..31 with the next block's first reads},
 * then {epilogue cycles, K blocks, tiles, unused}.  The output is the GEMM's; the launch is a few percent slower.
 * ablate != 0 leaves instructions out (the output is then garbage) to price them: 2 = the weight-fragment loads, 4 = the
 * activation and scale copies, 8 = the scale FMAs, 16 = the LDS fragment reads; built are 6 (no memory instructions), 8,
 * 14 (only MFMAs and LDS reads left), 30 (only MFMAs, barriers and scalar code left) and 64 = every tile reads the
 * operands of tile (0, 0), i.e. all operand traffic hits in the L2. */
int pf8_debug_grouped_gemm_fm_cycles(const uint8_t* a, const float* sa, const uint8_t* b_fm, const float* sb, int E,
                                     int64_t Mtot, int64_t N, int64_t K, const int32_t* m_indices, uint16_t* out,
                                     int64_t* cycles, int64_t workgroups, int ablate, pf8_stream_t stream);

/* Measurement hook: pf8_grouped_wgrad_pow2 sends the experts whose reduction axis is at least `blocks` 128-row blocks long
 * to the kernel with the 256x256 accumulator tile and the others to the 128x128-tile kernel (both give the same bits);
 * 0 = every expert to the 128x128-tile kernel.  Returns the previous setting (default 6). */
int pf8_debug_set_wgrad_tile256_min_blocks(int blocks);

#ifdef __cplusplus
}
#endif
#endif /* PF8_SELFTEST_H */
