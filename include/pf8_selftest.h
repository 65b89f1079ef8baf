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

#ifdef __cplusplus
}
#endif
#endif /* PF8_SELFTEST_H */
