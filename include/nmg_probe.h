/* C ABI of libnmg_probe.so: a measurement aid of bench.py, kept out of the product library
 * (libnmg_hip.so, include/nmg_hip.h).  Status codes: 0 ok, 1 bad argument, 2 launch failed. */
#ifndef NMG_PROBE_H
#define NMG_PROBE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* The rate the matrix cores sustain when nothing else happens.
 * No counterpart in the reference.  Every wavefront of 1024 workgroups issues the instructions of a
 * 128 x 128 x 64 slab from registers, `iters` times, with no memory traffic inside the loop.
 * kind 0: V_MFMA_F32_32X32X16_F16, 1: V_MFMA_F32_16X16X32_F16, 2: V_SMFMAC_F32_32X32X32_F16,
 * 3: V_SMFMAC_F32_16X16X64_F16.  d_operands: 1 MiB of fp16 operand values (zeros show the issue
 * rate, random values what the power limit leaves), 16-byte aligned; d_out: 1 MiB of sums that only
 * keep the loop alive.  The caller times the launch; nmg_probe_matrix_rate_flops gives the flops of
 * one launch (dense-equivalent for the sparse kinds). */
int nmg_probe_matrix_rate(int kind, const void *d_operands, float *d_out, int iters, void *stream);
int64_t nmg_probe_matrix_rate_flops(int kind, int iters);

#ifdef __cplusplus
}
#endif
#endif /* NMG_PROBE_H */
