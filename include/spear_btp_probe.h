/*
 * spear_btp_probe.h -- measurement aids of the MI355X (gfx950) Block Two-Pass library.
 *
 * Not part of the operator and without a counterpart in the reference: a copy kernel of known traffic and
 * bandwidth probes in the operator's own access shape, used by the benchmark to calibrate hardware counters and
 * to show what the memory system gives kernels shaped like the operator's. They live in the same shared library
 * (spear_amd/csrc/btp_probe.hip) and follow the conventions of spear_btp.h: device pointers, a hipStream_t passed
 * as void*, 0 or a negative SPEAR_BTP_E* code, spear_btp_last_error() for the message.
 */
#ifndef SPEAR_BTP_PROBE_H_
#define SPEAR_BTP_PROBE_H_

#include "spear_btp.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Measurement aid, not part of the operator: a plain device-to-device copy kernel of known
 * traffic (reads `bytes`, writes `bytes`; `bytes` a multiple of 16), used to calibrate hardware
 * counters and to measure the copy bandwidth the BTP kernels are compared with. */
int spear_btp_copy(const void* src, void* dst, unsigned long long bytes, void* stream);

/* Measurement aid as well: the operator's own access shape and cache policy without its arithmetic.
 * Every wavefront moves one 4 KiB slab with non-temporal 16-byte loads and stores; with src_b == NULL
 * it is a copy (reads `bytes`, writes `bytes`), otherwise dst = src_a ^ src_b (reads 2 x `bytes`, writes
 * `bytes`: the backward kernel's read/write mix). `bytes` a multiple of 4096. What this reaches is what
 * the memory system gives kernels of this shape, which is the practical ceiling the BTP kernels are
 * compared with beside the 8 TB/s peak. */
int spear_btp_stream_probe(const void* src_a, const void* src_b, void* dst, unsigned long long bytes, void* stream);

/* The same traffic in other launch shapes, to show where the kernels' own shape stands among the
 * alternatives: shape 0 = spear_btp_stream_probe (one 4 KiB slab per wavefront); 1 = two slabs per
 * wavefront, all loads issued before the first store; 2 = four slabs per wavefront in a loop that issues
 * the next slab's loads before the current slab's stores; 3 = that loop as a persistent grid striding over
 * the buffer; 4 = one 16-byte element per thread; 5 = reads only (src_a, and src_b if given; `dst` is not
 * written unless every input word is all ones); 6 = writes only (`dst` is filled, nothing is read). HBM serves
 * reads and writes one after the other, so shapes 5 and 6 give the two rates from which the floor of a mixed
 * kernel follows: R bytes read and W bytes written take at least R / read rate + W / write rate; 7 = shape 0
 * with 640 dependent FMAs between loads and stores (the output's last word may differ from shape 0's in its
 * lowest bit). Same arguments and result as spear_btp_stream_probe. */
#define SPEAR_BTP_PROBE_SHAPES 8
int spear_btp_stream_probe_shape(const void* src_a, const void* src_b, void* dst, unsigned long long bytes, int shape,
                                 void* stream);

/* The probe with the stream counts of the fused layer kernels (measurement aid, no counterpart in the
 * reference): `n_src` inputs of `bytes` each are combined (xor) into `n_dst` identical outputs of `bytes` each, in
 * the shape of spear_btp_stream_probe (one 4 KiB piece per wavefront and tensor, non-temporal 16-byte accesses).
 * (n_src, n_dst) = (3, 1): the fused forward's and the prefill kernel's mix; (4, 3): the fused backward's;
 * (1, 2): the stand-alone forward's with an fp32 result (the op's default output type).
 * `compute` != 0 puts a chain of dependent FMAs between loads and stores (640 for (3, 1), 1280 for (4, 3), 320
 * for (1, 2); the
 * outputs' last word may then differ in its lowest bit). `src`, `dst`: host arrays of device pointers, 16-byte
 * aligned; `bytes` a multiple of 4096. */
int spear_btp_stream_probe_mix(const void* const* src, int n_src, void* const* dst, int n_dst, unsigned long long bytes,
                               int compute, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SPEAR_BTP_PROBE_H_ */
