/*
 * aptserve_probes.h — C ABI of libaptserve_probes.so: measurement kernels for
 * MI355X (gfx950) that belong to the benchmark, not to the hybrid-cache
 * library.  They have no counterpart in the reference; they exist so that the
 * kernels of libaptserve_hip.so can be held against what plain streams and
 * bare matrix-core instruction streams sustain on the same GPU, and so that
 * hardware counters can be scaled against a kernel of known traffic.
 * Conventions (device pointers, stream, status codes) as in aptserve_hip.h.
 */
#ifndef APTSERVE_PROBES_H
#define APTSERVE_PROBES_H

#include "aptserve_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Plain device copy of nbytes (16-byte aligned pointers): the known-size
 * kernel that hardware counters of the kernels above are scaled against. */
int aps_copy_bytes(void* dst, const void* src, int64_t nbytes,
                   aps_stream_t stream);

/* Plain streams over nbytes (16-byte aligned), for measuring what the part
 * sustains: mode 0 copies src to dst (as aps_copy_bytes), mode 1 only reads
 * src (dst: 4 bytes that are practically never written), mode 2 only writes
 * dst with a non-constant pattern (src unused).  chunks_per_thread 1 or 4
 * 16-byte chunks in flight per thread.  The ceilings the row movers and the
 * attention are compared against come from these. */
int aps_stream_probe(int mode, int chunks_per_thread, void* dst,
                     const void* src, int64_t nbytes, aps_stream_t stream);

/* Matrix-core instructions alone, for measuring what the part sustains under
 * the power they draw: `workgroups` workgroups of 4 wavefronts (one per SIMD)
 * run `iters` rounds of 16 v_mfma_f32_32x32x16 (shape 0) or 32
 * v_mfma_f32_16x16x32 (shape 1) on operands kept in registers, which they load
 * once from `operands` (32 KiB of f16 / bf16 values, 16-byte aligned: random
 * values make the part throttle, zeros do not).  Flops of a launch:
 * workgroups * 4 * iters * 2 * 16 * 32*32*16.  `sink` receives one float per
 * thread (workgroups * 256 floats).  Shapes 2..6 measure how a SIMD issues
 * matrix and vector instructions side by side; a round is 16
 * v_mfma_f32_32x32x16 and / or 16 vector units (one v_exp_f32 and three
 * v_fma_f32 on registers): 2 the two kinds alternating instruction by
 * instruction, 3 all the MFMAs and then all the vector units, 4 the vector
 * units alone, all with one wavefront per SIMD; 5 and 6 are 2 and 3 with two
 * wavefronts per SIMD (workgroups of 8 wavefronts; sink: workgroups * 512
 * floats).  No counterpart in the reference: the ceilings the re-projection
 * GEMM and the prompt attention are compared against come from this. */
int aps_mfma_probe(int shape, int dtype, const void* operands, void* sink,
                   int workgroups, int iters, aps_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* APTSERVE_PROBES_H */
