/*
 * C ABI of librq_probe.so: machine-peak probe kernels for gfx950. A measurement aid with no counterpart in the
 * reference's operator (its method is the reference's rig/membench/stream_bench.hip:1-60 and
 * rig/bench_valu.cu:1-129). Not part of the operator's library: only the benchmark and its test load it.
 */
#ifndef RQ_PROBE_H
#define RQ_PROBE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Launches ONE probe kernel on `stream` (a hipStream_t passed as void*); the caller times a batch of launches.
 * buf: device scratch, 256-byte aligned, `bytes` long (>= 8192). Returns 0, a hipError_t (> 0) or -3 for arguments
 * the kernels cannot take.
 *   RQ_PROBE_EMPTY : a0 workgroups of 256 threads that do nothing (cost of a launch).
 *   RQ_PROBE_STREAM: reads a0 bytes of buf with non-temporal 16-byte loads, a1 loads in flight per thread
 *                    (4, 5, 8, 10, 16 or 20), a2 workgroups (0: one per chunk of a1 * 4 KiB).
 *   RQ_PROBE_MIX   : a0 = sub-kind | VALU instruction << 8 | one-wavefront-per-SIMD << 16 | MFMA form << 20,
 *                    a1 workgroups, a2 MFMA iterations (16 MFMAs each), a3 VALU iterations (128 instructions each).
 *                    Sub-kinds: 0 all wavefronts MFMA; 1 all VALU; 2 wavefronts 0..3 MFMA and 4..7 VALU (one of each
 *                    per SIMD); 3 wavefronts 0..3 MFMA, others idle; 4 wavefronts 4..7 VALU, others idle; 5 / 6 every
 *                    wavefront 1 MFMA + 8 / 16 VALU interleaved; 7 every wavefront its MFMAs, then its VALU work.
 *                    VALU instruction: 0 v_add_u32, 1 v_ashrrev_i32, 2 v_mul_i32_i24, 3 v_dot8c_i32_i4, 4 v_fma_f32, 5 v_add_f32.
 *                    MFMA form: 0 v_mfma_i32_16x16x64_i8 (with every VALU instruction), 1 v_mfma_i32_32x32x32_i8,
 *                    2 v_mfma_f32_32x32x64_f8f6f4 on fp8 operands, 3 the same on fp6 operands (forms 1..3 with VALU
 *                    instructions 0 and 4). The SIMD id each wavefront of workgroup 0 ran on is written to the 8 ints
 *                    at buf + 4096. */
#define RQ_PROBE_EMPTY  0
#define RQ_PROBE_STREAM 1
#define RQ_PROBE_MIX    2
int rq_probe(int kind, int64_t a0, int64_t a1, int64_t a2, int64_t a3, void *buf, size_t bytes, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* RQ_PROBE_H */
