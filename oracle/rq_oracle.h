/*
 * CPU oracle for the ruquant W4A4 / W4A4H MUL_MAT path.
 *
 * TEST INFRASTRUCTURE ONLY. This is a plain-C restatement of the reference's CPU arithmetic
 * (patches/llama.cpp-ruquant.patch in the reference tree; cited below as P:line). It exists so
 * that the HIP kernels can be checked bit for bit and so that a CPU baseline can be timed next to
 * them. Nothing that ships (the HIP library, its C ABI, the host bindings) links, loads or calls
 * it; only tests, the smoke check and the benchmark's cpu_baseline leg do.
 *
 * Every function here performs the same floating-point operations, in the same order, as the
 * reference function it cites. Build with -ffp-contract=off.
 */
#ifndef RQ_ORACLE_H
#define RQ_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 144-byte storage block of 256 int4 codes (P:44-50). Weights and quantized activations share it. */
typedef struct {
    float    d;      /* weights: row unit s_w; activations: token unit u                            */
    int32_t  sum;    /* weights: multiplier encoding or legacy code sum; activations: zero points   */
    int32_t  pad[2]; /* weights: {row / Hadamard length, clip bits}; activations: {m_g bytes, len}  */
    uint32_t qs[32]; /* element 8w+j lives in bits [4j+3:4j] of qs[w], two's-complement int4        */
} rqo_block;

enum { RQO_TYPE_W4A4 = 44, RQO_TYPE_W4A4H = 45, RQO_TYPE_A4 = 46, RQO_TYPE_A4H = 47 }; /* P:10-13 */

/* P:2419-2430. Returns 1 and fills p, m when n = p * m with m a power of two and p = 1 or a Paley order. */
int  rqo_hadamard_factor(int64_t n, int *p, int *m);
/* P:2433-2448. A is p*p entries of +-1 (row-major), Paley construction I. */
void rqo_paley(int p, int8_t *A);
/* P:2450-2485. In place x <- x H (or x H^T), H = (H_p kron H_m) / sqrt(n). */
void rqo_hadamard(float *x, int64_t n, int transpose);

/* P:2590-2600 without the process-wide cache: env_clip <= 0 means "not set". */
float rqo_resolve_clip(float env_clip, float tensor_clip);
/* Reads RQ_ACT_CLIP / RQ_ACT_CLIP_H the way P:2592-2597 does (atof, _H falls back to the plain one);
 * returns -1 when unset. Not cached, so one process can test several settings. */
float rqo_env_clip(int hadamard);
/* P:2602-2606, P:2608-2620: header fields of block 0. rot_check returns -1 where the reference aborts. */
float   rqo_tensor_clip(const void *blocks);
int64_t rqo_rot_check(int32_t n, int64_t k);

/* P:2639-2679. G is 64, 128 or 256 (P:2623-2631 picks it from RQ_ACT_GROUP; here it is an argument). */
void rqo_quantize_row_a(const float *x, rqo_block *y, int64_t k, float clip, int G);
/* P:2728-2736: copy, rotate every n_rot-long block, quantize, pad[1] = n_rot. */
void rqo_quantize_row_a4h(const float *x, rqo_block *y, int64_t k, float clip, int64_t n_rot, int G);

/* P:148-177. One weight row against one activation row, n = K. */
void rqo_vec_dot(int64_t n, float *s, const rqo_block *w, const rqo_block *a);

/* Weight side (P:2489-2580, P:2681-2710). wgroup: 0 = one scale per row, 256 or 64 = integer multipliers. */
void rqo_quantize_row_w(const float *x, rqo_block *y, int64_t k, int wgroup);
void rqo_quantize_row_w4a4h(const float *x, rqo_block *y, int64_t k, int64_t n_rot, int wgroup);
/* P:2738-2789. */
void rqo_dequantize_row_w(const rqo_block *x, float *y, int64_t k, int hadamard);
void rqo_dequantize_row_a(const rqo_block *x, float *y, int64_t k, int hadamard);

/* The MUL_MAT of P:92-132 + P:71-82 for one 2-D problem: y[M][N] (row stride ldy floats) =
 * W[N rows of K] x X[M rows, stride ldx floats]. Phase 1 quantizes tokens (tokens striped over threads),
 * phase 2 runs vec_dot over chunks of weight rows. Returns 0, or -1 on an impossible shape. */
int rqo_mul_mat(int type, const void *w_blocks, int64_t K, int64_t N,
                const float *x, int64_t ldx, int64_t M, float *y, int64_t ldy,
                float clip, int64_t n_rot, int G, int n_threads);

#ifdef __cplusplus
}
#endif
#endif
