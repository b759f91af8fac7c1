/*
 * C ABI of the MI355X (gfx950) implementation of ruquant's W4A4 / W4A4H MUL_MAT.
 *
 * Plain pointers and sizes only. Every device pointer is memory of the current HIP device; `stream` is a
 * hipStream_t passed as void* (the reference's Rust host passes its stream the same way,
 * src/kernels.rs:14). Citations "P:n" are lines of patches/llama.cpp-ruquant.patch in the reference.
 *
 * Life cycle of one weight tensor, mirroring the reference's first-use / steady-state split
 * (P:2027-2075, P:295-299):
 *   first use   (may synchronize, must not be captured in a graph):
 *       read block 0's header on the host -> rq_w4a4_resolve_clip / rq_w4a4_tensor_rot;
 *       rq_w4a4_prepare() rewrites the 144-byte blocks into the streaming layout, OUT OF PLACE
 *       (the reference repacks in place and leaves the tensor unreadable as blocks; this does not).
 *   steady state (no allocation, no synchronization, no host reads: safe inside HIP graph capture):
 *       rq_w4a4_mul_mat() on the prepared weights.
 *
 * Return values: 0 = success; > 0 = a hipError_t; < 0 = one of the RQ_E_* codes below.
 */
#ifndef RQ_W4A4_H
#define RQ_W4A4_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RQ_TYPE_W4A4   44   /* GGML_TYPE_W4A4  (P:10) */
#define RQ_TYPE_W4A4H  45   /* GGML_TYPE_W4A4H (P:11) */
#define RQ_TYPE_A4     46   /* GGML_TYPE_A4    (P:12) */
#define RQ_TYPE_A4H    47   /* GGML_TYPE_A4H   (P:13) */

#define RQ_BLOCK_CODES 256  /* QK_W4A4 (P:38) */
#define RQ_BLOCK_BYTES 144  /* sizeof(block_w4a4) (P:44-50) */
#define RQ_MAX_K       32768 /* QK_W4A4 * RQ_MAX_BLOCKS (P:1748, P:1982) */

#define RQ_E_UNSUPPORTED  (-1)  /* shape/type the op does not take (the reference says so via supports_op) */
#define RQ_E_WORKSPACE    (-2)  /* workspace or prepared buffer too small or misaligned */
#define RQ_E_ARGUMENT     (-3)  /* null pointer, bad clip, bad rotation length */
#define RQ_E_LIMIT        (-4)  /* rq_w4a4_mul_mat_static: the problem needs more than RQ_STATIC_SCRATCH_BYTES */

typedef void *rq_stream_t;

/* block_w4a4 as stored in a W4A4 / W4A4H tensor (P:44-50). */
typedef struct {
    float    d;       /* row unit s_w, repeated in every block of the row */
    int32_t  sum;     /* 1<<30 | k, or 3<<29 | k0 | k1<<4 | k2<<8 | k3<<12, or the legacy row code sum (k = 1) */
    int32_t  pad[2];  /* pad[0] = row length (W4A4) / Hadamard length (W4A4H); pad[1] = clip as float bits */
    uint32_t qs[32];  /* element 8w+j in bits [4j+3:4j] of qs[w] */
} rq_block_w4a4;

/* ---- host-side queries (no GPU work) -------------------------------------------------------------- */

/* Replaces ggml_cuda_rq_w4a4_supported (P:1977-1994): 1 if rq_w4a4_mul_mat takes this problem.
 * src1 / dst must be fp32 with element stride 4; ldx_bytes / ldy_bytes are their row strides in bytes. */
int rq_w4a4_supported(int type, int64_t K, int64_t N, int64_t M, int64_t ldx_bytes, int64_t ldy_bytes);

/* Replaces ggml_rq_hadamard_factor (P:2419-2430). Returns 1 and n = p * m, else 0. */
int rq_w4a4_hadamard_factor(int64_t n, int *p, int *m);

/* Replaces ggml_rq_act_clip_for(ggml_rq_tensor_clip(blocks), had) (P:2590-2606): RQ_ACT_CLIP[_H] from the
 * environment (read once per process, as the reference does), else the header's pad[1], else 1.
 * host_block0 points at the first 16 bytes (or more) of the tensor, in host memory. */
float rq_w4a4_resolve_clip(const void *host_block0, int type);

/* Replaces ggml_rq_tensor_rot / ggml_rq_rot_check (P:2608-2620): the Hadamard length in pad[0] if it is
 * positive, divides K and factors; -1 where the reference aborts. For RQ_TYPE_W4A4 returns 0. */
int64_t rq_w4a4_tensor_rot(const void *host_block0, int type, int64_t K);

/* Replaces ggml_rq_act_group (P:2623-2631): 64, or RQ_ACT_GROUP = 128 / 256 (read once). */
int rq_w4a4_act_group(void);

/* The weight-multiplier encoding of a tensor, from block 0's sum field (RQ_W_MULT / RQ_W_MULT_G, P:40-43): 0 = legacy
 * row code sum (multiplier 1), 256 = one multiplier per block (1 << 30 | k), 64 = one per 64 inputs (3 << 29 | ...).
 * Weight groups of 64 need activation groups of 64: ggml_vec_dot_w4a4_a4 asserts it (P:169-170), so a caller's first
 * use refuses such a tensor when rq_w4a4_act_group() != 64 (the adapter aborts, the Python host raises). */
int rq_w4a4_weight_group(const void *host_block0);

/* ---- first use ------------------------------------------------------------------------------------ */

/* Bytes of the prepared (streaming) form of an N x K weight; a multiple of 256. */
size_t rq_w4a4_prepared_bytes(int64_t K, int64_t N);

/* Replaces rq_repack_once (P:2046-2075), out of place: reads N rows of K/256 blocks at w_blocks_dev, writes
 * prepared_dev (256-byte aligned, rq_w4a4_prepared_bytes). The input is not modified. Outside graph capture the
 * call ends by waiting for `stream` and reading one word of the result back: whether the tensor carries weight
 * multipliers, which the wide-batch launcher remembers per prepared address to choose between two kernels (both are
 * right for every tensor; a prepared weight that is copied to another address, or prepared under capture, runs the
 * one that is slow on tensors with multipliers). */
int rq_w4a4_prepare(const void *w_blocks_dev, int64_t K, int64_t N,
                    void *prepared_dev, size_t prepared_bytes, rq_stream_t stream);

/* The same rewrite IN PLACE, as the reference does it (rq_repack_once, P:2046-2075): afterwards w_blocks_dev is the
 * prepared weight (pass it as prepared_dev) and no longer readable as blocks, so one copy of the codes is resident
 * instead of two. The codes, row scales, multipliers and flag word take 33 bytes per 64 codes against the blocks' 36
 * and so fit where the blocks were (RQ_E_WORKSPACE for the few tiny shapes where the padding to 64 rows does not). The
 * fp6 plane of the wide-batch kernel does not fit there: it goes to plane6_dev, rq_w4a4_plane6_bytes(K, N) bytes that
 * the caller owns for as long as the weight is used (0 bytes and a null pointer under RQ_GEMM_FP6=0). staging_dev: at
 * least rq_w4a4_inplace_staging_bytes(K, N) of scratch, free again when the stream has passed this call (a
 * workspace will do). w_blocks_dev, plane6_dev and staging_dev 256-byte aligned. First use only: not graph-safe. */
size_t rq_w4a4_plane6_bytes(int64_t K, int64_t N);
size_t rq_w4a4_inplace_staging_bytes(int64_t K, int64_t N);
int rq_w4a4_prepare_inplace(void *w_blocks_dev, int64_t K, int64_t N, void *plane6_dev, size_t plane6_bytes,
                            void *staging_dev, size_t staging_bytes, rq_stream_t stream);

/* ---- steady state --------------------------------------------------------------------------------- */

/* Scratch the op needs for this problem (quantized activations, multipliers, split-K sums); a multiple of
 * 256. The reference takes the same buffers from the backend pool (P:2106-2109, P:2232-2235). */
size_t rq_w4a4_workspace_bytes(int type, int64_t K, int64_t N, int64_t M);

/* Replaces ggml_cuda_mul_mat_rq_w4a4 (P:2341-2347, rq_mul_mat P:2145-2338):
 *   y[t][n] = W[n] . x[t], t < M, n < N, bit-identical to ggml_vec_dot_w4a4_a4 (P:148-177) on activations
 *   quantized by quantize_row_a4_clip / quantize_row_a4h_clip_n (P:2639-2679, P:2728-2736).
 * x_dev: M rows of K floats, row stride ldx floats (ldx * 4 a multiple of 16); y_dev: M rows of N floats,
 * row stride ldy floats. clip > 0 (rq_w4a4_resolve_clip); n_rot = rq_w4a4_tensor_rot (ignored for W4A4).
 * workspace_dev: 256-byte aligned, at least rq_w4a4_workspace_bytes; its contents need not be preserved
 * between calls, and two calls that overlap in time must not share it. */
int rq_w4a4_mul_mat(int type, const void *prepared_dev, int64_t K, int64_t N,
                    const float *x_dev, int64_t ldx, int64_t M,
                    float *y_dev, int64_t ldy,
                    float clip, int64_t n_rot,
                    void *workspace_dev, size_t workspace_bytes, rq_stream_t stream);

/* rq_w4a4_mul_mat for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): no counterpart in the reference, which takes its scratch from the backend pool.
 * Same arguments and results as rq_w4a4_mul_mat without the workspace: the scratch is a 16 MiB array inside the
 * library's code object (one copy per GPU, held until the process ends). Allocates nothing and frees nothing.
 * Returns RQ_E_LIMIT when rq_w4a4_workspace_bytes(type, K, N, M) exceeds RQ_STATIC_SCRATCH_BYTES (decode and
 * verify batches fit: K = 5120, N = 17408 up to 128 tokens; K = 32768, N = 65536 at 8). All calls on one GPU share
 * the array: calls that overlap in time on one GPU (two streams, two threads) race; serialize them or give the
 * others rq_w4a4_mul_mat with workspaces of their own. rq_w4a4_prepare on the same GPU must have run before (it
 * resolves the array's device address, which must not happen under capture). */
#define RQ_STATIC_SCRATCH_BYTES (16 << 20)
int rq_w4a4_mul_mat_static(int type, const void *prepared_dev, int64_t K, int64_t N,
                           const float *x_dev, int64_t ldx, int64_t M,
                           float *y_dev, int64_t ldy,
                           float clip, int64_t n_rot, rq_stream_t stream);

/* rq_w4a4_mul_mat in its two stages, for the reference's shared quantized activation (rq_act_cache, P:1996-2023,
 * P:2160-2172): consecutive MUL_MATs of one x (q / k / v, gate / up) that were not fused rotate and quantize x once.
 * stages = 1: activation transform only (Hadamard + quantizer; also clears the split-K cells of N rows);
 * stages = 2: product + epilogue only, on a workspace that a stages-1 or stages-3 call filled for the same type, K, M,
 *             x, clip and n_rot and for at least as many weight rows (cells of more rows were not cleared);
 * stages = 3: both (identical to rq_w4a4_mul_mat). The workspace must have been zero-filled once when it was
 * allocated if stage 2 is ever used on it with a different N than the filling call. One token on the one-launch
 * decode path has no separate activation stage: stage 1 does nothing there and stage 2 is the whole operator.
 * bench.py also uses the split to time the product kernel alone. */
int rq_w4a4_mul_mat_stages(int type, const void *prepared_dev, int64_t K, int64_t N,
                           const float *x_dev, int64_t ldx, int64_t M,
                           float *y_dev, int64_t ldy,
                           float clip, int64_t n_rot,
                           void *workspace_dev, size_t workspace_bytes, rq_stream_t stream, int stages);

/* Replaces ggml_cuda_mul_mat_rq_w4a4_fused (P:2371-2380): n <= 3 weights of one type, K, clip and rotation
 * length against the same x (q/k/v, gate/up): one activation transform, then the products.
 * workspace: rq_w4a4_workspace_bytes for N = the sum of the weights' row counts, each rounded up to 64: the streaming
 * kernels (M <= 64) then serve all the weights from one launch, as the reference's skinny kernel does. A workspace
 * sized for the largest N alone is also accepted; the products are then launched one per weight. */
int rq_w4a4_mul_mat_fused(int type, int n, const void *const *prepared_dev, int64_t K, const int64_t *N,
                          const float *x_dev, int64_t ldx, int64_t M,
                          float *const *y_dev, const int64_t *ldy,
                          float clip, int64_t n_rot,
                          void *workspace_dev, size_t workspace_bytes, rq_stream_t stream);

/* ---- the activation side on its own (the A4 / A4H from_float of the CPU type traits, P:71-88) ------- */

/* Replaces ggml_rq_hadamard per rotation block (P:2450-2485, P:2697-2699): out[t] = x[t] diag(H, H, ...),
 * M rows of K floats, each n_rot-long block rotated; out row stride ldo floats. */
int rq_w4a4_hadamard(const float *x_dev, int64_t ldx, int64_t M, int64_t K, int64_t n_rot,
                     float *out_dev, int64_t ldo, rq_stream_t stream);

/* Replaces quantize_row_a4_clip / quantize_row_a4h_clip_n (P:2639-2679, P:2728-2736): writes M rows of
 * K/256 activation blocks in the reference's A4 / A4H storage layout (byte-identical to the CPU's work
 * buffer). type is RQ_TYPE_A4 (no rotation) or RQ_TYPE_A4H. */
int rq_w4a4_quantize_act(int type, const float *x_dev, int64_t ldx, int64_t M, int64_t K,
                         float clip, int64_t n_rot, void *blocks_dev, rq_stream_t stream);

/* ---- on-disk format tools (host memory, no GPU work) --------------------------------------------- */

/* Replaces `pack` of the reference's converter (src/gptq.rs:210-231): N rows of K int4 codes (as int8, -8..7) and
 * one scale per row -> N * K/256 blocks with d = scale, sum = the row's code sum (legacy header, multiplier 1),
 * pad[0] = K, pad[1] = 0. */
int rq_w4a4_pack(const int8_t *codes, const float *scales, int64_t N, int64_t K, void *blocks);

/* Replaces `pack_groups` (src/gptq.rs:193-207): as rq_w4a4_pack, then sum = 1<<30 | k (mults_per_block = 1) or
 * 3<<29 | k0 | k1<<4 | k2<<8 | k3<<12 (mults_per_block = 4); mults holds mults_per_block bytes per block. */
int rq_w4a4_pack_groups(const int8_t *codes, const float *units, const uint8_t *mults, int mults_per_block,
                        int64_t N, int64_t K, void *blocks);

/* Replaces the block loop of `ruquant setclip` (src/convert.rs:876-878): activation clip into pad[1] of every
 * block; 0 clears it (back to 1, or the environment). */
void rq_w4a4_set_clip(void *blocks, int64_t n_blocks, float clip);

/* Replaces `set_rot_len` (src/convert.rs:99-101): Hadamard length into pad[0] of every block. */
void rq_w4a4_set_rot_len(void *blocks, int64_t n_blocks, int32_t n);

/* Replaces dequantize_row_w4a4 (P:2738-2742), the type's to_float: y = code * ((float) k_g * d) for N rows of K. */
int rq_w4a4_dequantize_rows(const void *blocks, int64_t N, int64_t K, float *out);

/* Replaces quantize_row_w4a4_ref / quantize_row_w4a4h_ref (P:2681-2683, P:2701-2710; the types' from_float_ref) and
 * the row loops of quantize_w4a4 / quantize_w4a4h (P:2775-2789) for a whole tensor on the GPU: N rows of K floats at
 * w_dev (row stride ldw floats, 16-byte aligned) -> N * K/256 blocks at blocks_dev, bit-identical to the reference's
 * output. W4A4H rows are rotated first (x diag(H_n_rot, ...), P:2697-2699); n_rot is the reference's K / RQ_ROT_BLOCKS
 * (P:2687-2694) and lands in pad[0]. wgroup is the reference's RQ_WGROUP switch (P:2531-2538): 0 = one scale per row
 * from the 13-ratio clip search (P:2509-2527) and the legacy row-sum header; 256 or 64 = a scale per block or per 64
 * inputs, stored as multipliers 1..15 of the row's unit (P:2555-2575). No allocation, no synchronization. */
size_t rq_w4a4_quantize_weights_workspace_bytes(int type, int64_t K, int64_t N, int wgroup);
int rq_w4a4_quantize_weights(int type, const float *w_dev, int64_t ldw, int64_t N, int64_t K, int64_t n_rot, int wgroup,
                             void *blocks_dev, void *workspace_dev, size_t workspace_bytes, rq_stream_t stream);

/* Replaces dequantize_row_w4a4 / _w4a4h / _a4 / _a4h (P:2738-2773; the types' to_float) on the GPU: rows x K/256
 * blocks of `type` (44..47) at blocks_dev -> rows of K floats at out_dev (row stride ldo floats). The rotated types
 * are taken back to the original basis with the transposed Hadamard of length n_rot, which the caller reads from
 * block 0 as the reference does (pad[0] of weights, pad[1] of activations; P:2757-2763); other types ignore n_rot. */
int rq_w4a4_dequantize(int type, const void *blocks_dev, int64_t rows, int64_t K, int64_t n_rot, float *out_dev,
                       int64_t ldo, rq_stream_t stream);

/* Which stages of rq_w4a4_mul_mat_stages launch kernels for this problem: bit 0 = stage 1 (activation side), bit 1 =
 * stage 2 (products). 2 for a one-token call that the single-launch kernel takes (stage 1 is then a no-op), 3
 * otherwise, 0 for arguments the operator refuses. No counterpart in the reference (its act cache is internal,
 * P:2163-2172); for hosts and benchmarks that time or capture the stages separately. */
int rq_w4a4_stage_mask(int type, int64_t K, int64_t M, int64_t n_rot);

/* Library version, for the host binding to check: bumped whenever an entry point, an error code or the meaning of an
 * argument changes. A binding built against this header refuses a library that reports another number. */
#define RQ_ABI_VERSION 3
int rq_w4a4_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif
