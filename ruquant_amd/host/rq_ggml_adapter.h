// The reference's backend entry points for W4A4 / W4A4H MUL_MAT (rq-w4a4.cuh, lines 2391-2401 of
// patches/llama.cpp-ruquant.patch), with the same names, argument meaning and error behaviour, over the C ABI of
// include/rq_w4a4.h. `rq_tensor` mirrors the fields of ggml_tensor that the op reads, so that in a ggml-hip build the
// bodies below work on ggml_tensor unchanged (type, ne, nb, data, extra, op, src).
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "../../include/rq_w4a4.h"

enum rq_ggml_type { RQ_GGML_TYPE_F32 = 0, RQ_GGML_TYPE_W4A4 = RQ_TYPE_W4A4, RQ_GGML_TYPE_W4A4H = RQ_TYPE_W4A4H };
enum rq_ggml_op { RQ_GGML_OP_NONE = 0, RQ_GGML_OP_MUL_MAT = 1 };

struct rq_tensor {
    int        type;
    int        op;
    int64_t    ne[4];   // elements per dimension: weights {K, N, 1, 1}, activations {K, M, 1, 1}, output {N, M, 1, 1}
    size_t     nb[4];   // strides in bytes
    void      *data;    // device memory
    void      *extra;   // first-use state of a weight (the reference's rq_tensor_info)
    rq_tensor *src[2];
};

// The quantized activation the scratch buffer currently holds (the reference's rq_act_cache, P:1996-2023): consecutive
// MUL_MATs of one x (q / k / v, gate / up) that were not fused still share one rotation + quantization. Keyed like
// the reference's (P:2163-2166) on the src1 tensor, its data pointer, the type and the weight-side parameters; dropped
// at every graph evaluation (ggml_cuda_rq_graph_begin), because x may have changed in place since.
struct rq_act_cache {
    const void *src1 = nullptr, *data = nullptr;
    int         type = 0;
    float       clip = 0.0f;
    int64_t     n_rot = 0, K = 0, M = 0;
    int64_t     rows_cleared = 0;   // split-K cells of this many weight rows were cleared when the activation was made
    bool        valid = false;
};

// Stands in for ggml_backend_cuda_context: the stream every launch goes to and a scratch pool. The pool here is
// one device buffer owned by the context (ggml's is stream ordered; the op only needs "memory that stays valid until
// the stream has passed this call"). It is sized at a weight's first use, which is outside graph capture, for every
// token count up to max_tokens (the backend's micro-batch), so that steady-state calls never allocate; a call that
// needs more grows it when the stream is not capturing and aborts with a message when it is.
struct rq_backend_context {
    void        *stream = nullptr;
    void        *scratch = nullptr;
    size_t       scratch_bytes = 0;
    int64_t      max_tokens = 512;
    // first use rewrites a weight's own buffer into the prepared form, as the reference does (P:2046-2075): one copy of
    // the codes stays resident and the tensor is no longer readable as blocks. false: the prepared form goes to a
    // buffer of its own and the tensor's bytes stay valid ggml blocks (twice the memory).
    bool         in_place = true;
    rq_act_cache act;
    long long    act_hits = 0, act_misses = 0;
    ~rq_backend_context();
};

// true if the backend takes this MUL_MAT (reference: P:1977-1994). cc is unused on this single-target build.
bool ggml_cuda_rq_w4a4_supported(int cc, const rq_tensor *src0, const rq_tensor *src1, const rq_tensor *dst);
// false until the weight has been through its first use, which synchronizes and allocates and therefore must stay
// out of graph capture (reference: P:1972-1974)
bool ggml_cuda_rq_w4a4_ready(const rq_tensor *src0);
// dst = src0 x src1 (reference: P:2341-2347). Aborts on errors the reference aborts on.
void ggml_cuda_mul_mat_rq_w4a4(rq_backend_context &ctx, const rq_tensor *src0, const rq_tensor *src1, rq_tensor *dst);
// b can share a's activation transform: both MUL_MAT nodes of the same x, type, K, clip and rotation length, at
// most 16 tokens, both weights already used once (reference: P:2350-2369)
bool ggml_cuda_rq_w4a4_can_fuse(const rq_tensor *a, const rq_tensor *b);
// n <= 3 such products as one call (reference: P:2371-2380)
void ggml_cuda_mul_mat_rq_w4a4_fused(rq_backend_context &ctx, const rq_tensor *const *src0s, rq_tensor *const *dsts, int n,
                                     const rq_tensor *src1);
// starts a new graph evaluation (reference: P:2021-2023): drops the shared quantized activation
void ggml_cuda_rq_graph_begin(rq_backend_context &ctx);
// frees what a weight's first use allocated (the reference never frees its rq_tensor_info; a backend that unloads
// models calls this from its buffer-free path)
void ggml_cuda_rq_w4a4_release(rq_tensor *src0);
