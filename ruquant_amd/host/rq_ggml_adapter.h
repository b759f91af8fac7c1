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

// Stands in for ggml_backend_cuda_context: the stream every launch goes to and a scratch pool. The pool here is
// one growing device buffer owned by the context (ggml's is stream ordered; the op only needs "memory that stays
// valid until the stream has passed this call").
struct rq_backend_context {
    void  *stream = nullptr;
    void  *scratch = nullptr;
    size_t scratch_bytes = 0;
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
// starts a new graph evaluation (reference: P:2021-2023). This implementation keeps no cross-call activation cache,
// so there is nothing to drop.
void ggml_cuda_rq_graph_begin(rq_backend_context &ctx);
