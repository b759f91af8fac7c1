#include "rq_ggml_adapter.h"

#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>

namespace {

// what the reference keeps per weight after its first use (rq_tensor_info, P:1820-1826)
struct rq_first_use {
    float   clip;
    int64_t n_rot;
    void   *prepared;        // the tensor's own buffer (prepared in place) or a buffer of this struct's
    size_t  prepared_bytes;
    void   *plane6;          // in place: the fp6 plane of the wide-batch kernel, which does not fit the tensor's buffer
    bool    owns_prepared;
};

[[noreturn]] void rq_abort(const char *what, long long a = 0, long long b = 0) {
    fprintf(stderr, "ruquant W4A4: %s (%lld, %lld)\n", what, a, b);
    abort();
}

void hip_check(hipError_t e, const char *what) {
    if (e != hipSuccess) {
        fprintf(stderr, "ruquant W4A4: %s: %s\n", what, hipGetErrorString(e));
        abort();
    }
}

bool is_rq_type(int t) { return t == RQ_GGML_TYPE_W4A4 || t == RQ_GGML_TYPE_W4A4H; }

bool contiguous_blocks(const rq_tensor *t) {
    const size_t row = (size_t) (t->ne[0] / RQ_BLOCK_CODES) * RQ_BLOCK_BYTES;
    return t->nb[0] == RQ_BLOCK_BYTES && t->nb[1] == row;
}

bool capturing(rq_backend_context &ctx) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t) ctx.stream, &st) != hipSuccess) return false;
    return st != hipStreamCaptureStatusNone;
}

// Makes the scratch buffer at least `bytes` long. Growing synchronizes, frees and allocates, none of which may happen
// under graph capture: there the call aborts with a message instead (first_use sizes the buffer for max_tokens, so a
// steady-state call gets here only with more tokens than the context was told to expect).
void *scratch(rq_backend_context &ctx, size_t bytes) {
    if (ctx.scratch_bytes < bytes) {
        if (capturing(ctx)) {
            rq_abort("scratch too small under graph capture: raise rq_backend_context::max_tokens", (long long) bytes,
                     (long long) ctx.scratch_bytes);
        }
        hip_check(hipStreamSynchronize((hipStream_t) ctx.stream), "scratch");
        if (ctx.scratch) hip_check(hipFree(ctx.scratch), "scratch");
        hip_check(hipMalloc(&ctx.scratch, bytes), "scratch");
        // the split-K cells inside must read zero before their first use (the kernels leave them zero)
        hip_check(hipMemsetAsync(ctx.scratch, 0, bytes, (hipStream_t) ctx.stream), "scratch");
        ctx.scratch_bytes = bytes;
        ctx.act.valid = false;
    }
    return ctx.scratch;
}

// largest workspace any token count up to max_tokens needs for this weight
size_t workspace_for(int type, int64_t K, int64_t N, int64_t max_tokens) {
    size_t need = 0;
    const int64_t probes[] = { 1, 3, 4, 8, 9, 16, 17, 64, 65, max_tokens };
    for (int64_t m : probes) {
        if (m > max_tokens) continue;
        const size_t b = rq_w4a4_workspace_bytes(type, K, N, m);
        if (b > need) need = b;
    }
    return need;
}

// first use, never inside a graph capture: read block 0's header, resolve clip and rotation length, prepare
rq_first_use *first_use(rq_backend_context &ctx, const rq_tensor *src0) {
    if (src0->extra) return (rq_first_use *) src0->extra;
    if (rq_w4a4_abi_version() != RQ_ABI_VERSION) {
        rq_abort("librq_w4a4.so is not the version this adapter was built against", rq_w4a4_abi_version(), RQ_ABI_VERSION);
    }
    rq_block_w4a4 hdr;
    hipStream_t stream = (hipStream_t) ctx.stream;
    hip_check(hipMemcpyAsync(&hdr, src0->data, 16, hipMemcpyDeviceToHost, stream), "header read");
    hip_check(hipStreamSynchronize(stream), "header read");
    rq_first_use *fu = new rq_first_use;
    fu->clip = rq_w4a4_resolve_clip(&hdr, src0->type);
    fu->n_rot = rq_w4a4_tensor_rot(&hdr, src0->type, src0->ne[0]);
    if (fu->n_rot < 0) {
        rq_abort("W4A4H: Hadamard length does not divide this row slice (ruquant convert --rot-blocks)", hdr.pad[0],
                 src0->ne[0]);
    }
    if (rq_w4a4_weight_group(&hdr) == 64 && rq_w4a4_act_group() != 64) {
        // ggml_vec_dot_w4a4_a4 asserts the same (P:169-170): one weight multiplier per activation group
        rq_abort("weight groups of 64 need activation groups of 64 (RQ_ACT_GROUP)", rq_w4a4_act_group());
    }
    const int64_t K = src0->ne[0], N = src0->ne[1];
    fu->prepared_bytes = rq_w4a4_prepared_bytes(K, N);
    fu->plane6 = nullptr;
    fu->owns_prepared = true;
    // the workspace of every later call with up to max_tokens tokens: allocated now, outside capture; it also stages
    // the in-place rewrite
    size_t ws_bytes = workspace_for(src0->type, K, N, ctx.max_tokens);
    const size_t staging = rq_w4a4_inplace_staging_bytes(K, N);
    if (ctx.in_place && staging > ws_bytes) ws_bytes = staging;
    void *ws = scratch(ctx, ws_bytes);
    int rc = RQ_E_WORKSPACE;
    if (ctx.in_place && (reinterpret_cast<uintptr_t>(src0->data) & 255) == 0) {
        const size_t n6 = rq_w4a4_plane6_bytes(K, N);
        if (n6) hip_check(hipMalloc(&fu->plane6, n6), "fp6 plane");
        rc = rq_w4a4_prepare_inplace(src0->data, K, N, fu->plane6, n6, ws, ctx.scratch_bytes, ctx.stream);
        if (rc == 0) {
            fu->prepared = src0->data;
            fu->owns_prepared = false;
            // the staging area held blocks: the split-K cells inside the scratch must read zero again
            hip_check(hipMemsetAsync(ctx.scratch, 0, ctx.scratch_bytes, stream), "scratch");
            ctx.act.valid = false;
        } else if (rc != RQ_E_WORKSPACE) {
            rq_abort("rq_w4a4_prepare_inplace failed", rc);
        } else if (fu->plane6) {   // (a shape whose prepared form does not fit its blocks: out of place after all)
            hip_check(hipFree(fu->plane6), "fp6 plane");
            fu->plane6 = nullptr;
        }
    }
    if (rc != 0) {
        hip_check(hipMalloc(&fu->prepared, fu->prepared_bytes), "prepared weight");
        rc = rq_w4a4_prepare(src0->data, K, N, fu->prepared, fu->prepared_bytes, ctx.stream);
        if (rc != 0) rq_abort("rq_w4a4_prepare failed", rc);
    }
    const_cast<rq_tensor *>(src0)->extra = fu;
    return fu;
}

}  // namespace

rq_backend_context::~rq_backend_context() {
    if (scratch) (void) hipFree(scratch);
}

bool ggml_cuda_rq_w4a4_supported(int cc, const rq_tensor *src0, const rq_tensor *src1, const rq_tensor *dst) {
    (void) cc;
    return is_rq_type(src0->type) && src1->type == RQ_GGML_TYPE_F32 && dst->type == RQ_GGML_TYPE_F32 &&
           src0->ne[2] == 1 && src0->ne[3] == 1 && src1->ne[2] == 1 && src1->ne[3] == 1 && contiguous_blocks(src0) &&
           src1->nb[0] == sizeof(float) && dst->nb[0] == sizeof(float) && src1->ne[0] == src0->ne[0] &&
           rq_w4a4_supported(src0->type, src0->ne[0], src0->ne[1], src1->ne[1], (int64_t) src1->nb[1],
                             (int64_t) dst->nb[1]) != 0;
}

bool ggml_cuda_rq_w4a4_ready(const rq_tensor *src0) { return src0->extra != nullptr; }

void ggml_cuda_mul_mat_rq_w4a4_fused(rq_backend_context &ctx, const rq_tensor *const *src0s, rq_tensor *const *dsts, int n,
                                     const rq_tensor *src1) {
    if (n < 1 || n > 3) rq_abort("fused call takes 1..3 weights", n);
    const void *prepared[3];
    float *ys[3];
    int64_t Ns[3], ldys[3];
    const rq_first_use *fu0 = nullptr;
    int64_t Nmax = 0;
    for (int i = 0; i < n; ++i) {
        const rq_first_use *fu = first_use(ctx, src0s[i]);
        if (i == 0) fu0 = fu;
        if (src0s[i]->type != src0s[0]->type || src0s[i]->ne[0] != src0s[0]->ne[0] || fu->clip != fu0->clip ||
            fu->n_rot != fu0->n_rot) {
            rq_abort("fused weights must share type, K, clip and rotation length");
        }
        prepared[i] = fu->prepared;
        ys[i] = (float *) dsts[i]->data;
        Ns[i] = src0s[i]->ne[1];
        ldys[i] = (int64_t) (dsts[i]->nb[1] / sizeof(float));
        if (Ns[i] > Nmax) Nmax = Ns[i];
    }
    const int64_t K = src0s[0]->ne[0], M = src1->ne[1];
    // split-K cells for the rows of all weights (each padded to 64): the streaming kernels then take one launch
    int64_t Nws = Nmax;
    if (n > 1) {
        Nws = 0;
        for (int i = 0; i < n; ++i) Nws += (Ns[i] + 63) / 64 * 64;
    }
    size_t ws_bytes = rq_w4a4_workspace_bytes(src0s[0]->type, K, Nws, M);
    if (ws_bytes > ctx.scratch_bytes && n > 1 && capturing(ctx)) {
        // a fused set that was not sized for: cells for the largest weight are enough (one product launch per weight)
        ws_bytes = rq_w4a4_workspace_bytes(src0s[0]->type, K, Nmax, M);
        Nws = Nmax;
    }
    void *ws = scratch(ctx, ws_bytes);
    const int type = src0s[0]->type;
    const float *x = (const float *) src1->data;
    const int64_t ldx = (int64_t) (src1->nb[1] / sizeof(float));
    rq_act_cache &c = ctx.act;
    int rc;
    if (n == 1 && c.valid && c.src1 == src1 && c.data == src1->data && c.type == type && c.clip == fu0->clip &&
        c.n_rot == fu0->n_rot && c.K == K && c.M == M && (Ns[0] + 63) / 64 * 64 <= c.rows_cleared) {
        // the scratch still holds this x rotated and quantized: the product alone (reference: P:2167-2172)
        ++ctx.act_hits;
        rc = rq_w4a4_mul_mat_stages(type, prepared[0], K, Ns[0], x, ldx, M, ys[0], ldys[0], fu0->clip, fu0->n_rot, ws,
                                    ctx.scratch_bytes, ctx.stream, 2);
    } else {
        ++ctx.act_misses;
        rc = rq_w4a4_mul_mat_fused(type, n, prepared, K, Ns, x, ldx, M, ys, ldys, fu0->clip, fu0->n_rot, ws, ws_bytes,
                                   ctx.stream);
        c.src1 = src1;
        c.data = src1->data;
        c.type = type;
        c.clip = fu0->clip;
        c.n_rot = fu0->n_rot;
        c.K = K;
        c.M = M;
        // (a fused call may have cleared the cells of all its weights; the largest one is what it surely cleared)
        c.rows_cleared = (Nmax + 63) / 64 * 64;
        c.valid = rc == 0;
    }
    if (rc != 0) rq_abort("no path for this shape", rc);   // the reference: GGML_ABORT (P:2337)
}

void ggml_cuda_mul_mat_rq_w4a4(rq_backend_context &ctx, const rq_tensor *src0, const rq_tensor *src1, rq_tensor *dst) {
    ggml_cuda_mul_mat_rq_w4a4_fused(ctx, &src0, &dst, 1, src1);
}

bool ggml_cuda_rq_w4a4_can_fuse(const rq_tensor *a, const rq_tensor *b) {
    if (a->op != RQ_GGML_OP_MUL_MAT || b->op != RQ_GGML_OP_MUL_MAT) return false;
    const rq_tensor *wa = a->src[0], *wb = b->src[0], *x = a->src[1];
    if (b->src[1] != x || !is_rq_type(wa->type) || wb->type != wa->type || wb->ne[0] != wa->ne[0] ||
        x->type != RQ_GGML_TYPE_F32 || x->ne[2] != 1 || x->ne[3] != 1 || x->ne[1] > 16 ||
        a->type != RQ_GGML_TYPE_F32 || b->type != RQ_GGML_TYPE_F32) {
        return false;
    }
    // both weights seen before: a first use synchronizes, so it stays unfused
    const rq_first_use *ia = (const rq_first_use *) wa->extra, *ib = (const rq_first_use *) wb->extra;
    return ia != nullptr && ib != nullptr && ia->clip == ib->clip && ia->n_rot == ib->n_rot;
}

void ggml_cuda_rq_graph_begin(rq_backend_context &ctx) { ctx.act.valid = false; }

void ggml_cuda_rq_w4a4_release(rq_tensor *src0) {
    rq_first_use *fu = (rq_first_use *) src0->extra;
    if (!fu) return;
    if (fu->owns_prepared) (void) hipFree(fu->prepared);
    if (fu->plane6) (void) hipFree(fu->plane6);
    delete fu;
    src0->extra = nullptr;
}
