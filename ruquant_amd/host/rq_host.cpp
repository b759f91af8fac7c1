// Host program over the adapter, in the role of the reference's Rust host (src/custom_op.rs, src/bench.rs): it owns
// the device buffers, builds the MUL_MAT node, runs it through the backend entry points and reports timings as JSON.
//
//   rq_host <type 44|45> <K> <N> <M> <weights.bin> <x.bin> <y.bin> [iters]
//
// weights.bin: N rows of K/256 blocks (144 bytes each) as a W4A4 / W4A4H tensor stores them; x.bin: M x K floats;
// y.bin (written): M x N floats. With three extra arguments "fuse <weights2.bin> <N2> <y2.bin>" a second weight of
// the same x goes through ggml_cuda_rq_w4a4_can_fuse / _fused. With "cache <weights2.bin> <N2> <y2.bin>" the two
// weights run as separate calls inside one graph evaluation (the second reuses the first's quantized activation),
// then x is negated in place and a new evaluation runs both again: y.bin / y2.bin hold the results for -x, and
// <y2.bin>.first the second weight's result of the first evaluation; the JSON carries the hit / miss counts.
#include "rq_ggml_adapter.h"

#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <chrono>
#include <string>
#include <vector>

#define CK(x)                                                                      \
    do {                                                                           \
        hipError_t e_ = (x);                                                       \
        if (e_ != hipSuccess) {                                                    \
            fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                \
            return 1;                                                              \
        }                                                                          \
    } while (0)

static bool read_file(const char *path, std::vector<char> &buf, size_t want) {
    FILE *f = fopen(path, "rb");
    if (!f) return false;
    buf.resize(want);
    const size_t got = fread(buf.data(), 1, want, f);
    fclose(f);
    return got == want;
}

static rq_tensor weight_tensor(int type, int64_t K, int64_t N, void *dev) {
    rq_tensor t;
    memset(&t, 0, sizeof t);
    t.type = type;
    t.ne[0] = K; t.ne[1] = N; t.ne[2] = t.ne[3] = 1;
    t.nb[0] = RQ_BLOCK_BYTES;
    t.nb[1] = (size_t) (K / RQ_BLOCK_CODES) * RQ_BLOCK_BYTES;
    t.nb[2] = t.nb[3] = t.nb[1] * (size_t) N;
    t.data = dev;
    return t;
}

static rq_tensor f32_tensor(int64_t cols, int64_t rows, void *dev) {
    rq_tensor t;
    memset(&t, 0, sizeof t);
    t.type = RQ_GGML_TYPE_F32;
    t.ne[0] = cols; t.ne[1] = rows; t.ne[2] = t.ne[3] = 1;
    t.nb[0] = sizeof(float);
    t.nb[1] = (size_t) cols * sizeof(float);
    t.nb[2] = t.nb[3] = t.nb[1] * (size_t) rows;
    t.data = dev;
    return t;
}

int main(int argc, char **argv) {
    if (argc < 8) {
        fprintf(stderr, "usage: %s type K N M weights.bin x.bin y.bin [iters] [fuse weights2.bin N2 y2.bin]\n", argv[0]);
        return 2;
    }
    const int type = atoi(argv[1]);
    const int64_t K = atoll(argv[2]), N = atoll(argv[3]), M = atoll(argv[4]);
    int iters = 20;
    int argi = 8;
    if (argc > argi && strcmp(argv[argi], "fuse") != 0) iters = atoi(argv[argi++]);
    const bool cache = argc > argi + 3 && strcmp(argv[argi], "cache") == 0;
    const bool fuse = argc > argi + 3 && (strcmp(argv[argi], "fuse") == 0 || cache);
    const int64_t N2 = fuse ? atoll(argv[argi + 2]) : 0;

    int n_dev = 0;
    CK(hipGetDeviceCount(&n_dev));
    if (n_dev < 1) {
        fprintf(stderr, "no HIP device\n");
        return 1;
    }
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));

    const size_t w_bytes = (size_t) N * (K / RQ_BLOCK_CODES) * RQ_BLOCK_BYTES, x_bytes = (size_t) M * K * 4;
    std::vector<char> wh, xh, w2h;
    if (!read_file(argv[5], wh, w_bytes) || !read_file(argv[6], xh, x_bytes)) {
        fprintf(stderr, "cannot read inputs\n");
        return 1;
    }
    void *wd, *xd, *yd, *w2d = nullptr, *y2d = nullptr;
    CK(hipMalloc(&wd, w_bytes));
    CK(hipMalloc(&xd, x_bytes));
    CK(hipMalloc(&yd, (size_t) M * N * 4));
    CK(hipMemcpy(wd, wh.data(), w_bytes, hipMemcpyHostToDevice));
    CK(hipMemcpy(xd, xh.data(), x_bytes, hipMemcpyHostToDevice));

    hipStream_t stream;
    CK(hipStreamCreate(&stream));
    rq_backend_context ctx;
    ctx.stream = stream;
    // RQ_HOST_IN_PLACE=0: keep the tensor's bytes as blocks and the prepared weight in a buffer of its own
    const char *ip = getenv("RQ_HOST_IN_PLACE");
    ctx.in_place = ip ? atoi(ip) != 0 : true;

    rq_tensor w = weight_tensor(type, K, N, wd), x = f32_tensor(K, M, xd), y = f32_tensor(N, M, yd);
    y.op = RQ_GGML_OP_MUL_MAT;
    y.src[0] = &w;
    y.src[1] = &x;
    if (!ggml_cuda_rq_w4a4_supported(0, &w, &x, &y)) {
        printf("{\"supported\": false}\n");   // ggml would schedule this node on the CPU backend
        return 3;
    }
    rq_tensor w2, y2;
    if (fuse) {
        const size_t w2_bytes = (size_t) N2 * (K / RQ_BLOCK_CODES) * RQ_BLOCK_BYTES;
        if (!read_file(argv[argi + 1], w2h, w2_bytes)) return 1;
        CK(hipMalloc(&w2d, w2_bytes));
        CK(hipMalloc(&y2d, (size_t) M * N2 * 4));
        CK(hipMemcpy(w2d, w2h.data(), w2_bytes, hipMemcpyHostToDevice));
        w2 = weight_tensor(type, K, N2, w2d);
        y2 = f32_tensor(N2, M, y2d);
        y2.op = RQ_GGML_OP_MUL_MAT;
        y2.src[0] = &w2;
        y2.src[1] = &x;
    }

    const bool ready_before = ggml_cuda_rq_w4a4_ready(&w);
    bool fused_ran = false;
    // first evaluation: first use of every weight, unfused (as the reference's graph gate forces). Device memory taken
    // by the first use of the LAST weight (the scratch buffer has its size by then when the weights have one shape) =
    // what stays resident for a weight besides its tensor.
    size_t free_before = 0, free_after = 0, total_mem = 0;
    ggml_cuda_rq_graph_begin(ctx);
    if (fuse) ggml_cuda_mul_mat_rq_w4a4(ctx, &w2, &x, &y2);
    CK(hipStreamSynchronize(stream));
    const size_t scratch_before = ctx.scratch_bytes;
    CK(hipMemGetInfo(&free_before, &total_mem));
    ggml_cuda_mul_mat_rq_w4a4(ctx, &w, &x, &y);
    CK(hipStreamSynchronize(stream));
    CK(hipMemGetInfo(&free_after, &total_mem));
    const long long first_use_bytes = (long long) free_before - (long long) free_after -
                                      ((long long) ctx.scratch_bytes - (long long) scratch_before);
    if (fuse) ggml_cuda_mul_mat_rq_w4a4(ctx, &w2, &x, &y2);   // (in the order of the graph: after w)
    CK(hipStreamSynchronize(stream));
    const bool ready_after = ggml_cuda_rq_w4a4_ready(&w);

    long long hits_first = 0, misses_first = 0, hits_again = 0, misses_again = 0;
    if (cache) {
        // one graph evaluation, two separate calls of the same x: the second finds x already rotated and quantized
        ctx.act_hits = ctx.act_misses = 0;
        ggml_cuda_rq_graph_begin(ctx);
        ggml_cuda_mul_mat_rq_w4a4(ctx, &w, &x, &y);
        ggml_cuda_mul_mat_rq_w4a4(ctx, &w2, &x, &y2);
        CK(hipStreamSynchronize(stream));
        hits_first = ctx.act_hits;
        misses_first = ctx.act_misses;
        {
            std::vector<float> y2h((size_t) M * N2);
            CK(hipMemcpy(y2h.data(), y2d, y2h.size() * 4, hipMemcpyDeviceToHost));
            const std::string first = std::string(argv[argi + 3]) + ".first";
            FILE *ff = fopen(first.c_str(), "wb");
            if (!ff || fwrite(y2h.data(), 4, y2h.size(), ff) != y2h.size()) return 1;
            fclose(ff);
        }
        // x changes in place between evaluations: the new evaluation must not reuse the old activation
        float *xf = reinterpret_cast<float *>(xh.data());
        for (size_t i = 0; i < (size_t) M * K; ++i) xf[i] = -xf[i];
        CK(hipMemcpy(xd, xh.data(), x_bytes, hipMemcpyHostToDevice));
        ctx.act_hits = ctx.act_misses = 0;
        ggml_cuda_rq_graph_begin(ctx);
        ggml_cuda_mul_mat_rq_w4a4(ctx, &w, &x, &y);
        ggml_cuda_mul_mat_rq_w4a4(ctx, &w2, &x, &y2);
        CK(hipStreamSynchronize(stream));
        hits_again = ctx.act_hits;
        misses_again = ctx.act_misses;
        iters = 0;
    }

    // steady state
    std::vector<double> times;
    for (int i = 0; i < iters; ++i) {
        const auto t0 = std::chrono::steady_clock::now();
        ggml_cuda_rq_graph_begin(ctx);
        if (fuse && !cache && ggml_cuda_rq_w4a4_can_fuse(&y, &y2)) {
            const rq_tensor *ws[2] = { &w, &w2 };
            rq_tensor *ds[2] = { &y, &y2 };
            ggml_cuda_mul_mat_rq_w4a4_fused(ctx, ws, ds, 2, &x);
            fused_ran = true;
        } else {
            ggml_cuda_mul_mat_rq_w4a4(ctx, &w, &x, &y);
            if (fuse) ggml_cuda_mul_mat_rq_w4a4(ctx, &w2, &x, &y2);
        }
        CK(hipStreamSynchronize(stream));
        times.push_back(std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count());
    }
    double best = 1e30, sum = 0;
    for (double t : times) { best = t < best ? t : best; sum += t; }

    std::vector<float> yh((size_t) M * N);
    CK(hipMemcpy(yh.data(), yd, yh.size() * 4, hipMemcpyDeviceToHost));
    FILE *f = fopen(argv[7], "wb");
    if (!f || fwrite(yh.data(), 4, yh.size(), f) != yh.size()) return 1;
    fclose(f);
    if (fuse) {
        std::vector<float> y2h((size_t) M * N2);
        CK(hipMemcpy(y2h.data(), y2d, y2h.size() * 4, hipMemcpyDeviceToHost));
        f = fopen(argv[argi + 3], "wb");
        if (!f || fwrite(y2h.data(), 4, y2h.size(), f) != y2h.size()) return 1;
        fclose(f);
    }
    printf("{\"supported\": true, \"device\": \"%s\", \"type\": %d, \"K\": %lld, \"N\": %lld, \"M\": %lld, "
           "\"ready_before\": %s, \"ready_after\": %s, \"fused\": %s, \"iters\": %d, \"best_us\": %.2f, \"mean_us\": %.2f, "
           "\"act_hits_first\": %lld, \"act_misses_first\": %lld, \"act_hits_again\": %lld, \"act_misses_again\": %lld, "
           "\"in_place\": %s, \"tensor_bytes\": %lld, \"first_use_bytes_beside_tensor\": %lld, \"plane6_bytes\": %lld, "
           "\"prepared_bytes\": %lld}\n",
           prop.name, type, (long long) K, (long long) N, (long long) M, ready_before ? "true" : "false",
           ready_after ? "true" : "false", fused_ran ? "true" : "false", iters, iters ? best : 0.0,
           iters ? sum / iters : 0.0, hits_first, misses_first, hits_again, misses_again, ctx.in_place ? "true" : "false",
           (long long) w_bytes, first_use_bytes, (long long) rq_w4a4_plane6_bytes(K, N),
           (long long) rq_w4a4_prepared_bytes(K, N));
    return 0;
}
