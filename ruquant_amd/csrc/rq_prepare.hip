// One-time rewrite of a W4A4 / W4A4H tensor (rows of 144-byte blocks) into the streaming layout described in
// rq_common.h, and into the fp6 fragment plane of the wide-batch MFMA kernel. Out of place: the tensor's own bytes
// stay valid ggml blocks.
#include "rq_common.h"

namespace rq {

namespace {

// weight multiplier of 64-input group sg of a block, from the header's sum field (reference patch lines 40-43)
__device__ __forceinline__ int weight_mult(uint32_t sum, int sg) {
    if ((sum >> 29) == 3u) return (int) ((sum >> (4 * sg)) & 0xF);
    if ((sum >> 30) == 1u) return (int) (sum & 0xF);
    return 1;
}

__global__ void rq_clear_flags_kernel(int32_t *flags) {
    if (threadIdx.x < 64) flags[threadIdx.x] = 0;
}

// one thread per (padded row, group): 32 bytes of codes in, two 16-byte halves out
__global__ void __launch_bounds__(256) rq_prepare_kernel(const rq_block_w4a4 *__restrict__ blocks, int64_t N, int ng,
                                                         int n_panels, uint4 *__restrict__ codes,
                                                         float *__restrict__ s_w, uint8_t *__restrict__ kmul,
                                                         int32_t *__restrict__ flags) {
    const int64_t idx = (int64_t) blockIdx.x * 256 + threadIdx.x;
    const int64_t total = (int64_t) n_panels * kPanelRows * ng;
    if (idx >= total) return;
    const int g = (int) (idx % ng);
    const int64_t n = idx / ng;
    const int panel = (int) (n / kPanelRows), r = (int) (n % kPanelRows);
    uint4 lo = make_uint4(0, 0, 0, 0), hi = lo;
    int kw = 1;
    float d = 0.0f;
    if (n < N) {
        const rq_block_w4a4 *blk = blocks + n * (ng / 4) + (g >> 2);
        const uint4 *q = reinterpret_cast<const uint4 *>(blk->qs) + (g & 3) * 2;
        lo = q[0];
        hi = q[1];
        kw = weight_mult((uint32_t) blk->sum, g & 3);
        d = blk->d;
    }
    const size_t cell = (size_t) panel * ng + g;
    codes[(cell * 2 + 0) * kPanelRows + r] = lo;
    codes[(cell * 2 + 1) * kPanelRows + r] = hi;
    kmul[cell * kPanelRows + r] = (uint8_t) kw;
    if (g == 0) s_w[n] = d;
    if (kw != 1) atomicOr(flags, 1);
}

// fp6 plane: one thread per (padded row, group, half): 32 int4 codes in, 32 sign-magnitude six-bit values out
__global__ void __launch_bounds__(256) rq_prepare6_kernel(const rq_block_w4a4 *__restrict__ blocks, int64_t N, int ng,
                                                          int n_rtiles, uint8_t *__restrict__ w6) {
    const int64_t idx = (int64_t) blockIdx.x * 256 + threadIdx.x;
    const int64_t total = (int64_t) n_rtiles * kRowTile6 * ng * 2;
    if (idx >= total) return;
    // consecutive threads take consecutive rows, so that the 16- and 8-byte pieces they write are neighbours
    const int r32 = (int) (idx & 31);
    const int half = (int) ((idx >> 5) & 1);
    const int64_t rest = idx >> 6;
    const int g = (int) (rest % ng);
    const int64_t frag = rest / ng;                 // 32-row fragment of the whole tensor
    const int64_t n = frag * 32 + r32;
    uint32_t out[6] = { 0, 0, 0, 0, 0, 0 };
    if (n < N) {
        const rq_block_w4a4 *blk = blocks + n * (ng / 4) + (g >> 2);
        const uint4 q = reinterpret_cast<const uint4 *>(blk->qs)[(g & 3) * 2 + half];
        const uint32_t wds[4] = { q.x, q.y, q.z, q.w };
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            const int v = ((int) (wds[j >> 3] << (28 - 4 * (j & 7)))) >> 28;   // signed nibble
            const uint32_t code = v < 0 ? (32u | (uint32_t) (-v)) : (uint32_t) v;
            const int bit = 6 * j;
            out[bit >> 5] |= code << (bit & 31);
            if ((bit & 31) > 26) out[(bit >> 5) + 1] |= code >> (32 - (bit & 31));
        }
    }
    const int64_t rtile = frag >> 3;
    const int f = (int) (frag & 7);
    uint8_t *dst = w6 + (((size_t) rtile * ng + g) * 8 + f) * kFrag6;
    const int lane = r32 + 32 * half;
    *reinterpret_cast<uint4 *>(dst + lane * 16) = make_uint4(out[0], out[1], out[2], out[3]);
    *reinterpret_cast<uint2 *>(dst + 1024 + lane * 8) = make_uint2(out[4], out[5]);
}

}  // namespace

hipError_t launch_prepare(const void *blocks, const PreparedLayout &L, uint8_t *prepared, hipStream_t stream) {
    int32_t *flags = reinterpret_cast<int32_t *>(prepared + L.off_flags);
    hipLaunchKernelGGL(rq_clear_flags_kernel, dim3(1), dim3(64), 0, stream, flags);
    const int64_t total = (int64_t) L.n_panels * kPanelRows * L.ng;
    const int grid = (int) ((total + 255) / 256);
    hipLaunchKernelGGL(rq_prepare_kernel, dim3(grid), dim3(256), 0, stream,
                       reinterpret_cast<const rq_block_w4a4 *>(blocks), L.N, L.ng, L.n_panels,
                       reinterpret_cast<uint4 *>(prepared + L.off_codes),
                       reinterpret_cast<float *>(prepared + L.off_sw), prepared + L.off_kmul, flags);
    if (L.off_w6 != 0) {
        const int64_t total6 = (int64_t) L.n_rtiles * kRowTile6 * L.ng * 2;
        hipLaunchKernelGGL(rq_prepare6_kernel, dim3((unsigned) ((total6 + 255) / 256)), dim3(256), 0, stream,
                           reinterpret_cast<const rq_block_w4a4 *>(blocks), L.N, L.ng, L.n_rtiles, prepared + L.off_w6);
    }
    return hipGetLastError();
}

}  // namespace rq
