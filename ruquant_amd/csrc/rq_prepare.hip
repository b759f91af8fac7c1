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

// fp6 plane: one thread per (row, group, half) of the 32-row fragments frag0 .. frag0 + n_frags - 1 of the tensor: 32
// int4 codes in, 32 sign-magnitude six-bit values out. `blocks` points at the blocks of row `row0` (the whole tensor,
// or a staged chunk of it); rows from N on are written as zeros.
__global__ void __launch_bounds__(256) rq_prepare6_kernel(const rq_block_w4a4 *__restrict__ blocks, int64_t row0,
                                                          int64_t N, int ng, int64_t frag0, int64_t n_frags,
                                                          uint8_t *__restrict__ w6) {
    const int64_t idx = (int64_t) blockIdx.x * 256 + threadIdx.x;
    const int64_t total = n_frags * 32 * ng * 2;
    if (idx >= total) return;
    // consecutive threads take consecutive rows, so that the 16- and 8-byte pieces they write are neighbours
    const int r32 = (int) (idx & 31);
    const int half = (int) ((idx >> 5) & 1);
    const int64_t rest = idx >> 6;
    const int g = (int) (rest % ng);
    const int64_t frag = frag0 + rest / ng;         // 32-row fragment of the whole tensor
    const int64_t n = frag * 32 + r32;
    uint32_t out[6] = { 0, 0, 0, 0, 0, 0 };
    if (n < N) {
        const rq_block_w4a4 *blk = blocks + (n - row0) * (ng / 4) + (g >> 2);
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

// the flag word of a prepared weight and, beside it, the device address of its fp6 plane (0: none), which the fp6
// GEMM reads from here: the plane may live inside the prepared buffer or, for a weight prepared in place, elsewhere
__global__ void rq_finish_flags_kernel(int32_t *flags, const int32_t *from, const uint8_t *plane6) {
    const int32_t f = from ? from[0] : flags[0];
    if (threadIdx.x == 0) {
        flags[0] = f;
        *reinterpret_cast<unsigned long long *>(flags + 2) = (unsigned long long) (uintptr_t) plane6;
    }
    if (threadIdx.x < kFlagReplicas) flags[64 + 16 * threadIdx.x] = f;   // (the copies: a 64-byte line each)
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
        const int64_t n_frags = (int64_t) L.n_rtiles * 8;
        const int64_t total6 = n_frags * 32 * L.ng * 2;
        hipLaunchKernelGGL(rq_prepare6_kernel, dim3((unsigned) ((total6 + 255) / 256)), dim3(256), 0, stream,
                           reinterpret_cast<const rq_block_w4a4 *>(blocks), (int64_t) 0, L.N, L.ng, (int64_t) 0, n_frags,
                           prepared + L.off_w6);
    }
    hipLaunchKernelGGL(rq_finish_flags_kernel, dim3(1), dim3(64), 0, stream, flags, (const int32_t *) nullptr,
                       L.off_w6 != 0 ? prepared + L.off_w6 : (const uint8_t *) nullptr);
    return hipGetLastError();
}

// In place (the reference's rq_repack_once, reference patch lines 2046-2075): the tensor's own buffer ends up holding
// the prepared codes, scales, multipliers and flags (32 + 1 bytes per 64 codes against the blocks' 36: it fits), the
// fp6 plane goes to `plane6`. Panels are taken in ascending order, a chunk at a time through `staging`: a chunk's
// blocks are copied out, then its codes are written over the blocks of the chunks before it (a panel's codes end in
// front of where its blocks began). Scales, multipliers and the flag word collect in the staging buffer and move to
// their places behind the codes at the end, when every block has been read.
hipError_t launch_prepare_inplace(void *blocks, const PreparedLayout &L, uint8_t *plane6, uint8_t *staging,
                                  size_t staging_bytes, hipStream_t stream) {
    uint8_t *base = reinterpret_cast<uint8_t *>(blocks);
    const size_t row_bytes = (size_t) (L.ng / 4) * sizeof(rq_block_w4a4);
    const size_t panel_src = kPanelRows * row_bytes;
    const size_t sw_bytes = align_up((size_t) L.n_panels * kPanelRows * sizeof(float), 256);
    const size_t kmul_bytes = align_up((size_t) L.n_panels * L.ng * kPanelRows, 256);
    const size_t side = sw_bytes + kmul_bytes + 256;
    if (staging_bytes < side + panel_src) return hipErrorInvalidValue;
    float *side_sw = reinterpret_cast<float *>(staging);
    uint8_t *side_kmul = staging + sw_bytes;
    int32_t *side_flags = reinterpret_cast<int32_t *>(staging + sw_bytes + kmul_bytes);
    uint8_t *chunk = staging + side;
    const int chunk_panels = (int) ((staging_bytes - side) / panel_src);
    hipLaunchKernelGGL(rq_clear_flags_kernel, dim3(1), dim3(64), 0, stream, side_flags);
    for (int p0 = 0; p0 < L.n_panels; p0 += chunk_panels) {
        const int np = L.n_panels - p0 < chunk_panels ? L.n_panels - p0 : chunk_panels;
        const int64_t row0 = (int64_t) p0 * kPanelRows;
        const int64_t rows = L.N - row0 < (int64_t) np * kPanelRows ? L.N - row0 : (int64_t) np * kPanelRows;
        hipError_t e = hipMemcpyAsync(chunk, base + (size_t) row0 * row_bytes, (size_t) rows * row_bytes,
                                      hipMemcpyDeviceToDevice, stream);
        if (e != hipSuccess) return e;
        const int64_t total = (int64_t) np * kPanelRows * L.ng;
        hipLaunchKernelGGL(rq_prepare_kernel, dim3((unsigned) ((total + 255) / 256)), dim3(256), 0, stream,
                           reinterpret_cast<const rq_block_w4a4 *>(chunk), rows, L.ng, np,
                           reinterpret_cast<uint4 *>(base + L.off_codes) + (size_t) p0 * L.ng * 128, side_sw + row0,
                           side_kmul + (size_t) p0 * L.ng * kPanelRows, side_flags);
        if (plane6 != nullptr) {
            // this chunk's fragments; the last chunk also writes the zero fragments that pad the plane to whole row tiles
            const int64_t frag0 = (int64_t) p0 * 2;
            const int64_t frag1 = p0 + np >= L.n_panels ? (int64_t) L.n_rtiles * 8 : (int64_t) (p0 + np) * 2;
            const int64_t total6 = (frag1 - frag0) * 32 * L.ng * 2;
            hipLaunchKernelGGL(rq_prepare6_kernel, dim3((unsigned) ((total6 + 255) / 256)), dim3(256), 0, stream,
                               reinterpret_cast<const rq_block_w4a4 *>(chunk), row0, row0 + rows, L.ng, frag0, frag1 - frag0,
                               plane6);
        }
    }
    hipError_t e = hipMemcpyAsync(base + L.off_sw, side_sw, (size_t) L.n_panels * kPanelRows * sizeof(float),
                                  hipMemcpyDeviceToDevice, stream);
    if (e != hipSuccess) return e;
    e = hipMemcpyAsync(base + L.off_kmul, side_kmul, (size_t) L.n_panels * L.ng * kPanelRows, hipMemcpyDeviceToDevice, stream);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(rq_finish_flags_kernel, dim3(1), dim3(64), 0, stream,
                       reinterpret_cast<int32_t *>(base + L.off_flags), side_flags, plane6);
    return hipGetLastError();
}

}  // namespace rq
