// int4 x int4 GEMM on the gfx950 matrix cores (v_mfma_i32_16x16x64_i8) for wide token batches.
//
// One MFMA consumes K = 64 inputs, which is exactly one activation group, so each MFMA result is one
// group's integer S = sum w * (q - z) for a 16 row x 16 token tile. Feeding q - z (range -15..15) instead of the
// stored code q - 8 makes S equal to acc + (8 - z) * colsum of the reference, so no column sums are needed.
// Weight codes are widened on the way into LDS by masking a nibble into the HIGH half of a byte (w * 16,
// no sign extension needed); the per-group fold then shifts by 8 instead of 4:
//     total += (k * m_g * 16 S) >> 8  ==  (k * m_g * S) >> 4          (reference patch lines 148-177)
// The fold is three full-rate VALU ops per output and group (24-bit multiply, arithmetic shift, add); the
// floor per group cannot be moved through the MFMA accumulator, so it stays on the vector ALU.
//
// Workgroup tile: 128 rows (two panels) x 128 tokens, four wavefronts in a 2 x 2 arrangement, each 64 x 64 as
// 4 x 4 MFMA tiles. LDS is double buffered: [quarter of the group][row or token][16 bytes] for both operands,
// so the 16 lanes that share a quarter read 256 contiguous bytes.
#include "rq_common.h"

#pragma clang fp contract(off)

namespace rq {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kBN = 128;   // rows per workgroup
constexpr int kBT = 128;   // tokens per workgroup
constexpr int kThreads = 256;

struct Stage {
    uint4   a[4][kBN];   // weights, int8 = code * 16
    uint4   b[4][kBT];   // activations, int8 = q - z
    uint8_t m[kBT];      // activation multipliers
    uint8_t k[kBN];      // weight multipliers (only read when the tensor has them)
};

// 8 int4 codes (nibble j = element j) -> the four even elements and the four odd elements, each as code * 16
__device__ __forceinline__ void widen(uint32_t w, uint32_t &even, uint32_t &odd) {
    even = (w << 4) & 0xF0F0F0F0u;
    odd = w & 0xF0F0F0F0u;
}

template <bool HASK>
__device__ __forceinline__ void gemm_body(const uint4 *__restrict__ codes, const uint8_t *__restrict__ kmul,
                                          const uint4 *__restrict__ act8, const uint8_t *__restrict__ m8,
                                          Stage (&st)[2], int panel0, int n_panels, int t0, int Mp, int ng,
                                          int32_t (&acc)[4][4][4]) {
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wr = wave & 1, wc = wave >> 1;
    const int l16 = lane & 15, quad = lane >> 4;

    // global -> register staging assignments
    const int w_pp = tid >> 7, w_idx = tid & 127;           // weights: panel of the pair, 16-byte cell in the group
    const bool w_on = panel0 + w_pp < n_panels;
    const uint4 *w_src = codes + (size_t) (panel0 + (w_on ? w_pp : 0)) * ng * 128 + w_idx;
    const int w_row = w_pp * 64 + (w_idx & 63), w_half = w_idx >> 6;
    const uint8_t *k_src = kmul + (size_t) (panel0 + (w_on ? w_pp : 0)) * ng * kPanelRows + (w_idx & 63);

    uint4 wq, aq[2];
    uint32_t mq = 0;
    uint8_t kq = 1;

    auto fetch = [&](int g) {
        wq = w_on ? w_src[(size_t) g * 128] : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + kThreads * i;  // quarter = c >> 7, token = c & 127
            aq[i] = act8[((size_t) g * 4 + (c >> 7)) * Mp + t0 + (c & 127)];
        }
        if (tid < kBT / 4) mq = *reinterpret_cast<const uint32_t *>(m8 + (size_t) g * Mp + t0 + 4 * tid);
        if (HASK && w_half == 0) kq = w_on ? k_src[(size_t) g * kPanelRows] : (uint8_t) 1;
    };
    auto stash = [&](Stage &s) {
        uint4 q0, q1;
        widen(wq.x, q0.x, q0.y);
        widen(wq.y, q0.z, q0.w);
        widen(wq.z, q1.x, q1.y);
        widen(wq.w, q1.z, q1.w);
        s.a[2 * w_half][w_row] = q0;
        s.a[2 * w_half + 1][w_row] = q1;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + kThreads * i;
            s.b[c >> 7][c & 127] = aq[i];
        }
        if (tid < kBT / 4) *reinterpret_cast<uint32_t *>(s.m + 4 * tid) = mq;
        if (HASK && w_half == 0) s.k[w_row] = kq;
    };

    fetch(0);
    stash(st[0]);
    __syncthreads();

    for (int g = 0; g < ng; ++g) {
        const Stage &s = st[g & 1];
        if (g + 1 < ng) fetch(g + 1);

        v4i A[4], B[4];
        int mm[4];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            const uint4 v = s.a[quad][64 * wr + 16 * rt + l16];
            A[rt] = v4i{ (int) v.x, (int) v.y, (int) v.z, (int) v.w };
        }
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
            const uint4 v = s.b[quad][64 * wc + 16 * ct + l16];
            B[ct] = v4i{ (int) v.x, (int) v.y, (int) v.z, (int) v.w };
            mm[ct] = s.m[64 * wc + 16 * ct + l16];
        }
        int kk[4][4];
        if (HASK) {
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                const uint32_t k4 = *reinterpret_cast<const uint32_t *>(s.k + 64 * wr + 16 * rt + 4 * quad);
#pragma unroll
                for (int i = 0; i < 4; ++i) kk[rt][i] = (k4 >> (8 * i)) & 0xFF;
            }
        }
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                const v4i S = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[rt], B[ct], v4i{ 0, 0, 0, 0 }, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int mult = HASK ? kk[rt][i] * mm[ct] : mm[ct];
                    acc[rt][ct][i] += __mul24(mult, S[i]) >> 8;
                }
            }
        }

        if (g + 1 < ng) stash(st[(g + 1) & 1]);
        __syncthreads();
    }
}

__global__ void __launch_bounds__(kThreads)
rq_gemm_kernel(const uint4 *__restrict__ codes, const float *__restrict__ s_w, const uint8_t *__restrict__ kmul,
               const int32_t *__restrict__ flags, const uint4 *__restrict__ act8, const uint8_t *__restrict__ m8,
               const float *__restrict__ u, float *__restrict__ y, int64_t ldy, int64_t N, int M, int Mp, int ng,
               int n_panels, int n_row_tiles, int n_tok_tiles) {
    __shared__ Stage st[2];

    // Workgroups go to the eight XCDs round robin. Give every XCD a contiguous run of row tiles with the token
    // tiles running fastest, so the workgroups resident on one XCD share weight and activation tiles in its L2.
    const int total = n_row_tiles * n_tok_tiles;
    int v = blockIdx.x;
    const int per_xcd = total / 8;
    if (v < per_xcd * 8) v = (v & 7) * per_xcd + (v >> 3);
    const int row_tile = v / n_tok_tiles, tok_tile = v - row_tile * n_tok_tiles;
    const int panel0 = row_tile * 2, t0 = tok_tile * kBT;

    int32_t acc[4][4][4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int ct = 0; ct < 4; ++ct)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[rt][ct][i] = 0;

    if (flags[0] & 1) {
        gemm_body<true>(codes, kmul, act8, m8, st, panel0, n_panels, t0, Mp, ng, acc);
    } else {
        gemm_body<false>(codes, kmul, act8, m8, st, panel0, n_panels, t0, Mp, ng, acc);
    }

    // epilogue (reference patch line 176): y = ((float(total) * 16) * u) * s_w
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wr = wave & 1, wc = wave >> 1;
    const int l16 = lane & 15, quad = lane >> 4;
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
        const int t = t0 + 64 * wc + 16 * ct + l16;
        if (t >= M) continue;
        const float ut = u[t];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            const int64_t n = (int64_t) panel0 * kPanelRows + 64 * wr + 16 * rt + 4 * quad;
            float *dst = y + (int64_t) t * ldy + n;
            if (n + 3 < N && ((reinterpret_cast<uintptr_t>(dst) & 15) == 0)) {
                const float4 sw = *reinterpret_cast<const float4 *>(s_w + n);
                float4 o;
                o.x = (((float) acc[rt][ct][0] * 16.0f) * ut) * sw.x;
                o.y = (((float) acc[rt][ct][1] * 16.0f) * ut) * sw.y;
                o.z = (((float) acc[rt][ct][2] * 16.0f) * ut) * sw.z;
                o.w = (((float) acc[rt][ct][3] * 16.0f) * ut) * sw.w;
                *reinterpret_cast<float4 *>(dst) = o;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (n + i < N) dst[i] = (((float) acc[rt][ct][i] * 16.0f) * ut) * s_w[n + i];
                }
            }
        }
    }
}

}  // namespace

hipError_t launch_gemm(const GemmArgs &a, hipStream_t stream) {
    const uint8_t *p = a.prepared;
    const int n_row_tiles = (a.L.n_panels + 1) / 2;
    const int n_tok_tiles = a.Mp / kBT;
    hipLaunchKernelGGL(rq_gemm_kernel, dim3(n_row_tiles * n_tok_tiles), dim3(kThreads), 0, stream,
                       reinterpret_cast<const uint4 *>(p + a.L.off_codes),
                       reinterpret_cast<const float *>(p + a.L.off_sw), p + a.L.off_kmul,
                       reinterpret_cast<const int32_t *>(p + a.L.off_flags),
                       reinterpret_cast<const uint4 *>(a.act8), a.m8, a.u, a.y, a.ldy, a.L.N, a.M, a.Mp, a.L.ng,
                       a.L.n_panels, n_row_tiles, n_tok_tiles);
    return hipGetLastError();
}

}  // namespace rq
