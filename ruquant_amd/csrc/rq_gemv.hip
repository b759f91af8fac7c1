// HBM-bound int4 x int4 GEMV for 1..8 tokens (decode and narrow verify widths) on gfx950.
//
// A workgroup of eight wavefronts owns one panel of 64 weight rows and one slice of K. Inside a wavefront
// lane = row: the prepared layout makes each group of 64 inputs two fully coalesced 1 KiB loads per
// wavefront, the activation codes of that group are the same for all 64 lanes and arrive through scalar
// loads, and v_dot8_i32_i4 consumes weight word x activation word directly. No lane ever exchanges data
// with another lane until the per-wave totals meet in LDS. The per-group fold, the exact int32 total and
// the fp32 epilogue are those of ggml_vec_dot_w4a4_a4 (reference patch lines 148-177):
//     total += (k * m_g * (acc_g + (8 - z_g) * colsum_g)) >> 4;   y = ((float(total) * 16) * u) * s_w.
// colsum_g is recomputed from the codes (dot8 against 0x11111111) instead of being stored.
#include "rq_common.h"

#include <stdlib.h>

#pragma clang fp contract(off)

namespace rq {

namespace {

constexpr int kWaves = 8;
constexpr int kUnroll = 4;  // groups in flight per wavefront: 8 x 16-byte loads per lane

__device__ __forceinline__ int dot8(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot8((int) a, (int) b, c, false);
}

template <int T, bool HASK>
__device__ __forceinline__ void gemv_body(const uint4 *__restrict__ codes, const uint8_t *__restrict__ kmul,
                                          const uint32_t *__restrict__ act, const int32_t *__restrict__ mz,
                                          int panel, int ng, int g_begin, int g_end, int wave, int lane,
                                          int32_t (&tot)[T]) {
    const uint4 *wp = codes + (size_t) panel * ng * 128 + lane;
    const uint8_t *kp = kmul + (size_t) panel * ng * kPanelRows + lane;
    for (int g0 = g_begin + wave; g0 < g_end; g0 += kWaves * kUnroll) {
        uint4 q[kUnroll][2];
        int kw[kUnroll];
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            const int g = g0 + k * kWaves;
            if (g < g_end) {
                q[k][0] = wp[(size_t) g * 128];
                q[k][1] = wp[(size_t) g * 128 + 64];
                if (HASK) kw[k] = kp[(size_t) g * kPanelRows];
            }
        }
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            const int g = g0 + k * kWaves;
            if (g < g_end) {
                const uint32_t w[8] = { q[k][0].x, q[k][0].y, q[k][0].z, q[k][0].w,
                                        q[k][1].x, q[k][1].y, q[k][1].z, q[k][1].w };
                int cs = 0;
#pragma unroll
                for (int i = 0; i < 8; ++i) cs = dot8(w[i], 0x11111111u, cs);
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    const uint32_t *ap = act + ((size_t) g * kGemvTokens + t) * 8;  // wave-uniform: scalar loads
                    int acc = 0;
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc = dot8(w[i], ap[i], acc);
                    const int32_t mzv = mz[(size_t) g * kGemvTokens + t];
                    const int mult = mzv & 0xFF;
                    const int zc = (int) (int8_t) ((mzv >> 8) & 0xFF);
                    int term = mult * (acc + zc * cs);
                    if (HASK) term *= kw[k];
                    tot[t] += term >> kTermShift;
                }
            }
        }
    }
}

template <int T>
__global__ void __launch_bounds__(kWaves * 64)
rq_gemv_kernel(const uint4 *__restrict__ codes, const float *__restrict__ s_w, const uint8_t *__restrict__ kmul,
               const int32_t *__restrict__ flags, const uint32_t *__restrict__ act, const int32_t *__restrict__ mz,
               const float *__restrict__ u, float *__restrict__ y, int64_t ldy, int64_t N, int ng,
               int32_t *__restrict__ tot_g, int32_t *__restrict__ cnt_g, int n_rows_pad) {
    __shared__ int32_t red[kWaves][T][64];
    __shared__ int s_last;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int panel = blockIdx.x;
    const int nks = gridDim.y, ks = blockIdx.y;
    const int g_begin = (int) ((int64_t) ng * ks / nks), g_end = (int) ((int64_t) ng * (ks + 1) / nks);

    int32_t tot[T];
#pragma unroll
    for (int t = 0; t < T; ++t) tot[t] = 0;

    if (flags[0] & 1) {
        gemv_body<T, true>(codes, kmul, act, mz, panel, ng, g_begin, g_end, wave, lane, tot);
    } else {
        gemv_body<T, false>(codes, kmul, act, mz, panel, ng, g_begin, g_end, wave, lane, tot);
    }

#pragma unroll
    for (int t = 0; t < T; ++t) red[wave][t][lane] = tot[t];
    __syncthreads();

    const int64_t n = (int64_t) panel * kPanelRows + lane;
    if (nks == 1) {
        if (tid < T * 64) {
            const int t = tid >> 6;
            int32_t sum = 0;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) sum += red[w][t][lane];
            if (n < N) y[(int64_t) t * ldy + n] = (((float) sum * 16.0f) * u[t]) * s_w[n];
        }
        return;
    }

    // K is split over gridDim.y workgroups: exact int32 sums meet in global memory, the last arrival finishes
    if (tid < T * 64) {
        const int t = tid >> 6;
        int32_t sum = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) sum += red[w][t][lane];
        atomicAdd(&tot_g[(size_t) t * n_rows_pad + n], sum);
    }
    __threadfence();
    __syncthreads();
    if (tid == 0) s_last = atomicAdd(&cnt_g[panel], 1) == nks - 1;
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    if (tid < T * 64) {
        const int t = tid >> 6;
        // read through the atomic unit (coherent across the chip) and leave the cell zero for the next pass
        const int32_t sum = atomicExch(&tot_g[(size_t) t * n_rows_pad + n], 0);
        if (n < N) y[(int64_t) t * ldy + n] = (((float) sum * 16.0f) * u[t]) * s_w[n];
    }
    if (tid == 0) atomicExch(&cnt_g[panel], 0);
}

template <int T>
hipError_t launch_t(const GemvArgs &a, int nks, hipStream_t stream) {
    const uint8_t *p = a.prepared;
    hipLaunchKernelGGL((rq_gemv_kernel<T>), dim3(a.L.n_panels, nks), dim3(kWaves * 64), 0, stream,
                       reinterpret_cast<const uint4 *>(p + a.L.off_codes),
                       reinterpret_cast<const float *>(p + a.L.off_sw), p + a.L.off_kmul,
                       reinterpret_cast<const int32_t *>(p + a.L.off_flags), a.act, a.mz, a.u, a.y, a.ldy, a.L.N,
                       a.L.ng, a.tot, a.cnt, a.L.n_panels * kPanelRows);
    return hipGetLastError();
}

}  // namespace

// How many workgroups share K for one panel: enough workgroups to cover the chip about twice, and at least
// two groups per wavefront so the loads of a wavefront overlap.
int gemv_ksplit(const PreparedLayout &L) {
    static const int forced = getenv("RQ_GEMV_KSPLIT") ? atoi(getenv("RQ_GEMV_KSPLIT")) : 0;
    int nks = 1;
    if (forced > 0) {
        nks = forced;
    } else {
        while (L.n_panels * nks < 512 && L.ng / (nks * 2) >= kWaves * 2) nks *= 2;
    }
    if (nks > L.ng) nks = L.ng;
    return nks < 1 ? 1 : nks;
}

hipError_t launch_gemv(const GemvArgs &a, hipStream_t stream) {
    const int nks = gemv_ksplit(a.L);
    switch (a.T) {
        case 1: return launch_t<1>(a, nks, stream);
        case 2: return launch_t<2>(a, nks, stream);
        case 3: return launch_t<3>(a, nks, stream);
        case 4: return launch_t<4>(a, nks, stream);
        case 5: return launch_t<5>(a, nks, stream);
        case 6: return launch_t<6>(a, nks, stream);
        case 7: return launch_t<7>(a, nks, stream);
        case 8: return launch_t<8>(a, nks, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace rq
