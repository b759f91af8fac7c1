// HBM-bound int4 x int4 GEMV for 1..8 tokens (decode and narrow verify widths) on gfx950.
//
// A workgroup of four wavefronts owns one panel of 64 weight rows and one slice of K. Inside a wavefront
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

constexpr int kGemvWaves = 4;
constexpr int kUnroll = 5;  // groups in flight per wavefront: 10 x 16-byte loads per lane

__device__ __forceinline__ int dot8(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot8((int) a, (int) b, c, false);
}

// One batch = up to kUnroll groups of this wavefront. All weight loads of the batch are issued first; the
// activation words of one token for the whole batch are fetched with scalar loads one token ahead of their use, so
// their latency hides behind the weight loads (first token) or behind the previous token's arithmetic.
template <int T, int kWaves>
__device__ __forceinline__ void gemv_body(const uint4 *__restrict__ codes, const uint8_t *__restrict__ kmul,
                                          const uint32_t *__restrict__ act, const int32_t *__restrict__ mz,
                                          const int32_t *__restrict__ flags, int panel, int ng, int g_begin, int g_end,
                                          int wave, int lane, int32_t (&tot)[T]) {
    const uint4 *wp = codes + (size_t) panel * ng * 128 + lane;
    const uint8_t *kp = kmul + (size_t) panel * ng * kPanelRows + lane;
    for (int g0 = g_begin + wave; g0 < g_end; g0 += kWaves * kUnroll) {
        uint4 q[kUnroll][2];
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            const int g = min(g0 + k * kWaves, g_end - 1);  // past the end: reread the last group, contribute nothing
            q[k][0] = wp[(size_t) g * 128];
            q[k][1] = wp[(size_t) g * 128 + 64];
        }
        // (token, group) pairs in the order t * kUnroll + k; their activation words ride a ring of scalar
        // registers kRing pairs deep
        constexpr int kPairs = T * kUnroll;
        constexpr int kRing = kPairs < 6 ? kPairs : 6;
        uint32_t a[kRing][8];
        int32_t mzv[kRing];
        auto fetch_pair = [&](int j) {
            const int t = j / kUnroll, k = j % kUnroll;
            const int g = min(g0 + k * kWaves, g_end - 1);
            const uint32_t *ap = act + ((size_t) g * kGemvTokens + t) * 8;  // wave-uniform address: scalar loads
#pragma unroll
            for (int i = 0; i < 8; ++i) a[j % kRing][i] = ap[i];
            mzv[j % kRing] = mz[(size_t) g * kGemvTokens + t];
        };
#pragma unroll
        for (int j = 0; j < kRing - 1; ++j) fetch_pair(j);
        // the multiplier flag is read here, after the weight loads are on their way (a volatile load cannot be
        // hoisted in front of them)
        const bool hask = *reinterpret_cast<const volatile int32_t *>(flags) & 1;
        int kw[kUnroll];
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            kw[k] = 1;
            if (hask) kw[k] = kp[(size_t) min(g0 + k * kWaves, g_end - 1) * kPanelRows];
        }
        int cs[kUnroll];
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            const uint32_t w[8] = { q[k][0].x, q[k][0].y, q[k][0].z, q[k][0].w, q[k][1].x, q[k][1].y, q[k][1].z, q[k][1].w };
            int c = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) c = dot8(w[i], 0x11111111u, c);
            cs[k] = c;
        }
#pragma unroll
        for (int j = 0; j < kPairs; ++j) {
            if (j + kRing - 1 < kPairs) fetch_pair(j + kRing - 1);
            const int t = j / kUnroll, k = j % kUnroll, slot = j % kRing;
            const uint32_t w[8] = { q[k][0].x, q[k][0].y, q[k][0].z, q[k][0].w, q[k][1].x, q[k][1].y, q[k][1].z, q[k][1].w };
            int acc = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc = dot8(w[i], a[slot][i], acc);
            const int mult = mzv[slot] & 0xFF;
            const int zc = (int) (int8_t) ((mzv[slot] >> 8) & 0xFF);
            int term = mult * (acc + zc * cs[k]);
            if (hask) term *= kw[k];
            if (g0 + k * kWaves < g_end) tot[t] += term >> kTermShift;
        }
    }
}

template <int T, int kWaves>
__global__ void __launch_bounds__(kWaves * 64)
rq_gemv_kernel(const uint4 *__restrict__ codes, const float *__restrict__ s_w, const uint8_t *__restrict__ kmul,
               const int32_t *__restrict__ flags, const uint32_t *__restrict__ act, const int32_t *__restrict__ mz,
               const float *__restrict__ u, float *__restrict__ y, int64_t ldy, int64_t N, int ng,
               unsigned long long *__restrict__ cells, int n_rows_pad) {
    __shared__ int32_t red[kWaves][T][64];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int panel = blockIdx.x;
    const int nks = gridDim.y, ks = blockIdx.y;
    const int g_begin = (int) ((int64_t) ng * ks / nks), g_end = (int) ((int64_t) ng * (ks + 1) / nks);

    int32_t tot[T];
#pragma unroll
    for (int t = 0; t < T; ++t) tot[t] = 0;

    gemv_body<T, kWaves>(codes, kmul, act, mz, flags, panel, ng, g_begin, g_end, wave, lane, tot);

#pragma unroll
    for (int t = 0; t < T; ++t) red[wave][t][lane] = tot[t];
    __syncthreads();

    for (int item = tid; item < T * 64; item += kWaves * 64) {
        const int t = item >> 6;
        const int64_t n = (int64_t) panel * kPanelRows + lane;
        int32_t sum = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) sum += red[w][t][lane];
        if (nks > 1) {
            // K is split over gridDim.y workgroups. Each output has one 64-bit cell: the low 48 bits collect the
            // exact integer sum, the bits above count arrivals. One device-scope atomic add does both, and the
            // value it returns tells the lane whether it was the last of the nks contributors; that lane alone
            // finishes the output and clears the cell for the next call. No fences, no second round trip: the
            // only cross-workgroup traffic is this one read-modify-write, performed in one place for the chip.
            unsigned long long *cell = cells + (size_t) t * n_rows_pad + n;
            const unsigned long long mine = (1ull << 48) + (unsigned long long) (long long) sum;
            const unsigned long long now =
                __hip_atomic_fetch_add(cell, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + mine;
            if ((int) ((now + (1ull << 47)) >> 48) != nks) continue;
            __hip_atomic_store(cell, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            sum = (int32_t) (uint32_t) now;  // the total fits int32 by construction of the format
        }
        if (n < N) y[(int64_t) t * ldy + n] = (((float) sum * 16.0f) * u[t]) * s_w[n];
    }
}

template <int T, int kWaves>
hipError_t launch_tw(const GemvArgs &a, int nks, hipStream_t stream) {
    const uint8_t *p = a.prepared;
    hipLaunchKernelGGL((rq_gemv_kernel<T, kWaves>), dim3(a.L.n_panels, nks), dim3(kWaves * 64), 0, stream,
                       reinterpret_cast<const uint4 *>(p + a.L.off_codes),
                       reinterpret_cast<const float *>(p + a.L.off_sw), p + a.L.off_kmul,
                       reinterpret_cast<const int32_t *>(p + a.L.off_flags), a.act, a.mz, a.u, a.y, a.ldy, a.L.N,
                       a.L.ng, reinterpret_cast<unsigned long long *>(a.tot), a.L.n_panels * kPanelRows);
    return hipGetLastError();
}

template <int T>
hipError_t launch_t(const GemvArgs &a, int nks, hipStream_t stream) {
    static const int waves = getenv("RQ_GEMV_WAVES") ? atoi(getenv("RQ_GEMV_WAVES")) : kGemvWaves;
    switch (waves) {
        case 2:  return launch_tw<T, 2>(a, nks, stream);
        case 8:  return launch_tw<T, 8>(a, nks, stream);
        default: return launch_tw<T, 4>(a, nks, stream);
    }
}

}  // namespace

// How many workgroups share K for one panel. The kernel is a pure stream with a latency-bound start and end, so
// it wants many small workgroups: their starts and tails overlap and the last wave of workgroups is short. Aim for
// about a thousand workgroups, at least a batch (kGemvWaves x kUnroll groups) each when K allows, and never fewer
// than four groups per workgroup.
int gemv_ksplit(const PreparedLayout &L) {
    static const int forced = getenv("RQ_GEMV_KSPLIT") ? atoi(getenv("RQ_GEMV_KSPLIT")) : 0;
    int nks;
    if (forced > 0) {
        nks = forced;
    } else {
        const int by_batch = (L.ng + kGemvWaves * kUnroll - 1) / (kGemvWaves * kUnroll);
        const int by_grid = (1024 + L.n_panels - 1) / L.n_panels;
        nks = by_batch > by_grid ? by_batch : by_grid;
        if (nks > L.ng / 4) nks = L.ng / 4;
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
