// HBM-bound int4 x int4 GEMV for 1..8 tokens (decode and narrow verify widths) on gfx950.
//
// A workgroup of four wavefronts owns one panel of 64 weight rows and one slice of K. Inside a wavefront
// lane = row: the prepared layout makes each group of 64 inputs two fully coalesced 1 KiB loads per
// wavefront, and v_dot8_i32_i4 consumes weight word x activation word directly. No lane exchanges data with another
// lane until the per-wave totals meet in LDS.
//
// The activation quantizer is part of this kernel. Its inputs are the (rotated) fp32 rows and the clipped range of
// every 64-wide group; a workgroup first puts the weight loads of its first batch in flight, then derives the
// token units from all ranges (reference patch lines 2646-2655: R = widest range, u = R / 3825), quantizes just the
// groups of its own K slice into LDS (lines 2662-2677: m, 1 / (m u), z, q, op for op) and meets its weights. So
// the quantizer costs no launch, no trip through memory for the codes, and its latency hides behind the first
// weight loads.
//
// The per-group fold, the exact int32 total and the fp32 epilogue are those of ggml_vec_dot_w4a4_a4 (lines 148-177):
//     total += (k * m_g * (acc_g + (8 - z_g) * colsum_g)) >> 4;   y = ((float(total) * 16) * u) * s_w.
// colsum_g is recomputed from the codes (dot8 against 0x11111111) instead of being stored.
#include "rq_hadamard.h"


#pragma clang fp contract(off)

namespace rq {

namespace {

constexpr int kGemvWaves = 4;
constexpr int kUnroll = 5;        // groups in flight per wavefront: 10 x 16-byte loads per lane
constexpr int kMaxSlice = 48;     // most groups one workgroup may own (bounds its LDS)

__device__ __forceinline__ int dot8(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot8((int) a, (int) b, c, false);
}

// a * b + c with a and b of at most 24 bits, as the one full-rate instruction (from __mul24(a, b) + c the compiler
// makes a 64-bit multiply-add, which runs at a quarter of the rate)
__device__ __forceinline__ int mad24(int a, int b, int c) {
    int r;
    asm("v_mad_i32_i24 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// Activation groups wider than 64 (GF = 2 or 4 runs of 64 per group): a group's runs share one multiplier and zero
// point and are folded once, so a wavefront takes whole groups ("units"). A batch is U runs of 64 per wavefront.
template <int GF>
constexpr int batch_runs() { return GF == 1 ? kUnroll : 4; }

template <int U>
struct Batch {
    uint4 q[U][2];
};

// u0: this wavefront's first unit of the batch; its next ones are kWaves units further on
template <int kWaves, int U, int GF>
__device__ __forceinline__ void load_batch(Batch<U> &b, const uint4 *wp, int u0, int u_end) {
#pragma unroll
    for (int k = 0; k < U; ++k) {
        const int u = min(u0 + (k / GF) * kWaves, u_end - 1);  // past the end: reread the last unit, contribute nothing
        const int g = u * GF + k % GF;
        // weights are read once per call: non-temporal, so they do not displace the activations and ranges in L2
        typedef unsigned v4u __attribute__((ext_vector_type(4)));
        const v4u q0 = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(wp + (size_t) g * 128));
        const v4u q1 = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(wp + (size_t) g * 128 + 64));
        b.q[k][0] = make_uint4(q0.x, q0.y, q0.z, q0.w);
        b.q[k][1] = make_uint4(q1.x, q1.y, q1.z, q1.w);
    }
}

// act: [run of 64 of the slice][token][8 words] codes q - 8 in the tensor's nibble order; mz: [unit of the slice][token]
// m | (8 - z) << 8. The weight multiplier of a unit is that of its first run (reference patch line 168).
// HASK (weight multipliers, a format variant) is a compile-time constant: as a run-time flag the compiler multiplies
// every term by a multiplier that is 1, a full 32-bit multiply at a quarter of the rate.
template <int T, int kWaves, int U, int GF, bool HASK>
__device__ __forceinline__ void compute_batch(const Batch<U> &b, const uint8_t *kp, const uint32_t *act,
                                              const int32_t *mz, int u0, int u_begin, int u_end, int32_t (&tot)[T]) {
#pragma unroll
    for (int j = 0; j < U / GF; ++j) {
        const int u = u0 + j * kWaves;
        if (u >= u_end) break;   // wave-uniform
        const int ul = u - u_begin;
        int part[T];
#pragma unroll
        for (int t = 0; t < T; ++t) part[t] = 0;
#pragma unroll
        for (int sub = 0; sub < GF; ++sub) {
            const int k = j * GF + sub;
            const uint32_t w[8] = { b.q[k][0].x, b.q[k][0].y, b.q[k][0].z, b.q[k][0].w,
                                    b.q[k][1].x, b.q[k][1].y, b.q[k][1].z, b.q[k][1].w };
            int cs = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) cs = dot8(w[i], 0x11111111u, cs);
            const int gl = ul * GF + sub;
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const uint4 a0 = *reinterpret_cast<const uint4 *>(act + (gl * T + t) * 8);      // same address in every lane
                const uint4 a1 = *reinterpret_cast<const uint4 *>(act + (gl * T + t) * 8 + 4);
                int acc = 0;
                acc = dot8(w[0], a0.x, acc);
                acc = dot8(w[1], a0.y, acc);
                acc = dot8(w[2], a0.z, acc);
                acc = dot8(w[3], a0.w, acc);
                acc = dot8(w[4], a1.x, acc);
                acc = dot8(w[5], a1.y, acc);
                acc = dot8(w[6], a1.z, acc);
                acc = dot8(w[7], a1.w, acc);
                const int zc = (int) (int8_t) ((mz[ul * T + t] >> 8) & 0xFF);
                part[t] += mad24(zc, cs, acc);   // |cs| <= 512, |zc| <= 8
            }
        }
        int kw = 1;
        if (HASK) kw = kp[(size_t) (u * GF) * kPanelRows];
#pragma unroll
        for (int t = 0; t < T; ++t) {
            // |part| <= 4 x 64 x 8 x 15 (an activation group of 256) and m <= 255: the 24-bit multiply is exact
            int term = __mul24(mz[ul * T + t] & 0xFF, part[t]);
            if (HASK) term *= kw;
            tot[t] += term >> kTermShift;
        }
    }
}

// slice_base / slice_extra: the split of K in units (activation groups)
template <int T, int kWaves, int GF>
__global__ void __launch_bounds__(kWaves * 64)
rq_gemv_kernel(const WeightSet ws, const float *__restrict__ x, int64_t ldx, const float *__restrict__ lohi,
               const float *__restrict__ rpart, unsigned long long *__restrict__ cells, int n_rows_pad, int slice_base,
               int slice_extra) {
    constexpr int NT = kWaves * 64;
    __shared__ int32_t red[kWaves][T][64];
    __shared__ float s_R[T], s_u[T];
    __shared__ float s_inv[kMaxSlice * T], s_zf[kMaxSlice * T];
    __shared__ uint32_t s_act[kMaxSlice * T * 8];
    __shared__ int32_t s_mz[kMaxSlice * T];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int panel = blockIdx.x;          // of the launch: the panels of up to three weights in a row
    const int wsel = (panel >= ws.first[1]) + (panel >= ws.first[2]);
    const int wpanel = panel - (wsel == 0 ? 0 : wsel == 1 ? ws.first[1] : ws.first[2]);
    const uint4 *__restrict__ codes = reinterpret_cast<const uint4 *>(wsel == 0 ? ws.codes[0] : wsel == 1 ? ws.codes[1] : ws.codes[2]);
    const uint8_t *__restrict__ kmul = wsel == 0 ? ws.kmul[0] : wsel == 1 ? ws.kmul[1] : ws.kmul[2];
    const int32_t *__restrict__ flags = wsel == 0 ? ws.flags[0] : wsel == 1 ? ws.flags[1] : ws.flags[2];
    constexpr int U = batch_runs<GF>();
    const int ng = ws.ng;
    const int nks = gridDim.y, ks = blockIdx.y;
    // slices of nu / nks units, the first nu % nks one longer (no division on the device)
    const int u_begin = ks * slice_base + (ks < slice_extra ? ks : slice_extra);
    const int u_end = u_begin + slice_base + (ks < slice_extra ? 1 : 0);
    const int g_begin = u_begin * GF, g_end = u_end * GF;   // the same in runs of 64
    const int cnt = g_end - g_begin;

    // The three inputs of the quantizer prologue do not depend on each other: fetch this thread's share of all of
    // them first (partial range maxima, its first (group, token) range, its first code word's eight values), so the
    // prologue pays one memory latency, not three in a row.
    const int n_ut = (u_end - u_begin) * T;        // (unit, token) pairs of the slice
    const int n_words = cnt * T * 8;               // code words of the slice
    float pre_r = 0.0f;
    if (GF == 1 && tid < T * 64 && lane < kRangeParts) pre_r = rpart[(tid >> 6) * kRangeParts + lane];
    float2 pre_lh = make_float2(0.0f, 0.0f);
    if (GF == 1 && tid < n_ut) pre_lh = reinterpret_cast<const float2 *>(lohi)[(size_t) (tid % T) * ng + g_begin + tid / T];
    float4 pre_x0 = make_float4(0.f, 0.f, 0.f, 0.f), pre_x1 = pre_x0;
    if (tid < n_words) {
        const int gt = tid >> 3;
        const float4 *xp = reinterpret_cast<const float4 *>(x + (int64_t) (gt % T) * ldx +
                                                            (int64_t) (g_begin + gt / T) * kGroup + (tid & 7) * 8);
        pre_x0 = xp[0];
        pre_x1 = xp[1];
    }

    // The epilogue's operands too (the row's scale, the weight's flag word): fetched at the end they would put one
    // more trip to memory behind the last split-K arrival, on the critical path of the whole launch.
    const float *__restrict__ s_w = wsel == 0 ? ws.s_w[0] : wsel == 1 ? ws.s_w[1] : ws.s_w[2];
    const int64_t N = wsel == 0 ? ws.N[0] : wsel == 1 ? ws.N[1] : ws.N[2];
    const int64_t n = (int64_t) wpanel * kPanelRows + lane;       // row of its weight
    const float pre_sw = n < N ? s_w[n] : 0.0f;
    const int32_t pre_flags = *reinterpret_cast<const volatile int32_t *>(flags);

    // ... and right behind them the weights of the first batch. This order matters: a wavefront's loads complete in
    // issue order, so the small prologue inputs must be the OLDER loads or they would wait for 10 KiB of weights.
    const uint4 *wp = codes + (size_t) wpanel * ng * 128 + lane;
    const uint8_t *kp = kmul + (size_t) wpanel * ng * kPanelRows + lane;
    Batch<U> b0;
    load_batch<kWaves, U, GF>(b0, wp, u_begin + wave, u_end);

    // ---- token units: R = widest clipped group range of the whole token (the activation kernel left 32 partial
    // maxima per token), 2 if the token is all zero; u = R / 3825
    if (tid < T * 64) {
        for (int tt = tid >> 6; tt < T; tt += kWaves) {   // wavefront w handles tokens w, w + kWaves, ...
            float r = 0.0f;
            if constexpr (GF == 1) {
                r = tt == (tid >> 6) ? pre_r : (lane < kRangeParts ? rpart[tt * kRangeParts + lane] : 0.0f);
            } else {
                // wide groups: the partial maxima are those of the runs of 64; the token's widest *group* comes from
                // the runs' ranges (min and max commute with the multiplication by the positive clip)
                for (int u = lane; u < ng / GF; u += 64) {
                    float2 c = reinterpret_cast<const float2 *>(lohi)[(size_t) tt * ng + u * GF];
#pragma unroll
                    for (int sub = 1; sub < GF; ++sub) {
                        const float2 o = reinterpret_cast<const float2 *>(lohi)[(size_t) tt * ng + u * GF + sub];
                        c.x = fminf(c.x, o.x);
                        c.y = fmaxf(c.y, o.y);
                    }
                    r = fmaxf(r, c.y - c.x);
                }
            }
            r = wave_max(r);
            if (r == 0.0f) r = 2.0f;
            if (lane == 0) {
                s_R[tt] = r;
                s_u[tt] = r / 3825.0f;  // 15 * 255
            }
        }
    }
    had::lds_barrier();   // not __syncthreads(): the weight loads stay in flight across the prologue

    // ---- per (group of the slice, token): multiplier, 1 / (m u), zero point (reference lines 2662-2665)
    for (int gt = tid; gt < n_ut; gt += NT) {
        const int t = gt % T, g = (u_begin + gt / T) * GF;
        float2 r = GF == 1 && gt == tid ? pre_lh : reinterpret_cast<const float2 *>(lohi)[(size_t) t * ng + g];
#pragma unroll
        for (int sub = 1; sub < GF; ++sub) {
            const float2 o = reinterpret_cast<const float2 *>(lohi)[(size_t) t * ng + g + sub];
            r.x = fminf(r.x, o.x);
            r.y = fmaxf(r.y, o.y);
        }
        const float lo = r.x, hi = r.y;
        const int mg = (int) fminf(fmaxf(ceilf(((hi - lo) * 255.0f) / s_R[t]), 1.0f), 255.0f);
        const float inv = 1.0f / ((float) mg * s_u[t]);
        const float zf = fminf(fmaxf(rintf(-lo * inv), 0.0f), 15.0f);
        s_inv[gt] = inv;
        s_zf[gt] = zf;
        s_mz[gt] = mg | ((8 - (int) zf) & 0xFF) << 8;
    }
    had::lds_barrier();

    // ---- codes: a thread per code word (8 values), q = clamp(rint(x * inv) + z, 0, 15) (lines 2670-2675)
    for (int id = tid; id < n_words; id += NT) {
        const int wi = id & 7, gt = id >> 3;
        const int t = gt % T, g = g_begin + gt / T;
        const int ut = (gt / T / GF) * T + t;     // its (unit, token) pair
        const float inv = s_inv[ut], zf = s_zf[ut];
        float4 v0 = pre_x0, v1 = pre_x1;
        if (id != tid) {
            const float4 *xp = reinterpret_cast<const float4 *>(x + (int64_t) t * ldx + (int64_t) g * kGroup + wi * 8);
            v0 = xp[0];
            v1 = xp[1];
        }
        const float f[8] = { v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w };
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int q = (int) fminf(fmaxf(rintf(f[j] * inv) + zf, 0.0f), 15.0f);
            word |= (uint32_t) ((q - 8) & 0xF) << (4 * j);
        }
        s_act[id] = word;
    }
    had::lds_barrier();

    // ---- the product
    const bool hask = pre_flags & 1;
    int32_t tot[T];
#pragma unroll
    for (int t = 0; t < T; ++t) tot[t] = 0;
    if (hask) {
        compute_batch<T, kWaves, U, GF, true>(b0, kp, s_act, s_mz, u_begin + wave, u_begin, u_end, tot);
    } else {
        compute_batch<T, kWaves, U, GF, false>(b0, kp, s_act, s_mz, u_begin + wave, u_begin, u_end, tot);
    }
    for (int u0 = u_begin + wave + kWaves * (U / GF); u0 < u_end; u0 += kWaves * (U / GF)) {
        Batch<U> b;
        load_batch<kWaves, U, GF>(b, wp, u0, u_end);
        if (hask) {
            compute_batch<T, kWaves, U, GF, true>(b, kp, s_act, s_mz, u0, u_begin, u_end, tot);
        } else {
            compute_batch<T, kWaves, U, GF, false>(b, kp, s_act, s_mz, u0, u_begin, u_end, tot);
        }
    }

#pragma unroll
    for (int t = 0; t < T; ++t) red[wave][t][lane] = tot[t];
    __syncthreads();

    float *__restrict__ y = wsel == 0 ? ws.y[0] : wsel == 1 ? ws.y[1] : ws.y[2];
    const int64_t ldy = wsel == 0 ? ws.ldy[0] : wsel == 1 ? ws.ldy[1] : ws.ldy[2];
    for (int item = tid; item < T * 64; item += NT) {
        const int t = item >> 6;
        const int64_t cell_row = (int64_t) panel * kPanelRows + lane;   // row of the launch (split-K cell)
        int32_t sum = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) sum += red[w][t][lane];
        if (nks > 1) {
            // K is split over gridDim.y workgroups. Each output has one 64-bit cell: the low 48 bits collect the
            // exact integer sum, the bits above count arrivals. One device-scope atomic add does both, and the
            // value it returns tells the lane whether it was the last of the nks contributors; that lane alone
            // finishes the output and clears the cell for the next call. No fences, no second round trip: the
            // only cross-workgroup traffic is this one read-modify-write, performed in one place for the chip.
            unsigned long long *cell = cells + (size_t) t * n_rows_pad + cell_row;
            const unsigned long long mine = (1ull << 48) + (unsigned long long) (long long) sum;
            const unsigned long long now =
                __hip_atomic_fetch_add(cell, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + mine;
            if ((int) ((now + (1ull << 47)) >> 48) != nks) continue;
            __hip_atomic_store(cell, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            sum = (int32_t) (uint32_t) now;  // the total fits int32 by construction of the format
        }
        if (n < N) y[(int64_t) t * ldy + n] = (((float) sum * 16.0f) * s_u[t]) * pre_sw;
    }
}

template <int T, int kWaves, int GF>
hipError_t launch_twg(const GemvArgs &a, int nks, hipStream_t stream) {
    const WeightSet ws = make_weight_set(a.w);
    const int n_panels = ws.first[kMaxFused];
    const int nu = ws.ng / GF;
    hipLaunchKernelGGL((rq_gemv_kernel<T, kWaves, GF>), dim3(n_panels, nks), dim3(kWaves * 64), 0, stream, ws, a.x, a.ldx,
                       a.lohi, a.rpart, reinterpret_cast<unsigned long long *>(a.tot), n_panels * kPanelRows,
                       nu / nks, nu % nks);
    return hipGetLastError();
}

template <int T>
hipError_t launch_t(const GemvArgs &a, int nks, hipStream_t stream) {
    // activation groups of 128 / 256 (a format variant): one configuration
    if (a.gf == 2) return launch_twg<T, kGemvWaves, 2>(a, nks, stream);
    if (a.gf == 4) return launch_twg<T, kGemvWaves, 4>(a, nks, stream);
    if (a.gf != 1) return hipErrorInvalidValue;
    return launch_twg<T, kGemvWaves, 1>(a, nks, stream);
}

}  // namespace

// How many workgroups share K for one panel. The kernel is a pure stream with a latency-bound start and end, so
// it wants many small workgroups: their starts and tails overlap and the last wave of workgroups is short. Aim for
// about a thousand workgroups, at least a batch (kGemvWaves x kUnroll groups) each when K allows, at least ten groups
// per workgroup, and never more than kMaxSlice (the slice's codes live in LDS).
int gemv_ksplit(int n_panels, int ng) {
    int nks;
    {
        const int by_batch = (ng + kGemvWaves * kUnroll - 1) / (kGemvWaves * kUnroll);
        const int by_grid = (1024 + n_panels - 1) / n_panels;
        // more splits than ng / 10 cost more in atomics and short workgroups than they gain in parallelism (measured
        // on 16..96 panels)
        const int cap = ng / 10 > by_batch ? ng / 10 : by_batch;
        nks = by_batch > by_grid ? by_batch : by_grid;
        if (nks > cap) nks = cap;
    }
    const int least = (ng + kMaxSlice - 1) / kMaxSlice;   // ceil(ng / nks) <= kMaxSlice
    if (nks < least) nks = least;
    if (nks > ng) nks = ng;
    return nks < 1 ? 1 : nks;
}

hipError_t launch_gemv(const GemvArgs &a, hipStream_t stream) {
    int n_panels = 0;
    for (int i = 0; i < a.w.n; ++i) n_panels += a.w.L[i].n_panels;
    const int ng = a.w.L[0].ng;
    int nks = gemv_ksplit(n_panels, ng);
    if (a.gf > 1) {
        // whole groups per slice, and no slice longer than the LDS of a workgroup holds
        const int nu = ng / a.gf;
        if (ng % a.gf != 0) return hipErrorInvalidValue;
        if (nks > nu) nks = nu;
        while (nks < nu && (nu + nks - 1) / nks * a.gf > kMaxSlice) ++nks;
    }
    switch (a.T) {
        case 1: return launch_t<1>(a, nks, stream);
        case 2: return launch_t<2>(a, nks, stream);
        case 3: return launch_t<3>(a, nks, stream);
        case 4: return launch_t<4>(a, nks, stream);
        default: return hipErrorInvalidValue;   // (the dispatcher sends five tokens and more to the MFMA kernels)
    }
}

}  // namespace rq
