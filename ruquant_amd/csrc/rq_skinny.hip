// int4 x int4 product for a handful to 64 tokens (wide decode batches, verify batches, short prefill chunks) on the gfx950 matrix cores.
//
// Still a weight stream: with so few tokens the weights are read once and the work per byte is small, so the kernel
// is shaped like the GEMV (a workgroup = one panel of 64 rows x one slice of K, no LDS staging and no barriers in
// the main loop, groups of the slice dealt round-robin to the wavefronts, totals summed in LDS) and borrows the
// arithmetic of the MFMA GEMM: tokens fill the 16-wide side of v_mfma_i32_16x16x64_i8, one MFMA = one activation
// group, activations arrive as the two int8 digits of m (q - z) (p = 64 hi + lo), so that
//     floor(m S / 16) = 4 Xhi + floor(Xlo / 16):
// Xhi accumulates across groups inside the MFMA accumulator, Xlo takes one shift and one add per output and group
// (reference patch lines 148-177 for the fold it reproduces). Weight nibbles are widened into the high half of a
// byte (w * 16); the shifts absorb the factor.
//
// A wavefront owns all four 16-row tiles of the panel and one or two 16-token tiles, so every fragment it loads is
// used four (weights: one or two) times from registers. It reads the A fragments straight from the prepared layout
// (8 bytes per lane: lanes that share a half of the group read 256 contiguous bytes) and the B fragments straight
// from the quantizer's digit planes (L2 resident: they are shared by every panel), through a register ring several
// groups deep: that depth is what covers the HBM latency. More than 32 tokens are split over workgroups that are
// dispatched next to each other on the same XCD, so the second read of the weights comes from that XCD's L2.
//
// Splitting K across workgroups costs one 64-bit L2 atomic per output and split, and device-scope atomics run at
// only about 0.15 per nanosecond on this part, so the launcher splits K inside the workgroup first.
#include "rq_common.h"

#include <stdlib.h>

#pragma clang fp contract(off)

namespace rq {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kWaves = 8, kThreads = kWaves * 64;
constexpr int depth_of(int) { return 3; }   // groups of loads in flight per wavefront

__device__ __forceinline__ void widen(uint32_t w, int &even, int &odd) {
    even = (int) ((w << 4) & 0xF0F0F0F0u);
    odd = (int) (w & 0xF0F0F0F0u);
}

// SINGLE: the activations arrive as one plane of q - z plus the multiplier m of (group, token) as a byte (half the
// activation bytes per group); otherwise as the two digit planes of m (q - z), which the GEMM's leftover rows use.
template <int TT, bool SINGLE>
struct Frag {
    uint2 a[4];                  // packed weights of the four 16-row tiles: this lane's quarter of the group
    uint4 b[TT][SINGLE ? 1 : 2]; // activation bytes of the token tiles: this lane's quarter
    uint8_t mv[TT];              // SINGLE: multiplier of this lane's token
};

// Addresses are a uniform base (the panel's codes, the digit planes) plus a 32-bit offset per lane. `live` is uniform
// over the wavefront. A ring slot past the end of the wavefront's share still issues its loads (the loop stays
// branch-free, so the wait counts stay exact) but with offset 0 in every lane, a few bytes that all lanes share:
// memory throughput per compute unit is what bounds this kernel, and a ring that fetched real groups past the end
// would add up to `depth` groups to every wavefront's share.
template <int TT, bool SINGLE>
__device__ __forceinline__ void load_frag(Frag<TT, SINGLE> &f, const uint8_t *a_panel, uint32_t a_lane,
                                          const uint8_t *b_planes, uint32_t b_lane, const uint8_t *mvals,
                                          uint32_t m_lane, int g, int Mp, bool live) {
    // weights are read once (twice with two token blocks, and then from L2 at once): non-temporal, so they do not
    // displace the activation planes, which every workgroup re-reads
    typedef unsigned v2u __attribute__((ext_vector_type(2)));
    const uint32_t ao = live ? a_lane + (uint32_t) g * 2048u : 0u;
    const uint32_t bo = live ? b_lane + (uint32_t) g * (SINGLE ? 64u : 128u) * (uint32_t) Mp : 0u;
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        const v2u v = __builtin_nontemporal_load(reinterpret_cast<const v2u *>(a_panel + ao + rt * 256));
        f.a[rt] = make_uint2(v.x, v.y);
    }
    if constexpr (SINGLE) {
        const uint32_t mo = live ? m_lane + (uint32_t) g * (uint32_t) Mp : 0u;
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            f.b[tt][0] = *reinterpret_cast<const uint4 *>(b_planes + bo + 256 * tt);
            f.mv[tt] = mvals[mo + 16 * tt];
        }
    } else {
        const uint32_t plane = 64u * (uint32_t) Mp;   // bytes from the low digits of a group to its high digits
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            f.b[tt][0] = *reinterpret_cast<const uint4 *>(b_planes + bo + 256 * tt);
            f.b[tt][1] = *reinterpret_cast<const uint4 *>(b_planes + bo + plane + 256 * tt);
        }
    }
}

template <int TT, bool HASK, bool SINGLE>
__device__ __forceinline__ void mma_frag(const Frag<TT, SINGLE> &f, const uint8_t *k_base, int g, v4i (&hi)[4][TT],
                                         int32_t (&lo)[4][TT][4]) {
    v4i A[4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        int e0, o0, e1, o1;
        widen(f.a[rt].x, e0, o0);
        widen(f.a[rt].y, e1, o1);
        A[rt] = v4i{ e0, o0, e1, o1 };
    }
    int kk[4][4];
    if (HASK) {
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            const uint32_t k4 = *reinterpret_cast<const uint32_t *>(k_base + (size_t) g * kPanelRows + 16 * rt);
#pragma unroll
            for (int i = 0; i < 4; ++i) kk[rt][i] = (k4 >> (8 * i)) & 0xFF;
        }
    }
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        const v4i Blo = v4i{ (int) f.b[tt][0].x, (int) f.b[tt][0].y, (int) f.b[tt][0].z, (int) f.b[tt][0].w };
        if constexpr (SINGLE) {
            // S = 16 sum w (q - z); the group's term is floor(k m sum / 16) = (k m S) >> 8: |S| < 2^17, k m < 2^12
            const int mg = (int) f.mv[tt];
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                const v4i S = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[rt], Blo, v4i{ 0, 0, 0, 0 }, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; ++i) lo[rt][tt][i] += __mul24(S[i], HASK ? kk[rt][i] * mg : mg) >> 8;
            }
        } else {
            const v4i Bhi = v4i{ (int) f.b[tt][1].x, (int) f.b[tt][1].y, (int) f.b[tt][1].z, (int) f.b[tt][1].w };
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                if (!HASK) {
                    hi[rt][tt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[rt], Bhi, hi[rt][tt], 0, 0, 0);
                    const v4i S = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[rt], Blo, v4i{ 0, 0, 0, 0 }, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; ++i) lo[rt][tt][i] += S[i] >> 8;
                } else {
                    const v4i H = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[rt], Bhi, v4i{ 0, 0, 0, 0 }, 0, 0, 0);
                    const v4i S = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[rt], Blo, v4i{ 0, 0, 0, 0 }, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; ++i) lo[rt][tt][i] += (kk[rt][i] * ((H[i] << 6) + S[i])) >> 8;
                }
            }
        }
    }
}

// Activation groups of 128 / 256 (RQ_ACT_GROUP), single plane: the quantizer's multiplier, and with it the floor of
// the fold, covers gf = 2 or 4 consecutive runs of 64 (reference patch lines 160-170). The runs' sums chain through
// the MFMA accumulator (`acc`) and are folded once, at the group's last run, with the weight multiplier of its first
// run, as the reference takes it. `g` is the run's index in the row, so g % gf is its place in the group (uniform).
// |16 sum| < 2^19 and k m < 2^12: the 24-bit multiply and its 32-bit result are exact.
template <int TT, bool HASK>
__device__ __forceinline__ void mma_frag_wide(const Frag<TT, true> &f, const uint8_t *k_base, int g, int gf,
                                              v4i (&acc)[4][TT], int32_t (&lo)[4][TT][4]) {
    v4i A[4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        int e0, o0, e1, o1;
        widen(f.a[rt].x, e0, o0);
        widen(f.a[rt].y, e1, o1);
        A[rt] = v4i{ e0, o0, e1, o1 };
    }
    const int pos = g & (gf - 1);
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        const v4i B = v4i{ (int) f.b[tt][0].x, (int) f.b[tt][0].y, (int) f.b[tt][0].z, (int) f.b[tt][0].w };
        if (pos == 0) {
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) acc[rt][tt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[rt], B, v4i{ 0, 0, 0, 0 }, 0, 0, 0);
        } else {
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) acc[rt][tt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[rt], B, acc[rt][tt], 0, 0, 0);
        }
    }
    if (pos != gf - 1) return;
    int kk[4][4];
    if (HASK) {
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            const uint32_t k4 = *reinterpret_cast<const uint32_t *>(k_base + (size_t) (g - pos) * kPanelRows + 16 * rt);
#pragma unroll
            for (int i = 0; i < 4; ++i) kk[rt][i] = (k4 >> (8 * i)) & 0xFF;
        }
    }
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        const int mg = (int) f.mv[tt];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
            for (int i = 0; i < 4; ++i) lo[rt][tt][i] += __mul24(acc[rt][tt][i], HASK ? kk[rt][i] * mg : mg) >> 8;
        }
    }
}

// One wavefront's share of the K slice: activation groups u_first, u_first + kWaves, ... of gf = 1 << gsh runs each
// (n runs in all; gf = 1: the runs g_first, g_first + kWaves, ...). Ring slot j % D holds
// the wavefront's run j; the slot is refilled with group j + D as soon as group j's MFMAs have been issued. The scheduling
// barriers keep the compiler from sinking those loads to their first use (which would expose the whole memory
// latency once per group). Past the end the ring issues idle loads, and nothing consumes them.
__device__ __forceinline__ int run_at(int u_first, int gsh, int j) {
    return ((u_first + (j >> gsh) * kWaves) << gsh) + (j & ((1 << gsh) - 1));
}

template <int TT, bool SINGLE>
__device__ __forceinline__ void fill_ring(Frag<TT, SINGLE> (&ring)[depth_of(TT)], const uint8_t *a_panel, uint32_t a_lane,
                                          const uint8_t *b_planes, uint32_t b_lane, const uint8_t *mvals,
                                          uint32_t m_lane, int Mp, int u_first, int gsh, int n) {
#pragma unroll
    for (int i = 0; i < depth_of(TT); ++i) {
        load_frag<TT, SINGLE>(ring[i], a_panel, a_lane, b_planes, b_lane, mvals, m_lane, run_at(u_first, gsh, i), Mp, i < n);
    }
}

template <int TT, bool HASK, bool SINGLE, bool WIDE>
__device__ __forceinline__ void stream_slice(Frag<TT, SINGLE> (&ring)[depth_of(TT)], const uint8_t *a_panel,
                                             uint32_t a_lane, const uint8_t *b_planes, uint32_t b_lane,
                                             const uint8_t *mvals, uint32_t m_lane, const uint8_t *k_base, int Mp,
                                             int u_first, int gsh, int n, v4i (&hi)[4][TT], int32_t (&lo)[4][TT][4]) {
    auto mma = [&](const Frag<TT, SINGLE> &f, int g) __attribute__((always_inline)) {
        if constexpr (WIDE) {
            mma_frag_wide<TT, HASK>(f, k_base, g, 1 << gsh, hi, lo);
        } else {
            mma_frag<TT, HASK, SINGLE>(f, k_base, g, hi, lo);
        }
    };
    constexpr int D = depth_of(TT);
    // whole rounds of the ring: branch-free, so the wait counts before each group's MFMAs are exact
    const int rounds = n / D;
    for (int r = 0; r < rounds; ++r) {
#pragma unroll
        for (int i = 0; i < D; ++i) {
            const int j = r * D + i;
            __builtin_amdgcn_sched_barrier(0);
            mma(ring[i], run_at(u_first, gsh, j));
            __builtin_amdgcn_sched_barrier(0);
            load_frag<TT, SINGLE>(ring[i], a_panel, a_lane, b_planes, b_lane, mvals, m_lane, run_at(u_first, gsh, j + D), Mp, j + D < n);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // the last n % D groups are already in the ring
    const int rem = n - rounds * D;
#pragma unroll
    for (int i = 0; i < D - 1; ++i) {
        if (i < rem) mma(ring[i], run_at(u_first, gsh, rounds * D + i));
    }
}

// WIDE: activation groups of gf = 1 << gsh runs of 64 (single plane only); slices of K are then counted in groups.
template <int TT, bool SINGLE, bool WIDE = false>
__global__ void __launch_bounds__(kThreads, TT == 1 ? 4 : (SINGLE && TT == 2) ? 3 : 2)   // wavefronts per SIMD: 4 = two workgroups per CU
rq_skinny_kernel(const WeightSet ws, const uint4 *__restrict__ act8, const uint8_t *__restrict__ mvals,
                 const float *__restrict__ u, int M, int Mp, int gsh,
                 int n_units, int nz,
                 unsigned long long *__restrict__ cells, int n_rows_pad, int main_panels, int tail_split,
                 int slice_base, int slice_extra, int panel0) {
    constexpr int kTok = TT * 16;
    constexpr int kStride = kTok + 1;             // padded: the epilogue reads a column of this array
    __shared__ int32_t s_tot[64 * kStride];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, quad = lane >> 4;
    // workgroups of one panel's token blocks sit 8 apart in dispatch order: same XCD (ids go round-robin over the
    // eight XCDs), close in time
    const int bid = blockIdx.x;
    const int chunk = nz == 1 ? bid / kXcds : nz == 2 ? bid / (2 * kXcds) : bid / (kXcds * nz);   // (shifts for 1 and 2)
    const int within = bid - chunk * kXcds * nz;
    const int unit = chunk * kXcds + within % kXcds, z = within / kXcds;
    if (unit >= n_units) return;
    const int t0 = z * kTok;                       // first token of this workgroup
    // Units of work: main_panels panels take their whole K in one workgroup (no atomics); each panel after them is
    // cut into tail_split slices of K, one workgroup each, which meet in the arrival cells. The launcher picks the
    // cut so that the workgroups fill whole rounds of the chip. The slices come first in dispatch order: their
    // critical path has one more trip to memory (the arrival atomics), and trips are short while the chip is still
    // filling up.
    const int ng = ws.ng;
    const int tail_units = n_units - main_panels;
    // (g_begin, g_end: in activation groups, i.e. runs of 64 unless WIDE)
    int panel = unit - tail_units, ks = 0, nks = 1, g_begin = 0, g_end = WIDE ? ng >> gsh : ng;
    if (unit < tail_units) {
        const int q = unit / tail_split;
        panel = main_panels + q;
        ks = unit - q * tail_split;
        nks = tail_split;
        // slices of ng / nks groups, the first ng % nks one longer
        g_begin = ks * slice_base + (ks < slice_extra ? ks : slice_extra);
        g_end = g_begin + slice_base + (ks < slice_extra ? 1 : 0);
    }

    panel += panel0;   // a launch over a sub-range of the panels (the tail of a GEMM launch)
    // `panel` counts through the panels of up to three weights: which weight, and which of its panels
    const int wsel = (panel >= ws.first[1]) + (panel >= ws.first[2]);
    const int wpanel = panel - (wsel == 0 ? 0 : wsel == 1 ? ws.first[1] : ws.first[2]);
    const uint8_t *__restrict__ codes = wsel == 0 ? ws.codes[0] : wsel == 1 ? ws.codes[1] : ws.codes[2];
    const uint8_t *__restrict__ kmul = wsel == 0 ? ws.kmul[0] : wsel == 1 ? ws.kmul[1] : ws.kmul[2];
    const int32_t *__restrict__ flags = wsel == 0 ? ws.flags[0] : wsel == 1 ? ws.flags[1] : ws.flags[2];
    const float *__restrict__ s_w = wsel == 0 ? ws.s_w[0] : wsel == 1 ? ws.s_w[1] : ws.s_w[2];
    float *__restrict__ y = wsel == 0 ? ws.y[0] : wsel == 1 ? ws.y[1] : ws.y[2];
    const int64_t ldy = wsel == 0 ? ws.ldy[0] : wsel == 1 ? ws.ldy[1] : ws.ldy[2];
    const int64_t N = wsel == 0 ? ws.N[0] : wsel == 1 ? ws.N[1] : ws.N[2];

    // this lane's byte of the panel: half quad >> 1, row l16 (+ 16 per row tile), 8 bytes at (quad & 1) * 8
    const uint8_t *a_panel = codes + (size_t) wpanel * ng * 2048;
    const uint32_t a_lane = (quad >> 1) * 1024 + l16 * 16 + (quad & 1) * 8;
    // this lane's cell of the digit planes: quarter quad, token t0 + l16 (+ 16 per token tile)
    const uint8_t *b_planes = reinterpret_cast<const uint8_t *>(act8);
    const uint32_t b_lane = ((uint32_t) quad * Mp + t0 + l16) * 16u;
    const uint32_t m_lane = (uint32_t) (t0 + l16);   // SINGLE: the multiplier of this lane's token (+ 16 per token tile)
    const uint8_t *k_base = kmul + (size_t) wpanel * ng * kPanelRows + 4 * quad;

    v4i hi[4][TT];
    int32_t lo[4][TT][4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            hi[rt][tt] = v4i{ 0, 0, 0, 0 };
#pragma unroll
            for (int i = 0; i < 4; ++i) lo[rt][tt][i] = 0;
        }
    }

    // What the epilogue needs from memory is asked for first: loads return in order, so by the time the first group
    // of weights is here these are too, and the tail of the kernel has no trip to memory left but its own stores.
    const int64_t nrow = (int64_t) wpanel * kPanelRows + lane;      // row of its weight
    const int64_t cell_row = (int64_t) panel * kPanelRows + lane;   // row of the launch (split-K cell)
    const float sw_row = s_w[nrow];                 // rows past N are stored as zero
    float u_tok[kTok / kWaves];
#pragma unroll
    for (int i = 0; i < kTok / kWaves; ++i) u_tok[i] = u[t0 + wave + i * kWaves];   // u has a slot for every padded token
    const int32_t has_k = *reinterpret_cast<const volatile int32_t *>(flags) & 1;

    // the first loads go out before anything that waits (the LDS clear)
    const int g_first = g_begin + wave;
    const int gs = WIDE ? gsh : 0;
    const int n = g_first < g_end ? ((g_end - g_first + kWaves - 1) / kWaves) << gs : 0;   // runs of this wavefront
    Frag<TT, SINGLE> ring[depth_of(TT)];
    fill_ring<TT, SINGLE>(ring, a_panel, a_lane, b_planes, b_lane, mvals, m_lane, Mp, g_first, gs, n);
    __builtin_amdgcn_sched_barrier(0);

    for (int i = tid; i < 64 * kStride; i += kThreads) s_tot[i] = 0;

    if (n > 0) {
        if (has_k) {
            stream_slice<TT, true, SINGLE, WIDE>(ring, a_panel, a_lane, b_planes, b_lane, mvals, m_lane, k_base, Mp, g_first, gs, n, hi, lo);
        } else {
            stream_slice<TT, false, SINGLE, WIDE>(ring, a_panel, a_lane, b_planes, b_lane, mvals, m_lane, k_base, Mp, g_first, gs, n, hi, lo);
        }
    }

    // the wavefronts' partial totals meet in LDS (integer adds: any order)
    __syncthreads();
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int32_t tot = SINGLE ? lo[rt][tt][i] : (hi[rt][tt][i] >> 2) + lo[rt][tt][i];
                atomicAdd(&s_tot[(16 * rt + 4 * quad + i) * kStride + 16 * tt + l16], tot);
            }
        }
    }
    __syncthreads();

    // epilogue: lane = row, a wavefront per token (coalesced rows of y); split-K through the arrival cells
#pragma unroll
    for (int i = 0; i < kTok / kWaves; ++i) {
        const int tl = wave + i * kWaves;
        const int t = t0 + tl;
        if (t >= M) break;
        int32_t sum = s_tot[lane * kStride + tl];
        if (nks > 1) {
            unsigned long long *cell = cells + (size_t) t * n_rows_pad + cell_row;
            const unsigned long long mine = (1ull << 48) + (unsigned long long) (long long) sum;
            const unsigned long long now =
                __hip_atomic_fetch_add(cell, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + mine;
            if ((int) ((now + (1ull << 47)) >> 48) != nks) continue;
            __hip_atomic_store(cell, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            sum = (int32_t) (uint32_t) now;
        }
        if (nrow < N) y[(int64_t) t * ldy + nrow] = (((float) sum * 16.0f) * u_tok[i]) * sw_row;
    }
}

template <int TT, bool SINGLE, bool WIDE = false>
hipError_t launch_tt(const SkinnyArgs &a, hipStream_t stream) {
    const WeightSet ws = make_weight_set(a.w);
    const int n_panels = a.panels > 0 ? a.panels : ws.first[kMaxFused];
    const int nz = (a.M + TT * 16 - 1) / (TT * 16);
    const int gf = WIDE ? a.runs_per_group : 1, gsh = gf == 4 ? 2 : gf == 2 ? 1 : 0;
    const int n_groups = ws.ng / gf;   // what a slice of K is counted in
    SkinnyPlan plan;
    if (a.panels > 0) {   // whole K per workgroup: no arrival cells
        plan.main_panels = n_panels;
        plan.tail_split = 1;
    } else {
        plan = skinny_plan(n_panels, ws.ng, a.M, nz, gf);
    }
    const int n_units = plan.main_panels + (n_panels - plan.main_panels) * plan.tail_split;
    const int blocks = (n_units + 7) / 8 * 8 * nz;
    hipLaunchKernelGGL((rq_skinny_kernel<TT, SINGLE, WIDE>), dim3(blocks), dim3(kThreads), 0, stream, ws,
                       reinterpret_cast<const uint4 *>(a.act8), a.mvals, a.u, a.M, a.Mp, gsh, n_units, nz,
                       reinterpret_cast<unsigned long long *>(a.tot), ws.first[kMaxFused] * kPanelRows,
                       plan.main_panels, plan.tail_split, n_groups / plan.tail_split, n_groups % plan.tail_split,
                       a.panels > 0 ? a.panel0 : 0);
    return hipGetLastError();
}

}  // namespace

// How the panels are dealt to workgroups. One workgroup keeps a compute unit's memory pipeline full, and workgroups
// go to the compute units round robin, so the kernel takes as long as the busiest compute unit: 272 whole panels on
// 256 compute units cost two rounds (measured: 16.9 us against 10.6 us for 256 panels). So the panels that fill
// whole rounds run as whole-K workgroups, and the remainder is cut along K into slices small enough to spread over
// the chip: `tail_split` slices per panel, which meet in 64-bit arrival cells. Device-scope atomics cost about 7 ns
// per thousand, so the cut is chosen by a small cost model (busiest compute unit + atomics) rather than maximised.
SkinnyPlan skinny_plan(int n_panels, int ng, int M, int nz, int runs_per_group) {
    const int kCUs = device_compute_units();
    SkinnyPlan plan;
    // at least four runs of 64 per slice, and whole activation groups (runs_per_group runs each)
    const int per_slice = runs_per_group > 4 ? runs_per_group : 4;
    const int smax = ng / per_slice < 1 ? 1 : (ng / per_slice > 16 ? 16 : ng / per_slice);
    const int per_round = kCUs / nz;                       // panels in one round of the chip
    plan.main_panels = n_panels / per_round * per_round;
    plan.tail_split = 1;
    const int b = n_panels - plan.main_panels;
    if (b == 0) return plan;
    // microseconds: a panel's weights at the rate one compute unit sustains, atomics at 7 ns per thousand (mostly
    // hidden behind the whole panels when there are any)
    const double t_panel = (double) ng * 2048.0 / (M <= 16 ? 19000.0 : 13000.0);
    const double atomics_weight = plan.main_panels > 0 ? 0.25 : 1.0;
    double best = 1e30;
    for (int s = 1; s <= smax; ++s) {
        const int rounds = (b * nz * s + kCUs - 1) / kCUs;
        const double cost = rounds * t_panel / s
                            + (s > 1 ? atomics_weight * 0.007e-3 * (double) b * kPanelRows * M * s : 0.0);
        if (cost < best - 1e-9) {
            best = cost;
            plan.tail_split = s;
        }
    }
    return plan;
}

hipError_t launch_skinny(const SkinnyArgs &a, hipStream_t stream) {
    constexpr int tt1_max = 16;   // most tokens served with one token tile of 16 per wavefront
    if (a.panels > 0) return launch_tt<2, false>(a, stream);   // the tail of a GEMM launch: blocks of 32 tokens
    if (a.mvals != nullptr && a.runs_per_group > 1) {
        // activation groups of 128 / 256: one or two token tiles per wavefront, more tokens as blocks of 32
        if (a.M <= 16) return launch_tt<1, true, true>(a, stream);
        return launch_tt<2, true, true>(a, stream);
    }
    if (a.mvals != nullptr) {   // the caller wrote single-plane activations
        // 33..64 tokens: one workgroup with four token tiles per wavefront reads the weights once and halves the
        // workgroup count, two blocks of 32 tokens give twice the workgroups. The former wins on long rows and on
        // weights with a whole round of panels (K=17408, N=5120, M=64: 22.7 against 26.9 us; K=5120, N=17408: 27.1
        // against 27.9), the latter on small weights (K=5120, N=5120: 10.9 against 15.8 us).
        int n_panels = 0;
        for (int i = 0; i < a.w.n; ++i) n_panels += a.w.L[i].n_panels;
        const bool wide = a.w.L[0].ng >= 160 || n_panels >= device_compute_units();
        if (a.M > 32 && wide) return launch_tt<4, true>(a, stream);
        if (a.M <= 16) return launch_tt<1, true>(a, stream);
        return launch_tt<2, true>(a, stream);
    }
    if (a.M <= (tt1_max > 64 ? 64 : tt1_max)) return launch_tt<1, false>(a, stream);
    return launch_tt<2, false>(a, stream);
}

}  // namespace rq
