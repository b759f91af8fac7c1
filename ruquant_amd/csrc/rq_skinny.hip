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

template <int TT>
struct Frag {
    uint2 a[4];        // packed weights of the four 16-row tiles: this lane's quarter of the group
    uint4 b[TT][2];    // activation digits (lo, hi) of the token tiles: this lane's quarter
};

template <int TT>
__device__ __forceinline__ void load_frag(Frag<TT> &f, const uint8_t *a_base, const uint4 *b_base, int g, int Mp) {
    // weights are read once (twice with two token blocks, and then from L2 at once): non-temporal, so they do not
    // displace the digit planes, which every workgroup re-reads
    typedef unsigned v2u __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        const v2u v = __builtin_nontemporal_load(reinterpret_cast<const v2u *>(a_base + (size_t) g * 2048 + rt * 256));
        f.a[rt] = make_uint2(v.x, v.y);
    }
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        f.b[tt][0] = b_base[(size_t) g * 8 * Mp + 16 * tt];
        f.b[tt][1] = b_base[(size_t) g * 8 * Mp + (size_t) 4 * Mp + 16 * tt];
    }
}

template <int TT, bool HASK>
__device__ __forceinline__ void mma_frag(const Frag<TT> &f, const uint8_t *k_base, int g, v4i (&hi)[4][TT],
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

// One wavefront's share of the K slice: groups g_first, g_first + kWaves, ... (n of them). Ring slot j % D holds
// group j; the slot is refilled with group j + D as soon as group j's MFMAs have been issued. The scheduling
// barriers keep the compiler from sinking those loads to their first use (which would expose the whole memory
// latency once per group). Past the end the ring refetches the last group, and nothing consumes it.
template <int TT>
__device__ __forceinline__ void fill_ring(Frag<TT> (&ring)[depth_of(TT)], const uint8_t *a_base, const uint4 *b_base,
                                          int Mp, int g_first, int g_last) {
#pragma unroll
    for (int i = 0; i < depth_of(TT); ++i) {
        const int g = g_first + i * kWaves;
        load_frag<TT>(ring[i], a_base, b_base, g < g_last ? g : g_last, Mp);
    }
}

template <int TT, bool HASK>
__device__ __forceinline__ void stream_slice(Frag<TT> (&ring)[depth_of(TT)], const uint8_t *a_base,
                                             const uint4 *b_base, const uint8_t *k_base, int Mp, int g_first, int n,
                                             int g_last, v4i (&hi)[4][TT], int32_t (&lo)[4][TT][4]) {
    constexpr int D = depth_of(TT);
    // whole rounds of the ring: branch-free, so the wait counts before each group's MFMAs are exact
    const int rounds = n / D;
    for (int r = 0; r < rounds; ++r) {
#pragma unroll
        for (int i = 0; i < D; ++i) {
            const int g = g_first + (r * D + i) * kWaves;
            const int gn = g + D * kWaves;
            __builtin_amdgcn_sched_barrier(0);
            mma_frag<TT, HASK>(ring[i], k_base, g, hi, lo);
            __builtin_amdgcn_sched_barrier(0);
            load_frag<TT>(ring[i], a_base, b_base, gn < g_last ? gn : g_last, Mp);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // the last n % D groups are already in the ring
    const int rem = n - rounds * D;
#pragma unroll
    for (int i = 0; i < D - 1; ++i) {
        if (i < rem) mma_frag<TT, HASK>(ring[i], k_base, g_first + (rounds * D + i) * kWaves, hi, lo);
    }
}

template <int TT>
__global__ void __launch_bounds__(kThreads, TT == 1 ? 4 : 2)   // wavefronts per SIMD: two workgroups per CU at TT = 1
rq_skinny_kernel(const uint8_t *__restrict__ codes, const float *__restrict__ s_w, const uint8_t *__restrict__ kmul,
                 const int32_t *__restrict__ flags, const uint4 *__restrict__ act8, const float *__restrict__ u,
                 float *__restrict__ y, int64_t ldy, int64_t N, int M, int Mp, int ng, int n_panels, int nz,
                 unsigned long long *__restrict__ cells, int n_rows_pad, int slice_base, int slice_extra) {
    constexpr int kTok = TT * 16;
    constexpr int kStride = kTok + 1;             // padded: the epilogue reads a column of this array
    __shared__ int32_t s_tot[64 * kStride];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, quad = lane >> 4;
    // workgroups of one panel's token blocks sit 8 apart in dispatch order: same XCD (ids go round-robin over the
    // eight XCDs), close in time
    const int bid = blockIdx.x;
    const int chunk = bid >> (nz == 2 ? 4 : 3), within = bid - chunk * 8 * nz;   // nz is 1 or 2
    const int panel = chunk * 8 + (within & 7), z = within >> 3;
    if (panel >= n_panels) return;
    const int t0 = z * kTok;                       // first token of this workgroup
    const int nks = gridDim.y, ks = blockIdx.y;
    // slices of ng / nks groups, the first ng % nks one longer (no division on the device)
    const int g_begin = ks * slice_base + (ks < slice_extra ? ks : slice_extra);
    const int g_end = g_begin + slice_base + (ks < slice_extra ? 1 : 0);

    // this lane's byte of the panel: half quad >> 1, row l16 (+ 16 per row tile), 8 bytes at (quad & 1) * 8
    const uint8_t *a_base = codes + (size_t) panel * ng * 2048 + (quad >> 1) * 1024 + l16 * 16 + (quad & 1) * 8;
    // this lane's cell of the digit planes: quarter quad, token t0 + l16 (+ 16 per token tile)
    const uint4 *b_base = act8 + (size_t) quad * Mp + t0 + l16;
    const uint8_t *k_base = kmul + (size_t) panel * ng * kPanelRows + 4 * quad;

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

    // the first loads go out before anything that waits (the flag word, the LDS clear)
    const int g_first = g_begin + wave;
    const int n = g_first < g_end ? (g_end - g_first + kWaves - 1) / kWaves : 0;
    const int g_last = n > 0 ? g_first + (n - 1) * kWaves : g_begin;
    Frag<TT> ring[depth_of(TT)];
    fill_ring<TT>(ring, a_base, b_base, Mp, n > 0 ? g_first : g_begin, g_last);
    __builtin_amdgcn_sched_barrier(0);

    for (int i = tid; i < 64 * kStride; i += kThreads) s_tot[i] = 0;

    if (n > 0) {
        if (*reinterpret_cast<const volatile int32_t *>(flags) & 1) {
            stream_slice<TT, true>(ring, a_base, b_base, k_base, Mp, g_first, n, g_last, hi, lo);
        } else {
            stream_slice<TT, false>(ring, a_base, b_base, k_base, Mp, g_first, n, g_last, hi, lo);
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
                const int32_t tot = (hi[rt][tt][i] >> 2) + lo[rt][tt][i];
                atomicAdd(&s_tot[(16 * rt + 4 * quad + i) * kStride + 16 * tt + l16], tot);
            }
        }
    }
    __syncthreads();

    // epilogue: lane = row, a wavefront per token (coalesced rows of y); split-K through the arrival cells
    const int64_t nrow = (int64_t) panel * kPanelRows + lane;
    for (int tl = wave; tl < kTok; tl += kWaves) {
        const int t = t0 + tl;
        if (t >= M) break;
        int32_t sum = s_tot[lane * kStride + tl];
        if (nks > 1) {
            unsigned long long *cell = cells + (size_t) t * n_rows_pad + nrow;
            const unsigned long long mine = (1ull << 48) + (unsigned long long) (long long) sum;
            const unsigned long long now =
                __hip_atomic_fetch_add(cell, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + mine;
            if ((int) ((now + (1ull << 47)) >> 48) != nks) continue;
            __hip_atomic_store(cell, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            sum = (int32_t) (uint32_t) now;
        }
        if (nrow < N) y[(int64_t) t * ldy + nrow] = (((float) sum * 16.0f) * u[t]) * s_w[nrow];
    }
}

template <int TT>
hipError_t launch_tt(const SkinnyArgs &a, hipStream_t stream) {
    const uint8_t *p = a.prepared;
    const int nz = (a.M + TT * 16 - 1) / (TT * 16);
    const int nks = skinny_ksplit(a.L, a.M);
    const int blocks = (a.L.n_panels + 7) / 8 * 8 * nz;
    hipLaunchKernelGGL((rq_skinny_kernel<TT>), dim3(blocks, nks), dim3(kThreads), 0, stream, p + a.L.off_codes,
                       reinterpret_cast<const float *>(p + a.L.off_sw), p + a.L.off_kmul,
                       reinterpret_cast<const int32_t *>(p + a.L.off_flags), reinterpret_cast<const uint4 *>(a.act8),
                       a.u, a.y, a.ldy, a.L.N, a.M, a.Mp, a.L.ng, a.L.n_panels, nz,
                       reinterpret_cast<unsigned long long *>(a.tot), a.L.n_panels * kPanelRows, a.L.ng / nks, a.L.ng % nks);
    return hipGetLastError();
}

}  // namespace

// K splits across workgroups: enough workgroups to cover the chip twice, within a budget of L2 atomics (one per
// output and split), and at least two groups per wavefront
int skinny_ksplit(const PreparedLayout &L, int M) {
    static const int forced = getenv("RQ_SKINNY_KSPLIT") ? atoi(getenv("RQ_SKINNY_KSPLIT")) : 0;
    const int nz = M <= 16 ? 1 : (M + 31) / 32;
    int nks = (512 + L.n_panels * nz - 1) / (L.n_panels * nz);
    const int64_t budget = 400000 / ((int64_t) M * L.n_panels * kPanelRows);
    if (nks > budget) nks = (int) budget;
    if (forced > 0) nks = forced;
    if (nks > L.ng / (2 * kWaves)) nks = L.ng / (2 * kWaves);
    return nks < 1 ? 1 : nks;
}

hipError_t launch_skinny(const SkinnyArgs &a, hipStream_t stream) {
    if (a.M <= 16) return launch_tt<1>(a, stream);
    return launch_tt<2>(a, stream);
}

}  // namespace rq
