// int4 x int4 GEMM on the gfx950 matrix cores (v_mfma_i32_16x16x64_i8) for wide token batches.
//
// The reference total is sum over 64-input groups g of floor(m_g * S_g / 16), S_g = sum_k w_k (q_k - z_g)
// (ggml_vec_dot_w4a4_a4, reference patch lines 148-177, with acc + (8 - z) colsum written as one sum). One MFMA
// has K = 64 = exactly one group, but the floor per group is not linear, and a multiply + shift + add per output
// and group on the vector ALU would cost several times the MFMA itself. So the multiplier goes INTO the matrix
// operand: the quantizer emits p = m_g (q - z) (|p| <= 3825) as two balanced int8 digits, p = 64 hi + lo with
// lo in [-32, 31] and hi in [-60, 60]. Then
//     m_g S_g = 64 Xhi_g + Xlo_g,   floor(m_g S_g / 16) = 4 Xhi_g + floor(Xlo_g / 16),
// where Xhi_g = sum w hi accumulates ACROSS groups inside the MFMA accumulator (no vector work at all) and only
// Xlo_g = sum w lo needs the per-group floor: one arithmetic shift and one add per output and group, both
// full-rate ops. Two MFMAs per group instead of one, but the vector ALU no longer paces the loop.
//
// Weight codes stay packed (int4) all the way into LDS and are widened when a wavefront reads its A fragment, by
// masking each nibble into the HIGH half of a byte (w * 16, no sign extension needed), so every X above arrives
// times 16: the fold shifts by 8, the final hi sum by 2.
//
// Tensors whose headers carry integer weight multipliers k (uniform branch on the prepared flag) restart both
// accumulators every group and fold floor(k (64 Xhi + Xlo) / 16) on the vector ALU.
//
// Data movement: a workgroup of eight wavefronts owns 256 rows (four panels) x 128 tokens; wavefront (wr, wc) owns
// rows 64 wr.. and tokens 64 wc.. as 4 x 4 MFMA tiles. The operands of one group (8 KiB of packed weights, 16 KiB of
// activation digits) go from global memory straight into LDS with global_load_lds_dwordx4 (no registers, no
// ds_write), kStages groups deep, so a fetch has several groups of arithmetic to complete. The prepared weight
// layout and the quantizer's output layout are exactly the LDS layouts: every wavefront-wide transfer is 1 KiB
// contiguous on both sides.
#include "rq_common.h"

#pragma clang fp contract(off)

namespace rq {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void global_cvoid;

constexpr int kBN = 256;        // rows per workgroup (four panels)
constexpr int kBT = 128;        // tokens per workgroup
constexpr int kThreads = 512;
constexpr int kStages = 6;      // LDS ring depth
constexpr int kLoads = 3;       // LDS-direct loads per thread and group: 1 weight cell + 2 activation cells

struct Stage {
    uint4 a[4][2][64];      // packed weights [panel][half of the group][row]: 16 bytes = 32 codes
    uint4 b[2][4][kBT];     // activation digits [0 = lo, 1 = hi][quarter of the group][token]
};
static_assert(sizeof(Stage) == 24576, "stage size");

// 8 int4 codes (nibble j = element j) -> the four even elements and the four odd elements, each as code * 16
__device__ __forceinline__ void widen(uint32_t w, int &even, int &odd) {
    even = (int) ((w << 4) & 0xF0F0F0F0u);
    odd = (int) (w & 0xF0F0F0F0u);
}

__device__ __forceinline__ v4i as_v4i(const uint4 v) { return v4i{ (int) v.x, (int) v.y, (int) v.z, (int) v.w }; }

struct Ctx {
    const uint4 *w_src;   // this thread's weight cell of group 0
    const uint4 *a_src;   // this thread's first activation cell of group 0
    size_t a_cell, a_step;
    int wave, wr, wc, l16, quad;
    int ng;
};

// One LDS-direct load: 64 lanes x 16 bytes from the lanes' global addresses to 1 KiB of LDS starting at `lds`
// (wave-uniform; the hardware adds lane * 16). Written as assembly so that the outstanding-load count stays under
// this file's control: the compiler's own bookkeeping would wait for every LDS-direct load before any LDS read.
// The LDS pointer is an operand and memory is clobbered, so the compiler treats the stage as written.
__device__ __forceinline__ void load_to_lds(const uint4 *gptr, uint4 *lds) {
    const uint32_t lds_addr = (uint32_t) (uintptr_t) (lds_void *) lds;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(lds_addr)
                 : "memory", "m0");
}

// fetch of group g into stage s: every wavefront moves three 1 KiB runs
__device__ __forceinline__ void fetch(const Ctx &c, Stage &s, int g) {
    const int gg = g < c.ng ? g : c.ng - 1;   // past the end: refetch the last group into a stage nobody reads
    uint4 *a_dst = &s.a[0][0][0] + c.wave * 64;
    uint4 *b_dst = &s.b[0][0][0] + c.wave * 64;
    load_to_lds(c.w_src + (size_t) gg * 128, a_dst);
    load_to_lds(c.a_src + (size_t) gg * c.a_step, b_dst);
    load_to_lds(c.a_src + (size_t) gg * c.a_step + c.a_cell, b_dst + 512);
}

template <bool HASK>
__device__ __forceinline__ void compute(const Ctx &c, const Stage &s, const uint8_t *__restrict__ k_src, int g,
                                        v4i (&hi)[4][4], int32_t (&lo)[4][4][4]) {
    v4i A[4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        // quarter `quad` of the group = 8 bytes of the row's cell in half quad >> 1
        const uint2 pk = *(reinterpret_cast<const uint2 *>(&s.a[c.wr][c.quad >> 1][16 * rt + c.l16]) + (c.quad & 1));
        int e0, o0, e1, o1;
        widen(pk.x, e0, o0);
        widen(pk.y, e1, o1);
        A[rt] = v4i{ e0, o0, e1, o1 };
    }
    int kk[4][4];
    if (HASK) {
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            const uint32_t k4 = *reinterpret_cast<const uint32_t *>(k_src + (size_t) g * kPanelRows + 16 * rt);
#pragma unroll
            for (int i = 0; i < 4; ++i) kk[rt][i] = (k4 >> (8 * i)) & 0xFF;
        }
    }
    if (!HASK) {
        // Software pipeline over the four token tiles: the eight MFMAs of tile ct are issued back to back while the
        // vector ALU folds the four results of tile ct - 1, so neither unit waits for the other.
        v4i S[2][4];
#pragma unroll
        for (int ct = 0; ct < 5; ++ct) {
            if (ct < 4) {
                const v4i Blo = as_v4i(s.b[0][c.quad][64 * c.wc + 16 * ct + c.l16]);
                const v4i Bhi = as_v4i(s.b[1][c.quad][64 * c.wc + 16 * ct + c.l16]);
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) {
                    S[ct & 1][rt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[rt], Blo, v4i{ 0, 0, 0, 0 }, 0, 0, 0);
                    hi[rt][ct] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[rt], Bhi, hi[rt][ct], 0, 0, 0);
                }
            }
            if (ct > 0) {
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) lo[rt][ct - 1][i] += S[(ct - 1) & 1][rt][i] >> 8;
                }
            }
            if (ct > 0 && ct < 4) {
                // 8 MFMAs interleaved with the 32 vector ops of the previous tile's fold: 1 MFMA, 4 VALU, ...
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
                    __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);  // VALU
                }
            }
        }
    } else {
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
            const v4i Blo = as_v4i(s.b[0][c.quad][64 * c.wc + 16 * ct + c.l16]);
            const v4i Bhi = as_v4i(s.b[1][c.quad][64 * c.wc + 16 * ct + c.l16]);
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                const v4i H = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[rt], Bhi, v4i{ 0, 0, 0, 0 }, 0, 0, 0);
                const v4i S = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[rt], Blo, v4i{ 0, 0, 0, 0 }, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; ++i) lo[rt][ct][i] += (kk[rt][i] * ((H[i] << 6) + S[i])) >> 8;
            }
        }
    }
}

// One group: wait for its operands, meet the other wavefronts, refill the stage that was just released, compute.
// At the wait, the loads this thread has issued after group g's are those of groups g+1 .. g+kStages-2.
template <bool HASK>
__device__ __forceinline__ void step(const Ctx &c, const Stage &cur, Stage &refill, const uint8_t *__restrict__ k_src,
                                     int g, v4i (&hi)[4][4], int32_t (&lo)[4][4][4]) {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kStages - 2) * kLoads) : "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    fetch(c, refill, g + kStages - 1);
    compute<HASK>(c, cur, k_src, g, hi, lo);
}

template <bool HASK>
__device__ __forceinline__ void gemm_body(const Ctx &c, Stage &s0, Stage &s1, Stage &s2, Stage &s3, Stage &s4,
                                          Stage &s5, const uint8_t *__restrict__ k_src, v4i (&hi)[4][4],
                                          int32_t (&lo)[4][4][4]) {
    fetch(c, s0, 0);
    fetch(c, s1, 1);
    fetch(c, s2, 2);
    fetch(c, s3, 3);
    fetch(c, s4, 4);
    for (int g = 0; g < c.ng; g += kStages) {
        step<HASK>(c, s0, s5, k_src, g, hi, lo);
        if (g + 1 < c.ng) step<HASK>(c, s1, s0, k_src, g + 1, hi, lo);
        if (g + 2 < c.ng) step<HASK>(c, s2, s1, k_src, g + 2, hi, lo);
        if (g + 3 < c.ng) step<HASK>(c, s3, s2, k_src, g + 3, hi, lo);
        if (g + 4 < c.ng) step<HASK>(c, s4, s3, k_src, g + 4, hi, lo);
        if (g + 5 < c.ng) step<HASK>(c, s5, s4, k_src, g + 5, hi, lo);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // drain the refetches of the last group before LDS is released
}

__global__ void __launch_bounds__(kThreads)
rq_gemm_kernel(const uint4 *__restrict__ codes, const float *__restrict__ s_w, const uint8_t *__restrict__ kmul,
               const int32_t *__restrict__ flags, const uint4 *__restrict__ act8, const float *__restrict__ u,
               float *__restrict__ y, int64_t ldy, int64_t N, int M, int Mp, int ng, int n_panels, int n_row_tiles,
               int n_tok_tiles) {
    // one array per stage: the compiler tracks LDS-direct loads per destination object
    __shared__ Stage s0;
    __shared__ Stage s1;
    __shared__ Stage s2;
    __shared__ Stage s3;
    __shared__ Stage s4;
    __shared__ Stage s5;

    // Workgroups go to the eight XCDs round robin. Give every XCD a contiguous run of row tiles with the token
    // tiles running fastest, so the workgroups resident on one XCD share weight and activation tiles in its L2.
    const int total = n_row_tiles * n_tok_tiles;
    int v = blockIdx.x;
    const int per_xcd = total / 8;
    if (v < per_xcd * 8) v = (v & 7) * per_xcd + (v >> 3);
    const int row_tile = v / n_tok_tiles, tok_tile = v - row_tile * n_tok_tiles;
    const int panel0 = row_tile * 4, t0 = tok_tile * kBT;

    const int tid = threadIdx.x;
    Ctx c;
    c.wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    c.wr = c.wave & 3;
    c.wc = c.wave >> 2;
    c.l16 = tid & 15;
    c.quad = (tid & 63) >> 4;
    c.ng = ng;
    // weights: thread tid moves cell tid of the tile's 512 (panel = tid >> 7, half = (tid >> 6) & 1, row = tid & 63);
    // panels past the tensor read panel n_panels - 1 again (their outputs are never stored)
    const int w_panel = min(panel0 + (tid >> 7), n_panels - 1);
    c.w_src = codes + (size_t) w_panel * ng * 128 + (tid & 127);
    // activations: the tile of one group is 1024 cells [digit][quarter][token]; thread tid moves cells tid and
    // tid + 512 (digit = cell >> 9, quarter = (cell >> 7) & 3, token = cell & 127)
    c.a_src = act8 + (size_t) (tid >> 7) * Mp + t0 + (tid & 127);
    c.a_cell = (size_t) 4 * Mp;   // + 512 cells = the other digit
    c.a_step = (size_t) 8 * Mp;   // cells per group
    const uint8_t *k_src = kmul + (size_t) min(panel0 + c.wr, n_panels - 1) * ng * kPanelRows + 4 * c.quad;

    v4i hi[4][4];
    int32_t lo[4][4][4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
            hi[rt][ct] = v4i{ 0, 0, 0, 0 };
#pragma unroll
            for (int i = 0; i < 4; ++i) lo[rt][ct][i] = 0;
        }
    }

    if (flags[0] & 1) {
        gemm_body<true>(c, s0, s1, s2, s3, s4, s5, k_src, hi, lo);
    } else {
        gemm_body<false>(c, s0, s1, s2, s3, s4, s5, k_src, hi, lo);
    }

    // epilogue (reference patch line 176): y = ((float(total) * 16) * u) * s_w, total = 4 Xhi + sum of floors
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
        const int t = t0 + 64 * c.wc + 16 * ct + c.l16;
        if (t >= M) continue;
        const float ut = u[t];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            const int64_t n = (int64_t) (panel0 + c.wr) * kPanelRows + 16 * rt + 4 * c.quad;
            float *dst = y + (int64_t) t * ldy + n;
            int32_t tot[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) tot[i] = (hi[rt][ct][i] >> 2) + lo[rt][ct][i];
            if (n + 3 < N && ((reinterpret_cast<uintptr_t>(dst) & 15) == 0)) {
                const float4 sw = *reinterpret_cast<const float4 *>(s_w + n);
                float4 o;
                o.x = (((float) tot[0] * 16.0f) * ut) * sw.x;
                o.y = (((float) tot[1] * 16.0f) * ut) * sw.y;
                o.z = (((float) tot[2] * 16.0f) * ut) * sw.z;
                o.w = (((float) tot[3] * 16.0f) * ut) * sw.w;
                *reinterpret_cast<float4 *>(dst) = o;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (n + i < N) dst[i] = (((float) tot[i] * 16.0f) * ut) * s_w[n + i];
                }
            }
        }
    }
}

}  // namespace

hipError_t launch_gemm(const GemmArgs &a, hipStream_t stream) {
    const uint8_t *p = a.prepared;
    const int n_row_tiles = (a.L.n_panels + 3) / 4;
    const int n_tok_tiles = a.Mp / kBT;
    hipLaunchKernelGGL(rq_gemm_kernel, dim3(n_row_tiles * n_tok_tiles), dim3(kThreads), 0, stream,
                       reinterpret_cast<const uint4 *>(p + a.L.off_codes),
                       reinterpret_cast<const float *>(p + a.L.off_sw), p + a.L.off_kmul,
                       reinterpret_cast<const int32_t *>(p + a.L.off_flags),
                       reinterpret_cast<const uint4 *>(a.act8), a.u, a.y, a.ldy, a.L.N, a.M, a.Mp, a.L.ng,
                       a.L.n_panels, n_row_tiles, n_tok_tiles);
    return hipGetLastError();
}

}  // namespace rq
