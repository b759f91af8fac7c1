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
// Xlo_g = sum w lo needs the per-group floor. That floor rides on the accumulator too: the low-digit accumulator
// holds 256 h + r (h = floors so far, r = the last group's remainder); clearing r with one AND per output and
// group and handing the result to the next group's MFMA as its C operand yields Xlo' + 256 h, whose floor by 256
// is floor(Xlo' / 256) + h (Xlo' = 16 Xlo, see below). Two MFMAs per group instead of one, and one full-rate
// vector instruction per output and group.
//
// Weight codes stay packed (int4) all the way into LDS and are widened when a wavefront reads its A fragment, by
// masking each nibble into the HIGH half of a byte (w * 16, no sign extension needed), so every X above arrives
// times 16: the fold shifts by 8, the final hi sum by 2.
//
// Tensors whose headers carry integer weight multipliers k (uniform branch on the prepared flag) restart both
// accumulators every group and fold floor(k (64 Xhi + Xlo) / 16) on the vector ALU.
//
// Data movement: a workgroup of eight wavefronts owns 256 rows (four panels) x 128 tokens; wavefront (wr, wc) owns
// rows 64 wr.. and tokens 64 wc.. as 4 x 4 MFMA tiles (narrow and half-width variants for launches and tails that wide
// tiles do not fill: see the tile shapes below and launch_gemm). The operands of one group (8 KiB of packed weights, 16 KiB of
// activation digits) go from global memory straight into LDS with global_load_lds_dwordx4 (no registers, no
// ds_write), kStages groups deep, so a fetch has several groups of arithmetic to complete. The prepared weight
// layout and the quantizer's output layout are exactly the LDS layouts: every wavefront-wide transfer is 1 KiB
// contiguous on both sides.
#include "rq_common.h"

#include <string.h>

#include <stdlib.h>

#pragma clang fp contract(off)

namespace rq {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void global_cvoid;

constexpr int kBT = 128;        // tokens per workgroup, wide tiles
constexpr int kBTn = 32;        // tokens per workgroup, narrow tiles
constexpr int kBTh = 64;        // tokens per workgroup, half tiles
constexpr int kThreads = 512;
constexpr int kStages = 6;      // LDS ring depth

// Tile shapes (the kernel's template argument). All are 256 rows; a wavefront owns 64 rows x TT token tiles of 16.
//   kWide  : 128 tokens, wavefront columns = token halves of 64
//   kNarrow:  32 tokens, wavefront columns = alternate groups of K (they meet in LDS at the end)
//   kHalf  :  64 tokens, wavefront columns = token halves of 32: the wide tile's data flow at half its width, for
//             launches whose wide tiles would not fill one round of the chip
constexpr int kWide = 0, kNarrow = 1, kHalf = 2;
constexpr int tiles_of(int mode) { return mode == kWide ? 4 : 2; }          // token tiles of 16 per wavefront
constexpr int loads_of(int mode) { return mode == kHalf ? 2 : 3; }          // LDS-direct loads per thread and step

// One ring stage = 1536 cells of 16 bytes = 24 KiB.
//   wide tile  : [0, 512)    packed weights of one group  [panel 4][half 2][row 64]
//                [512, 1536) activation digits            [digit 2][quarter 4][token 128]
//   narrow tile: [0, 1024)   packed weights of two groups [group 2][panel 4][half 2][row 64]
//                [1024,1536) activation digits            [group 2][digit 2][quarter 4][token 32]
//   half tile  : [0, 512)    packed weights of one group; [512, 1024) activation digits [digit 2][quarter 4][token 64]
struct Stage {
    uint4 cell[1536];
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
    const uint4 *a_src;   // this thread's (first) activation cell of group 0
    size_t a_cell, a_step;
    int wave, wr, wc, l16, quad;   // wc: token half (wide) or K half (narrow)
    int ng;
    int gs;                        // 64-wide groups per activation group (narrow tiles only): 1, 2 or 4
};

// One LDS-direct load: 64 lanes x 16 bytes from the lanes' global addresses to 1 KiB of LDS starting at `lds`
// (wave-uniform; the hardware adds lane * 16). Written as assembly so that the outstanding-load count stays under
// this file's control: the compiler's own bookkeeping would wait for every LDS-direct load before any LDS read.
// The LDS pointer is an operand and memory is clobbered, so the compiler treats the stage as written.
__device__ __forceinline__ void load_to_lds(const uint4 *gptr, uint4 *lds) {
    const uint32_t lds_addr = (uint32_t) (uintptr_t) (lds_void *) lds;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 :  "v"(gptr), "s"(lds_addr)
                 : "memory", "m0");
}

// 64 lanes x 4 bytes to 256 bytes of LDS
__device__ __forceinline__ void load_to_lds_dword(const float *gptr, float *lds) {
    const uint32_t lds_addr = (uint32_t) (uintptr_t) (lds_void *) lds;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
                 :
                 :  "v"(gptr), "s"(lds_addr)
                 : "memory", "m0");
}

// fetch of step `st` into stage s: every wavefront moves three 1 KiB runs. Groups past the end are clamped to the
// last one (refetched into cells nobody reads).
template <int MODE>
__device__ __forceinline__ void fetch(const Ctx &c, Stage &s, int st) {
    uint4 *dst = &s.cell[0] + c.wave * 64;
    if (MODE == kHalf) {
        const int g = st < c.ng ? st : c.ng - 1;
        load_to_lds(c.w_src + (size_t) g * 128, dst);
        load_to_lds(c.a_src + (size_t) g * c.a_step, dst + 512);   // both digits: thread tid moves cell tid of 512
    } else if (MODE == kWide) {
        const int g = st < c.ng ? st : c.ng - 1;
        load_to_lds(c.w_src + (size_t) g * 128, dst);
        load_to_lds(c.a_src + (size_t) g * c.a_step, dst + 512);
        load_to_lds(c.a_src + (size_t) g * c.a_step + c.a_cell, dst + 1024);
    } else {
        const int last = c.ng - 1;
        const int g0 = 2 * st < last ? 2 * st : last, g1 = 2 * st + 1 < last ? 2 * st + 1 : last;
        const int gb = 2 * st + (c.wave >> 2) < last ? 2 * st + (c.wave >> 2) : last;   // this wavefront's digit cells
        load_to_lds(c.w_src + (size_t) g0 * 128, dst);
        load_to_lds(c.w_src + (size_t) g1 * 128, dst + 512);
        load_to_lds(c.a_src + (size_t) gb * c.a_step, dst + 1024);
    }
}

// One step of one wavefront: 64 rows x TT token tiles of 16 against one group (wide: group `st`, token half wc;
// narrow: group 2 st + wc).
template <bool HASK, int MODE>
__device__ __forceinline__ void compute(const Ctx &c, const Stage &s, const uint8_t *__restrict__ k_src, int st,
                                        v4i (&hi)[4][tiles_of(MODE)], int32_t (&lo)[4][tiles_of(MODE)][4]) {
    constexpr bool NARROW = MODE == kNarrow;
    constexpr int TT = tiles_of(MODE);
    const int g = NARROW ? 2 * st + c.wc : st;
    if (NARROW && g >= c.ng) return;   // odd group count: the second K half sits out the last step (wave-uniform)
    // A: quarter `quad` of the group = 8 bytes of the row's cell in half quad >> 1
    const uint4 *a_cells = &s.cell[0] + (NARROW ? c.wc * 512 : 0) + (c.wr * 2 + (c.quad >> 1)) * 64 + c.l16;
    // B: [digit][quarter][token]
    const uint4 *b_cells = NARROW         ? &s.cell[1024] + c.wc * 256 + c.quad * kBTn + c.l16
                           : MODE == kHalf ? &s.cell[512] + c.quad * kBTh + 32 * c.wc + c.l16
                                           : &s.cell[512] + c.quad * kBT + 64 * c.wc + c.l16;
    constexpr int kDigit = NARROW ? 4 * kBTn : MODE == kHalf ? 4 * kBTh : 4 * kBT;   // cells between the lo and the hi plane
    v4i A[4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        const uint2 pk = *(reinterpret_cast<const uint2 *>(a_cells + 16 * rt) + (c.quad & 1));
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
        // Software pipeline over the token tiles: the eight MFMAs of tile ct are issued back to back while the
        // vector ALU folds the four results of tile ct - 1, so neither unit waits for the other.
        v4i S[2][4];
#pragma unroll
        for (int ct = 0; ct < TT + 1; ++ct) {
            if (ct < TT) {
                const v4i Blo = as_v4i(b_cells[16 * ct]);
                const v4i Bhi = as_v4i(b_cells[kDigit + 16 * ct]);
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
            if (ct > 0 && ct < TT) {
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
        for (int ct = 0; ct < TT; ++ct) {
            const v4i Blo = as_v4i(b_cells[16 * ct]);
            const v4i Bhi = as_v4i(b_cells[kDigit + 16 * ct]);
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

// Two groups of a tile at once (the fast path: no weight multipliers), in units of one 16 x 16 tile (x two groups =
// 4 MFMAs); the second group of a unit is issued one unit later, when the first group's result has arrived.
template <int MODE>
__device__ __forceinline__ void compute_pair(const Ctx &c, const Stage &sa, const Stage &sb,
                                             v4i (&hi)[4][tiles_of(MODE)], int32_t (&lo)[4][tiles_of(MODE)][4]) {
    constexpr bool NARROW = MODE == kNarrow;
    constexpr int TT = tiles_of(MODE);
    constexpr int kDigit = NARROW ? 4 * kBTn : MODE == kHalf ? 4 * kBTh : 4 * kBT;   // cells between the lo and the hi plane
    const int a_off = (NARROW ? c.wc * 512 : 0) + (c.wr * 2 + (c.quad >> 1)) * 64 + c.l16;
    const int b_off = NARROW         ? 1024 + c.wc * 256 + c.quad * kBTn + c.l16
                      : MODE == kHalf ? 512 + c.quad * kBTh + 32 * c.wc + c.l16
                                      : 512 + c.quad * kBT + 64 * c.wc + c.l16;
    v4i Aa[4], Ab[4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        const uint2 pa = *(reinterpret_cast<const uint2 *>(&sa.cell[a_off + 16 * rt]) + (c.quad & 1));
        const uint2 pb = *(reinterpret_cast<const uint2 *>(&sb.cell[a_off + 16 * rt]) + (c.quad & 1));
        int e0, o0, e1, o1;
        widen(pa.x, e0, o0);
        widen(pa.y, e1, o1);
        Aa[rt] = v4i{ e0, o0, e1, o1 };
        widen(pb.x, e0, o0);
        widen(pb.y, e1, o1);
        Ab[rt] = v4i{ e0, o0, e1, o1 };
    }
    // lo[rt][ct] is a chained accumulator here: value = 256 h + r, h = the sum of the floors so far, 0 <= r < 256.
    // Clearing r (one AND per value) and feeding the result to the next group's low-digit MFMA as its C operand gives
    // X + 256 h, whose floor by 256 is floor(X / 256) + h: the MFMA adds the floors up, and the vector ALU spends one
    // instruction per value and group instead of a shift and half a three-operand add. The kernel shifts once at the end.
    // (|X| <= 16 x 64 x 8 x 32 = 2^18 per group, so |256 h| < 2^18 x K / 64 <= 2^27 for the longest row: no overflow.)
    auto cleared = [](const v4i &v) { return v4i{ v[0] & ~255, v[1] & ~255, v[2] & ~255, v[3] & ~255 }; };
    v4i T[2];      // after group a, per unit in flight
    v4i B[2][4];   // [buffer][lo a, hi a, lo b, hi b] of one token tile; the next tile's are fetched a unit ahead
    auto load_b = [&](int buf, int ct) {
        B[buf][0] = as_v4i(sa.cell[b_off + 16 * ct]);
        B[buf][1] = as_v4i(sa.cell[b_off + kDigit + 16 * ct]);
        B[buf][2] = as_v4i(sb.cell[b_off + 16 * ct]);
        B[buf][3] = as_v4i(sb.cell[b_off + kDigit + 16 * ct]);
    };
    load_b(0, 0);
#pragma unroll
    for (int un = 0; un < 4 * TT + 1; ++un) {
        const int ct = un >> 2, rt = un & 3;
        if (rt == 0) __builtin_amdgcn_sched_barrier(0);   // keeps the LDS reads of later tiles from piling up early
        if (un > 0) {
            // group b of the previous unit: its group-a result has had a unit's worth of MFMAs to arrive. (Before the
            // next tile's B fragments are fetched: they go into the buffer that unit 4 ct - 1 still reads.)
            const int pct = (un - 1) >> 2, prt = (un - 1) & 3;
            const v4i r = __builtin_amdgcn_mfma_i32_16x16x64_i8(Ab[prt], B[pct & 1][2], cleared(T[(un - 1) & 1]), 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) lo[prt][pct][i] = r[i];
            hi[prt][pct] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Ab[prt], B[pct & 1][3], hi[prt][pct], 0, 0, 0);
        }
        if (un < 4 * TT) {
            if (rt == 0 && ct < TT - 1) load_b((ct + 1) & 1, ct + 1);
            const v4i cur = v4i{ lo[rt][ct][0], lo[rt][ct][1], lo[rt][ct][2], lo[rt][ct][3] };
            T[un & 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aa[rt], B[ct & 1][0], cleared(cur), 0, 0, 0);
            hi[rt][ct] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aa[rt], B[ct & 1][1], hi[rt][ct], 0, 0, 0);
        }
    }
}

// Narrow tiles with activation groups of 128 or 256 (RQ_ACT_GROUP): the quantizer's multiplier and zero point, and
// with them the floor of the fold, cover gs = 2 or 4 consecutive groups of 64. A pair of steps holds groups
// 4i .. 4i+3 (two per stage). gs = 2: wave column wc owns the two groups of stage wc. gs = 4: the four groups are one
// unit; the wave columns take such units alternately. The digit sums of a unit chain through the MFMA accumulator
// and are floored once. A format variant: correct first, no software pipeline.
template <bool HASK>
__device__ __forceinline__ void compute_units(const Ctx &c, const Stage &cur0, const Stage &cur1,
                                              const uint8_t *__restrict__ k_src, int st, v4i (&hi)[4][2],
                                              int32_t (&lo)[4][2][4]) {
    int g0;
    if (c.gs == 2) {
        g0 = 2 * (st + c.wc);
    } else {
        if (((st >> 1) & 1) != c.wc) return;
        g0 = 2 * st;
    }
    if (g0 >= c.ng) return;   // ng is a multiple of gs: a unit is whole or absent (wave-uniform)
    const int a_off = (c.wr * 2 + (c.quad >> 1)) * 64 + c.l16;
    const int b_off = 1024 + c.quad * kBTn + c.l16;
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        int kk[4] = { 1, 1, 1, 1 };
        if (HASK) {
            // the multiplier of the unit's first 64 inputs, as RQ_W_MULT_G(sum, sg << (2 - lsub)) picks it
            // (reference patch line 171)
            const uint32_t k4 = *reinterpret_cast<const uint32_t *>(k_src + (size_t) g0 * kPanelRows + 16 * rt);
#pragma unroll
            for (int i = 0; i < 4; ++i) kk[i] = (k4 >> (8 * i)) & 0xFF;
        }
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) {
            v4i S = v4i{ 0, 0, 0, 0 };
            v4i H = HASK ? v4i{ 0, 0, 0, 0 } : hi[rt][ct];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (j < c.gs) {
                    const Stage &sg = c.gs == 2 ? (c.wc ? cur1 : cur0) : (j < 2 ? cur0 : cur1);
                    const int gi = j & 1;   // group within the stage
                    const uint2 pk = *(reinterpret_cast<const uint2 *>(&sg.cell[gi * 512 + a_off + 16 * rt]) + (c.quad & 1));
                    int e0, o0, e1, o1;
                    widen(pk.x, e0, o0);
                    widen(pk.y, e1, o1);
                    const v4i A = v4i{ e0, o0, e1, o1 };
                    const v4i Blo = as_v4i(sg.cell[b_off + gi * 256 + 16 * ct]);
                    const v4i Bhi = as_v4i(sg.cell[b_off + gi * 256 + 4 * kBTn + 16 * ct]);
                    S = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, Blo, S, 0, 0, 0);
                    H = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, Bhi, H, 0, 0, 0);
                }
            }
            if (!HASK) {
                hi[rt][ct] = H;
#pragma unroll
                for (int i = 0; i < 4; ++i) lo[rt][ct][i] += S[i] >> 8;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) lo[rt][ct][i] += (kk[i] * ((H[i] << 6) + S[i])) >> 8;
            }
        }
    }
}

// One pair of steps: wait for their operands, meet the other wavefronts, refill the two stages that were just
// released, compute. At the wait, the loads this thread has issued after this pair's are those of the next pair.
template <bool HASK, int MODE>
__device__ __forceinline__ void pair_step(const Ctx &c, const Stage &cur0, const Stage &cur1, Stage &refill0,
                                          Stage &refill1, const uint8_t *__restrict__ k_src, int st, int n_steps,
                                          v4i (&hi)[4][tiles_of(MODE)], int32_t (&lo)[4][tiles_of(MODE)][4]) {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * loads_of(MODE)) : "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    fetch<MODE>(c, refill0, st + 4);
    fetch<MODE>(c, refill1, st + 5);
    if constexpr (MODE == kNarrow) {
        if (c.gs > 1) {
            compute_units<HASK>(c, cur0, cur1, k_src, st, hi, lo);
            return;
        }
    }
    if constexpr (!HASK) {
        // K is a multiple of 256, so the number of groups is a multiple of 4: a pair of steps (two groups wide, four
        // narrow) is always whole
        compute_pair<MODE>(c, cur0, cur1, hi, lo);
    } else {
        compute<HASK, MODE>(c, cur0, k_src, st, hi, lo);
        if (st + 1 < n_steps) compute<HASK, MODE>(c, cur1, k_src, st + 1, hi, lo);
    }
}

template <bool HASK, int MODE>
__device__ __forceinline__ void gemm_body(const Ctx &c, Stage &s0, Stage &s1, Stage &s2, Stage &s3, Stage &s4,
                                          Stage &s5, const uint8_t *__restrict__ k_src,
                                          v4i (&hi)[4][tiles_of(MODE)], int32_t (&lo)[4][tiles_of(MODE)][4]) {
    const int n_steps = MODE == kNarrow ? (c.ng + 1) / 2 : c.ng;
    fetch<MODE>(c, s0, 0);
    fetch<MODE>(c, s1, 1);
    fetch<MODE>(c, s2, 2);
    fetch<MODE>(c, s3, 3);
    for (int st = 0; st < n_steps; st += kStages) {
        pair_step<HASK, MODE>(c, s0, s1, s4, s5, k_src, st, n_steps, hi, lo);
        if (st + 2 < n_steps) pair_step<HASK, MODE>(c, s2, s3, s0, s1, k_src, st + 2, n_steps, hi, lo);
        if (st + 4 < n_steps) pair_step<HASK, MODE>(c, s4, s5, s2, s3, k_src, st + 4, n_steps, hi, lo);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // drain the refetches of the last steps before LDS is reused
}

// Wide tiles (256 rows x 128 tokens) are the efficient shape, but a launch of T of them keeps the chip busy for
// ceil(T / 256) rounds. So only whole rounds (or none, or all: see launch_gemm) run wide, and the rest (`first_tile`
// onwards) run as narrow tiles: the same 256 rows x 32 tokens, with the two wavefront columns taking alternate groups of K instead of
// token halves and meeting in LDS at the end. Four times as many workgroups of a quarter of the work each.
template <int MODE>
__global__ void __launch_bounds__(kThreads)
rq_gemm_kernel(const uint4 *__restrict__ codes, const float *__restrict__ s_w, const uint8_t *__restrict__ kmul,
               const int32_t *__restrict__ flags, const uint4 *__restrict__ act8, const float *__restrict__ u,
               float *__restrict__ y, int64_t ldy, int64_t N, int M, int Mp, int ng, int n_panels, int n_tok_tiles,
               int first_tile, int n_tiles, int gs, int live_last) {
    // one array per stage: the compiler tracks LDS-direct loads per destination object
    __shared__ Stage s0;
    __shared__ Stage s1;
    __shared__ Stage s2;
    __shared__ Stage s3;
    __shared__ Stage s4;
    __shared__ Stage s5;
    // the epilogue's operands, fetched with the first groups: the scales of the tile's 256 rows, then the units of its
    // tokens (at the end of the tile, their trip from memory, two microseconds, would stand between the last group
    // and the stores)
    __shared__ __align__(16) float s_pre[256 + kBT];
    constexpr bool NARROW = MODE == kNarrow;
    constexpr int TT = tiles_of(MODE);
    constexpr int kTok = MODE == kHalf ? kBTh : kBT;   // tokens of a wide or half tile

    // Workgroups go to the eight XCDs round robin. Wide: give every XCD a contiguous run of row tiles with the token
    // tiles running fastest, so the workgroups resident on one XCD share weight and activation tiles in its L2.
    int row_tile, t0;
    if (!NARROW) {
        int v = blockIdx.x;
        const int per_xcd = n_tiles / kXcds;
        if (v < per_xcd * kXcds) v = (v % kXcds) * per_xcd + v / kXcds;
        if (gs) {
            // (wide tiles only: gs carries the flag) super-tiles of 8 row tiles x 4 token tiles = the 32 workgroups an
            // XCD runs at a time: together they read 8 weight tiles and 4 activation tiles, the mix that puts the
            // least through that XCD's L2
            const int s = v >> 5, i = v & 31;
            const int spr = n_tok_tiles >> 2;
            const int sr = s / spr;
            row_tile = sr * 8 + (i >> 2);
            t0 = ((s - sr * spr) * 4 + (i & 3)) * kTok;
        } else {
            row_tile = v / n_tok_tiles;
            t0 = (v - row_tile * n_tok_tiles) * kTok;   // (half tiles: n_tok_tiles counts tiles of 64 tokens)
        }
    } else {
        // Narrow workgroups cover whole row tiles from `first_tile / n_tok_tiles` on; only token quarters that hold
        // tokens are enumerated (an empty workgroup would still take a slot of the round-robin dispatch). Each XCD
        // gets a contiguous run, so the quarters of one row tile share its weights in one L2.
        int b = blockIdx.x;
        const int per_xcd = n_tiles / kXcds;          // here: number of narrow workgroups
        if (b < per_xcd * kXcds) b = (b % kXcds) * per_xcd + b / kXcds;
        const int per_row = 4 * (n_tok_tiles - 1) + live_last;
        const int r = b / per_row, slot = b - r * per_row;
        row_tile = first_tile / n_tok_tiles + r;
        t0 = slot * kBTn;                          // quarters are consecutive in token order
    }
    const int panel0 = row_tile * 4;
    const int tid = threadIdx.x;
    Ctx c;
    c.wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    c.wr = c.wave & 3;
    c.wc = c.wave >> 2;
    c.l16 = tid & 15;
    c.quad = (tid & 63) >> 4;
    c.ng = ng;
    c.gs = gs;
    // weights: thread tid moves cell tid of a group's 512 (panel = tid >> 7, half = (tid >> 6) & 1, row = tid & 63);
    // panels past the tensor read panel n_panels - 1 again (their outputs are never stored)
    const int w_panel = min(panel0 + (tid >> 7), n_panels - 1);
    c.w_src = codes + (size_t) w_panel * ng * 128 + (tid & 127);
    c.a_step = (size_t) 8 * Mp;   // cells per group
    c.a_cell = (size_t) 4 * Mp;   // the other digit
    if (MODE == kHalf) {
        // the tile of one group is 512 cells [digit][quarter][token 64]; thread tid moves cell tid (digit and quarter =
        // tid >> 6, which is also their order in the planes)
        c.a_src = act8 + (size_t) (tid >> 6) * Mp + t0 + (tid & 63);
    } else if (!NARROW) {
        // the tile of one group is 1024 cells [digit][quarter][token]; thread tid moves cells tid and tid + 512
        // (digit = cell >> 9, quarter = (cell >> 7) & 3, token = cell & 127)
        c.a_src = act8 + (size_t) (tid >> 7) * Mp + t0 + (tid & 127);
    } else {
        // two groups of 256 cells [digit][quarter][token 32]; thread tid moves cell tid & 255 of group tid >> 8
        // (the group is added per step: it is uniform per wavefront)
        c.a_src = act8 + (size_t) ((tid >> 5) & 7) * Mp + t0 + (tid & 31);
    }
    const uint8_t *k_src = kmul + (size_t) min(panel0 + c.wr, n_panels - 1) * ng * kPanelRows + 4 * c.quad;

    v4i hi[4][TT];
    int32_t lo[4][TT][4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
        for (int ct = 0; ct < TT; ++ct) {
            hi[rt][ct] = v4i{ 0, 0, 0, 0 };
#pragma unroll
            for (int i = 0; i < 4; ++i) lo[rt][ct][i] = 0;
        }
    }

    {
        const int lane = tid & 63;
        if (c.wave < 4) {
            const int64_t n = (int64_t) panel0 * kPanelRows + 64 * c.wave + lane;
            load_to_lds_dword(s_w + (n < N ? n : N - 1), &s_pre[64 * c.wave]);
        } else if (c.wave < 6) {
            const int t = t0 + 64 * (c.wave - 4) + lane;
            load_to_lds_dword(u + (t < M ? t : M - 1), &s_pre[256 + 64 * (c.wave - 4)]);
        }
    }
    if (flags[0] & 1) {
        gemm_body<true, MODE>(c, s0, s1, s2, s3, s4, s5, k_src, hi, lo);
    } else {
        gemm_body<false, MODE>(c, s0, s1, s2, s3, s4, s5, k_src, hi, lo);
    }

    // (the fast path leaves the sum of the floors in the bits above the low byte: see compute_pair)
    const bool chained = !(flags[0] & 1) && !(NARROW && c.gs > 1);
    int32_t tot[4][TT][4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
        for (int ct = 0; ct < TT; ++ct) {
#pragma unroll
            for (int i = 0; i < 4; ++i) tot[rt][ct][i] = (hi[rt][ct][i] >> 2) + (chained ? lo[rt][ct][i] >> 8 : lo[rt][ct][i]);
        }
    }
    if (NARROW) {
        // the odd-group half hands its totals to the even-group half through LDS (the stages are free now):
        // 32 values per lane, 16 KiB per pair of row tiles
        __syncthreads();
        int32_t *xch0 = reinterpret_cast<int32_t *>(&s0.cell[0]) + (c.wr * 64 + (tid & 63));
        int32_t *xch1 = reinterpret_cast<int32_t *>(&s1.cell[0]) + (c.wr * 64 + (tid & 63));
        if (c.wc == 1) {
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
                for (int ct = 0; ct < TT; ++ct) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) (rt < 2 ? xch0 : xch1)[(((rt & 1) * TT + ct) * 4 + i) * 256] = tot[rt][ct][i];
                }
            }
        }
        __syncthreads();
        if (c.wc == 1) return;
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
            for (int ct = 0; ct < TT; ++ct) {
#pragma unroll
                for (int i = 0; i < 4; ++i) tot[rt][ct][i] += (rt < 2 ? xch0 : xch1)[(((rt & 1) * TT + ct) * 4 + i) * 256];
            }
        }
    }

    // epilogue (reference patch line 176): y = ((float(total) * 16) * u) * s_w, total = 4 Xhi + sum of floors
#pragma unroll
    for (int ct = 0; ct < TT; ++ct) {
        const int t = t0 + (NARROW ? 0 : MODE == kHalf ? 32 * c.wc : 64 * c.wc) + 16 * ct + c.l16;
        if (t >= M) continue;
        const float ut = s_pre[256 + (t - t0)];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            const int64_t n = (int64_t) (panel0 + c.wr) * kPanelRows + 16 * rt + 4 * c.quad;
            float *dst = y + (int64_t) t * ldy + n;
            const float4 sw = *reinterpret_cast<const float4 *>(&s_pre[64 * c.wr + 16 * rt + 4 * c.quad]);
            if (n + 3 < N && ((reinterpret_cast<uintptr_t>(dst) & 15) == 0)) {
                float4 o;
                o.x = (((float) tot[rt][ct][0] * 16.0f) * ut) * sw.x;
                o.y = (((float) tot[rt][ct][1] * 16.0f) * ut) * sw.y;
                o.z = (((float) tot[rt][ct][2] * 16.0f) * ut) * sw.z;
                o.w = (((float) tot[rt][ct][3] * 16.0f) * ut) * sw.w;
                // the output is written once and not read back by this launch: non-temporal, so that 4 M N bytes of y
                // do not push weight and activation tiles out of L2
                typedef float v4f __attribute__((ext_vector_type(4)));
                __builtin_nontemporal_store(v4f{ o.x, o.y, o.z, o.w }, reinterpret_cast<v4f *>(dst));
            } else {
                const float swv[4] = { sw.x, sw.y, sw.z, sw.w };
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (n + i < N) dst[i] = (((float) tot[rt][ct][i] * 16.0f) * ut) * swv[i];
                }
            }
        }
    }
}

}  // namespace

constexpr double kHalfRound = 1.5;   // a round of half tiles, in rounds of narrow tiles

hipError_t launch_gemm(const GemmArgs &a, hipStream_t stream) {
    const uint8_t *p = a.prepared;
    const int n_row_tiles = (a.L.n_panels + 3) / 4;
    const int n_tok_tiles = a.Mp / kBT;
    const int n_tiles = n_row_tiles * n_tok_tiles;
    // How many tiles run wide. A round of 256 wide tiles takes about 2.6 times a round of 256 narrow ones (a
    // quarter of the work each, at two thirds of the efficiency); rounds are whole. Candidates: all narrow, whole
    // wide rounds (in whole row tiles) with a narrow tail, all wide.
    const int kCUs = device_compute_units();
    const int live_last = ((a.M + kBTn - 1) / kBTn + 3) % 4 + 1;     // token quarters of the last tile that hold tokens
    const int per_row = 4 * (n_tok_tiles - 1) + live_last;           // narrow workgroups per row tile
    auto cost = [&](int nw) {                                        // nw: a multiple of n_tok_tiles (whole row tiles)
        const int64_t nn = (int64_t) (n_row_tiles - nw / n_tok_tiles) * per_row;
        return 2.6 * ((nw + kCUs - 1) / kCUs) + 1.0 * ((nn + kCUs - 1) / kCUs);
    };
    int n_wide = 0;
    const int whole = n_tiles / kCUs * kCUs / n_tok_tiles * n_tok_tiles;
    if (cost(whole) < cost(n_wide)) n_wide = whole;
    if (cost(n_tiles) < cost(n_wide)) n_wide = n_tiles;
    if (a.groups_per_fold > 1) n_wide = 0;   // wider activation groups: narrow tiles only
    // A third way to run the rows that the whole wide rounds leave over: the skinny kernel (rq_skinny.hip), a
    // workgroup per panel of 64 rows and block of 32 tokens, whole K, no LDS staging. A round of 256 of those takes
    // about 0.65 of a narrow round (measured: 20 us against 31 us at K = 5120) but holds an eighth of a narrow tile
    // each: it wins when the leftover is a few row tiles and the token count moderate (K=5120, N=17408, M=512: 256
    // wide tiles + 16 panels x 16 token blocks, 116.6 -> 102.4 us; at M=1024 the narrow tiles stay ahead).
    bool skinny_tail = false;
    double best = cost(n_wide);
    // (the skinny kernel addresses the digit planes with 32-bit offsets)
    const bool planes_fit = (int64_t) a.L.ng * 128 * a.Mp < ((int64_t) 1 << 32);
    if (a.groups_per_fold == 1 && whole > 0 && whole < n_tiles && planes_fit) {
        const int tail_panels = a.L.n_panels - whole / n_tok_tiles * 4;
        const int64_t wgs = (int64_t) tail_panels * ((a.M + 31) / 32);
        const double c = 2.6 * (whole / kCUs) + 0.65 * ((wgs + kCUs - 1) / kCUs);
        if (c < best) {
            n_wide = whole;
            skinny_tail = true;
            best = c;
        }
    }
    // A fourth way: half tiles (256 rows x 64 tokens) for the whole launch, when that many tiles fill the rounds of
    // the chip better than the mixes above (K = 5120, N = 6144, M = 512: 192 half tiles in one round against 384
    // narrow tiles in two). A round of half tiles takes about 1.5 rounds of narrow ones (46 us against 31 us at K = 5120).
    const int n_half_tok = (a.M + kBTh - 1) / kBTh;
    const int n_half = n_row_tiles * n_half_tok;
    const bool half_tiles = a.groups_per_fold == 1 && kHalfRound * ((n_half + kCUs - 1) / kCUs) < best;
    // the super-tile order of the wide kernel needs a wide region of whole blocks of 8 row tiles x 4 token tiles
    const int super_tiles = n_wide > 0 && n_tok_tiles % 4 == 0 && n_wide % n_tok_tiles == 0 &&
                            (n_wide / n_tok_tiles) % 8 == 0;
    const uint4 *codes = reinterpret_cast<const uint4 *>(p + a.L.off_codes);
    const float *s_w = reinterpret_cast<const float *>(p + a.L.off_sw);
    const int32_t *flags = reinterpret_cast<const int32_t *>(p + a.L.off_flags);
    const uint4 *act8 = reinterpret_cast<const uint4 *>(a.act8);
    if (half_tiles) {
        hipLaunchKernelGGL(rq_gemm_kernel<kHalf>, dim3(n_half), dim3(kThreads), 0, stream, codes, s_w,
                           p + a.L.off_kmul, flags, act8, a.u, a.y, a.ldy, a.L.N, a.M, a.Mp, a.L.ng, a.L.n_panels,
                           n_half_tok, 0, n_half, 0, 4);
        return hipGetLastError();
    }
    if (n_wide > 0) {
        hipLaunchKernelGGL(rq_gemm_kernel<kWide>, dim3(n_wide), dim3(kThreads), 0, stream, codes, s_w,
                           p + a.L.off_kmul, flags, act8, a.u, a.y, a.ldy, a.L.N, a.M, a.Mp, a.L.ng, a.L.n_panels,
                           n_tok_tiles, 0, n_wide, super_tiles, 4);
    }
    if (n_wide < n_tiles && skinny_tail) {
        SkinnyArgs t;
        memset(&t, 0, sizeof t);
        t.w.n = 1;
        t.w.prepared[0] = a.prepared;
        t.w.L[0] = a.L;
        t.w.y[0] = a.y;
        t.w.ldy[0] = a.ldy;
        t.act8 = a.act8;
        t.u = a.u;
        t.M = a.M;
        t.Mp = a.Mp;
        t.tot = nullptr;   // whole K per workgroup
        t.panel0 = n_wide / n_tok_tiles * 4;
        t.panels = a.L.n_panels - t.panel0;
        return launch_skinny(t, stream);
    }
    if (n_wide < n_tiles) {
        const int n_blocks = (n_row_tiles - n_wide / n_tok_tiles) * per_row;
        hipLaunchKernelGGL(rq_gemm_kernel<kNarrow>, dim3(n_blocks), dim3(kThreads), 0, stream, codes, s_w,
                           p + a.L.off_kmul, flags, act8, a.u, a.y, a.ldy, a.L.N, a.M, a.Mp, a.L.ng, a.L.n_panels,
                           n_tok_tiles, n_wide, n_blocks, a.groups_per_fold, live_last);
    }
    return hipGetLastError();
}

}  // namespace rq
