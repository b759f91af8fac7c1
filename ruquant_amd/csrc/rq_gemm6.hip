// int4 x int4 GEMM for wide token batches on the gfx950 matrix cores, through v_mfma_f32_32x32x64_f8f6f4 with fp6
// (E2M3) operands: the MFMA form that runs at twice the rate of the int8 one and whose K = 64 is exactly one
// activation group.
//
// Why fp6 is exact here. An E2M3 value with sign s and the five exponent / mantissa bits read as the integer n
// (0 .. 31) is n / 8 for n <= 15 (subnormals 0 .. 7 / 8, then 1 .. 1.875 in steps of 1 / 8): the sign-magnitude code
// of an integer |v| <= 15 IS the fp6 encoding of v / 8. Weight codes w (-8 .. 7) and activation values q - z
// (-15 .. 15) both fit, every product w (q - z) / 64 is a multiple of 1 / 64 below 2, and a group's sum
// S / 64 (|S| <= 7680) is exact in the fp32 accumulator. One MFMA per 32 x 32 outputs and group yields
// S_g = sum_k w_k (q_k - z_g), which equals the reference's acc + (8 - z) colsum (ggml_vec_dot_w4a4_a4, reference
// patch lines 160-172).
//
// The per-group floor. The reference adds floor(m_g S_g / 16) per group (reference patch lines 35-39, 173). With the
// wavefront's fp32 rounding mode set toward minus infinity, acc = fma(S / 64, 4 m, acc) on an accumulator that
// holds an integer in [2^23, 2^24) (where one unit in the last place is 1) is acc + floor(m S / 16): the FMA forms
// m S / 16 + acc exactly and rounds once, downwards, to an integer. One full-rate vector instruction per output and
// group. The accumulator starts at 1.5 x 2^23; a group moves it by at most 255 x 7680 / 16 = 122,400, so after 32
// groups (3,916,800 < 2^22) its offset from the start is moved into an int32 total (two integer instructions per
// value: the float's bit pattern minus the bit pattern of 1.5 x 2^23 is that offset) and it starts again.
//
// Tensors with integer weight multipliers k (uniform branch on the prepared flag) fold
// floor(k m S / 16) in integers instead. Activation groups of 128 / 256 (RQ_ACT_GROUP) chain the 2 or 4 MFMAs of a
// group through the accumulator operand before the one fold.
//
// Data movement: a workgroup of eight wavefronts owns 256 rows x 128 tokens; wavefront (wr, wc) owns rows 64 wr .. and
// tokens 64 wc .. as 2 x 2 MFMA tiles of 32 x 32. Operands go from global memory straight into LDS
// (global_load_lds_dwordx4), two groups per ring stage, four stages. Both the fp6 weight plane that
// rq_w4a4_prepare writes and the activation plane of the quantizer are stored as MFMA fragments (32 rows or tokens x
// 64 inputs = 1536 bytes: a 16-byte and an 8-byte piece per lane, each piece contiguous across the lanes), so a
// stage is filled by whole 1 KiB runs and read back without bank conflicts.
#include "rq_common.h"

#include <string.h>

#pragma clang fp contract(off)

// Timing-only builds (-DRQ6_VARIANT=n, results are wrong): the loop with one ingredient left out, to see what each
// costs. 1: no fetches; 2: no MFMAs or folds (groups of 128 / 256 only); 3: operands made up in registers instead of
// read from LDS; 4: no barrier; 5: MFMAs and folds alone (1 + 3 + 4).
#ifndef RQ6_VARIANT
#define RQ6_VARIANT 0
#endif

namespace rq {

namespace {

constexpr bool kWithFetch = RQ6_VARIANT != 1 && RQ6_VARIANT != 5;
constexpr bool kWithCompute = RQ6_VARIANT != 2;
constexpr bool kWithLdsReads = RQ6_VARIANT != 3 && RQ6_VARIANT != 5;
constexpr bool kWithBarrier = RQ6_VARIANT != 4 && RQ6_VARIANT != 5;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void lds_void;

constexpr int kThreads = 512;
constexpr int kTileRows = 256;                 // rows of a workgroup's tile
constexpr int kTileTok = 128;                  // tokens of a workgroup's tile
constexpr int kCellsA = 8 * kFrag6 / 16;       // 768 cells: eight weight fragments of one group
constexpr int kCellsB = 4 * kFrag6 / 16;       // 384 cells: four activation fragments of one group
constexpr int kCellsM = kTileTok * 4 / 16;     // 32 cells: the 128 tokens' multipliers of one group (4 m as float)
// One ring stage = two groups: [A g0][A g1][B g0][B g1][m g0][m g1][k g0][k g1] = 2400 cells of 16 bytes = 37.5 KiB
constexpr int kCellsK = kTileRows / 16;         // 16 cells: the 256 rows' weight multipliers of one group (a byte each)
constexpr int kOffA = 0, kOffB = 2 * kCellsA, kOffM = kOffB + 2 * kCellsB, kOffK = kOffM + 2 * kCellsM;
constexpr int kStageCellsPlain = kOffK;                 // without the rows' weight multipliers
constexpr int kStageCellsK = kOffK + 2 * kCellsK;       // with them
constexpr int kRing = 4;
static_assert(kStageCellsPlain == 2368 && kStageCellsK == 2400, "stage size");
// Each wavefront moves four whole 1 KiB runs per step (cells 0 .. 2047: the weights and the first 512 activation
// cells) and 44 lanes' worth of a fifth (cells 2048 .. 2399: the rest of the activations, the tokens' multipliers and the
// rows' weight multipliers).
constexpr int kTailCell = 2048;
static_assert(kTailCell + 8 * 40 == kStageCellsPlain && kTailCell + 8 * 44 == kStageCellsK, "tail split");
constexpr int kLoadsPerStep = 5;

constexpr int kXposeStride = 36;               // floats between tokens of a wavefront's output block in LDS (32 rows + 4)
constexpr float kBias = 12582912.0f;           // 1.5 x 2^23
constexpr int kBiasBits = 0x4B400000;
constexpr int kFlushSteps = 16;                // 32 groups
constexpr int kRsrcWord3 = 0x00020000;         // last word of a raw buffer descriptor on this target (32-bit data format)
constexpr int kDeviceScope = 16;               // cache policy of a buffer access: the sc1 bit

// WITHK: the stage of the kernel form that folds with weight multipliers from LDS. (Two layouts, because the 512
// bytes shift the stages' LDS offsets, and with them the plain kernel's loop needs base registers it does not have.)
template <bool WITHK>
struct StageT {
    static constexpr int kCells = WITHK ? kStageCellsK : kStageCellsPlain;
    static constexpr int kTailLanes = WITHK ? 44 : 40;   // lanes of a wavefront's fifth load
    uint4 cell[kCells];
};

// 64 lanes x 16 bytes from base + lane offset to 1 KiB of LDS at `lds` (wave-uniform; the hardware adds lane * 16).
// Assembly, so that the count of outstanding loads stays under this file's control (the s_waitcnt of step()).
// a wave-uniform address, said so explicitly: the compiler then keeps it in scalar registers
__device__ __forceinline__ const uint8_t *uniform(const uint8_t *p) {
    const uint64_t b = (uint64_t) (uintptr_t) p;
    return reinterpret_cast<const uint8_t *>(
        (uintptr_t) ((uint64_t) (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) b) |
                     (uint64_t) (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (b >> 32)) << 32));
}

__device__ __forceinline__ void load_run(const uint8_t *base, uint32_t lane_off, uint4 *lds) {
    const uint32_t lds_addr = (uint32_t) (uintptr_t) (lds_void *) lds;
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(lane_off), "s"(base), "s"(lds_addr)
                 : "memory", "m0");
}

// the same from per-lane addresses, for the lanes of `mask` only (the others move nothing). The execution mask is
// switched inside the statement: a branch around the load would cut the step into several basic blocks, and the
// compiler then sinks the folds of one step behind the barrier of the next (their inputs, 128 registers, spill).
__device__ __forceinline__ void load_cells(const uint8_t *gptr, uint4 *lds, uint64_t mask) {
    const uint32_t lds_addr = (uint32_t) (uintptr_t) (lds_void *) lds;
    uint64_t saved;
    asm volatile("s_mov_b32 m0, %2\n\ts_mov_b64 %0, exec\n\ts_mov_b64 exec, %3\n\t"
                 "global_load_lds_dwordx4 %1, off\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "v"(gptr), "s"(lds_addr), "s"(mask)
                 : "memory", "m0");
}

__device__ __forceinline__ void load_to_lds_dword(const float *gptr, float *lds) {
    const uint32_t lds_addr = (uint32_t) (uintptr_t) (lds_void *) lds;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
                 :
                 : "v"(gptr), "s"(lds_addr)
                 : "memory", "m0");
}

struct Ctx {
    // the four whole runs this wavefront moves per step: address of step 0 and advance per step (wave-uniform)
    const uint8_t *run_src[4];
    size_t run_step[4];
    const uint8_t *tail_src; // this lane's cell of the fifth load, current step
    uint32_t tail_step;      // its advance per step (bytes: under 4 GiB for any batch the workspace can hold)
    const uint8_t *k_src;    // weight multipliers of this wavefront's panel, row offset of the lane's first quad
    int wave, wr, wc, lane;
    int n_steps;             // steps (two groups each) of this workgroup
    int g0;                  // its first group
};

// fetch of step `st` (two groups) into stage s, then advance the sources; past the last step they stay where they
// are (the last step is fetched again, into cells nobody reads), so every step issues the same number of loads.
// In pieces, so that the loop can deal them out between its MFMAs: five loads issued back to back by all eight
// wavefronts right behind the barrier queue up in front of the memory pipeline, and a wavefront that waits to issue a
// load issues no MFMA either.
template <class Stage>
__device__ __forceinline__ void fetch_run(Ctx &c, Stage &s, int st, int i) {
    load_run(c.run_src[i], (uint32_t) c.lane * 16, &s.cell[(i * 8 + c.wave) * 64]);
    c.run_src[i] = uniform(c.run_src[i] + (st + 1 < c.n_steps ? c.run_step[i] : 0));
}
template <class Stage>
__device__ __forceinline__ void fetch_tail(Ctx &c, Stage &s, int st) {
    load_cells(c.tail_src, &s.cell[kTailCell + c.wave * Stage::kTailLanes], ((uint64_t) 1 << Stage::kTailLanes) - 1);
    c.tail_src += st + 1 < c.n_steps ? c.tail_step : 0;
}
template <class Stage>
__device__ __forceinline__ void fetch(Ctx &c, Stage &s, int st) {
#pragma unroll
    for (int i = 0; i < 4; ++i) fetch_run(c, s, st, i);
    fetch_tail(c, s, st);
}

template <class Stage>
__device__ __forceinline__ v8i fragment(const Stage &s, int cell0, int lane) {
    const uint4 p0 = s.cell[cell0 + lane];
    const uint2 p1 = *(reinterpret_cast<const uint2 *>(&s.cell[cell0 + 64]) + lane);
    v8i v;
    v[0] = (int) p0.x; v[1] = (int) p0.y; v[2] = (int) p0.z; v[3] = (int) p0.w;
    v[4] = (int) p1.x; v[5] = (int) p1.y;
    // (the fp6 form reads six registers: elements 6 and 7 are left undefined)
    return v;
}

// fast path: acc += floor(m S / 16) for the 16 outputs of one tile (round toward minus infinity is set)
__device__ __forceinline__ void fold_fast(const v16f &S, float m4, float (&acc)[16]) {
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = __builtin_fmaf(S[r], m4, acc[r]);
}

// weight multipliers (reference patch lines 169-173): acc += floor(k m S / 16), the same single FMA with 4 m k in
// place of 4 m (k <= 15, so a group moves the accumulator by at most 15 x 122,400: flush after every second group).
// kw: the multipliers of the lane's sixteen rows, four bytes per register.
__device__ __forceinline__ void fold_km(const v16f &S, float m4, const uint32_t (&kw)[4], float (&acc)[16]) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const float kf = (float) ((kw[r >> 2] >> (8 * (r & 3))) & 0xFFu);
        acc[r] = __builtin_fmaf(S[r], kf * m4, acc[r]);
    }
}
// the sixteen multipliers a lane needs for row block a (rows 32 a + 8 q + 4 (lane / 32) + 0 .. 3, q = 0 .. 3) of group gi
template <class Stage>
__device__ __forceinline__ void read_kw(const Ctx &c, const Stage &s, int gi, int a, uint32_t (&kw)[4]) {
    // (the lane's part of the address is worked out here each time: kept across the loop, the eight addresses that the
    // compiler forms from it, one per stage and group, are registers the loop does not have, and their reloads from
    // scratch wait for every load in flight)
    uint32_t h = (uint32_t) c.lane >> 5;
    asm volatile("" : "+v"(h));
    const uint32_t *k = reinterpret_cast<const uint32_t *>(&s.cell[kOffK + gi * kCellsK]) + 16 * c.wr + 8 * a + h;
#pragma unroll
    for (int q = 0; q < 4; ++q) kw[q] = k[2 * q];
}

// the same in integers, from multipliers in global memory (the forms for activation groups of 128 / 256)
__device__ __forceinline__ void fold_k(const v16f &S, float m4, const int (&kk)[16], int32_t (&tot)[16]) {
    const int mi = (int) (m4 * 0.25f);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int Si = (int) (S[r] * 64.0f);
        tot[r] += (kk[r] * mi * Si) >> kTermShift;
    }
}

// One step (two groups of 64 inputs) of one wavefront: 64 rows x 64 tokens as 2 x 2 tiles. GS = runs of 64 per
// activation group (1, 2, 4). A unit = one tile x one activation group's runs inside this step: its MFMAs chain through
// the accumulator operand; the fold of unit i runs behind the MFMAs of unit i + 1.
template <bool HASK, int GS, class Stage>
__device__ __forceinline__ void compute(const Ctx &c, const Stage &s, int st, float (&acc)[2][2][16],
                                        int32_t (&tot)[2][2][16], v16f (&carry)[2][2]) {
    constexpr int kRuns = GS == 1 ? 1 : 2;        // runs of a unit inside one step
    constexpr int kUnits = GS == 1 ? 8 : 4;
    v8i A[2][2], B[2][2];
    float m4[2][2];
#pragma unroll
    for (int gi = 0; gi < 2; ++gi) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#if RQ6_VARIANT == 3 || RQ6_VARIANT == 5
            for (int e = 0; e < 6; ++e) { A[gi][i][e] = c.lane * (e + gi + 1) + st; B[gi][i][e] = c.lane * (e + i + 3) + st; }
            m4[gi][i] = 4.0f;
            asm volatile("" : "+v"(A[gi][i]), "+v"(B[gi][i]));
            continue;
#endif
            A[gi][i] = fragment(s, kOffA + gi * kCellsA + (2 * c.wr + i) * (kFrag6 / 16), c.lane);
            B[gi][i] = fragment(s, kOffB + gi * kCellsB + (2 * c.wc + i) * (kFrag6 / 16), c.lane);
            m4[gi][i] = reinterpret_cast<const float *>(&s.cell[kOffM + gi * kCellsM])[64 * c.wc + 32 * i + (c.lane & 31)];
        }
    }
    // with groups of 256 a unit spans two steps: the even step leaves its half in `carry`, the odd step folds
    const bool folds = GS < 4 || (st & 1);
    const bool starts = GS < 4 || !(st & 1);
    const v16f zero = {};
    v16f S[2];
    int prev_a = 0, prev_b = 0, prev_gi = 0;
#pragma unroll
    for (int un = 0; un < kUnits + 1; ++un) {
        if (un < kUnits) {
            const int gi = GS == 1 ? un >> 2 : 0, a = (un >> 1) & 1, b = un & 1;
            v16f C = GS == 4 && !starts ? carry[a][b] : zero;
#pragma unroll
            for (int run = 0; run < kRuns; ++run) {
                C = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(A[gi + run][a], B[gi + run][b], C, 2, 2, 0, 0, 0, 0);
            }
            if (GS == 4 && !folds) carry[a][b] = C;
            S[un & 1] = C;
        }
        if (un > 0 && folds) {
            const v16f &P = S[(un - 1) & 1];
            if (!HASK) {
                fold_fast(P, m4[prev_gi][prev_b], acc[prev_a][prev_b]);
            } else {
                // the multiplier of the group's first run (reference patch line 171: RQ_W_MULT_G(sum, sg << (2 - lsub)))
                const int g = c.g0 + (GS == 4 ? 2 * (st & ~1) : 2 * st) + prev_gi;
                int k16[16];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t k4 = *reinterpret_cast<const uint32_t *>(c.k_src + (size_t) g * kPanelRows + 32 * prev_a + 8 * q);
#pragma unroll
                    for (int i = 0; i < 4; ++i) k16[4 * q + i] = (k4 >> (8 * i)) & 0xFF;
                }
                fold_k(P, m4[prev_gi][prev_b], k16, tot[prev_a][prev_b]);
            }
        }
        if (un < kUnits) {
            prev_gi = GS == 1 ? un >> 2 : 0;
            prev_a = (un >> 1) & 1;
            prev_b = un & 1;
        }
        // A unit's MFMAs and the previous unit's fold stay together, MFMAs first: the fold then runs while the matrix
        // pipe works on the next unit. (Left alone, the scheduler issues all the independent MFMAs of a step first and
        // their results, 16 registers each, spill; with a plain barrier it puts the fold in front of the MFMA, so that
        // every fold waits for the MFMA issued right before it.)
        if (un < kUnits) __builtin_amdgcn_sched_group_barrier(0x008, kRuns, 0);   // MFMA
        if (un > 0 && folds && !HASK) __builtin_amdgcn_sched_group_barrier(0x002, 16, 0);   // VALU
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <bool HASK, int GS, class Stage>
__device__ __forceinline__ void step(Ctx &c, const Stage &cur, Stage &refill, int st, float (&acc)[2][2][16],
                                     int32_t (&tot)[2][2][16], v16f (&carry)[2][2]) {
    // the loads of steps st + 1 and st + 2 may still be in flight
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kLoadsPerStep) : "memory");
    if (kWithBarrier) __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (kWithFetch) fetch(c, refill, st + 3);
    if (kWithCompute) compute<HASK, GS>(c, cur, st, acc, tot, carry);
}

__device__ __forceinline__ void flush(float (&acc)[2][2][16], int32_t (&tot)[2][2][16]) {
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                tot[a][b][r] += __builtin_bit_cast(int, acc[a][b][r]) - kBiasBits;
                acc[a][b][r] = kBias;
            }
        }
    }
}

template <bool HASK, int GS, class Stage>
__device__ __forceinline__ void body(Ctx &c, Stage &s0, Stage &s1, Stage &s2, Stage &s3,
                                     float (&acc)[2][2][16], int32_t (&tot)[2][2][16]) {
    v16f carry[2][2] = {};
    fetch(c, s0, 0);
    fetch(c, s1, 1);
    fetch(c, s2, 2);
    for (int st = 0; st < c.n_steps; st += kRing) {
        // (K is a multiple of 256: the number of steps is even, so steps come in pairs)
        step<HASK, GS>(c, s0, s3, st, acc, tot, carry);
        step<HASK, GS>(c, s1, s0, st + 1, acc, tot, carry);
        if (st + 2 < c.n_steps) {
            step<HASK, GS>(c, s2, s1, st + 2, acc, tot, carry);
            step<HASK, GS>(c, s3, s2, st + 3, acc, tot, carry);
        }
        if (!HASK && ((st / kRing + 1) % (kFlushSteps / kRing)) == 0) flush(acc, tot);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the refetches of the last steps
}

// ---- groups of 64 (the common case): the same steps with the LDS reads taken out of the critical path.
// The operands of a group are read from LDS while the previous group is being computed: the reads of a step's second
// group are issued in front of the first group's MFMAs, and the wait for the next stage (vmcnt + barrier) sits between
// the two groups, so that the next step's first group can be read behind the second group's MFMAs. (With all reads at
// the top of a step every wavefront waited for 12 KiB from LDS at the same moment, right behind the barrier: a
// quarter of the step.)
struct Operands {
    v8i A[2], B[2];
    float m4[2];
};

template <class Stage>
__device__ __forceinline__ void read_operands(const Ctx &c, const Stage &s, int gi, Operands &o) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        o.A[i] = fragment(s, kOffA + gi * kCellsA + (2 * c.wr + i) * (kFrag6 / 16), c.lane);
        o.B[i] = fragment(s, kOffB + gi * kCellsB + (2 * c.wc + i) * (kFrag6 / 16), c.lane);
        o.m4[i] = reinterpret_cast<const float *>(&s.cell[kOffM + gi * kCellsM])[64 * c.wc + 32 * i + (c.lane & 31)];
    }
}

// the four tiles of one group; the fold of a tile runs behind the MFMA of the next one, the last tile's result is
// handed to the next group (P, pm, and the tile it belongs to is always (1, 1))
// (with weight multipliers: `sk`, `gi` = the stage and the group in it that `o` was read from, `sp`, `gp` = those of
// the group before it, whose last tile is folded behind this group's first MFMA; the multipliers of a fold's rows are
// read from LDS in front of the MFMA that the fold stands behind)
// KFMA: the one-FMA fold with multipliers from LDS; otherwise (a kernel that is launched when nothing says the tensor
// has weight multipliers, and must still be right when it has) the integer fold with multipliers from global memory.
template <bool HASK, bool KFMA, class Stage, class Between>
__device__ __forceinline__ void group_units(const Ctx &c, const Operands &o, int g, const Stage &sp, int gp, const Stage &sk, int gi,
                                            v16f &P, float &pm, float (&acc)[2][2][16], int32_t (&tot)[2][2][16], Between between) {
    const v16f zero = {};
#pragma unroll
    for (int un = 0; un < 4; ++un) {
        const int a = un >> 1, b = un & 1;
        const int pa = un == 0 ? 1 : (un - 1) >> 1, pb = un == 0 ? 1 : (un - 1) & 1;
        uint32_t kw[4];
        if (HASK && KFMA) read_kw(c, un == 0 ? sp : sk, un == 0 ? gp : gi, pa, kw);
        // The wavefront asks for issue priority while it hands over its MFMA. The two statements also pin the order
        // MFMA, load, fold: without them the compiler moves the load (an assembly statement) in front of the MFMA,
        // which then waits behind the load's issue (M=2048: 185.5 -> 180 us; with the priority left at 0 in both
        // statements, 181 us).
        __builtin_amdgcn_s_setprio(1);
        const v16f S = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(o.A[a], o.B[b], zero, 2, 2, 0, 0, 0, 0);
        __builtin_amdgcn_s_setprio(0);
        between(un);   // (a piece of the next stages' fetch: behind the MFMA, in front of the previous tile's fold)
        if (!HASK) {
            fold_fast(P, pm, acc[pa][pb]);
        } else if (KFMA) {
            fold_km(P, pm, kw, acc[pa][pb]);   // (a workgroup's first fold adds nothing: P and pm start as zero)
        } else {
            const int pg = un == 0 ? g - 1 : g;
            int k16[16];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t k4 = *reinterpret_cast<const uint32_t *>(c.k_src + (size_t) (pg < 0 ? 0 : pg) * kPanelRows + 32 * pa + 8 * q);
#pragma unroll
                for (int i = 0; i < 4; ++i) k16[4 * q + i] = (k4 >> (8 * i)) & 0xFF;
            }
            fold_k(P, pm, k16, tot[pa][pb]);
        }
        P = S;
        pm = o.m4[b];
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                // MFMA
        if (!HASK) __builtin_amdgcn_sched_group_barrier(0x002, 16, 0);    // VALU: the fold
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <bool HASK, bool KFMA, class Stage>
__device__ __forceinline__ void body64(Ctx &c, Stage &s0, Stage &s1, Stage &s2, Stage &s3, float (&acc)[2][2][16],
                                       int32_t (&tot)[2][2][16]) {
    Stage *ring[kRing] = { &s0, &s1, &s2, &s3 };
    Operands X, Y;
    if (!kWithLdsReads) {
        for (int i = 0; i < 2; ++i) for (int e = 0; e < 6; ++e) { X.A[i][e] = c.lane * (e + 1); X.B[i][e] = c.lane * (e + i + 3); Y.A[i][e] = c.lane * (e + 7); Y.B[i][e] = c.lane * (e + i + 2); }
        X.m4[0] = X.m4[1] = Y.m4[0] = Y.m4[1] = 4.0f;
    }
    v16f P = {};
    float pm = 0.0f;
    // stages 0 and 1 whole, of stage 2 the first three runs: its other two loads and everything after them is dealt
    // out between the MFMAs of the loop (three runs of step st + 3 behind the barrier of step st, the fourth run and the
    // fifth load in the first half of step st + 1)
    fetch(c, s0, 0);
    fetch(c, s1, 1);
#pragma unroll
    for (int i = 0; i < 3; ++i) fetch_run(c, s2, 2, i);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kLoadsPerStep - 2) : "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_operands(c, s0, 0, X);
    for (int st0 = 0; st0 < c.n_steps; st0 += kRing) {
#pragma unroll
        for (int j = 0; j < kRing; ++j) {
            const int st = st0 + j;
            if (j > 0 && st >= c.n_steps) break;   // (wave-uniform)
            const Stage &cur = *ring[j];
            const Stage &next = *ring[(j + 1) % kRing];
            Stage &refill2 = *ring[(j + 2) % kRing];
            Stage &refill3 = *ring[(j + 3) % kRing];
            if (kWithLdsReads) read_operands(c, cur, 1, Y);
            __builtin_amdgcn_sched_barrier(0);
            group_units<HASK, KFMA>(c, X, c.g0 + 2 * st, *ring[(j + 3) % kRing], 1, cur, 0, P, pm, acc, tot, [&](int un) {
                if (!kWithFetch) return;
                if (un == 0) fetch_run(c, refill2, st + 2, 3);
                if (un == 2) fetch_tail(c, refill2, st + 2);
            });
            // stage st + 1 is whole once every wavefront has seen its own loads of it arrive (those of step st + 2
            // may still be in flight); stage st - 1 is then free for step st + 3
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoadsPerStep) : "memory");
            if (kWithBarrier) __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (kWithLdsReads) read_operands(c, next, 0, X);   // (past the last step: stale cells, never used)
            __builtin_amdgcn_sched_barrier(0);
            group_units<HASK, KFMA>(c, Y, c.g0 + 2 * st + 1, cur, 0, cur, 1, P, pm, acc, tot, [&](int un) {
                if (!kWithFetch) return;
                if (un < 3) fetch_run(c, refill3, st + 3, un);
            });
            if (HASK && KFMA) flush(acc, tot);   // (every accumulator has taken two groups' terms since the last one)
        }
        if (!HASK && ((st0 / kRing + 1) % (kFlushSteps / kRing)) == 0) flush(acc, tot);
    }
    // the last tile of the last group
    if (!HASK) {
        fold_fast(P, pm, acc[1][1]);
    } else if (KFMA) {
        uint32_t kw[4];
        read_kw(c, *ring[(c.n_steps - 1) % kRing], 1, 1, kw);
        fold_km(P, pm, kw, acc[1][1]);
    } else {
        int k16[16];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t k4 = *reinterpret_cast<const uint32_t *>(c.k_src + (size_t) (c.g0 + 2 * c.n_steps - 1) * kPanelRows + 32 + 8 * q);
#pragma unroll
            for (int i = 0; i < 4; ++i) k16[4 * q + i] = (k4 >> (8 * i)) & 0xFF;
        }
        fold_k(P, pm, k16, tot[1][1]);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the refetches of the last steps
}

// KFMA (activation groups of 64 only): the form of the kernel for tensors with weight multipliers; see group_units
template <int GS, bool KFMA>
__global__ void __launch_bounds__(kThreads)
rq_gemm6_kernel(const float *__restrict__ s_w, const uint8_t *__restrict__ kmul,
                const int32_t *__restrict__ flags, const uint8_t *__restrict__ act6, const float *__restrict__ m4,
                const float *__restrict__ u, float *__restrict__ y, int64_t ldy, int64_t N, int M, int Mp, int ng,
                int n_panels, int n_tok_tiles, int n_tiles, int super_tiles, int n_whole, int parts,
                int *__restrict__ counters, unsigned long long *__restrict__ slabs) {
    using Stage = StageT<KFMA>;
    __shared__ Stage ring[kRing];
    Stage &s0 = ring[0], &s1 = ring[1], &s2 = ring[2], &s3 = ring[3];
    static_assert(8 * 32 * kXposeStride * 4 <= sizeof(Stage), "the epilogue's output blocks fit one stage");
    // the epilogue's operands, fetched ahead of the first groups: the scales of the tile's 256 rows, then the units of
    // its 128 tokens
    __shared__ __align__(16) float s_pre[kTileRows + kTileTok + 4];   // (+ a word for the arrival count of a slice)

    // Workgroups go to the eight XCDs round robin: every XCD gets a contiguous run of tiles, visited in super-tiles of
    // 8 row tiles x 4 token tiles (the 32 workgroups an XCD runs at a time then share 8 weight tiles and 4 activation
    // tiles in its L2), or with the token tiles running fastest where the launch is not made of whole super-tiles.
    // The first n_whole workgroups take a whole tile each. The tiles after them (fewer than would fill the chip once)
    // are cut along K into `parts` slices each, one workgroup per slice, which meet through memory (see the epilogue).
    int row_tile, t0, part = 0, slot = 0;
    {
        int v = blockIdx.x;
        if (v < n_whole) {
            const int per_xcd = n_whole / kXcds;
            if (v < per_xcd * kXcds) v = (v % kXcds) * per_xcd + v / kXcds;
        } else {
            // slices: an XCD gets a contiguous run of (tile, part) pairs, parts running slowest within the run, so that
            // neighbouring tiles' slices of the same stretch of K are resident together
            int j = v - n_whole;
            const int n_sl = (n_tiles - n_whole) * parts, per_xcd = n_sl / kXcds;
            if (j < per_xcd * kXcds) j = (j % kXcds) * per_xcd + j / kXcds;
            v = n_whole + j / parts;
            part = j - (j / parts) * parts;
        }
        if (super_tiles) {
            const int s = v >> 5, i = v & 31;
            const int spr = n_tok_tiles >> 2;
            const int sr = s / spr;
            row_tile = sr * 8 + (i >> 2);
            t0 = ((s - sr * spr) * 4 + (i & 3)) * kTileTok;
        } else {
            row_tile = v / n_tok_tiles;
            t0 = (v - row_tile * n_tok_tiles) * kTileTok;
        }
        slot = v - n_whole;
    }
    const bool sliced = (int) blockIdx.x >= n_whole;
    // this workgroup's steps (two groups each) of the tile's ng / 2
    const int s_begin = sliced ? (int) ((int64_t) (ng / 2) * part / parts) : 0;
    const int s_end = sliced ? (int) ((int64_t) (ng / 2) * (part + 1) / parts) : ng / 2;
    const int tid = threadIdx.x;
    // the fp6 plane's address stands beside the flag word (it is inside the prepared buffer, or, for a weight that was
    // prepared in place, a buffer of its own)
    const uint8_t *w6 = reinterpret_cast<const uint8_t *>((uintptr_t) *reinterpret_cast<const unsigned long long *>(flags + 2));
    Ctx c;
    c.wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    c.wr = c.wave & 3;
    c.wc = c.wave >> 2;
    c.lane = tid & 63;
    c.n_steps = s_end - s_begin;
    c.g0 = 2 * s_begin;
    const uint8_t *w_tile = w6 + (size_t) row_tile * ng * (kCellsA * 16);   // this tile's rows, group 0
    const size_t a_step = (size_t) (Mp / 32) * kFrag6;                       // bytes between groups of the activation plane
    const uint8_t *a_tile = act6 + (size_t) (t0 / 32) * kFrag6;              // this tile's tokens, group 0
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        // run L of the stage: runs 0 .. 23 are the weights of the step's two groups (12 each), 24 .. 35 the activations
        // (6 each; the last four belong to the fifth load)
        const int L = i * 8 + c.wave;
        if (L < 24) {
            c.run_step[i] = (size_t) 2 * kCellsA * 16;
            c.run_src[i] = uniform(w_tile + (size_t) (L / 12) * (kCellsA * 16) + (size_t) (L % 12) * 1024 + s_begin * c.run_step[i]);
        } else {
            c.run_step[i] = 2 * a_step;
            c.run_src[i] = uniform(a_tile + (size_t) ((L - 24) / 6) * a_step + (size_t) ((L - 24) % 6) * 1024 + s_begin * c.run_step[i]);
        }
    }
    {
        // fifth load: cells 2048 .. 2303 are the last 256 cells of the second group's activations, cells 2304 .. 2367
        // the tokens' multipliers of the two groups, cells 2368 .. 2399 the weight multipliers of the tile's 256 rows
        // for the two groups (a byte per row: 64 bytes per panel of 64 rows)
        const int cell = kTailCell + c.wave * Stage::kTailLanes + (c.lane < Stage::kTailLanes ? c.lane : 0);
        if (cell < kOffM) {
            c.tail_step = (uint32_t) (2 * a_step);
            c.tail_src = a_tile + a_step + (size_t) (cell - (kOffB + kCellsB)) * 16 + (size_t) s_begin * c.tail_step;
        } else if (cell < kOffK) {
            const int gi = (cell - kOffM) / kCellsM, off = (cell - kOffM) % kCellsM;
            c.tail_step = (uint32_t) (2 * Mp * sizeof(float));
            c.tail_src = reinterpret_cast<const uint8_t *>(m4 + (size_t) gi * Mp + t0) + (size_t) off * 16 + (size_t) s_begin * c.tail_step;
        } else {
            const int gi = (cell - kOffK) / kCellsK, x = (cell - kOffK) % kCellsK;
            const int pnl = min(row_tile * 4 + (x >> 2), n_panels - 1);
            c.tail_step = 2 * kPanelRows;
            c.tail_src = kmul + ((size_t) pnl * ng + gi) * kPanelRows + (size_t) (x & 3) * 16 + (size_t) s_begin * c.tail_step;
        }
    }
    const int panel = min(row_tile * 4 + c.wr, n_panels - 1);
    c.k_src = kmul + (size_t) panel * ng * kPanelRows + 4 * (c.lane >> 5);

    if (c.wave < 4) {
        const int64_t n = (int64_t) row_tile * kTileRows + 64 * c.wave + c.lane;
        load_to_lds_dword(s_w + (n < N ? n : N - 1), &s_pre[64 * c.wave]);
    } else if (c.wave < 6) {
        const int t = t0 + 64 * (c.wave - 4) + c.lane;
        load_to_lds_dword(u + (t < M ? t : M - 1), &s_pre[kTileRows + 64 * (c.wave - 4)]);
    }

    float acc[2][2][16];
    int32_t tot[2][2][16];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                acc[a][b][r] = kBias;
                tot[a][b][r] = 0;
            }
        }
    }
    const bool hask = flags[0] & 1;
    // fp32 rounding toward minus infinity for the folds (MODE bits 1:0); the MFMA sums are exact in any mode
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 2" ::: "memory");
    if (KFMA || hask) {   // (the form for weight multipliers takes every tensor that way: multipliers of 1 where there are none)
        if constexpr (GS == 1) body64<true, KFMA>(c, s0, s1, s2, s3, acc, tot);
        else body<true, GS>(c, s0, s1, s2, s3, acc, tot);
    } else {
        if constexpr (GS == 1) body64<false, KFMA>(c, s0, s1, s2, s3, acc, tot);
        else body<false, GS>(c, s0, s1, s2, s3, acc, tot);
    }
    flush(acc, tot);
    // Back to round to nearest even for the epilogue. The compiler does not know that fp32 arithmetic reads MODE, so
    // the totals pass through a statement on either side of the change: the one in front keeps the last folds (which
    // the totals depend on) from being scheduled behind it, the one behind keeps the conversions below from being
    // scheduled in front of it.
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
#pragma unroll
            for (int r = 0; r < 16; ++r) asm volatile("" : "+v"(tot[a][b][r]));
        }
    }
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 0" ::: "memory");
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
#pragma unroll
            for (int r = 0; r < 16; ++r) asm volatile("" : "+v"(tot[a][b][r]));
        }
    }

    if (sliced) {
        // A slice of K: its totals go to a slab of their own (64 ints per thread, written through to memory at
        // device scope: the slices of a tile run on different XCDs, each with its own L2), then one atomic per
        // workgroup counts the arrival. The workgroup that completes the count adds the other slices' slabs to the
        // totals it still holds and goes on to the epilogue; the others are done. (An atomic per output instead,
        // accumulating in 64-bit arrival cells, cost more than the slicing gained: 8 M device-scope atomics.)
        // (Slabs move as 16 bytes per lane with the cache policy of a device-scope access: written through to memory,
        // read past this XCD's L2.)
        constexpr int kSlabBytes = kTileRows * kTileTok * (int) sizeof(int32_t);
        uint8_t *slab_base = reinterpret_cast<uint8_t *>(slabs) + (size_t) slot * parts * kSlabBytes;
        const uint32_t lane_off = (uint32_t) tid * 16;
        {
            const __amdgpu_buffer_rsrc_t mine = __builtin_amdgcn_make_buffer_rsrc(slab_base + (size_t) part * kSlabBytes, 0, kSlabBytes, kRsrcWord3);
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int a = i >> 3, b = (i >> 2) & 1, r = 4 * (i & 3);
                __builtin_amdgcn_raw_buffer_store_b128(v4i{ tot[a][b][r], tot[a][b][r + 1], tot[a][b][r + 2], tot[a][b][r + 3] }, mine,
                                                       lane_off + i * (kThreads * 16), 0, kDeviceScope);
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this thread's stores have reached memory
        __syncthreads();                                    // ... and everybody else's
        int *s_flag = reinterpret_cast<int *>(&s_pre[kTileRows + kTileTok]);
        if (tid == 0) {
            const int before = __hip_atomic_fetch_add(counters + slot, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (before == parts - 1) __hip_atomic_store(counters + slot, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *s_flag = before;
        }
        __syncthreads();
        if (*s_flag != parts - 1) return;
        // the other parts' slabs, the loads of the next one in flight while one is added
        v4i in[2][16];
        auto load_part = [&](int k, v4i (&dst)[16]) {   // k-th of the other parts
            const int pp = k < part ? k : k + 1;
            const __amdgpu_buffer_rsrc_t other = __builtin_amdgcn_make_buffer_rsrc(slab_base + (size_t) pp * kSlabBytes, 0, kSlabBytes, kRsrcWord3);
#pragma unroll
            for (int i = 0; i < 16; ++i) dst[i] = __builtin_amdgcn_raw_buffer_load_b128(other, lane_off + i * (kThreads * 16), 0, kDeviceScope);
        };
        auto add_part = [&](const v4i (&src)[16]) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int a = i >> 3, b = (i >> 2) & 1, r = 4 * (i & 3);
#pragma unroll
                for (int e = 0; e < 4; ++e) tot[a][b][r + e] += src[i][e];
            }
        };
        const int others = parts - 1;
        load_part(0, in[0]);
        for (int k = 0; k < others; k += 2) {
            if (k + 1 < others) load_part(k + 1, in[1]);
            add_part(in[0]);
            if (k + 1 < others) {
                if (k + 2 < others) load_part(k + 2, in[0]);
                add_part(in[1]);
            }
        }
    }

    // epilogue (reference patch line 176): y = ((float(total) * 16) * u) * s_w. In the MFMA result a lane holds one
    // token (column) and, per tile, rows 8 q + 4 (lane / 32) + 0 .. 3 for q = 0 .. 3: stored as they are, a wavefront's
    // stores would be 32-byte pieces of 32 different rows of y (a third of the kernel's time went there). So every
    // wavefront turns its four 32 x 32 blocks through LDS one after the other (4.5 KiB per wavefront, all eight inside
    // the last ring stage, which no fetch is aimed at when the loop ends) and writes 128 contiguous bytes per token.
    __syncthreads();   // every wavefront is done reading the ring
    float *xp = reinterpret_cast<float *>(&s3.cell[0]) + c.wave * (32 * kXposeStride);
    const int h = c.lane >> 5;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        const float ut = s_pre[kTileRows + 64 * c.wc + 32 * b + (c.lane & 31)];
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int rw = 8 * q + 4 * h;   // row within the block
                const float4 sw = *reinterpret_cast<const float4 *>(&s_pre[64 * c.wr + 32 * a + rw]);
                float4 o;
                o.x = (((float) tot[a][b][4 * q + 0] * 16.0f) * ut) * sw.x;
                o.y = (((float) tot[a][b][4 * q + 1] * 16.0f) * ut) * sw.y;
                o.z = (((float) tot[a][b][4 * q + 2] * 16.0f) * ut) * sw.z;
                o.w = (((float) tot[a][b][4 * q + 3] * 16.0f) * ut) * sw.w;
                *reinterpret_cast<float4 *>(&xp[(c.lane & 31) * kXposeStride + rw]) = o;
            }
            // (a wavefront reads back only what it wrote itself, and its LDS operations complete in order)
            const int64_t n = (int64_t) row_tile * kTileRows + 64 * c.wr + 32 * a + 4 * (c.lane & 7);
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int tw = 8 * it + (c.lane >> 3);   // token within the block
                const int t = t0 + 64 * c.wc + 32 * b + tw;
                const float4 o = *reinterpret_cast<const float4 *>(&xp[tw * kXposeStride + 4 * (c.lane & 7)]);
                if (t >= M) continue;
                float *dst = y + (int64_t) t * ldy + n;
                if (n + 3 < N && ((reinterpret_cast<uintptr_t>(dst) & 15) == 0)) {
                    // the output is written once and not read back by this launch: non-temporal
                    typedef float v4f __attribute__((ext_vector_type(4)));
                    __builtin_nontemporal_store(v4f{ o.x, o.y, o.z, o.w }, reinterpret_cast<v4f *>(dst));
                } else {
                    const float ov[4] = { o.x, o.y, o.z, o.w };
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (n + i < N) dst[i] = ov[i];
                    }
                }
            }
        }
    }
}

}  // namespace

Gemm6Plan gemm6_plan(int64_t N, int64_t M, int ng, int groups_per_fold) {
    Gemm6Plan pl;
    const int n_row_tiles = (int) ((N + kTileRows - 1) / kTileRows);
    const int n_tok_tiles = (int) ((M + kTileTok - 1) / kTileTok);
    pl.n_tiles = n_row_tiles * n_tok_tiles;
    pl.n_whole = pl.n_tiles;
    pl.parts = 1;
    // Whole rounds of the chip run a tile per workgroup. What is left over (fewer tiles than compute units) would
    // keep the chip busy for one more whole tile time; cut along K into `parts` slices per tile it takes 1 / parts of
    // that. (The count of compute units is taken as the 256 of the part this library is written for: the plan must
    // not depend on the device, because the workspace is sized from it.)
    const int left = pl.n_tiles % kPlanUnits;
    if (left > 0 && kPlanUnits / left >= 2) {
        // more slices = less work per slice, but the workgroup that completes a tile reads the other slices' slabs one
        // after the other (about 2 us each) and every slice pays its own start (about 5 us): per step 1.1 us
        const int steps = ng / 2;
        int best = 1;
        double best_cost = 1.1 * steps;
        for (int parts = 2; parts <= kPlanUnits / left && parts <= steps / 2; ++parts) {
            // wider activation groups: a slice holds whole groups and an even number of steps
            if (groups_per_fold > 1 && steps % (2 * parts) != 0) continue;
            const double cost = 1.1 * ((steps + parts - 1) / parts) + 5.0 + 2.0 * (parts - 1);
            if (cost < best_cost) {
                best_cost = cost;
                best = parts;
            }
        }
        if (best >= 2) {   // (left * parts <= kPlanUnits slices: the workspace holds a slab for each)
            pl.parts = best;
            pl.n_whole = pl.n_tiles - left;
        }
    }
    // one arrival counter per cut tile, then a slab of 256 x 128 ints per slice
    pl.cell_bytes = pl.parts > 1 ? kGemm6CounterBytes + (size_t) (pl.n_tiles - pl.n_whole) * pl.parts * kTileRows * kTileTok * sizeof(int32_t) : 0;
    return pl;
}

hipError_t launch_gemm6(const GemmArgs &a, hipStream_t stream) {
    const uint8_t *p = a.prepared;
    const int n_row_tiles = a.L.n_rtiles;
    const int n_tok_tiles = a.Mp / kTileTok;
    Gemm6Plan pl = gemm6_plan(a.L.N, a.M, a.L.ng, a.groups_per_fold);
    if (pl.n_tiles != n_row_tiles * n_tok_tiles) return hipErrorInvalidValue;
    if (a.cells == nullptr) {   // a workspace without slabs: every tile whole
        pl.n_whole = pl.n_tiles;
        pl.parts = 1;
    }
    const int super_tiles = n_tok_tiles % 4 == 0 && n_row_tiles % 8 == 0;
    const int grid = pl.n_whole + (pl.n_tiles - pl.n_whole) * pl.parts;
    const float *m4 = reinterpret_cast<const float *>(a.act8 + act6_plane_bytes(a.L.ng, a.Mp));
#define RQ_LAUNCH6(GS, KFMA)                                                                                        \
    hipLaunchKernelGGL((rq_gemm6_kernel<GS, KFMA>), dim3(grid), dim3(kThreads), 0, stream,                            \
                       reinterpret_cast<const float *>(p + a.L.off_sw), p + a.L.off_kmul,                           \
                       reinterpret_cast<const int32_t *>(p + a.L.off_flags), a.act8, m4, a.u, a.y, a.ldy, a.L.N, a.M, \
                       a.Mp, a.L.ng, a.L.n_panels, n_tok_tiles, pl.n_tiles, super_tiles, pl.n_whole, pl.parts,      \
                       reinterpret_cast<int *>(a.cells),                                                             \
                       reinterpret_cast<unsigned long long *>(reinterpret_cast<uint8_t *>(a.cells) + kGemm6CounterBytes))
    // (a.weight_multipliers: what the host knows about the tensor; only a choice between two kernels that are both
    // right for every tensor)
    if (a.groups_per_fold == 1 && a.weight_multipliers) RQ_LAUNCH6(1, true);
    else if (a.groups_per_fold == 1) RQ_LAUNCH6(1, false);
    else if (a.groups_per_fold == 2) RQ_LAUNCH6(2, false);
    else RQ_LAUNCH6(4, false);
#undef RQ_LAUNCH6
    return hipGetLastError();
}

}  // namespace rq
