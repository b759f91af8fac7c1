// One-token W4A4 / W4A4H MUL_MAT in ONE launch: online Hadamard, activation quantizer, int4 x int4 product and the
// fp32 epilogue (kernels 1-4 of the decode path) with no second kernel, no split-K cells and no atomics in memory.
//
// Why one launch: a dependent launch costs about 1.8 us on this part even inside a HIP graph, and the rotation of a
// single row is a chain of short latency-bound phases that cannot fill the chip. Here every workgroup repeats the
// (cheap) rotation + quantization of the token for itself, hidden behind its own share of the weight stream:
//
//   * wavefronts 8..15 ("stream") put ALL of the workgroup's weight bytes in flight into registers right away
//     (about 170 KiB per compute unit for a 44 MB weight; a wavefront that has queued loads stalls at issue once the
//     memory queue is full, which is why these wavefronts do nothing else), then wait at the workgroup's barriers;
//   * wavefronts 0..7 ("rotate") load the row, run the Sylvester butterflies and the Paley stage in LDS with the
//     reference's order of additions (ggml_rq_hadamard, reference patch lines 2450-2485), reduce the clipped group
//     ranges, derive the token unit, the group multipliers and zero points and the 4-bit codes
//     (rq_quantize_row_a, lines 2639-2679) into LDS;
//   * the stream wavefronts then fold group by group (ggml_vec_dot_w4a4_a4, lines 148-177) as their loads arrive,
//     add the exact int32 terms into per-row cells in LDS, and the epilogue writes y = ((float(total) * 16) * u) * s_w.
//
// Work is dealt in whole rows (never along K, so no reduction between workgroups exists): the rows of the launch are
// cut into quads, workgroup s takes quads [s Q / G, (s + 1) Q / G), and G is the number of compute units, so every
// compute unit streams the same number of bytes to within one quad. A stream wavefront reads the prepared layout as
// items of 8 rows x 4 groups: lane = (row of the octet, half of the group, group of the item), one 16-byte load per
// lane, eight full 128-byte lines per wavefront load. An octet that two workgroups share is read by both (its lines
// hold both quads); the slot order puts such neighbours on one XCD, where the second read is an L2 hit.
#include "rq_hadamard.h"

#pragma clang fp contract(off)

#ifdef RQ_DECODE_TIMING
// Phase timestamps of workgroup 0 (wavefronts 0 and 8), kept in registers and written out at the very end: a store in
// the middle of the kernel would queue behind the weight stream and distort what it measures.
__device__ unsigned long long rq_decode_stamps[64];   // [0, 16) rotate wavefront, [32, 48) stream wavefront
#define RQ_STAMP_DECL unsigned long long rq_st[16] = {}
#define RQ_STAMP(i) do { rq_st[(i)] = __builtin_readcyclecounter(); } while (0)
#define RQ_STAMP_AT(st, i) do { (st)[(i)] = __builtin_readcyclecounter(); } while (0)
#define RQ_STAMP_PTR rq_st
#define RQ_STAMP_FLUSH do { if (blockIdx.x == 0 && (threadIdx.x == 0 || threadIdx.x == 512)) { \
        for (int i_ = 0; i_ < 16; ++i_) rq_decode_stamps[i_ + (threadIdx.x ? 32 : 0)] = rq_st[i_]; } } while (0)
extern "C" int rq_w4a4_decode_stamps(unsigned long long *out) {
    return (int) hipMemcpyFromSymbol(out, HIP_SYMBOL(rq_decode_stamps), sizeof(rq_decode_stamps));
}
#else
#define RQ_STAMP_DECL do { } while (0)
#define RQ_STAMP(i) do { } while (0)
#define RQ_STAMP_AT(st, i) do { } while (0)
#define RQ_STAMP_PTR nullptr
#define RQ_STAMP_FLUSH do { } while (0)
#endif

namespace rq {

namespace {

using namespace had;

constexpr int kRotWaves = 8;
constexpr int kStrWaves = 8;
constexpr int kRotThreads = kRotWaves * 64;
constexpr int kDecThreads = (kRotWaves + kStrWaves) * 64;

struct DecodeKernelArgs {
    WeightSet    ws;        // up to three weights of one K; first[] counts panels
    const float *x;         // the token's row of K floats
    int          K, rotate, n_rot, m;
    float        scale, clip;
    int          main_panels;       // whole panels per workgroup: panels s, s + G, ... (G = workgroups)
    int          tail_panel0;       // first panel of the remainder, which is dealt in quads of rows
    int          q_base, q_extra;   // remainder quads per workgroup: q_base, the first q_extra slots one more
    int          inv_nblk;          // floor(2^22 / nblk) + 1, nblk = K / 256: i / nblk = (i * inv_nblk) >> 22 for every item index
    int          syncs;             // bits 0-7: times the rotate wavefronts meet (rot_sync) until the codes are in LDS
                                    // bits 8-9: 1 / 2: every rotate wavefront has that many pairs of Paley items and
                                    // quantizes their sums from its registers (paley_quantize); 0: the sums go through
                                    // LDS. (One word: the arguments end where a 64-byte line of the kernel-argument
                                    // segment ends, and a word on the next line, asked for behind the first barrier,
                                    // is a miss of its own in front of every wavefront's first wait: K = 5120,
                                    // N = 5120: 6.5 -> 6.4 us with the two packed into one word.)
};

__device__ __forceinline__ int dot8(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot8((int) a, (int) b, c, false);
}

// a * b + c with a and b of at most 24 bits as the one full-rate instruction (from __mul24(a, b) + c the compiler
// makes a 64-bit multiply-add, which runs at a quarter of the rate); the first form takes `a` from a scalar register
__device__ __forceinline__ int mad24_s(int a, int b, int c) {
    int r;
    asm("v_mad_i32_i24 %0, %1, %2, %3" : "=v"(r) : "s"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ int mad24(int a, int b, int c) {
    int r;
    asm("v_mad_i32_i24 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

__device__ __forceinline__ int align4(int v) { return (v + 3) & ~3; }

// Barrier among the rotate wavefronts only, through a counter in LDS that only grows: a wavefront adds one when its
// LDS writes of the phase are done and waits until all kRotWaves have (`target` = kRotWaves x phases so far). The
// hardware barrier would also wait for the stream wavefronts, which sit blocked in the issue of their loads for
// microseconds (the memory queue is full): the phases of the rotation must not wait for that.
// (The counter is read through an LDS-typed pointer: a generic one makes the poll a FLAT load, which queues behind
// the weight stream.)
typedef __attribute__((address_space(3))) int lds_int;
template <bool SLEEP>
__device__ __forceinline__ void wait_count(const int *cnt, int target) {
    const volatile lds_int *c = (const volatile lds_int *) cnt;
    while (__builtin_amdgcn_readfirstlane(*c) < target) {
        if (SLEEP) __builtin_amdgcn_s_sleep(2);   // the stream waits for microseconds; the rotation for a straggler
    }
    asm volatile("" ::: "memory");
}
// (The add needs no wait for the wavefront's LDS writes in front of it: a wavefront's LDS instructions are carried out in
// the order of issue, so whoever sees the count sees the writes. It returns the count, and the wavefront that
// arrives last, the one the others wait for, knows so from the answer and does not poll: two LDS round trips less on
// the critical path of every phase. The ordering rests on that in-order LDS queue plus the compiler barrier in front of
// the add, which keeps the compiler from sinking the phase's plain LDS stores below the relaxed atomic.)
__device__ __forceinline__ void rot_sync(int *cnt, int &target, int lane) {
    target += kRotWaves;
    int seen = 0;
    asm volatile("" ::: "memory");
    if (lane == 0) seen = atomicAdd(cnt, 1) + 1;
    seen = __builtin_amdgcn_readfirstlane(seen);
    if (seen < target) wait_count<false>(cnt, target);
    asm volatile("" ::: "memory");
}

// The activation quantizer of the rotate wavefronts for R code words per thread (word w = r x 512 + thread, its eight
// values stay in registers between the two phases): group ranges [min(x, 0), max(x, 0)] x clip with eight lanes per
// group of 64 and the token's widest range (reference lines 2646-2654); then, behind the phase barrier, the unit, per
// group multiplier and zero point, and the 4-bit codes (reference lines 2662-2677). R is a compile-time constant so
// that the R rounds are one instruction stream: their LDS reads go out together and their dependent min / max / DPP
// chains interleave (as separate uniform branches the rounds ran one after the other).
template <int R>
__device__ __forceinline__ void quantize_rounds(const float *row, bool dense, int nw, float clip, int rt, int lane,
                                                int wave, float *s_part, float *s_unit, uint32_t *s_act,
                                                int32_t *s_mz, int *s_cnt, int &sync_target, unsigned long long *stamps) {
    (void) stamps;
    float f[R][8];
    float g_lo_r[R], g_hi_r[R];
#pragma unroll
    for (int wr = 0; wr < R; ++wr) {
        const int w = wr * kRotThreads + rt;
        const bool on = w < nw;
        if (dense) {
            const float4 *sp = reinterpret_cast<const float4 *>(row + 8 * (on ? w : 0));
            const float4 v0 = sp[0], v1 = sp[1];
            f[wr][0] = v0.x; f[wr][1] = v0.y; f[wr][2] = v0.z; f[wr][3] = v0.w;
            f[wr][4] = v1.x; f[wr][5] = v1.y; f[wr][6] = v1.z; f[wr][7] = v1.w;
        } else {
            const float *sp = row + padi(8 * (on ? w : 0));
#pragma unroll
            for (int j = 0; j < 8; ++j) f[wr][j] = sp[j];
        }
        if (!on) {
#pragma unroll
            for (int j = 0; j < 8; ++j) f[wr][j] = 0.0f;
        }
    }
#ifdef RQ_DECODE_TIMING
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // (the values have arrived from LDS)
#endif
    RQ_STAMP_AT(stamps, 10);
    float rmax = 0.0f;
#pragma unroll
    for (int wr = 0; wr < R; ++wr) {
        const bool on = wr * kRotThreads + rt < nw;
        float mn = 0.0f, mx = 0.0f;
        minmax8_raw(f[wr], mn, mx);
        mn = group8_reduce<false>(mn);
        mx = group8_reduce<true>(mx);
        g_lo_r[wr] = mn * clip;
        g_hi_r[wr] = mx * clip;
        if (on) rmax = fmaxf(rmax, g_hi_r[wr] - g_lo_r[wr]);
    }
    rmax = wave_max(rmax);
    if (lane == 0) s_part[wave] = rmax;
    RQ_STAMP_AT(stamps, 11);
    rot_sync(s_cnt, sync_target, lane);
    RQ_STAMP_AT(stamps, 5);

    float Rg = s_part[0];
#pragma unroll
    for (int i = 1; i < kRotWaves; ++i) Rg = fmaxf(Rg, s_part[i]);
    if (Rg == 0.0f) Rg = 2.0f;
    const float u = Rg / 3825.0f;  // 15 * 255
    if (rt == 0) s_unit[0] = u;
#pragma unroll
    for (int wr = 0; wr < R; ++wr) {
        const int w = wr * kRotThreads + rt;
        const float lo = g_lo_r[wr], hi = g_hi_r[wr];
        const int mg = (int) fminf(fmaxf(ceilf(((hi - lo) * 255.0f) / Rg), 1.0f), 255.0f);
        const float inv = 1.0f / ((float) mg * u);
        const float zf = fminf(fmaxf(rintf(-lo * inv), 0.0f), 15.0f);
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int q = (int) fminf(fmaxf(rintf(f[wr][j] * inv) + zf, 0.0f), 15.0f);
            word |= (uint32_t) ((q - 8) & 0xF) << (4 * j);
        }
        if (w < nw) {
            s_act[w] = word;
            if ((w & 7) == 0) s_mz[w >> 3] = mg | ((8 - (int) zf) & 0xFF) << 8;
        }
    }
    RQ_STAMP_AT(stamps, 12);
}

// LDS: [row, padded][Paley output, dense][codes][mz][cells][wave maxima, unit, phase counter]
__host__ __device__ inline size_t decode_lds_bytes(int K, bool two_rows) {
    const int Kp = ((K + (K >> 4) + 1) + 3) & ~3;
    const int ng = K / kGroup;
    return (size_t) (Kp + (two_rows ? K : 0) + K / 8 + ng + kDecodeCells + 8 + kRotWaves + 4) * 4;
}

// Two Paley items of one wavefront, column runs `cr` and `cr + 1` of slice `s` (a run = 64 neighbouring columns, a
// slice = P / 4 of a column's outputs), as one instruction stream: from the padded row `buf` to the dense row `alt`.
template <int P>
__device__ __forceinline__ void paley_pair(const float *buf, float *alt, int s, int cr, int lane, int lm, int m,
                                           int n_rot, int pm, float scale) {
    constexpr int kOut = P / 4;
    const int c0 = cr * 64 + lane, c1 = c0 + 64;
    const int b0 = (c0 >> lm) * n_rot + (c0 & (m - 1)), b1 = (c1 >> lm) * n_rot + (c1 & (m - 1));
    float out0[kOut], out1[kOut];
    if (m == 256) {
        paley_pick_stream2<P, kOut, 272>(s, buf + padi(b0), buf + padi(b1), 272, out0, out1);
    } else {
        paley_pick_stream2<P, kOut, 0>(s, buf + padi(b0), buf + padi(b1), pm, out0, out1);
    }
    float *d0 = alt + b0 + kOut * s * m, *d1 = alt + b1 + kOut * s * m;
#pragma unroll
    for (int o = 0; o < kOut; ++o) {
        d0[o * m] = out0[o] * scale;
        d1[o * m] = out1[o] * scale;
    }
}

// Maxima over the lanes of up to sixteen registers at once, each result delivered to the lanes that will work with
// it: a butterfly in which a lane keeps one register of a pair and hands the other to its partner, so every level
// halves the registers (three instructions per pair: two selects and a maximum whose operand is the lane permutation)
// where one all-lanes reduction per register costs six plus a transfer through a scalar register. The partners are the
// four exact lane exchanges of the DPP unit, in an order in which no exchange disturbs the lane bits chosen by earlier
// levels: lane ^ 7 (row_half_mirror, choosing by lane bit 2), ^ 1 (bit 0), ^ 2 (bit 1), ^ 8 (row_ror:8, bit 3); then
// the four rows of sixteen lanes are combined so that every row holds the results. Register i's result ends in the
// lanes l with scatter_index(l) == i; lanes whose index has no register hold the identity.
// SIGNED: maximum of the bit patterns as signed integers, which among floats of both signs is the largest positive
// value if there is one (else some negative value: the caller takes the maximum with 0 anyway); otherwise as unsigned
// integers: the most negative value if there is one.
__device__ __forceinline__ int scatter_index(int lane) {
    return ((lane >> 2) & 1) | ((lane & 1) << 1) | (((lane >> 1) & 1) << 2) | (lane & 8);
}
constexpr int scatter_lane(int i) { return ((i & 1) << 2) | ((i >> 1) & 1) | (((i >> 2) & 1) << 1) | (i & 8); }

template <bool SIGNED>
__device__ __forceinline__ uint32_t pattern_max(uint32_t a, uint32_t b) {
    return SIGNED ? (uint32_t) max((int) a, (int) b) : max(a, b);
}
template <bool SIGNED, int LEVEL>
__device__ __forceinline__ uint32_t exchange_max(uint32_t keep, uint32_t give) {
    constexpr int kCtrl = LEVEL == 0 ? 0x141 : LEVEL == 1 ? 0xB1 : LEVEL == 2 ? 0x4E : 0x128;
    return pattern_max<SIGNED>(keep, (uint32_t) __builtin_amdgcn_update_dpp(0, (int) give, kCtrl, 0xF, 0xF, true));
}
template <bool SIGNED, int N, int LEVEL>
__device__ __forceinline__ uint32_t scatter_max(const uint32_t (&v)[N], const bool (&upper)[4]) {
    constexpr uint32_t kIdentity = SIGNED ? 0x80000000u : 0u;
    if constexpr (LEVEL == 4) {
        static_assert(N == 1, "sixteen registers at most");
        typedef unsigned v2u __attribute__((ext_vector_type(2)));
        const v2u a = __builtin_amdgcn_permlane16_swap(v[0], v[0], false, false);   // rows 0 with 1, 2 with 3
        const uint32_t r = pattern_max<SIGNED>(a.x, a.y);
        const v2u b = __builtin_amdgcn_permlane32_swap(r, r, false, false);         // the halves of the wavefront
        return pattern_max<SIGNED>(b.x, b.y);
    } else {
        constexpr int H = (N + 1) / 2;
        uint32_t r[H];
#pragma unroll
        for (int j = 0; j < H; ++j) {
            const uint32_t A = v[2 * j], B = 2 * j + 1 < N ? v[2 * j + 1] : kIdentity;
            r[j] = exchange_max<SIGNED, LEVEL>(upper[LEVEL] ? B : A, upper[LEVEL] ? A : B);
        }
        return scatter_max<SIGNED, H, LEVEL + 1>(r, upper);
    }
}

// Paley stage and activation quantizer of one rotate wavefront without a trip through LDS in between, for rows where
// every wavefront has NPAIR pairs of Paley items (column runs cr, cr + 1, ... of slice s). The 64 lanes of one Paley
// output register hold 64 neighbouring columns of one output chunk: exactly one activation group. So the group's
// range is a reduction over the lanes of that register (reference lines 2646-2654), the lanes the reduction delivers
// group i to work out its multiplier, zero point and reciprocal step (lines 2662-2668: the two divisions once per
// group), and the codes are made where the values are (lines 2670-2675), eight neighbouring lanes gathering a code word.
template <int P, int NPAIR>
__device__ __forceinline__ void paley_quantize(const float *buf, int s, int cr, int lane, int wave, int lm, int m,
                                               int n_rot, int pm, float scale, float clip, float *s_part,
                                               float *s_unit, uint32_t *s_act, int32_t *s_mz, int *s_cnt,
                                               int &sync_target, unsigned long long *stamps) {
    (void) stamps;
    constexpr int kOut = P / 4;
    constexpr int NG = NPAIR * 2 * kOut;   // groups (= registers) of this wavefront
    constexpr int NB = (NG + 15) / 16;     // batches of sixteen registers: batch b is delivered to the lanes of row b
    static_assert(NB <= 2, "two rows of lanes take the parameters");
    float x[NG];
    int e_first = 0;   // element index of output 0 of the first run's first column; run r starts 64 r behind it
#pragma unroll
    for (int pr = 0; pr < NPAIR; ++pr) {
        const int c0 = (cr + 2 * pr) * 64 + lane, c1 = c0 + 64;
        const int b0 = (c0 >> lm) * n_rot + (c0 & (m - 1)), b1 = (c1 >> lm) * n_rot + (c1 & (m - 1));
        float out0[kOut], out1[kOut];
        if (m == 256) {
            paley_pick_stream2<P, kOut, 272>(s, buf + padi(b0), buf + padi(b1), 272, out0, out1);
        } else {
            paley_pick_stream2<P, kOut, 0>(s, buf + padi(b0), buf + padi(b1), pm, out0, out1);
        }
#pragma unroll
        for (int o = 0; o < kOut; ++o) {
            x[(2 * pr) * kOut + o] = out0[o] * scale;
            x[(2 * pr + 1) * kOut + o] = out1[o] * scale;
        }
        if (pr == 0) e_first = __builtin_amdgcn_readfirstlane(b0 + kOut * s * m);
    }
    RQ_STAMP_AT(stamps, 9);
    RQ_STAMP_AT(stamps, 4);
    RQ_STAMP_AT(stamps, 10);
    // ranges: min(0, x ...) and max(0, x ...) of each register over its lanes, delivered to the lanes of the group
    const bool upper[4] = { (lane & 4) != 0, (lane & 1) != 0, (lane & 2) != 0, (lane & 8) != 0 };
    const int g_l = ((lane >> 4) & 1) * 16 + scatter_index(lane);   // the group (of this wavefront) the lane works for
    uint32_t lo_bits = 0, hi_bits = 0;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        constexpr int kFull = 16;
        const int n = NG - b * kFull < kFull ? NG - b * kFull : kFull;
        uint32_t v[kFull];
#pragma unroll
        for (int i = 0; i < kFull; ++i) v[i] = b * kFull + i < NG ? __builtin_bit_cast(uint32_t, x[b * kFull + i < NG ? b * kFull + i : 0]) : 0u;
        uint32_t lo_b, hi_b;
        if (n > 8) {
            lo_b = scatter_max<false, 16, 0>(v, upper);
#pragma unroll
            for (int i = 0; i < kFull; ++i) if (b * kFull + i >= NG) v[i] = 0x80000000u;
            hi_b = scatter_max<true, 16, 0>(v, upper);
        } else {
            uint32_t w8[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) w8[i] = v[i];
            lo_b = scatter_max<false, 8, 0>(w8, upper);
#pragma unroll
            for (int i = 0; i < 8; ++i) if (b * kFull + i >= NG) w8[i] = 0x80000000u;
            hi_b = scatter_max<true, 8, 0>(w8, upper);
        }
        if (b == 0 || (lane & 16)) {
            lo_bits = lo_b;
            hi_bits = hi_b;
        }
    }
    const bool mine = g_l < NG && lane < 32;
    const float lo_l = fminf(__builtin_bit_cast(float, lo_bits), 0.0f) * clip;
    const float hi_l = fmaxf(__builtin_bit_cast(float, hi_bits), 0.0f) * clip;
    const float rmax = wave_max(mine ? hi_l - lo_l : 0.0f);
    if (lane == 0) s_part[wave] = rmax;
    RQ_STAMP_AT(stamps, 11);
    rot_sync(s_cnt, sync_target, lane);
    RQ_STAMP_AT(stamps, 5);

    float Rg = s_part[0];
#pragma unroll
    for (int i = 1; i < kRotWaves; ++i) Rg = fmaxf(Rg, s_part[i]);
    if (Rg == 0.0f) Rg = 2.0f;
    const float u = Rg / 3825.0f;  // 15 * 255
    if (wave == 0 && lane == 0) s_unit[0] = u;
    // the parameters of the lane's group
    const int mg_l = (int) fminf(fmaxf(ceilf(((hi_l - lo_l) * 255.0f) / Rg), 1.0f), 255.0f);
    const float inv_l = 1.0f / ((float) mg_l * u);
    const float zf_l = fminf(fmaxf(rintf(-lo_l * inv_l), 0.0f), 15.0f);
    if (mine) {
        // (group g: run g / kOut of the wavefront, output g % kOut; the wavefront's runs are neighbours in one rotation
        // block, so run r starts 64 r elements behind run 0)
        const int run = g_l / kOut, o = g_l - run * kOut;
        s_mz[(e_first >> 6) + run + o * (m >> 6)] = mg_l | ((8 - (int) zf_l) & 0xFF) << 8;
    }
    // (all code words first, then the stores under one lane mask: with a store per group in between, every group's
    // dependent chain ran alone, with the wait states of its lane permutations unfilled)
    const int nib_shift = 4 * (lane & 7);
    uint32_t word[NG];
#pragma unroll
    for (int i = 0; i < NG; ++i) {
        const int src = (i >> 4) * 16 + scatter_lane(i & 15);
        const float inv = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, inv_l), src));
        const float zf = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, zf_l), src));
        // (the median of three is the clamp: the sum is finite)
        const uint32_t q = (uint32_t) (int) __builtin_amdgcn_fmed3f(rintf(x[i] * inv) + zf, 0.0f, 15.0f);
        uint32_t w = q << nib_shift;
        w |= (uint32_t) __builtin_amdgcn_update_dpp(0, (int) w, 0xB1, 0xF, 0xF, true);
        w |= (uint32_t) __builtin_amdgcn_update_dpp(0, (int) w, 0x4E, 0xF, 0xF, true);
        w |= (uint32_t) __builtin_amdgcn_update_dpp(0, (int) w, 0x141, 0xF, 0xF, true);
        word[i] = w ^ 0x88888888u;   // q - 8 as 4-bit two's complement
    }
    if ((lane & 7) == 0) {
        uint32_t *dst = s_act + (lane >> 3);
#pragma unroll
        for (int i = 0; i < NG; ++i) {
            dst[(e_first >> 3) + 8 * (i / kOut) + (i % kOut) * (m >> 3)] = word[i];
        }
    }
    RQ_STAMP_AT(stamps, 12);
}

// MG: group-items (64 rows x one group: two loads) a stream wavefront has in flight per round of a whole panel;
// MT: remainder items (8 rows x 4 groups: one load) per round. The first round of both is issued up front.
template <int P, int MG, int MT>
__global__ void __launch_bounds__(kDecThreads) rq_decode_kernel(const DecodeKernelArgs a) {
    extern __shared__ __align__(16) float smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    RQ_STAMP_DECL;
    RQ_STAMP(0);
    const int K = a.K, ng = K / kGroup;

    // ---- the rotate wavefronts request the row before anything else: 16 consecutive floats per thread and unit.
    // Everything below (cells, row scales, item addresses) is computed while it travels.
    // Chunks of 256 floats (16 units): the 16 lanes of a DPP row hold one chunk, so the Sylvester stages with
    // strides 16 .. 128 run between lanes and the row makes no trip through LDS between its stages (dpp_unit_of_lane
    // says which unit a lane holds).
    const bool dpp256 = a.rotate && (a.m & 255) == 0;   // chunks of whole blocks of 256 floats
    const DppUnit du = dpp_unit_of_lane(lane);
    const int unit_of_lane = du.unit;
    constexpr int kUnits = 2;   // K <= 16384
    float4 qv[kUnits][4];
    if (wave < kRotWaves) {
#pragma unroll
        for (int ub = 0; ub < kUnits; ++ub) {
            int u = tid + ub * kRotThreads;
            if (dpp256) u = (u & ~15) | unit_of_lane;
            if (u < (K >> 4)) {
                const float4 *src = reinterpret_cast<const float4 *>(a.x + 16 * u);
#pragma unroll
                for (int j = 0; j < 4; ++j) qv[ub][j] = src[j];
            }
        }
    }
    const int Kp = align4(padi(K) + 1);
    float *buf = smem;
    float *alt = smem + Kp;   // Paley output, dense (its readers take 8 consecutive floats as two 16-byte reads)
    uint32_t *s_act = reinterpret_cast<uint32_t *>(smem + Kp + (P > 1 ? K : 0));   // [K / 8] code words, tensor nibble order
    int32_t *s_mz = reinterpret_cast<int32_t *>(s_act + K / 8);    // [ng] m | (8 - z) << 8
    int32_t *red = s_mz + ng;                                      // cells: [whole panels][64 rows], [octets][8 rows], one spare
    float *s_part = reinterpret_cast<float *>(red + kDecodeCells + 8);   // [kRotWaves] widest range per wavefront
    float *s_unit = s_part + kRotWaves;
    int *s_cnt = reinterpret_cast<int *>(s_unit + 1);   // phases the rotate wavefronts have finished, x kRotWaves

    if (tid < kDecodeCells + 8) red[tid] = 0;
    if (tid == 0) s_cnt[0] = 0;
    // The first of the kernel's two hardware barriers (the other one stands in front of the epilogue): the cells and
    // the phase counter are initialized before anybody adds to them. It comes early (behind the row request, in front
    // of everything that needs more arguments), where no wavefront is held up yet. The stream wavefronts do NOT wait
    // for the row: a compute unit's memory pipeline takes requests in issue order, and the row was requested by the
    // kernel's first instructions, so it is ahead of every weight by construction. (When the row was requested
    // further down, weight requests that got in front of it delayed it by the translation of their first page:
    // with 1, 2, 4 or 9 of a wavefront's 10 groups requested early the call took 11.9, 11.7, 12.5, 15.3 us instead of
    // 11.0, and a barrier held the stream back until the row had arrived. With the row first, that barrier only
    // cost time: 8.5 -> 7.7 us at N = 5120.)
    __builtin_amdgcn_s_barrier();
    RQ_STAMP(13);

    // ---- The stream wavefronts request the first round of their first whole panel here, in front of everything else
    // they work out (rows and cells, the remainder's addresses: 1700 cycles). The barrier above is what keeps the
    // token's row in front of them in the memory pipeline: the rotate wavefronts ask for it before they arrive there.
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    v4u w[MG > 0 ? MG : 1][2];
    // groups asked for here: their registers are live through all that follows. 2 take 0.03 us off the headline
    // call, 4 take 0.2, 6 take 0.24, 8 no longer fit the registers (+0.5 us). The 12-group form that also carries
    // remainder items has no register to spare: with any asked for early it spills more (K = 6144, N = 17408:
    // 13.6 -> 14.8 us).
    constexpr int kEarly = (MG >= 12 && MT > 0) ? 0 : MG < 6 ? MG : 6;
    if constexpr (MG > 0) {
        if (wave >= kRotWaves) {
            const int sw = wave - kRotWaves;
            const int panel = blockIdx.x;   // the first of panels s, s + G, ...
            const int wsel = (panel >= a.ws.first[1]) + (panel >= a.ws.first[2]);
            const int wpanel = panel - (wsel == 0 ? 0 : wsel == 1 ? a.ws.first[1] : a.ws.first[2]);
            const uint8_t *codes = wsel == 0 ? a.ws.codes[0] : wsel == 1 ? a.ws.codes[1] : a.ws.codes[2];
            const uint8_t *pbase = codes + (size_t) wpanel * ng * 2048 + lane * 16;
#pragma unroll
            for (int j = 0; j < kEarly; ++j) {
                int g = sw + j * kStrWaves;
                if (g >= ng) g = 0;   // past the end: the first group again, contributes nothing
                w[j][0] = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(pbase + (size_t) g * 2048));
                w[j][1] = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(pbase + (size_t) g * 2048 + 1024));
            }
        }
    }

    // ---- this workgroup's rows: whole panels s, s + G, ..., and a run of quads of the remainder panels. Remainder
    // slots run over the XCDs so that slots t and t + 1 (which may share an octet) sit on one XCD: workgroups go to
    // the eight XCDs round robin.
    const int G = gridDim.x;
    const int s_wg = blockIdx.x;
    int slot = s_wg;
    if (G % kXcds == 0) slot = (int) (blockIdx.x % kXcds) * (G / kXcds) + (int) (blockIdx.x / kXcds);
    const int q0 = a.tail_panel0 * 16 + slot * a.q_base + (slot < a.q_extra ? slot : a.q_extra);
    const int q1 = q0 + a.q_base + (slot < a.q_extra ? 1 : 0);
    const int oct0 = q0 >> 1, n_oct = q1 > q0 ? ((q1 + 1) >> 1) - oct0 : 0;
    const int nblk = ng >> 2;
    const int main_cells = a.main_panels * kPanelRows;

    // the epilogue's thread = one row of the workgroup; its row scale is requested before anything else
    float pre_sw = 0.0f;
    float *y_row = nullptr;
    if (tid < main_cells + n_oct * 8) {
        int panel, r;
        bool mine = true;
        if (tid < main_cells) {
            panel = (tid >> 6) * G + s_wg;
            r = tid & 63;
        } else {
            const int t = tid - main_cells;
            const int o = oct0 + (t >> 3);
            const int q = 2 * o + ((t & 7) >> 2);
            panel = o >> 3;
            r = (o & 7) * 8 + (t & 7);
            mine = q >= q0 && q < q1;
        }
        const int wsel = (panel >= a.ws.first[1]) + (panel >= a.ws.first[2]);
        const int wpanel = panel - (wsel == 0 ? 0 : wsel == 1 ? a.ws.first[1] : a.ws.first[2]);
        const float *s_w = wsel == 0 ? a.ws.s_w[0] : wsel == 1 ? a.ws.s_w[1] : a.ws.s_w[2];
        const int64_t N = wsel == 0 ? a.ws.N[0] : wsel == 1 ? a.ws.N[1] : a.ws.N[2];
        float *y = wsel == 0 ? a.ws.y[0] : wsel == 1 ? a.ws.y[1] : a.ws.y[2];
        const int64_t n = (int64_t) wpanel * kPanelRows + r;
        if (mine && n < N) {
            pre_sw = s_w[n];
            y_row = y + n;
        }
    }

    RQ_STAMP(14);
    if (wave >= kRotWaves) {
        // =========================================================== the weight stream
        const int sw = wave - kRotWaves;
        const int r8 = lane & 7, h = (lane >> 3) & 1, g4 = lane >> 4;
        const uint32_t lane_off = (uint32_t) (g4 * 2048 + h * 1024 + r8 * 16);
        // flag words of the weights (bit 0: some weight multiplier differs from 1)
        // (from the copy of this workgroup's turn: with all 2048 stream wavefronts of a launch on the one line of the
        // word itself, these loads, which sit in every wavefront's queue in front of most of its weights, took long to
        // come back, and loads come back in order: K = 5120, N = 17408 9.72 -> 9.55 us, N = 12288 7.98 -> 7.72)
        const int flag_copy = 64 + 16 * (int) (blockIdx.x % kFlagReplicas);
        const int32_t f0 = __builtin_nontemporal_load(a.ws.flags[0] + flag_copy);
        const int32_t f1 = __builtin_nontemporal_load(a.ws.flags[1] + flag_copy);
        const int32_t f2 = __builtin_nontemporal_load(a.ws.flags[2] + flag_copy);

        RQ_STAMP(1);

        const bool anyk = ((f0 | f1 | f2) & 1) != 0;
        const int n_items = n_oct * nblk;
        const int codes_ready = kRotWaves * (a.syncs & 255);
        bool waited = false;

        // remainder item `i` of this workgroup -> address of its 1 KiB (8 rows x 4 groups x 2 halves)
        // (items past the end read the first 16 bytes of the workgroup's own first item, every lane the same: one
        // request per load, and a different line for every workgroup; with the whole first KiB read again the load
        // path carried up to as many KiB of these as of real items. A workgroup without remainder rows takes the
        // remainder's first bytes: valid memory)
        auto tail_address = [&](int i, bool valid) -> const uint8_t * {
            const int ol = valid ? (int) (((uint32_t) i * (uint32_t) a.inv_nblk) >> 22) : 0;
            const int bb = valid ? i - ol * nblk : 0;
            const int o = n_items > 0 ? oct0 + ol : a.tail_panel0 * 8;
            const int panel = o >> 3;
            const int wsel = (panel >= a.ws.first[1]) + (panel >= a.ws.first[2]);
            const int wpanel = panel - (wsel == 0 ? 0 : wsel == 1 ? a.ws.first[1] : a.ws.first[2]);
            const uint8_t *codes = wsel == 0 ? a.ws.codes[0] : wsel == 1 ? a.ws.codes[1] : a.ws.codes[2];
            return codes + ((size_t) wpanel * ng + 4 * bb) * 2048 + (o & 7) * 128 + (valid ? lane_off : 0u);
        };
        // the first round of remainder items goes out with the first round of the whole panels
        v4u wt[MT > 0 ? MT : 1];
        if constexpr (MT > 0) {
#pragma unroll
            for (int it = 0; it < MT; ++it) {
                const int i = sw + it * kStrWaves;
                wt[it] = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(tail_address(i, i < n_items)));
            }
        }

        RQ_STAMP(15);
        // ---- whole panels: lane = row, a group is two 1 KiB loads; the wavefront takes groups sw, sw + 8, ...
        if constexpr (MG > 0) {
            const int gpw = (ng + kStrWaves - 1) / kStrWaves;   // groups per wavefront and panel
            for (int pl = 0; pl < a.main_panels; ++pl) {
                const int panel = pl * G + s_wg;
                const int wsel = (panel >= a.ws.first[1]) + (panel >= a.ws.first[2]);
                const int wpanel = panel - (wsel == 0 ? 0 : wsel == 1 ? a.ws.first[1] : a.ws.first[2]);
                const uint8_t *codes = wsel == 0 ? a.ws.codes[0] : wsel == 1 ? a.ws.codes[1] : a.ws.codes[2];
                const uint8_t *kmul = wsel == 0 ? a.ws.kmul[0] : wsel == 1 ? a.ws.kmul[1] : a.ws.kmul[2];
                const int32_t fl = wsel == 0 ? f0 : wsel == 1 ? f1 : f2;
                const uint8_t *pbase = codes + (size_t) wpanel * ng * 2048 + lane * 16;
                int tot = 0;
                for (int gi0 = 0; gi0 < gpw; gi0 += MG) {
                    // (the first groups of the first panel's first round are in flight since the kernel's start)
                    const bool first = pl == 0 && gi0 == 0;
#pragma unroll
                    for (int j = 0; j < MG; ++j) {
                        if (j < kEarly && first) continue;
                        int g = sw + (gi0 + j) * kStrWaves;
                        if (g >= ng) g = 0;   // past the end: the first group again, contributes nothing
                        w[j][0] = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(pbase + (size_t) g * 2048));
                        w[j][1] = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(pbase + (size_t) g * 2048 + 1024));
                    }
                    if (!waited) {
                        RQ_STAMP(2);
                        wait_count<true>(s_cnt, codes_ready);   // row in LDS, Sylvester passes, Paley, ranges, codes
                        waited = true;
                        RQ_STAMP(3);
                    }
                    // The activation words of a group are the same for all 64 rows. The wavefront's MG groups are
                    // MG x 8 code words and MG (m, z) words: fetched from LDS once, one word per lane, and handed to
                    // the dot products as scalars (v_readlane), so the fold of a group waits for no LDS round trip.
                    uint32_t aw[2];
                    int mzw;
                    {
                        const int gl = sw + (gi0 + (lane >> 3)) * kStrWaves, gh = sw + (gi0 + 8 + (lane >> 3)) * kStrWaves;
                        aw[0] = s_act[(gl < ng ? gl : 0) * 8 + (lane & 7)];
                        aw[1] = MG > 8 ? s_act[(gh < ng && lane < (MG - 8) * 8 ? gh : 0) * 8 + (lane & 7)] : 0u;
                        const int gm = sw + (gi0 + lane) * kStrWaves;
                        mzw = s_mz[gm < ng && lane < MG ? gm : 0];
                    }
#pragma unroll
                    for (int j = 0; j < MG; ++j) {
                        const int gq = sw + (gi0 + j) * kStrWaves;
                        const bool on = gq < ng;
                        const int g = on ? gq : 0;
                        uint32_t av[8];
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            av[i] = (uint32_t) __builtin_amdgcn_readlane((int) aw[(j * 8 + i) >> 6], (j * 8 + i) & 63);
                        }
                        const int mzv = __builtin_amdgcn_readlane(mzw, j);
                        int acc = 0, cs = 0;
                        acc = dot8(w[j][0].x, av[0], acc);
                        acc = dot8(w[j][0].y, av[1], acc);
                        acc = dot8(w[j][0].z, av[2], acc);
                        acc = dot8(w[j][0].w, av[3], acc);
                        acc = dot8(w[j][1].x, av[4], acc);
                        acc = dot8(w[j][1].y, av[5], acc);
                        acc = dot8(w[j][1].z, av[6], acc);
                        acc = dot8(w[j][1].w, av[7], acc);
                        cs = dot8(w[j][0].x, 0x11111111u, cs);
                        cs = dot8(w[j][0].y, 0x11111111u, cs);
                        cs = dot8(w[j][0].z, 0x11111111u, cs);
                        cs = dot8(w[j][0].w, 0x11111111u, cs);
                        cs = dot8(w[j][1].x, 0x11111111u, cs);
                        cs = dot8(w[j][1].y, 0x11111111u, cs);
                        cs = dot8(w[j][1].z, 0x11111111u, cs);
                        cs = dot8(w[j][1].w, 0x11111111u, cs);
                        // |acc|, |cs * (8 - z)| <= 4096 and m <= 255: 24-bit multiplies are exact
                        const int part = mad24_s((int) (int8_t) ((mzv >> 8) & 0xFF), cs, acc);
                        int term = __mul24(on ? (mzv & 0xFF) : 0, part);
                        if (fl & 1) term *= (int) kmul[((size_t) wpanel * ng + g) * kPanelRows + lane];
                        tot += term >> kTermShift;
                    }
                }
                atomicAdd(&red[pl * kPanelRows + lane], tot);
            }
        }

        // ---- remainder: lane = (row of the octet, half of the group, group of the item)
        if constexpr (MT > 0) {
            for (int i0 = 0; i0 < n_items || !waited; i0 += MT * kStrWaves) {
                if (i0 > 0) {
#pragma unroll
                    for (int it = 0; it < MT; ++it) {
                        const int i = i0 + sw + it * kStrWaves;
                        wt[it] = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(tail_address(i, i < n_items)));
                    }
                }
                if (!waited) {
                    RQ_STAMP(2);
                    wait_count<true>(s_cnt, codes_ready);
                    waited = true;
                    RQ_STAMP(3);
                }
#pragma unroll
                for (int it = 0; it < MT; ++it) {
                    const int iq = i0 + sw + it * kStrWaves;
                    const bool on = iq < n_items;
                    if (!on) break;   // (uniform over the wavefront; the items behind are past the end as well)
                    const int i = iq;
                    const int ol = (int) (((uint32_t) i * (uint32_t) a.inv_nblk) >> 22);
                    const int bb = i - ol * nblk;
                    const int g = 4 * bb + g4;
                    const uint4 av = *reinterpret_cast<const uint4 *>(s_act + g * 8 + 4 * h);
                    const int mzv = s_mz[g];
                    int acc = 0, cs = 0;
                    acc = dot8(wt[it].x, av.x, acc);
                    acc = dot8(wt[it].y, av.y, acc);
                    acc = dot8(wt[it].z, av.z, acc);
                    acc = dot8(wt[it].w, av.w, acc);
                    cs = dot8(wt[it].x, 0x11111111u, cs);
                    cs = dot8(wt[it].y, 0x11111111u, cs);
                    cs = dot8(wt[it].z, 0x11111111u, cs);
                    cs = dot8(wt[it].w, 0x11111111u, cs);
                    int part = mad24((int) (int8_t) ((mzv >> 8) & 0xFF), cs, acc);
                    // the other half of the group sits eight lanes away in the same row of 16 lanes
                    part += __builtin_amdgcn_update_dpp(0, part, 0x128 /* row_ror:8 */, 0xF, 0xF, false);
                    int term = __mul24(mzv & 0xFF, part);
                    if (anyk) {
                        // weight multipliers (a format variant): fetched here, behind the stream
                        const int o = oct0 + ol;
                        const int panel = o >> 3;
                        const int wsel = (panel >= a.ws.first[1]) + (panel >= a.ws.first[2]);
                        const int32_t fl = wsel == 0 ? f0 : wsel == 1 ? f1 : f2;
                        if (fl & 1) {
                            const int wpanel = panel - (wsel == 0 ? 0 : wsel == 1 ? a.ws.first[1] : a.ws.first[2]);
                            const uint8_t *kmul = wsel == 0 ? a.ws.kmul[0] : wsel == 1 ? a.ws.kmul[1] : a.ws.kmul[2];
                            term *= (int) kmul[((size_t) wpanel * ng + g) * kPanelRows + (o & 7) * 8 + r8];
                        }
                    }
                    term >>= kTermShift;
                    // rows of a shared octet that belong to the neighbour land in cells that nobody writes out; items
                    // past the end add nothing (a shared spare cell for them made all their lanes queue on one address)
                    if (h == 0 && on) atomicAdd(&red[main_cells + ol * 8 + r8], term);
                }
            }
        }
        RQ_STAMP(4);
        lds_barrier();   // all terms are in the cells
        RQ_STAMP(5);
    } else {
        // =========================================================== the activation side (512 threads)
        const int rt = tid;
        const int paley_pairs = a.syncs >> 8;
        int sync_target = 0;
        // the row (requested at the top of the kernel)
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        RQ_STAMP(1);
#pragma unroll
        for (int ub = 0; ub < kUnits; ++ub) {
            int u = rt + ub * kRotThreads;
            if (dpp256) u = (u & ~15) | unit_of_lane;
            if (u < (K >> 4)) {   // (whole DPP rows: K / 16 is a multiple of 16 when the chunks are 256 long)
                float v[16] = { qv[ub][0].x, qv[ub][0].y, qv[ub][0].z, qv[ub][0].w, qv[ub][1].x, qv[ub][1].y,
                                qv[ub][1].z, qv[ub][1].w, qv[ub][2].x, qv[ub][2].y, qv[ub][2].z, qv[ub][2].w,
                                qv[ub][3].x, qv[ub][3].y, qv[ub][3].z, qv[ub][3].w };
                if (a.rotate) {
                    // Sylvester stages with strides 1, 2, 4, 8 in registers (chunks are multiples of 16 floats)
#pragma unroll
                    for (int hh = 1; hh < 16; hh <<= 1) {
#pragma unroll
                        for (int j = 0; j < 16; ++j) {
                            if ((j & hh) == 0) {
                                const float lo = v[j], up = v[j + hh];
                                v[j] = lo + up;
                                v[j + hh] = lo - up;
                            }
                        }
                    }
                }
                if (dpp256) dpp_stages_256(v, du);   // strides 16 .. 128 between lanes
                float *d = buf + padi(16 * u);
#pragma unroll
                for (int j = 0; j < 16; ++j) d[j] = v[j];
            }
        }
        RQ_STAMP(8);
        rot_sync(s_cnt, sync_target, lane);
        RQ_STAMP(2);

        if (a.rotate) {
            const int m = a.m;
            const int lm = __ffs(m) - 1;
            {
                // the stages behind the ones done in registers (strides 1 .. 8) and between lanes (16 .. 128, for
                // chunks made of blocks of 256 floats), in ascending stride order through LDS
                for (int ls = dpp256 ? 8 : 4; ls < lm;) {
                    const int lr2 = lm - ls < 4 ? lm - ls : 4;
                    if (lr2 == 4) fwht_pass<4>(buf, K, lm, ls, rt, kRotThreads);
                    else if (lr2 == 3) fwht_pass<3>(buf, K, lm, ls, rt, kRotThreads);
                    else if (lr2 == 2) fwht_pass<2>(buf, K, lm, ls, rt, kRotThreads);
                    else fwht_pass<1>(buf, K, lm, ls, rt, kRotThreads);
                    ls += lr2;
                    rot_sync(s_cnt, sync_target, lane);
                }
            }
            RQ_STAMP(3);
            if constexpr (P > 1) {
                // Paley across the P chunks of every rotation block, into the second row buffer. A wave-item is
                // (slice of kOut outputs, run of 64 columns); the slice's sign pattern is straight-line code.
                constexpr int kOut = P / 4;
                constexpr int kSlices = 4;
                const int ncols = K / P;
                const int pm = m + (m >> 4);
                const int col_runs = (ncols + 63) >> 6;
                const int n_it = kSlices * col_runs;
                const int per_wave = (n_it + kRotWaves - 1) / kRotWaves;
                if (paley_pairs) {
                    // every wavefront has whole pairs of items: Paley sums, ranges and codes without leaving registers
                    int s = 0, cr = per_wave * wave;
                    while (cr >= col_runs) {
                        cr -= col_runs;
                        ++s;
                    }
                    if (paley_pairs == 1) {
                        paley_quantize<P, 1>(buf, s, cr, lane, wave, lm, m, a.n_rot, pm, a.scale, a.clip, s_part, s_unit,
                                             s_act, s_mz, s_cnt, sync_target, RQ_STAMP_PTR);
                    } else {
                        paley_quantize<P, 2>(buf, s, cr, lane, wave, lm, m, a.n_rot, pm, a.scale, a.clip, s_part, s_unit,
                                             s_act, s_mz, s_cnt, sync_target, RQ_STAMP_PTR);
                    }
                } else if (per_wave == 2 && (col_runs & 1) == 0 && (ncols & 63) == 0 && 2 * wave + 1 < n_it) {
                    // the wavefront's two items are neighbouring column runs of one slice: one instruction stream
                    // for both (whole row rotated as H20 x H256 or H12 x H256: 16 items for eight wavefronts)
                    int s = 0, cr = 2 * wave;
                    while (cr >= col_runs) {
                        cr -= col_runs;
                        ++s;
                    }
                    paley_pair<P>(buf, alt, s, cr, lane, lm, m, a.n_rot, pm, a.scale);
                } else if ((per_wave & 1) == 0 && col_runs % per_wave == 0 && (ncols & 63) == 0 &&
                           per_wave * (wave + 1) <= n_it) {
                    // four or eight items per wavefront (H12 x H512, H20 x H512: 32 items; H12 x H1024: 64): they are
                    // neighbouring column runs of one slice as well, taken two at a time (one at a time, K = 6144:
                    // 9.5 us for the call at N = 5120 against 8.9 us; four at a time: 8.8 us)
                    int s = 0, cr = per_wave * wave;
                    while (cr >= col_runs) {
                        cr -= col_runs;
                        ++s;
                    }
                    for (int pr = 0; pr < per_wave; pr += 2) paley_pair<P>(buf, alt, s, cr + pr, lane, lm, m, a.n_rot, pm, a.scale);
                } else
                for (int it = 0; it < per_wave; ++it) {
                    const int wi = wave * per_wave + it;
                    if (wi >= n_it) break;
                    int s = 0, cr = wi;   // wi / col_runs, wi % col_runs (a few uniform subtractions)
                    while (cr >= col_runs) {
                        cr -= col_runs;
                        ++s;
                    }
                    const int cidx = cr * 64 + lane;
                    if (cidx >= ncols) continue;
                    const int rb = cidx >> lm, j = cidx & (m - 1);   // chunk lengths are powers of two
                    const int b0 = rb * a.n_rot + j;
                    const float *src = buf + padi(b0);
                    float out[kOut];
                    if (m == 256) {
                        // chunks of 256: the chunk stride in the padded row is the constant 272, so the P loads are
                        // immediate offsets from one address
                        paley_pick_stream<P, kOut, 272>(s, src, 272, out);
                    } else {
                        paley_pick_stream<P, kOut, 0>(s, src, pm, out);
                    }
                    float *dst = alt + b0 + kOut * s * m;
#pragma unroll
                    for (int o = 0; o < kOut; ++o) dst[o * m] = out[o] * a.scale;
                }
                if (!paley_pairs) {
                    RQ_STAMP(9);
                    rot_sync(s_cnt, sync_target, lane);
                }
            } else {
                for (int i = rt; i < K; i += kRotThreads) buf[padi(i)] = buf[padi(i)] * a.scale;
                rot_sync(s_cnt, sync_target, lane);
            }
        }

        // ---- group ranges, the token's unit, multipliers, zero points and codes (quantize_rounds), with the number
        // of code words per thread as a compile-time constant
        if (!(P > 1 && a.rotate && paley_pairs)) {
            RQ_STAMP(4);
            const int nw = K >> 3;
            const bool dense = a.rotate && P > 1;            // the Paley stage wrote the dense buffer
            const float *row = dense ? alt : buf;
            switch ((nw + kRotThreads - 1) / kRotThreads) {   // K <= 16384: at most four words per thread
            case 1: quantize_rounds<1>(row, dense, nw, a.clip, rt, lane, wave, s_part, s_unit, s_act, s_mz, s_cnt, sync_target, RQ_STAMP_PTR); break;
            case 2: quantize_rounds<2>(row, dense, nw, a.clip, rt, lane, wave, s_part, s_unit, s_act, s_mz, s_cnt, sync_target, RQ_STAMP_PTR); break;
            case 3: quantize_rounds<3>(row, dense, nw, a.clip, rt, lane, wave, s_part, s_unit, s_act, s_mz, s_cnt, sync_target, RQ_STAMP_PTR); break;
            default: quantize_rounds<4>(row, dense, nw, a.clip, rt, lane, wave, s_part, s_unit, s_act, s_mz, s_cnt, sync_target, RQ_STAMP_PTR); break;
            }
        }
        rot_sync(s_cnt, sync_target, lane);   // codes, multipliers and unit are in LDS: the stream folds
        RQ_STAMP(6);
        lds_barrier();   // ... and has finished
        RQ_STAMP(7);
    }

    // ---- epilogue (reference line 176): three fp32 multiplies in the reference's order
    if (y_row != nullptr) *y_row = (((float) red[tid] * 16.0f) * s_unit[0]) * pre_sw;
    RQ_STAMP_FLUSH;
}

template <int P, int MG, int MT>
hipError_t launch_pmt(const DecodeKernelArgs &k, int grid, size_t lds, hipStream_t stream) {
    static bool attr_set = false;   // (also done per device by init_decode_kernels)
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&rq_decode_kernel<P, MG, MT>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 64);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    hipLaunchKernelGGL((rq_decode_kernel<P, MG, MT>), dim3(grid), dim3(kDecThreads), lds, stream, k);
    return hipGetLastError();
}

// whole panels: 10 groups per wavefront and round cover K = 5120 in one round (12: K = 6144); the remainder gets 4
// items per wavefront and round beside whole panels, 12 to 26 (the smallest even count that holds them) when the launch is
// remainder only
template <int P>
hipError_t launch_p(const DecodeKernelArgs &k, int grid, size_t lds, hipStream_t stream) {
    if (k.main_panels == 0) {
        // remainder only: all of a wavefront's items in flight when they are at most 26
        // most octets that a workgroup's run of quads touches (a run that starts or ends inside an octet shares it)
        int octets = 0;
        for (int s = 0; s < grid; ++s) {
            const int q0 = s * k.q_base + (s < k.q_extra ? s : k.q_extra), q1 = q0 + k.q_base + (s < k.q_extra ? 1 : 0);
            const int n = q1 > q0 ? ((q1 + 1) >> 1) - (q0 >> 1) : 0;
            if (n > octets) octets = n;
        }
        const int per_wave = (octets * (k.K / 256) + kStrWaves - 1) / kStrWaves;
        // The smallest form that holds them all: a slot too few is a second round of loads behind the first round's
        // fold (K = 5120, N = 11264, 15 items: 8.4 -> 10.2 us with 14 slots), and every slot too many costs 0.1 us
        // (N = 8192, 10 items: 6.9 us with 12 slots, 9.1 us with 26).
        if (per_wave > 24) return launch_pmt<P, 0, 26>(k, grid, lds, stream);
        if (per_wave > 22) return launch_pmt<P, 0, 24>(k, grid, lds, stream);
        if (per_wave > 20) return launch_pmt<P, 0, 22>(k, grid, lds, stream);
        if (per_wave > 18) return launch_pmt<P, 0, 20>(k, grid, lds, stream);
        if (per_wave > 16) return launch_pmt<P, 0, 18>(k, grid, lds, stream);
        if (per_wave > 14) return launch_pmt<P, 0, 16>(k, grid, lds, stream);
        if (per_wave > 12) return launch_pmt<P, 0, 14>(k, grid, lds, stream);
        return launch_pmt<P, 0, 12>(k, grid, lds, stream);
    }
    const int gpw = (k.K / kGroup + kStrWaves - 1) / kStrWaves;
    const bool tail = k.q_base > 0 || k.q_extra > 0;
    if (gpw % 12 == 0 || (gpw % 10 != 0 && gpw > 10)) {
        return tail ? launch_pmt<P, 12, 2>(k, grid, lds, stream) : launch_pmt<P, 12, 0>(k, grid, lds, stream);
    }
    return tail ? launch_pmt<P, 10, 4>(k, grid, lds, stream) : launch_pmt<P, 10, 0>(k, grid, lds, stream);
}

template <int P, int MG, int MT>
hipError_t allow_lds() {
    return hipFuncSetAttribute(reinterpret_cast<const void *>(&rq_decode_kernel<P, MG, MT>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 64);
}

template <int P>
hipError_t allow_lds_p() {
    hipError_t e = allow_lds<P, 0, 12>();
    if (e == hipSuccess) e = allow_lds<P, 0, 14>();
    if (e == hipSuccess) e = allow_lds<P, 0, 16>();
    if (e == hipSuccess) e = allow_lds<P, 0, 18>();
    if (e == hipSuccess) e = allow_lds<P, 0, 20>();
    if (e == hipSuccess) e = allow_lds<P, 0, 22>();
    if (e == hipSuccess) e = allow_lds<P, 0, 24>();
    if (e == hipSuccess) e = allow_lds<P, 0, 26>();
    if (e == hipSuccess) e = allow_lds<P, 10, 4>();
    if (e == hipSuccess) e = allow_lds<P, 10, 0>();
    if (e == hipSuccess) e = allow_lds<P, 12, 2>();
    if (e == hipSuccess) e = allow_lds<P, 12, 0>();
    return e;
}

}  // namespace

hipError_t init_decode_kernels() {
    hipError_t e = allow_lds_p<1>();
    if (e == hipSuccess) e = allow_lds_p<12>();
    if (e == hipSuccess) e = allow_lds_p<20>();
    return e;
}

// Which one-token problems the single-launch kernel takes: activation groups of 64, a rotation with a short Paley
// stage whose chunks are multiples of 16 floats (or no rotation), and a row that fits LDS twice.
bool decode_takes(int K, int rotate, int p, int m, int act_group) {
    if (act_group != kGroup) return false;
    if (K > 16384) return false;
    if (rotate) {
        // Long Paley stages stay with the rotation kernel that spreads a token over many workgroups: H68 x H256
        // (K = 17408) is 1.2 M additions per token, which one workgroup's eight wavefronts need 14 us for (measured:
        // 28 us for the whole call against 17.5 us with the two launches).
        if (p != 1 && p != 12 && p != 20) return false;
        if ((m & 15) != 0) return false;
    }
    return decode_lds_bytes(K, rotate && p > 1) <= 160 * 1024 - 64;
}

hipError_t launch_decode(const DecodeArgs &d, hipStream_t stream) {
    DecodeKernelArgs k;
    k.ws = make_weight_set(d.w);
    k.x = d.x;
    k.K = d.K;
    k.rotate = d.rotate;
    k.n_rot = d.n_rot;
    k.m = d.m;
    k.scale = d.scale;
    k.clip = d.clip;
    k.inv_nblk = (1 << 22) / (d.K / 256) + 1;
    const int lm = d.rotate ? __builtin_ctz((unsigned) d.m) : 0;
    // stages through LDS: those above stride 8, or above stride 128 when the chunks are whole blocks of 256 floats
    // (four more stages then run between lanes)
    const int lm0 = d.rotate && (d.m & 255) == 0 ? 8 : 4;
    const int n_pass = d.rotate && lm > lm0 ? (lm - lm0 + 3) / 4 : 0;   // Sylvester passes through LDS after the register pass
    int paley_pairs = 0;
    if (d.rotate && d.p > 1 && d.K % d.p == 0) {
        // the Paley items (4 slices x runs of 64 columns) deal out as one or two whole pairs of neighbouring runs to
        // each of the eight rotate wavefronts: H20 x H256, H12 x H256 (one pair), H12 x H512, H20 x H512 (two)
        const int ncols = d.K / d.p, col_runs = ncols / 64, n_it = 4 * col_runs;
        const int per_wave = n_it / kRotWaves;
        if ((ncols & 63) == 0 && (d.m & 63) == 0 && n_it == per_wave * kRotWaves && (per_wave == 2 || per_wave == 4) &&
            col_runs % per_wave == 0 && (d.m / 64) % per_wave == 0) {   // (a wavefront's runs lie in one rotation block)
            paley_pairs = per_wave / 2;
        }
    }
    // meetings: row in LDS, the Sylvester passes, Paley (or the scale) unless the sums stay in registers, ranges, codes
    k.syncs = (1 + n_pass + (d.rotate && !paley_pairs ? 1 : 0) + 2) | paley_pairs << 8;
    const int n_panels = k.ws.first[kMaxFused];
    // one workgroup per compute unit: whole panels as far as they go round, the remainder in quads of rows. More
    // workgroups (a multiple of the compute units) only when the rows of one would not fit its LDS cells.
    const int cus = d.compute_units > 0 ? d.compute_units : 256;
    int grid = cus;
    for (;;) {
        const int mp = n_panels / grid;
        const int tail_quads = (n_panels - mp * grid) * 16;
        const int octets = tail_quads ? (tail_quads + grid - 1) / grid / 2 + 2 : 0;
        if (mp * kPanelRows + octets * 8 <= kDecodeCells) break;
        grid += cus;
    }
    if (grid > n_panels * 16) grid = n_panels * 16;
    // Fewer panels than compute units, but most of them: one whole panel per workgroup on n_panels compute units and
    // the others idle. A panel streams as contiguous KiB with the lane as the row; rows dealt in quads over all
    // compute units are read as 128-byte pieces, and that form loses from about 55 % of the compute units on
    // (K = 5120: N = 8192 6.9 us in quads, 7.4 us in panels; N = 10240 7.7 and 7.55; N = 12288 8.5 and 8.0; N = 15360
    // 10.3 and 8.6; N = 16320 10.7 and 8.9; K = 4096, where the panel is shorter: N = 12288 7.5 and 7.7).
    if (grid == cus && n_panels < cus && n_panels * 8 >= cus * (d.K >= 5120 ? 5 : 7)) grid = n_panels;
    k.main_panels = n_panels / grid;
    k.tail_panel0 = k.main_panels * grid;
    const int tail_quads = (n_panels - k.tail_panel0) * 16;
    k.q_base = tail_quads / grid;
    k.q_extra = tail_quads % grid;
    const size_t lds = decode_lds_bytes(d.K, d.rotate && d.p > 1);
    switch (d.rotate ? d.p : 1) {
        case 1:  return launch_p<1>(k, grid, lds, stream);
        case 12: return launch_p<12>(k, grid, lds, stream);
        case 20: return launch_p<20>(k, grid, lds, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace rq
