// Building blocks of the online Hadamard shared by the activation kernels: the Paley sign table and its unrolled
// column sums, the register butterflies of the Sylvester transform, the padded LDS row.
#pragma once

#include "rq_common.h"

#pragma clang fp contract(off)

namespace rq {
namespace had {

// ---- Paley construction I, as signs: neg[i][a] is true where A[i][a] = -1 (reference lines 2433-2448) ----
template <int P>
struct PaleyTable {
    bool neg[P][P];
};

template <int P>
constexpr PaleyTable<P> make_paley() {
    PaleyTable<P> t{};
    constexpr int q = P - 1;
    bool residue[P] = {};
    for (int r = 1; r < q; ++r) residue[(r * r) % q] = true;
    for (int i = 0; i < P; ++i) {
        for (int a = 0; a < P; ++a) {
            bool n = false;
            if (i == a || i == 0) {
                n = false;                       // diagonal and first row are +1
            } else if (a == 0) {
                n = true;                        // first column below the diagonal is -1
            } else {
                n = !residue[(((a - i) % q) + q) % q];
            }
            t.neg[i][a] = n;
        }
    }
    return t;
}

// outputs 4S .. 4S+3 of one column: acc = ((0 +- c0) +- c1) ... in ascending chunk order. TR takes the signs of the
// transposed matrix (A[a][i] instead of A[i][a], reference line 2476): the inverse rotation of the dequantizers.
template <int P, int S, bool TR = false>
__device__ __forceinline__ void paley_slice(const float (&col)[P], float (&out)[4]) {
    constexpr PaleyTable<P> T = make_paley<P>();
#pragma unroll
    for (int o = 0; o < 4; ++o) {
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < P; ++i) {
            acc = (TR ? T.neg[4 * S + o][i] : T.neg[i][4 * S + o]) ? acc - col[i] : acc + col[i];
        }
        out[o] = acc;
    }
}

// outputs O * s .. O * s + O - 1 of one column, s uniform over the wavefront: the straight-line code of slice s
template <int P, int O, int S = 0>
__device__ __forceinline__ void paley_pick(int s, const float (&col)[P], float (&out)[O]) {
    if (s == S) {
        constexpr PaleyTable<P> T = make_paley<P>();
#pragma unroll
        for (int o = 0; o < O; ++o) {
            float acc = 0.0f;
#pragma unroll
            for (int i = 0; i < P; ++i) {
                acc = T.neg[i][O * S + o] ? acc - col[i] : acc + col[i];
            }
            out[o] = acc;
        }
    } else if constexpr (S + 1 < P / O) {
        paley_pick<P, O, S + 1>(s, col, out);
    }
}

// The same outputs with the column read on the fly (element i of the column at src[i * stride]): the loop runs over
// the column's elements and updates the O running sums, so every sum still receives its terms in ascending chunk
// order, one rounding per term, and a long column needs O + 1 registers instead of P.
template <int P, int O, int STRIDE, int S = 0>
__device__ __forceinline__ void paley_pick_stream(int s, const float *src, int stride, float (&out)[O]) {
    if (s == S) {
        constexpr PaleyTable<P> T = make_paley<P>();
#pragma unroll
        for (int o = 0; o < O; ++o) out[o] = 0.0f;
#pragma unroll
        for (int i = 0; i < P; ++i) {
            const float c = src[i * (STRIDE ? STRIDE : stride)];
#pragma unroll
            for (int o = 0; o < O; ++o) out[o] = T.neg[i][O * S + o] ? out[o] - c : out[o] + c;
        }
    } else if constexpr (S + 1 < P / O) {
        paley_pick_stream<P, O, STRIDE, S + 1>(s, src, stride, out);
    }
}

// The same for two columns at once (two runs of 64 columns of one slice): twice the independent sums per
// instruction stream, which is what hides the latency of the dependent additions and of the LDS reads when a
// wavefront has only two items.
template <int P, int O, int STRIDE, int S = 0>
__device__ __forceinline__ void paley_pick_stream2(int s, const float *src0, const float *src1, int stride,
                                                   float (&out0)[O], float (&out1)[O]) {
    if (s == S) {
        constexpr PaleyTable<P> T = make_paley<P>();
#pragma unroll
        for (int o = 0; o < O; ++o) {
            out0[o] = 0.0f;
            out1[o] = 0.0f;
        }
#pragma unroll
        for (int i = 0; i < P; ++i) {
            const float c0 = src0[i * (STRIDE ? STRIDE : stride)];
            const float c1 = src1[i * (STRIDE ? STRIDE : stride)];
#pragma unroll
            for (int o = 0; o < O; ++o) {
                out0[o] = T.neg[i][O * S + o] ? out0[o] - c0 : out0[o] + c0;
                out1[o] = T.neg[i][O * S + o] ? out1[o] - c1 : out1[o] + c1;
            }
        }
    } else if constexpr (S + 1 < P / O) {
        paley_pick_stream2<P, O, STRIDE, S + 1>(s, src0, src1, stride, out0, out1);
    }
}

// all P outputs of one column, written back in place (the column is private to the calling thread). STRIDE is the
// distance between the chunks of a column in the padded row when it is known at compile time (0: use `stride`): the
// P loads and P stores then share one or two address registers with immediate offsets, where a run-time stride costs
// an address register per element, which for long columns is what spills.
template <int P, int S = 0, bool TR = false, int STRIDE = 0>
__device__ __forceinline__ void paley_column(const float (&col)[P], float *dst, int stride, float scale) {
    float out[4];
    paley_slice<P, S, TR>(col, out);
#pragma unroll
    for (int o = 0; o < 4; ++o) dst[(4 * S + o) * (STRIDE ? STRIDE : stride)] = out[o] * scale;
    if constexpr (S + 1 < P / 4) paley_column<P, S + 1, TR, STRIDE>(col, dst, stride, scale);
}

template <int P, int STRIDE>
__device__ __forceinline__ void load_column(float (&col)[P], const float *src, int stride) {
#pragma unroll
    for (int i = 0; i < P; ++i) col[i] = src[i * (STRIDE ? STRIDE : stride)];
}

// same, for chunk lengths that are not a multiple of 16 (the padded stride is then not uniform)
template <int P, int S = 0, bool TR = false>
__device__ __forceinline__ void paley_column_generic(const float (&col)[P], float *buf, int b0, int m, float scale) {
    float out[4];
    paley_slice<P, S, TR>(col, out);
#pragma unroll
    for (int o = 0; o < 4; ++o) {
        const int i = b0 + (4 * S + o) * m;
        buf[i + (i >> 4)] = out[o] * scale;
    }
    if constexpr (S + 1 < P / 4) paley_column_generic<P, S + 1, TR>(col, buf, b0, m, scale);
}

// Wavefront-wide max / min, the same value in every lane. The steps are DPP lane permutations (swap within pairs,
// within quads, mirror the half rows, mirror the rows of 16, then carry across rows), which run at vector-ALU speed;
// six dependent LDS-crossbar permutes would cost several hundred cycles each time, and the rotation kernels reduce
// once per activation group.
// Each step is ONE instruction, v_max_f32 / v_min_f32 with the permutation on its first operand, written as
// assembly: from fmaxf(v, permuted v) the compiler makes four (a copy, the permutation as a move of its own, a
// v_max_f32 x, x, x that quiets a signalling NaN, the max), because the language-level maximum is defined on quieted
// operands. The instruction itself returns the other operand when one is a NaN, as fmaxf does. The s_nop in front is
// the two wait states a DPP operand needs behind the vector instruction that wrote it (the compiler does not look
// inside the assembly).
// The operand is tied to the result: a lane whose partner is switched off, and the rows that a row mask leaves out,
// keep their value.
#define RQ_DPP_MINMAX_ROWS(v, ctrl, rows)                                                                        \
    {                                                                                                            \
        if (MAX) asm("s_nop 1\n\tv_max_f32_dpp %0, %0, %0 " ctrl " row_mask:" rows " bank_mask:0xf" : "+v"(v));   \
        else     asm("s_nop 1\n\tv_min_f32_dpp %0, %0, %0 " ctrl " row_mask:" rows " bank_mask:0xf" : "+v"(v));   \
    }
#define RQ_DPP_MINMAX(v, ctrl) RQ_DPP_MINMAX_ROWS(v, ctrl, "0xf")
template <bool MAX>
__device__ __forceinline__ float wave_reduce(float v) {
    RQ_DPP_MINMAX(v, "quad_perm:[1,0,3,2]")
    RQ_DPP_MINMAX(v, "quad_perm:[2,3,0,1]")
    RQ_DPP_MINMAX(v, "row_half_mirror")
    RQ_DPP_MINMAX(v, "row_mirror")                    // every lane of a row now holds the row's value
    RQ_DPP_MINMAX_ROWS(v, "row_bcast:15", "0xa")      // into rows 1 and 3
    RQ_DPP_MINMAX_ROWS(v, "row_bcast:31", "0xc")      // into rows 2 and 3: lane 63 holds the wavefront's value
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
// min / max of three as the one instruction, for operands that come straight from memory (the compiler would quiet
// each of them first, an instruction per operand)
__device__ __forceinline__ float min3_raw(float a, float b, float c) {
    float r;
    asm("v_min3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
// min(lo, v[0..7]) and max(hi, v[0..7])
__device__ __forceinline__ void minmax8_raw(const float (&v)[8], float &lo, float &hi) {
    lo = min3_raw(min3_raw(lo, v[0], v[1]), min3_raw(v[2], v[3], v[4]), min3_raw(v[5], v[6], v[7]));
    hi = max3_raw(max3_raw(hi, v[0], v[1]), max3_raw(v[2], v[3], v[4]), max3_raw(v[5], v[6], v[7]));
}
// max / min over aligned runs of eight lanes, the same value in all eight
template <bool MAX>
__device__ __forceinline__ float group8_reduce(float v) {
    RQ_DPP_MINMAX(v, "quad_perm:[1,0,3,2]")
    RQ_DPP_MINMAX(v, "quad_perm:[2,3,0,1]")
    RQ_DPP_MINMAX(v, "row_half_mirror")   // lane i of a half row takes lane 7 - i, which sits in the other quad
    return v;
}
#undef RQ_DPP_MINMAX
#undef RQ_DPP_MINMAX_ROWS
__device__ __forceinline__ float wave_max(float v) { return wave_reduce<true>(v); }
__device__ __forceinline__ float wave_min(float v) { return wave_reduce<false>(v); }

// The row sits in LDS with one float of padding after every 16: element i lives at i + i / 16. With it the
// strided accesses of the register butterflies (16 elements 16, 256, ... apart) spread over all banks.
__device__ __forceinline__ int padi(int i) { return i + (i >> 4); }

// One pass of the Sylvester transform: R = 2^LR elements `1 << ls` apart go through LR butterfly stages in
// registers (strides 1 << ls, 2 << ls, ...; lower index gets a + b, upper a - b, as reference lines 2454-2464).
// Successive passes run in ascending stride order, so every element sees the reference's stage order.
template <int LR>
__device__ __forceinline__ void fwht_pass(float *buf, int K, int lm, int ls, int tid, int nt) {
    constexpr int R = 1 << LR;
    const int units = K >> LR;
    for (int u = tid; u < units; u += nt) {
        const int c = u >> (lm - LR), ul = u & ((1 << (lm - LR)) - 1);
        const int low = ul & ((1 << ls) - 1), high = ul >> ls;
        const int base = (c << lm) + ((high << (ls + LR)) | low);
        float v[R];
#pragma unroll
        for (int j = 0; j < R; ++j) v[j] = buf[padi(base + (j << ls))];
#pragma unroll
        for (int h = 1; h < R; h <<= 1) {
#pragma unroll
            for (int j = 0; j < R; ++j) {
                if ((j & h) == 0) {
                    const float lo = v[j], up = v[j + h];
                    v[j] = lo + up;
                    v[j + h] = lo - up;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < R; ++j) buf[padi(base + (j << ls))] = v[j];
    }
}


// Eight consecutive values of one activation group -> the two int8 digit words pairs of the MFMA operand layout.
// q = clamp(rint(x * inv) + zf, 0, 15) as the reference computes it (patch lines 2670-2675); p = m (q - z), |p| <= 3825,
// is formed in fp32 (small integers: exact) and split into balanced digits p = 64 hi + lo, lo in [-32, 31]. Bytes go
// in the order the weight unpack yields: the even values of the word (`*_e`), then the odd ones (`*_o`); v_perm_b32
// gathers four low bytes in three instructions.
__device__ __forceinline__ uint32_t pack_low_bytes(int x0, int x1, int x2, int x3) {
    const uint32_t t0 = __builtin_amdgcn_perm((uint32_t) x1, (uint32_t) x0, 0x0c0c0400u);
    const uint32_t t1 = __builtin_amdgcn_perm((uint32_t) x3, (uint32_t) x2, 0x0c0c0400u);
    return __builtin_amdgcn_perm(t1, t0, 0x05040100u);
}

__device__ __forceinline__ void digits_of_word(const float (&f)[8], float inv, float zf, float mgf, uint32_t &lo_e,
                                               uint32_t &lo_o, uint32_t &hi_e, uint32_t &hi_o) {
    int lo[8], hi[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float q = fminf(fmaxf(rintf(f[j] * inv) + zf, 0.0f), 15.0f);
        const int p = (int) ((q - zf) * mgf);
        hi[j] = (p + 32) >> 6;
        lo[j] = p - (hi[j] << 6);
    }
    lo_e = pack_low_bytes(lo[0], lo[2], lo[4], lo[6]);
    lo_o = pack_low_bytes(lo[1], lo[3], lo[5], lo[7]);
    hi_e = pack_low_bytes(hi[0], hi[2], hi[4], hi[6]);
    hi_o = pack_low_bytes(hi[1], hi[3], hi[5], hi[7]);
}

// Single-plane form: the bytes are q - z (-15 .. 15); the group multiplier travels beside the plane.
__device__ __forceinline__ void qz_of_word(const float (&f)[8], float inv, float zf, uint32_t &even, uint32_t &odd) {
    int d[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) d[j] = (int) (fminf(fmaxf(rintf(f[j] * inv) + zf, 0.0f), 15.0f) - zf);
    even = pack_low_bytes(d[0], d[2], d[4], d[6]);
    odd = pack_low_bytes(d[1], d[3], d[5], d[7]);
}

// Workgroup barrier for data that travels through LDS only: waits for this wavefront's LDS operations, not for its
// outstanding global loads (which __syncthreads() would also drain, stalling a kernel that keeps weight loads in
// flight across its prologue).
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// One row of K floats (K % 4 == 0) from global memory into the padded LDS row. All of a batch's loads are issued
// before the first LDS store: the row of a long K is several trips to memory per thread, and taken one at a time
// each trip would cost a full memory latency.
template <int NT>
__device__ __forceinline__ void load_row(float *buf, const float *__restrict__ xr, int K, int tid) {
    constexpr int kBatch = 8;
    for (int i0 = tid * 4; i0 < K; i0 += NT * 4 * kBatch) {
        float4 v[kBatch] = {};
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int i = i0 + b * NT * 4;
            if (i < K) v[b] = *reinterpret_cast<const float4 *>(xr + i);
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int i = i0 + b * NT * 4;
            if (i < K) {
                float *d = buf + padi(i);      // i % 4 == 0: the four land in one run of 16
                d[0] = v[b].x;
                d[1] = v[b].y;
                d[2] = v[b].z;
                d[3] = v[b].w;
            }
        }
    }
}

// The row from global memory through the first four Sylvester stages (strides 1, 2, 4, 8; chunks of at least 16
// floats) into the padded LDS row: a thread takes 16 consecutive floats, so the stages run in registers on the way in
// and the row makes one trip through LDS less (worth 10-15 % of the kernel for one token and for thousands).
// BATCH units per thread are requested before the first is worked on: a long row is several units per thread, and
// taken one at a time each would cost a full trip to memory.
template <int NT, int BATCH = 1>
__device__ __forceinline__ void load_row_fwht16(float *buf, const float *__restrict__ xr, int K, int tid) {
    for (int u0 = tid; u0 < (K >> 4); u0 += NT * BATCH) {
        float4 q[BATCH][4];
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            const int u = u0 + b * NT;
            if (u < (K >> 4)) {
                const float4 *src = reinterpret_cast<const float4 *>(xr + 16 * u);
#pragma unroll
                for (int j = 0; j < 4; ++j) q[b][j] = src[j];
            }
        }
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            const int u = u0 + b * NT;
            if (u >= (K >> 4)) break;
            float v[16] = { q[b][0].x, q[b][0].y, q[b][0].z, q[b][0].w, q[b][1].x, q[b][1].y, q[b][1].z, q[b][1].w,
                            q[b][2].x, q[b][2].y, q[b][2].z, q[b][2].w, q[b][3].x, q[b][3].y, q[b][3].z, q[b][3].w };
#pragma unroll
            for (int h = 1; h < 16; h <<= 1) {
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    if ((j & h) == 0) {
                        const float lo = v[j], up = v[j + h];
                        v[j] = lo + up;
                        v[j + h] = lo - up;
                    }
                }
            }
            float *d = buf + padi(16 * u);   // a run of 16 is contiguous in the padded row
#pragma unroll
            for (int j = 0; j < 16; ++j) d[j] = v[j];
        }
    }
}

// One Sylvester stage between lanes: `ctrl` swaps every lane with its partner (the lane whose unit differs in the
// stage's index bit); the lane of the lower unit gets a + b, the upper one a - b with a the lower unit's value
// (reference lines 2454-2464). t - v is formed as t + (-v): the same IEEE operation.
template <int CTRL>
__device__ __forceinline__ void dpp_stage(float (&v)[16], uint32_t upper_sign) {
    // (all sign flips first: taken value by value, every sum waited out the two wait states that an instruction with a
    // lane permutation needs behind the write of any of its operands)
    float sv[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) sv[j] = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v[j]) ^ upper_sign);
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const float t = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v[j]), CTRL,
                                                                              0xF, 0xF, false));
        v[j] = t + sv[j];
    }
}

// The unit of 16 floats that lane `lane` of a DPP row of 16 lanes takes when the row holds one block of 256 floats: the
// unit whose index bits (b0, b1, b2, b3) give lane = b0 ^ 2 b1 ^ 7 b2 ^ 8 b3, so that the partners of the stages with
// strides 16, 32, 64, 128 are lane ^ 1, ^ 2, ^ 7, ^ 8: quad_perm, quad_perm, row_half_mirror and row_ror:8.
struct DppUnit {
    int unit;                 // 0 .. 15: the unit within the block of 256 floats
    uint32_t s16, s32, s64, s128;   // sign bit of the lane's own value in each stage (set: upper partner, takes a - b)
};
__device__ __forceinline__ DppUnit dpp_unit_of_lane(int lane) {
    const int lr = lane & 15;
    const int hb3 = lr >> 3, hr = lr & 7, hb2 = hr >> 2, hr2 = hr ^ (hb2 ? 7 : 0);
    DppUnit d;
    d.unit = (hr2 & 1) | (hr2 & 2) | hb2 << 2 | hb3 << 3;
    d.s16 = (uint32_t) (hr2 & 1) << 31;
    d.s32 = (uint32_t) ((hr2 >> 1) & 1) << 31;
    d.s64 = (uint32_t) hb2 << 31;
    d.s128 = (uint32_t) hb3 << 31;
    return d;
}
// stages with strides 16 .. 128 of a block of 256 floats held by the 16 lanes of a DPP row, 16 values per lane
__device__ __forceinline__ void dpp_stages_256(float (&v)[16], const DppUnit &d) {
    dpp_stage<0xB1>(v, d.s16);     // quad_perm [1, 0, 3, 2]
    dpp_stage<0x4E>(v, d.s32);     // quad_perm [2, 3, 0, 1]
    dpp_stage<0x141>(v, d.s64);    // row_half_mirror
    dpp_stage<0x128>(v, d.s128);   // row_ror:8
}

// load_row_fwht16 for rows whose chunks are made of blocks of 256 floats (K is then a multiple of 256 and NT a multiple
// of 64, so the 16 lanes of a DPP row are in or out of every round together): eight stages on the way in, four in
// registers and four between lanes, and the row makes two trips through LDS less.
template <int NT, int BATCH = 1>
__device__ __forceinline__ void load_row_fwht256(float *buf, const float *__restrict__ xr, int K, int tid) {
    const DppUnit d = dpp_unit_of_lane(tid & 63);
    for (int u0 = tid; u0 < (K >> 4); u0 += NT * BATCH) {
        float4 q[BATCH][4];
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            const int u = ((u0 + b * NT) & ~15) | d.unit;
            if (u < (K >> 4)) {
                const float4 *src = reinterpret_cast<const float4 *>(xr + 16 * u);
#pragma unroll
                for (int j = 0; j < 4; ++j) q[b][j] = src[j];
            }
        }
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            const int u = ((u0 + b * NT) & ~15) | d.unit;
            if (u >= (K >> 4)) break;
            float v[16] = { q[b][0].x, q[b][0].y, q[b][0].z, q[b][0].w, q[b][1].x, q[b][1].y, q[b][1].z, q[b][1].w,
                            q[b][2].x, q[b][2].y, q[b][2].z, q[b][2].w, q[b][3].x, q[b][3].y, q[b][3].z, q[b][3].w };
#pragma unroll
            for (int h = 1; h < 16; h <<= 1) {
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    if ((j & h) == 0) {
                        const float lo = v[j], up = v[j + h];
                        v[j] = lo + up;
                        v[j + h] = lo - up;
                    }
                }
            }
            dpp_stages_256(v, d);
            float *dd = buf + padi(16 * u);
#pragma unroll
            for (int j = 0; j < 16; ++j) dd[j] = v[j];
        }
    }
}

// all Sylvester stages from stride 1 << ls0 up of every chunk of m = 1 << lm floats of a padded row, four stages per
// trip through LDS
__device__ __forceinline__ void fwht_row(float *buf, int K, int lm, int tid, int nt, int ls0 = 0) {
    for (int ls = ls0; ls < lm;) {
        const int lr = lm - ls < 4 ? lm - ls : 4;
        if (lr == 4) fwht_pass<4>(buf, K, lm, ls, tid, nt);
        else if (lr == 3) fwht_pass<3>(buf, K, lm, ls, tid, nt);
        else if (lr == 2) fwht_pass<2>(buf, K, lm, ls, tid, nt);
        else fwht_pass<1>(buf, K, lm, ls, tid, nt);
        ls += lr;
        __syncthreads();
    }
}

}  // namespace had
}  // namespace rq
