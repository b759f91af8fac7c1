// Online Hadamard (Paley x Sylvester) and per-token asymmetric int4 activation quantizer for gfx950.
//
// One workgroup owns one token: the whole row (up to 32768 floats) lives in the CU's 160 KiB LDS from the
// global load to the last code word, so the rotated activations never travel through HBM.
//
// Bit-exactness with the CPU reference (ggml_rq_hadamard, reference patch lines 2450-2485, and
// rq_quantize_row_a, lines 2639-2679) rests on three rules that this file keeps:
//   * Sylvester stages are exact pairs (a + b, a - b), stride ascending; which lane computes a pair is free, so
//     four stages at a time run in registers (16 elements per thread) between two trips through LDS.
//   * The Paley stage adds the p chunk values of a column strictly in ascending chunk order, starting from
//     +0.0f, one rounding per add; the signs are compile-time constants so each term is one v_add / v_sub.
//   * Every product, sum and quotient of the quantizer is a separate correctly rounded fp32 operation
//     (no contraction, IEEE division, denormals kept).
#include "rq_hadamard.h"

#pragma clang fp contract(off)

namespace rq {

namespace {

// Threads per token workgroup. Small batches (the sliced variant) with a short Paley stage get 1024: there the kernel
// is one workgroup per compute unit at most, bound by the latency of its own phases, and twice the threads halve the
// work per phase. Long Paley stages keep their columns in registers and need the 256-register budget of 512 threads.
template <int P, bool SLICED>
constexpr int threads_of() { return SLICED && P < 44 ? 1024 : 512; }

using namespace had;

template <int P, bool SLICED, bool ALONE = false>
// Registers are capped so that two workgroups (p >= 44: long columns, long rows) or three fit a compute unit: the
// stages of one token are separated by barriers, and it is the other workgroups that keep the vector ALU busy. (The
// sliced variant serves small batches, where occupancy is not the limit.) ALONE is the plain variant for rows so long
// that LDS holds one workgroup per compute unit anyway: the cap then only makes the p >= 60 columns spill (136 to 504
// bytes per lane), so it goes (2048 tokens, K = 26624, p = 104: 354 -> 269 us; K = 21504, p = 84: 204 -> 193 us).
__global__ void __launch_bounds__((threads_of<P, SLICED>()), SLICED ? (P < 44 ? 4 : 2) : ALONE ? 2 : P >= 44 ? 4 : 6)
rq_rotate_quant_kernel(const RotQuantArgs a) {
    constexpr int kNT = threads_of<P, SLICED>();
    extern __shared__ __align__(16) float smem[];
    __shared__ float s_red[kNT / 64];

    const int tid = threadIdx.x;
    if ((int) blockIdx.x >= a.token_blocks) {
        // blocks past the tokens clear the split-K cells of the product kernel
        const int64_t i0 = ((int64_t) (blockIdx.x - a.token_blocks) * kNT + tid) * 4;
        if (i0 + 3 < a.zero_ints) {
            *reinterpret_cast<int4 *>(a.zero_ptr + i0) = make_int4(0, 0, 0, 0);
        } else {
            for (int64_t i = i0; i < a.zero_ints; ++i) a.zero_ptr[i] = 0;
        }
        return;
    }

    // Which token. In the digit-plane layout eight consecutive tokens share a 128-byte line of every (group, digit,
    // quarter) run, and workgroups go to the eight XCDs round robin: taken in order, the eight writers of a line
    // would sit in eight different L2s and the line would reach memory as eight partial writes. So within blocks of
    // 64 tokens, workgroup b takes token 8 (b % 8) + (b / 8) % 8: the writers of a line share an XCD (same b % 8)
    // and are dispatched within 64 workgroups of each other.
    int t = blockIdx.x;
    if (a.mode == kActI8 && t < (a.M & ~63)) t = (t & ~63) | ((t & 7) << 3) | ((t >> 3) & 7);
    const int K = a.K;
    const int ng = K / kGroup;
    const int Kp = padi(K) + 1;                  // floats of one padded row
    float *buf = smem;
    float *alt = smem + Kp;                      // second row buffer (SLICED only)
    float *g_lo = smem + (SLICED ? 2 * Kp : Kp);
    float *g_hi = g_lo + ng;

    const float *xr = a.x + (int64_t) t * a.ldx;
    // the first four Sylvester stages ride on the load (one trip through LDS less per token). In the sliced variant
    // (small batches, bound by the latency of its phases) the next four ride too, between lanes, when the chunks are
    // made of blocks of 256 floats; large batches are bound by vector-ALU time, where the LDS pass is the cheaper
    // one (2048 tokens at K = 17408: 105 us against 128 us with the stages between lanes).
    const bool fused_first = a.rotate && (a.m & 15) == 0;
    const bool fused_256 = SLICED && a.rotate && (a.m & 255) == 0;
    if (fused_256) {
        load_row_fwht256<kNT, (P >= 44 ? 3 : 1)>(buf, xr, K, tid);
    } else if (fused_first) {
        // long Paley stages go with long rows (several units of 16 floats per thread): all of a thread's loads go
        // out before the first butterfly
        load_row_fwht16<kNT, (P >= 44 ? 3 : 1)>(buf, xr, K, tid);
    } else {
        load_row<kNT>(buf, xr, K, tid);
    }
    __syncthreads();

    if (a.rotate) {
        const int m = a.m;
        const int lm = __ffs(m) - 1;
        fwht_row(buf, K, lm, tid, kNT, fused_256 ? 8 : fused_first ? 4 : 0);
        if constexpr (P > 1) {
            // Paley across the P chunks of every rotation block (reference lines 2466-2482), then the scale
            const int ncols = K / P;  // columns of all rotation blocks of this token
            const bool m16 = (m & 15) == 0;
            const int pm = m + (m >> 4);
            if constexpr (SLICED) {
                // wave-items = (slice of kOut outputs, run of 64 columns); each wavefront takes a contiguous block
                // of them, so it stays in one slice's straight-line code for several items in a row. Short stages are
                // cut into four slices: with 256 or 512 columns that is one or two items for each of the sixteen
                // wavefronts, where slices of four outputs would leave a quarter of them a second item to do alone.
                constexpr int kOut = P < 44 ? P / 4 : 4;
                const int col_runs = (ncols + 63) >> 6;
                const int n_items = (P / kOut) * col_runs;
                const int per_wave = (n_items + kNT / 64 - 1) / (kNT / 64);
                const int wave = tid >> 6, lane = tid & 63;
                for (int it = 0; it < per_wave; ++it) {
                    const int wi = wave * per_wave + it;
                    if (wi >= n_items) break;
                    const int s = wi / col_runs, cidx = (wi - s * col_runs) * 64 + lane;
                    if (cidx >= ncols) continue;
                    const int rb = cidx / m, j = cidx - rb * m;
                    const int b0 = rb * a.n_rot + j;
                    float col[P];
                    if (m16) {
                        const float *src = buf + padi(b0);
#pragma unroll
                        for (int i = 0; i < P; ++i) col[i] = src[i * pm];
                    } else {
#pragma unroll
                        for (int i = 0; i < P; ++i) col[i] = buf[padi(b0 + i * m)];
                    }
                    float out[kOut];
                    paley_pick<P, kOut>(s, col, out);
#pragma unroll
                    for (int o = 0; o < kOut; ++o) alt[padi(b0 + (kOut * s + o) * m)] = out[o] * a.scale;
                }
                __syncthreads();
                float *tmp = buf; buf = alt; alt = tmp;
            } else {
                for (int cidx = tid; cidx < ncols; cidx += kNT) {
                    const int rb = cidx / m, j = cidx - rb * m;
                    const int b0 = rb * a.n_rot + j;
                    float col[P];
                    if (pm == 272) {   // chunks of 256 (K = 5120, 17408): the common case, compile-time stride
                        float *src = buf + padi(b0);
                        load_column<P, 272>(col, src, pm);
                        paley_column<P, 0, false, 272>(col, src, pm, a.scale);
                    } else if (m16) {
                        float *src = buf + padi(b0);
                        load_column<P, 0>(col, src, pm);
                        paley_column<P>(col, src, pm, a.scale);
                    } else {
#pragma unroll
                        for (int i = 0; i < P; ++i) col[i] = buf[padi(b0 + i * m)];
                        paley_column_generic<P>(col, buf, b0, m, a.scale);
                    }
                }
                __syncthreads();
            }
        } else {
            for (int i = tid; i < K; i += kNT) buf[padi(i)] = buf[padi(i)] * a.scale;
            __syncthreads();
        }
    }

    if (a.mode == kActRotateOnly) {
        float *o = a.out_f32 + (int64_t) t * a.ldo;
        for (int i = tid * 4; i < K; i += kNT * 4) {
            const float *sp = buf + padi(i);
            *reinterpret_cast<float4 *>(o + i) = make_float4(sp[0], sp[1], sp[2], sp[3]);
        }
        return;
    }

    // ---- group ranges [min(x,0), max(x,0)] * clip and the token's widest range (reference lines 2646-2654)
    const int nw = K >> 3;  // code words of this token: a thread per word, lpg lanes per activation group
    const int lpg = a.G >> 3, lgl = __ffs(lpg) - 1;   // 8, 16 or 32 lanes: groups of 64, 128 or 256 (RQ_ACT_GROUP)
    float rmax = 0.0f;
    for (int w0 = 0; w0 < nw; w0 += kNT) {
        const int w = w0 + tid;
        const bool on = w < nw;
        float mn = 0.0f, mx = 0.0f;
        if (on) {
            const float *sp = buf + padi(8 * w);   // 8 consecutive values never straddle a run of 16
            const float v8[8] = { sp[0], sp[1], sp[2], sp[3], sp[4], sp[5], sp[6], sp[7] };
            had::minmax8_raw(v8, mn, mx);
        }
        if (lpg == 8) {
            // groups of 64 = eight lanes: swap within pairs, within quads, mirror the half row; DPP steps at vector-ALU
            // speed instead of three trips through the LDS crossbar
            mn = had::group8_reduce<false>(mn);
            mx = had::group8_reduce<true>(mx);
        } else {
            for (int off = 1; off < lpg; off <<= 1) {
                mn = fminf(mn, __shfl_xor(mn, off, 64));
                mx = fmaxf(mx, __shfl_xor(mx, off, 64));
            }
        }
        const float lo = mn * a.clip, hi = mx * a.clip;
        if (on) {
            if ((tid & (lpg - 1)) == 0) {
                g_lo[w >> lgl] = lo;
                g_hi[w >> lgl] = hi;
            }
            rmax = fmaxf(rmax, hi - lo);
        }
    }
    if (a.mode == kActStats) {
        rmax = wave_max(rmax);
        if ((tid & 63) == 0) a.rpart[(size_t) t * kRangeParts + (tid >> 6)] = rmax;
        if (tid >= kNT / 64 && tid < kRangeParts) a.rpart[(size_t) t * kRangeParts + tid] = 0.0f;
        __syncthreads();
        float *lh = a.lohi + (size_t) t * ng * 2;
        for (int g = tid; g < ng; g += kNT) {
            lh[2 * g] = g_lo[g];
            lh[2 * g + 1] = g_hi[g];
        }
        if (a.out_f32 != nullptr) {
            float *o = a.out_f32 + (int64_t) t * a.ldo;
            for (int i = tid * 4; i < K; i += kNT * 4) {
                const float *sp = buf + padi(i);
                *reinterpret_cast<float4 *>(o + i) = make_float4(sp[0], sp[1], sp[2], sp[3]);
            }
        }
        return;
    }
    rmax = wave_max(rmax);
    if ((tid & 63) == 0) s_red[tid >> 6] = rmax;
    __syncthreads();
    float R = s_red[0];
#pragma unroll
    for (int i = 1; i < kNT / 64; ++i) R = fmaxf(R, s_red[i]);
    if (R == 0.0f) R = 2.0f;
    const float u = R / 3825.0f;  // 15 * 255
    if (tid == 0 && a.u != nullptr) a.u[t] = u;

    // ---- per group multiplier and zero point, per value code (reference lines 2662-2677)
    for (int w0 = 0; w0 < nw; w0 += kNT) {
        const int w = w0 + tid;
        const bool on = w < nw;
        const int wc = on ? w : 0;
        const int g = wc >> 3;                     // 64-wide group: where the digits go
        const float lo = g_lo[wc >> lgl], hi = g_hi[wc >> lgl];
        const int mg = (int) fminf(fmaxf(ceilf(((hi - lo) * 255.0f) / R), 1.0f), 255.0f);
        const float inv = 1.0f / ((float) mg * u);
        const float zf = fminf(fmaxf(rintf(-lo * inv), 0.0f), 15.0f);
        const int z = (int) zf;
        const float *sp = buf + padi(8 * wc);
        const float f[8] = { sp[0], sp[1], sp[2], sp[3], sp[4], sp[5], sp[6], sp[7] };
        if (a.mode == kActI8 && a.single == 2) {
            // fp6 fragment plane: q - z as sign and magnitude, six bits each (as fp6 E2M3 the value is (q - z) / 8);
            // this word's 48 bits are bytes 6 (w % 4) .. of the 24 bytes that lane token % 32 + 32 * (half of the group)
            // holds in the fragment of 32 tokens: bytes 0 .. 15 at lane * 16, bytes 16 .. 23 at 1024 + lane * 8
            uint64_t bits = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int d = (int) (fminf(fmaxf(rintf(f[j] * inv) + zf, 0.0f), 15.0f) - zf);
                const uint32_t code = d < 0 ? (32u | (uint32_t) (-d)) : (uint32_t) d;
                bits |= (uint64_t) code << (6 * j);
            }
            if (on) {
                const int c8 = w & 7;
                const int lane = (t & 31) + 32 * (c8 >> 2);
                uint8_t *frag = reinterpret_cast<uint8_t *>(a.act) + ((size_t) g * (a.Mp >> 5) + (t >> 5)) * kFrag6;
#pragma unroll
                for (int i = 0; i < 3; ++i) {
                    const int o = 6 * (c8 & 3) + 2 * i;   // byte of the lane's 24
                    uint8_t *dst = o < 16 ? frag + lane * 16 + o : frag + 1024 + lane * 8 + (o - 16);
                    *reinterpret_cast<uint16_t *>(dst) = (uint16_t) (bits >> (16 * i));
                }
                if (c8 == 0) a.m4[(size_t) g * a.Mp + t] = 4.0f * (float) mg;
            }
            continue;
        }
        if (a.mode == kActI8 && a.single) {
            uint32_t even, odd;
            qz_of_word(f, inv, zf, even, odd);
            if (on) {
                // [group][quarter of the group][token][16 bytes] and the multiplier of (group, token)
                const size_t cell = ((size_t) g * 4 + ((w & 7) >> 1)) * a.Mp + t;
                *reinterpret_cast<uint2 *>(a.act + cell * 4 + (w & 1) * 2) = make_uint2(even, odd);
                if ((w & 7) == 0) a.mvals[(size_t) g * a.Mp + t] = (uint8_t) mg;
            }
            continue;
        }
        if (a.mode == kActI8) {
            uint32_t lo_e, lo_o, hi_e, hi_o;
            digits_of_word(f, inv, zf, (float) mg, lo_e, lo_o, hi_e, hi_o);
            if (on) {
                // [group][digit][quarter of the group][token][16 bytes]: a token tile of one quarter is contiguous
                const size_t cell = (((size_t) g * 2 + 0) * 4 + ((w & 7) >> 1)) * a.Mp + t;
                uint32_t *dst = a.act + cell * 4 + (w & 1) * 2;
                *reinterpret_cast<uint2 *>(dst) = make_uint2(lo_e, lo_o);
                *reinterpret_cast<uint2 *>(dst + (size_t) 16 * a.Mp) = make_uint2(hi_e, hi_o);
            }
            continue;
        }

        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int q = (int) fminf(fmaxf(rintf(f[j] * inv) + zf, 0.0f), 15.0f);
            word |= (uint32_t) ((q - 8) & 0xF) << (4 * j);
        }

        {  // kActBlocks: the reference's A4 / A4H storage (reference lines 2656-2661, 2667-2669)
            const int base = tid & 32;  // lanes base, base + lpg, ... hold the block's 4, 2 or 1 groups
            uint32_t zs = 0, ms = 0;
#pragma unroll
            for (int sg = 0; sg < 4; ++sg) {
                const uint32_t zv = (uint32_t) __shfl(z, base + ((lpg * sg) & 31), 64);
                const uint32_t mv = (uint32_t) __shfl(mg, base + ((lpg * sg) & 31), 64);
                if (sg * lpg < 32) {
                    zs |= zv << (4 * sg);
                    ms |= mv << (8 * sg);
                }
            }
            const uint32_t lsub = a.G == 64 ? 2u : a.G == 128 ? 1u : 0u;
            if (on) {
                rq_block_w4a4 *blk = reinterpret_cast<rq_block_w4a4 *>(a.blocks) + (size_t) t * (K / RQ_BLOCK_CODES) + (w >> 5);
                blk->qs[w & 31] = word;
                if ((w & 31) == 0) {
                    blk->d = u;
                    blk->sum = (int32_t) ((lsub << 16) | zs);
                    blk->pad[0] = (int32_t) ms;
                    blk->pad[1] = a.len_field;
                }
            }
        }
    }
}

// the kernels keep a whole row in dynamic LDS: raise the per-kernel limit (once per device, see init_activation_kernels)
template <int P, bool SLICED, bool ALONE = false>
hipError_t allow_big_lds() {
    return hipFuncSetAttribute(reinterpret_cast<const void *>(&rq_rotate_quant_kernel<P, SLICED, ALONE>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 64);
}

// the plain variant has an ALONE build where the cap makes its columns spill and rows of up to RQ_MAX_K floats get that
// long (p = 68 and 72 would need chunks of 512: past RQ_MAX_K)
constexpr bool has_alone(int p) { return p == 60 || p >= 84; }

template <int P>
hipError_t allow_big_lds_both() {
    hipError_t e = allow_big_lds<P, false>();
    if (e == hipSuccess && P > 1) e = allow_big_lds<P, (P > 1)>();
    if (e == hipSuccess && has_alone(P)) e = allow_big_lds<P, false, has_alone(P)>();
    return e;
}

template <int P, bool SLICED, bool ALONE = false>
hipError_t launch_one(const RotQuantArgs &a, size_t lds, hipStream_t stream) {
    static bool attr_set = false;   // calls that never went through rq_w4a4_prepare on this device
    if (!attr_set) {
        hipError_t e = allow_big_lds<P, SLICED, ALONE>();
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    constexpr int kNT = threads_of<P, SLICED>();
    // blocks past the tokens clear the split-K cells, four ints per thread
    RotQuantArgs b = a;
    b.token_blocks = a.M;
    const int grid = a.M + (int) ((a.zero_ints + (int64_t) kNT * 4 - 1) / ((int64_t) kNT * 4));
    if (grid == 0) return hipSuccess;
    hipLaunchKernelGGL((rq_rotate_quant_kernel<P, SLICED, ALONE>), dim3(grid), dim3(kNT), lds, stream, b);
    return hipGetLastError();
}

// LDS: one padded row (two when the Paley stage is sliced over more threads) plus the group ranges. Slicing buys
// parallelism inside a token and costs occupancy, so it is for small batches only.
template <int P>
hipError_t launch_p(const RotQuantArgs &a, hipStream_t stream) {
    const size_t row = (size_t) (a.K + (a.K >> 4) + 1) * sizeof(float);
    const size_t stats = (size_t) 2 * (a.K / kGroup + 1) * sizeof(float);
    // long Paley stages: past kTwoStepTokens tokens the plain variant (two workgroups per CU) is the faster one
    if (P > 1 && a.M <= (P >= 44 ? kTwoStepTokens : 64) && 2 * row + stats <= 160 * 1024 - 64) {
        return launch_one<P, (P > 1)>(a, 2 * row + stats, stream);
    }
    // a second workgroup does not fit beside this one
    if (has_alone(P) && 2 * (row + stats + 64) > 160 * 1024) return launch_one<P, false, has_alone(P)>(a, row + stats, stream);
    return launch_one<P, false>(a, row + stats, stream);
}

}  // namespace

hipError_t init_rotate_quant_kernels() {
    hipError_t e = allow_big_lds_both<1>();
    if (e == hipSuccess) e = allow_big_lds_both<12>();
    if (e == hipSuccess) e = allow_big_lds_both<20>();
    if (e == hipSuccess) e = allow_big_lds_both<44>();
    if (e == hipSuccess) e = allow_big_lds_both<60>();
    if (e == hipSuccess) e = allow_big_lds_both<68>();
    if (e == hipSuccess) e = allow_big_lds_both<72>();
    if (e == hipSuccess) e = allow_big_lds_both<84>();
    if (e == hipSuccess) e = allow_big_lds_both<104>();
    if (e == hipSuccess) e = allow_big_lds_both<108>();
    return e;
}

hipError_t launch_rotate_quant(const RotQuantArgs &a, hipStream_t stream) {
    if (a.M == 0 && a.zero_ints == 0) return hipSuccess;
    const int p = a.rotate ? a.p : 1;
    switch (p) {
        case 1:   return launch_p<1>(a, stream);
        case 12:  return launch_p<12>(a, stream);
        case 20:  return launch_p<20>(a, stream);
        case 44:  return launch_p<44>(a, stream);
        case 60:  return launch_p<60>(a, stream);
        case 68:  return launch_p<68>(a, stream);
        case 72:  return launch_p<72>(a, stream);
        case 84:  return launch_p<84>(a, stream);
        case 104: return launch_p<104>(a, stream);
        case 108: return launch_p<108>(a, stream);
        default:  return hipErrorInvalidValue;
    }
}

}  // namespace rq
