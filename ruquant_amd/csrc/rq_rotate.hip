// Online Hadamard for the decode path: one token spread over several workgroups.
//
// A decode step has one to a few tokens, and a single workgroup per token would leave the rotation bound by the
// issue rate of eight wavefronts. The Paley stage is independent per column, so here a workgroup owns a slab of 64
// columns of every rotation block: it loads the whole row into LDS, runs the (cheap) Sylvester stages of all chunks
// itself, then the Paley sums of its own columns only. A run of 64 columns of one output chunk is exactly one
// activation group, so the wavefront that produced it also reduces its range [min(x,0), max(x,0)] * clip.
// Outputs: the rotated row (fp32) and the clipped group ranges; the GEMV quantizes from those.
// Arithmetic and its order are those of ggml_rq_hadamard (reference patch lines 2450-2485).
#include "rq_hadamard.h"

#pragma clang fp contract(off)

namespace rq {

namespace {

using namespace had;

constexpr int kRT = 512;  // threads per workgroup

// O = outputs of a column that one Paley item (one wavefront) forms: four, or two for a long stage and few tokens
// (twice the workgroups, half the chain of additions per wavefront: 6.9 -> 6.5 us for one token of K = 17408; at 16
// tokens the workgroups would no longer be resident together: 10.2 -> 11.5 us)
template <int P, int O>
__global__ void __launch_bounds__(kRT) rq_rotate_slab_kernel(const RotQuantArgs a, int slabs, int parts) {
    extern __shared__ __align__(16) float buf[];
    __shared__ float s_rmax[kRT / 64];

    const int tid = threadIdx.x;
    if ((int) blockIdx.x >= a.token_blocks) {
        // blocks past the tokens clear the split-K cells of the product kernel
        const int64_t i0 = ((int64_t) (blockIdx.x - a.token_blocks) * kRT + tid) * 4;
        if (i0 + 3 < a.zero_ints) {
            *reinterpret_cast<int4 *>(a.zero_ptr + i0) = make_int4(0, 0, 0, 0);
        } else {
            for (int64_t i = i0; i < a.zero_ints; ++i) a.zero_ptr[i] = 0;
        }
        return;
    }

    // workgroup = (token, slab of 64 columns, part): the slab's Paley items are dealt round-robin to `parts`
    // workgroups, so that a wavefront has one or two of them
    const int per_token = slabs * parts;
    const int t = blockIdx.x / per_token, sp = blockIdx.x - t * per_token;
    const int slab = sp / parts, part = sp - slab * parts;
    const int K = a.K, m = a.m, ng = K / kGroup;
    const int lm = __ffs(m) - 1;
    const int wave = tid >> 6, lane = tid & 63;
    constexpr int kO = O;

    const float *xr = a.x + (int64_t) t * a.ldx;
    // the first four Sylvester stages ride on the load (chunks here are multiples of 64), and the next four too,
    // between lanes, when the chunks are made of blocks of 256 floats
    const bool fused_256 = (m & 255) == 0;
    if (fused_256) load_row_fwht256<kRT>(buf, xr, K, tid);
    else load_row_fwht16<kRT>(buf, xr, K, tid);
    __syncthreads();
    fwht_row(buf, K, lm, tid, kRT, fused_256 ? 8 : 4);

    float *out = a.out_f32 + (int64_t) t * a.ldo;
    float *lh = a.lohi + (size_t) t * ng * 2;
    float rmax = 0.0f;   // widest range this wavefront has produced

    if constexpr (P == 1) {
        // no Paley stage: the slab is a share of the row's runs of 64
        const int runs = K >> 6;
        for (int r = sp * (kRT / 64) + wave; r < runs; r += per_token * (kRT / 64)) {
            const int idx = 64 * r + lane;
            const float v = buf[padi(idx)] * a.scale;
            out[idx] = v;
            const float lo = wave_min(fminf(v, 0.0f)) * a.clip, hi = wave_max(fmaxf(v, 0.0f)) * a.clip;
            if (lane == 0) {
                lh[2 * r] = lo;
                lh[2 * r + 1] = hi;
            }
            rmax = fmaxf(rmax, hi - lo);
        }
    } else {
        // wave-items = (rotation block, slice of O output chunks) for this slab's 64 columns
        const int n_rb = K / a.n_rot;
        const int n_items = n_rb * (P / kO);
        const int pm = m + (m >> 4);
        for (int wi = part + parts * wave; wi < n_items; wi += parts * (kRT / 64)) {
            const int s = wi / n_rb, rb = wi - s * n_rb;
            const int b0 = rb * a.n_rot + 64 * slab + lane;
            const float *src = buf + padi(b0);
            // (the sums advance together, one column element at a time, and the column is read on the fly: O + 1
            // registers instead of P; measured the same speed as one sum after the other from a column in registers)
            float res[kO];
            paley_pick_stream<P, kO, 0>(s, src, pm, res);
#pragma unroll
            for (int o = 0; o < kO; ++o) {
                const int idx = b0 + (kO * s + o) * m;
                const float v = res[o] * a.scale;
                out[idx] = v;
                const float lo = wave_min(fminf(v, 0.0f)) * a.clip, hi = wave_max(fmaxf(v, 0.0f)) * a.clip;
                if (lane == 0) {
                    lh[2 * (idx >> 6)] = lo;
                    lh[2 * (idx >> 6) + 1] = hi;
                }
                rmax = fmaxf(rmax, hi - lo);
            }
        }
    }
    // one slot of the token's partial maxima per workgroup; slots nobody owns are written as zero by the first one
    if (lane == 0) s_rmax[wave] = rmax;
    __syncthreads();
    if (tid == 0) {
        float r = s_rmax[0];
#pragma unroll
        for (int i = 1; i < kRT / 64; ++i) r = fmaxf(r, s_rmax[i]);
        a.rpart[(size_t) t * kRangeParts + sp] = r;
    }
    if (sp == 0 && tid >= per_token && tid < kRangeParts) a.rpart[(size_t) t * kRangeParts + tid] = 0.0f;
}

// The activation quantizer for tokens whose rotated rows and group ranges already exist (written by the kernel
// above): token unit from the partial range maxima, then per group the multiplier and zero point and per value the
// code, emitted as the two int8 digits of m (q - z) in the layout of the MFMA kernels. A thread per code word; same
// fp32 operations in the same order as the one-workgroup quantizer (reference patch lines 2639-2679).
__global__ void __launch_bounds__(kRT) rq_quantize_digits_kernel(const RotQuantArgs a, int blocks_per_token) {
    const int tid = threadIdx.x;
    const int t = blockIdx.x / blocks_per_token;
    const int w = (blockIdx.x - t * blocks_per_token) * kRT + tid;
    const int lane = tid & 63;
    float R = wave_max(lane < kRangeParts ? a.rpart[(size_t) t * kRangeParts + lane] : 0.0f);
    if (R == 0.0f) R = 2.0f;
    const float u = R / 3825.0f;  // 15 * 255
    if (w == 0) a.u[t] = u;
    if (w >= (a.K >> 3)) return;
    const int g = w >> 3;
    const float2 lh = reinterpret_cast<const float2 *>(a.lohi)[(size_t) t * (a.K / kGroup) + g];
    const int mg = (int) fminf(fmaxf(ceilf(((lh.y - lh.x) * 255.0f) / R), 1.0f), 255.0f);
    const float inv = 1.0f / ((float) mg * u);
    const float zf = fminf(fmaxf(rintf(-lh.x * inv), 0.0f), 15.0f);
    const float4 *src = reinterpret_cast<const float4 *>(a.out_f32 + (int64_t) t * a.ldo + 8 * w);
    const float4 v0 = src[0], v1 = src[1];
    const float f[8] = { v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w };
    if (a.single) {
        uint32_t even, odd;
        qz_of_word(f, inv, zf, even, odd);
        const size_t cell1 = ((size_t) g * 4 + ((w & 7) >> 1)) * a.Mp + t;
        *reinterpret_cast<uint2 *>(a.act + cell1 * 4 + (w & 1) * 2) = make_uint2(even, odd);
        if ((w & 7) == 0) a.mvals[(size_t) g * a.Mp + t] = (uint8_t) mg;
        return;
    }
    uint32_t lo_e, lo_o, hi_e, hi_o;
    digits_of_word(f, inv, zf, (float) mg, lo_e, lo_o, hi_e, hi_o);
    // [group][digit][quarter of the group][token][16 bytes]
    const size_t cell = (((size_t) g * 2 + 0) * 4 + ((w & 7) >> 1)) * a.Mp + t;
    uint32_t *dst = a.act + cell * 4 + (w & 1) * 2;
    *reinterpret_cast<uint2 *>(dst) = make_uint2(lo_e, lo_o);
    *reinterpret_cast<uint2 *>(dst + (size_t) 16 * a.Mp) = make_uint2(hi_e, hi_o);
}

template <int P, int O>
hipError_t allow_big_lds() {
    return hipFuncSetAttribute(reinterpret_cast<const void *>(&rq_rotate_slab_kernel<P, O>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 64);
}

// the two-output form exists for the long Paley stage only
constexpr bool has_pairs(int p) { return p > 44; }

template <int P>
hipError_t allow_big_lds_p() {
    hipError_t e = allow_big_lds<P, 4>();
    if constexpr (has_pairs(P)) {
        if (e == hipSuccess) e = allow_big_lds<P, 2>();
    }
    return e;
}

// workgroups per token that share a slab's Paley items: enough that a wavefront gets one item, within the token's
// range slots
inline int parts_of(int n_items, int slabs) {
    int parts = (n_items + kRT / 64 - 1) / (kRT / 64);
    while (parts > 1 && slabs * parts > kRangeParts) --parts;
    return parts;
}

template <int P>
hipError_t launch_slab(const RotQuantArgs &a, hipStream_t stream) {
    static bool attr_set = false;   // calls that never went through rq_w4a4_prepare on this device
    if (!attr_set) {
        hipError_t e = allow_big_lds_p<P>();
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    // one slab per 64 columns of a chunk; without a Paley stage, a few workgroups share the row's runs
    int slabs = P > 1 ? a.m / 64 : (a.K >= 4096 ? 4 : 1);
    if (slabs > kRangeParts) return launch_rotate_quant(a, stream);   // more slabs than range slots
    const int n_rb = a.K / a.n_rot;
    int parts = P > 1 ? parts_of(n_rb * (P / 4), slabs) : 1;
    bool pairs = false;
    if constexpr (has_pairs(P)) {
        // items of two outputs while all the workgroups are still resident together (one per compute unit)
        const int parts2 = parts_of(n_rb * (P / 2), slabs);
        if (a.M * slabs * parts2 <= device_compute_units()) {
            pairs = true;
            parts = parts2;
        }
    }
    const int zero_blocks = (int) ((a.zero_ints + (int64_t) kRT * 4 - 1) / ((int64_t) kRT * 4));
    RotQuantArgs b = a;
    b.token_blocks = a.M * slabs * parts;
    const size_t lds = (size_t) (a.K + (a.K >> 4) + 1) * sizeof(float);
    const dim3 grid(b.token_blocks + zero_blocks);
    if constexpr (has_pairs(P)) {
        if (pairs) {
            hipLaunchKernelGGL((rq_rotate_slab_kernel<P, 2>), grid, dim3(kRT), lds, stream, b, slabs, parts);
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL((rq_rotate_slab_kernel<P, 4>), grid, dim3(kRT), lds, stream, b, slabs, parts);
    return hipGetLastError();
}

}  // namespace

hipError_t init_rotate_slab_kernels() {
    hipError_t e = allow_big_lds_p<1>();
    if (e == hipSuccess) e = allow_big_lds_p<12>();
    if (e == hipSuccess) e = allow_big_lds_p<20>();
    if (e == hipSuccess) e = allow_big_lds_p<68>();
    return e;
}

hipError_t launch_rotate_stats(const RotQuantArgs &a, hipStream_t stream) {
    // The slab kernel needs whole groups per (chunk, slab): chunks that are a multiple of 64 long. Everything else,
    // and unrotated activations (ranges only), goes through the one-workgroup-per-token kernel.
    if (!a.rotate || (a.m & 63) != 0 || a.M > kSkinnyTokens) return launch_rotate_quant(a, stream);
    switch (a.p) {
        case 1:  return launch_slab<1>(a, stream);
        case 12: return launch_slab<12>(a, stream);
        case 20: return launch_slab<20>(a, stream);
        case 68: return launch_slab<68>(a, stream);
        default: return launch_rotate_quant(a, stream);
    }
}

hipError_t launch_quantize_digits(const RotQuantArgs &a, hipStream_t stream) {
    const int bpt = ((a.K >> 3) + kRT - 1) / kRT;
    hipLaunchKernelGGL(rq_quantize_digits_kernel, dim3(a.M * bpt), dim3(kRT), 0, stream, a, bpt);
    return hipGetLastError();
}

}  // namespace rq
