// Weight-side quantizer and the dequantizers of the four block types, on the GPU: what ggml calls from_float_ref and
// to_float for W4A4 / W4A4H / A4 / A4H (reference patch lines 2507-2580, 2681-2710, 2738-2773).
//
// A converter quantizes whole tensors; the reference does it a row at a time on the host. Here the row (or the weight
// group) is the unit of parallelism, and the results are bit-identical because the only order-sensitive quantity, the
// double-precision error sum of the scale search, is accumulated by one lane in the reference's element order:
//   * search kernel: sixteen lanes per segment (a row, a block of 256 or a group of 64); thirteen of them each try one
//     clip ratio over the whole segment, sequentially, and a scan in ratio order keeps the first smallest error;
//   * encode kernel: a workgroup per row turns the chosen scale(s) into codes, row sum / multiplier headers and
//     blocks;
//   * dequantize kernel: a workgroup per row decodes blocks into the padded LDS row and, for the rotated types, runs
//     the Sylvester butterflies and the transposed Paley stage before the row leaves for memory.
// The forward rotation of W4A4H weights is the activation kernel's rotate-only mode.
#include "rq_hadamard.h"

#include <math.h>
#include <string.h>

#pragma clang fp contract(off)

namespace rq {

hipError_t launch_rotate_quant(const RotQuantArgs &a, hipStream_t stream);

namespace {

using namespace had;

constexpr int kRatios = 13;          // clip ratios 1.0, 0.975, ... 0.7 (reference lines 2514-2524)
constexpr int kSearchThreads = 256;  // sixteen segments of sixteen lanes

struct SearchArgs {
    const float *x;    // rows of K floats, ld apart
    int64_t ld;
    int64_t segments;  // rows * per_row
    int per_row;       // segments per row
    int n;             // floats per segment
    float *scale;      // [segments]
};

__global__ void __launch_bounds__(kSearchThreads) rq_wsearch_kernel(const SearchArgs a) {
    const int tid = threadIdx.x, r = tid & 15;
    int64_t seg = (int64_t) blockIdx.x * (kSearchThreads / 16) + (tid >> 4);
    const bool live = seg < a.segments;
    if (!live) seg = a.segments - 1;   // idle lanes follow a live segment so that the shuffles below stay uniform
    const int64_t row = seg / a.per_row;
    const float *x = a.x + row * a.ld + (seg - row * a.per_row) * (int64_t) a.n;
    const int n = a.n;

    float amax = 0.0f;
    for (int i = r * 4; i < n; i += 64) {
        const float4 v = *reinterpret_cast<const float4 *>(x + i);
        amax = fmaxf(fmaxf(fmaxf(fmaxf(amax, fabsf(v.x)), fabsf(v.y)), fabsf(v.z)), fabsf(v.w));
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 16));

    float s = 0.0f;
    double err = INFINITY;
    if (amax > 0.0f && r < kRatios) {
        s = amax * (1.0f - 0.025f * (float) r) / 7.0f;
        err = 0.0;
        for (int i = 0; i < n; i += 4) {
            const float4 v = *reinterpret_cast<const float4 *>(x + i);
            const float xs[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float q = fminf(fmaxf(rintf(xs[j] / s), -8.0f), 7.0f);
                const double e = (double) (q * s) - (double) xs[j];
                err += e * e;
            }
        }
    }
    // first smallest error in ratio order, as the reference's `err < best_err` scan
    const int base = (tid & 63) & ~15;
    float best_s = 0.0f;
    double best_err = INFINITY;
#pragma unroll
    for (int k = 0; k < kRatios; ++k) {
        const double ek = __shfl(err, base + k, 64);
        const float sk = __shfl(s, base + k, 64);
        if (ek < best_err) {
            best_err = ek;
            best_s = sk;
        }
    }
    if (live && r == 0) a.scale[seg] = best_s;
}

struct EncodeArgs {
    const float *x;
    int64_t ld;
    int K;
    int per_row;        // scales per row: 1, K / 256 or K / 64
    int groups;         // 0: one scale per row, legacy header; 1: weight groups (multiplier headers)
    const float *scale; // [rows * per_row]
    rq_block_w4a4 *blocks;
    int32_t len_field;  // pad[0]: the row length, or the Hadamard length of a W4A4H tensor
};

__device__ __forceinline__ int code_for(float x, float s) {
    return s > 0.0f ? (int) fminf(fmaxf(rintf(x / s), -8.0f), 7.0f) : 0;
}

__global__ void __launch_bounds__(256) rq_wencode_kernel(const EncodeArgs a) {
    __shared__ int s_mult[512];   // multiplier of every weight group of the row (K <= 32768: at most 512 groups)
    __shared__ float s_red[4];
    __shared__ int s_sum;
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int K = a.K, nb = K / RQ_BLOCK_CODES, nw = K >> 3;
    const float *x = a.x + row * a.ld;
    rq_block_w4a4 *out = a.blocks + row * nb;
    float unit;   // the row's d
    if (!a.groups) {
        unit = a.scale[row];
        if (tid == 0) s_sum = 0;
        __syncthreads();
    } else {
        // the row's unit is the largest group scale / 15; every group scale becomes a multiple 1..15 of it
        const float *sb = a.scale + row * a.per_row;
        float smax = 0.0f;
        for (int g = tid; g < a.per_row; g += 256) smax = fmaxf(smax, sb[g]);
        smax = wave_max(smax);
        if ((tid & 63) == 0) s_red[tid >> 6] = smax;
        __syncthreads();
        smax = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
        unit = smax / 15.0f;
        for (int g = tid; g < a.per_row; g += 256) {
            s_mult[g] = unit > 0.0f ? (int) fminf(fmaxf(rintf(sb[g] / unit), 1.0f), 15.0f) : 1;
        }
        __syncthreads();
    }
    const int lgw = nw / a.per_row;   // code words per weight group (8 or 32)
    int sum = 0;
    for (int w = tid; w < nw; w += 256) {
        const float s = !a.groups ? unit : (float) s_mult[w / lgw] * unit;
        const float4 v0 = *reinterpret_cast<const float4 *>(x + 8 * w);
        const float4 v1 = *reinterpret_cast<const float4 *>(x + 8 * w + 4);
        const float xs[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int c = code_for(xs[j], s);
            sum += c;
            word |= (uint32_t) (c & 0xF) << (4 * j);
        }
        out[w >> 5].qs[w & 31] = word;
    }
    if (!a.groups) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
        if ((tid & 63) == 0) atomicAdd(&s_sum, sum);
        __syncthreads();
    }
    for (int b = tid; b < nb; b += 256) {
        int32_t header;
        if (!a.groups) {
            header = s_sum;   // legacy header: the row's code sum (multiplier 1)
        } else if (a.per_row == nb) {
            header = (int32_t) (1u << 30 | (uint32_t) s_mult[b]);
        } else {
            header = (int32_t) (3u << 29 | (uint32_t) s_mult[4 * b] | (uint32_t) s_mult[4 * b + 1] << 4 |
                                (uint32_t) s_mult[4 * b + 2] << 8 | (uint32_t) s_mult[4 * b + 3] << 12);
        }
        out[b].d = unit;
        out[b].sum = header;
        out[b].pad[0] = a.len_field;
        out[b].pad[1] = 0;
    }
}

// ---- dequantizers ------------------------------------------------------------------------------------------------

struct DequantArgs {
    const rq_block_w4a4 *blocks;
    int K;
    int act;       // 0: weight blocks (multiplier per 64 from the header); 1: activation blocks (zero point + multiplier)
    int rotate;    // the inverse rotation follows
    int n_rot, m;
    float scale;   // 1 / sqrtf(n_rot)
    float *out;
    int64_t ldo;
};

__device__ __forceinline__ int nibble(uint32_t word, int j) { return (int) (((word >> (4 * j)) & 0xF) ^ 8) - 8; }

__device__ __forceinline__ int weight_mult(int32_t sum, int g) {
    const uint32_t s = (uint32_t) sum;
    if ((s >> 29) == 3) return (int) ((s >> (4 * g)) & 0xF);
    if ((s >> 30) == 1) return (int) (s & 0xF);
    return 1;
}

template <int P>
__global__ void __launch_bounds__(512) rq_dequant_rows_kernel(const DequantArgs a) {
    extern __shared__ __align__(16) float smem[];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int K = a.K, nb = K / RQ_BLOCK_CODES, nw = K >> 3;
    const rq_block_w4a4 *in = a.blocks + row * nb;
    float *o = a.out + row * a.ldo;
    float *buf = smem;

    for (int w = tid; w < nw; w += 512) {
        const rq_block_w4a4 &blk = in[w >> 5];
        const int ww = w & 31;
        const uint32_t word = blk.qs[ww];
        float f;
        int bias = 0;
        if (a.act) {
            // reference lines 2744-2753: group of the word from the header's sub-group shift
            const int lsub = (blk.sum >> 16) & 3;
            const int sg = (8 * ww) >> (8 - lsub);
            const int z = (blk.sum >> (4 * sg)) & 0xF;
            const int mg = (int) (((uint32_t) blk.pad[0] >> (8 * sg)) & 0xFF);
            f = (float) mg * blk.d;
            bias = 8 - z;
        } else {
            f = (float) weight_mult(blk.sum, ww >> 3) * blk.d;
        }
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (float) (nibble(word, j) + bias) * f;
        if (a.rotate) {
            float *d = buf + padi(8 * w);   // 8 w % 8 == 0: the eight land in one run of 16
#pragma unroll
            for (int j = 0; j < 8; ++j) d[j] = v[j];
        } else {
            *reinterpret_cast<float4 *>(o + 8 * w) = make_float4(v[0], v[1], v[2], v[3]);
            *reinterpret_cast<float4 *>(o + 8 * w + 4) = make_float4(v[4], v[5], v[6], v[7]);
        }
    }
    if (!a.rotate) return;
    __syncthreads();

    const int m = a.m;
    const int lm = __ffs(m) - 1;
    fwht_row(buf, K, lm, tid, 512);
    if constexpr (P > 1) {
        const int ncols = K / P;
        const bool m16 = (m & 15) == 0;
        const int pm = m + (m >> 4);
        for (int cidx = tid; cidx < ncols; cidx += 512) {
            const int rb = cidx / m, j = cidx - rb * m;
            const int b0 = rb * a.n_rot + j;
            float col[P];
            if (m16) {
                float *src = buf + padi(b0);
#pragma unroll
                for (int i = 0; i < P; ++i) col[i] = src[i * pm];
                paley_column<P, 0, true>(col, src, pm, a.scale);
            } else {
#pragma unroll
                for (int i = 0; i < P; ++i) col[i] = buf[padi(b0 + i * m)];
                paley_column_generic<P, 0, true>(col, buf, b0, m, a.scale);
            }
        }
    } else {
        for (int i = tid; i < K; i += 512) buf[padi(i)] = buf[padi(i)] * a.scale;
    }
    __syncthreads();
    for (int i = tid * 4; i < K; i += 512 * 4) {
        const float *sp = buf + padi(i);
        *reinterpret_cast<float4 *>(o + i) = make_float4(sp[0], sp[1], sp[2], sp[3]);
    }
}

template <int P>
hipError_t launch_dequant(const DequantArgs &a, int64_t rows, hipStream_t stream) {
    const size_t lds = a.rotate ? (size_t) (a.K + (a.K >> 4) + 1) * sizeof(float) : 0;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&rq_dequant_rows_kernel<P>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 64);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    hipLaunchKernelGGL((rq_dequant_rows_kernel<P>), dim3((unsigned) rows), dim3(512), lds, stream, a);
    return hipGetLastError();
}

bool factor(int64_t n, int &p, int &m) { return rq_w4a4_hadamard_factor(n, &p, &m) != 0; }

struct QuantWorkspace {
    size_t off_rot, off_scale, bytes;
};

QuantWorkspace quant_workspace(int type, int64_t K, int64_t N, int wgroup) {
    QuantWorkspace w;
    size_t off = 0;
    w.off_rot = off;
    if (type == RQ_TYPE_W4A4H) off = align_up(off + (size_t) N * K * sizeof(float), 256);
    w.off_scale = off;
    const int64_t per_row = wgroup == 0 ? 1 : K / wgroup;
    off = align_up(off + (size_t) N * per_row * sizeof(float), 256);
    w.bytes = off;
    return w;
}

}  // namespace
}  // namespace rq

using namespace rq;

extern "C" {

size_t rq_w4a4_quantize_weights_workspace_bytes(int type, int64_t K, int64_t N, int wgroup) {
    if ((type != RQ_TYPE_W4A4 && type != RQ_TYPE_W4A4H) || K <= 0 || K % RQ_BLOCK_CODES != 0 || K > RQ_MAX_K || N <= 0) return 0;
    if (wgroup != 0 && wgroup != 64 && wgroup != RQ_BLOCK_CODES) return 0;
    return quant_workspace(type, K, N, wgroup).bytes;
}

int rq_w4a4_quantize_weights(int type, const float *w_dev, int64_t ldw, int64_t N, int64_t K, int64_t n_rot, int wgroup,
                             void *blocks_dev, void *workspace_dev, size_t workspace_bytes, rq_stream_t stream) {
    if (!w_dev || !blocks_dev || !workspace_dev) return RQ_E_ARGUMENT;
    if (type != RQ_TYPE_W4A4 && type != RQ_TYPE_W4A4H) return RQ_E_UNSUPPORTED;
    if (K <= 0 || K % RQ_BLOCK_CODES != 0 || K > RQ_MAX_K || N < 0 || N > 0x7fffffff) return RQ_E_UNSUPPORTED;
    if (wgroup != 0 && wgroup != 64 && wgroup != RQ_BLOCK_CODES) return RQ_E_ARGUMENT;
    if (ldw < K || (ldw * 4) % 16 != 0 || (reinterpret_cast<uintptr_t>(w_dev) & 15) != 0) return RQ_E_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(blocks_dev) & 15) != 0 || (reinterpret_cast<uintptr_t>(workspace_dev) & 255) != 0) return RQ_E_ARGUMENT;
    if (N == 0) return 0;
    const QuantWorkspace ws = quant_workspace(type, K, N, wgroup);
    if (workspace_bytes < ws.bytes) return RQ_E_WORKSPACE;
    char *base = reinterpret_cast<char *>(workspace_dev);
    hipStream_t st = (hipStream_t) stream;

    const float *src = w_dev;
    int64_t ld = ldw;
    int32_t len_field = (int32_t) K;
    if (type == RQ_TYPE_W4A4H) {
        // stores Q(W H): the forward rotation of every row, block-diagonal when n_rot < K (reference lines 2701-2710)
        int p, m;
        if (n_rot <= 0 || K % n_rot != 0 || !factor(n_rot, p, m)) return RQ_E_ARGUMENT;
        float *rot = reinterpret_cast<float *>(base + ws.off_rot);
        RotQuantArgs q;
        memset(&q, 0, sizeof q);
        q.x = w_dev;
        q.ldx = ldw;
        q.M = (int) N;
        q.K = (int) K;
        q.rotate = 1;
        q.n_rot = (int) n_rot;
        q.p = p;
        q.m = m;
        q.scale = 1.0f / sqrtf((float) n_rot);
        q.clip = 1.0f;
        q.G = kGroup;
        q.mode = kActRotateOnly;
        q.out_f32 = rot;
        q.ldo = K;
        hipError_t e = launch_rotate_quant(q, st);
        if (e != hipSuccess) return (int) e;
        src = rot;
        ld = K;
        len_field = (int32_t) n_rot;
    }

    const int per_row = wgroup == 0 ? 1 : (int) (K / wgroup);
    SearchArgs s;
    s.x = src;
    s.ld = ld;
    s.per_row = per_row;
    s.segments = N * per_row;
    s.n = (int) (K / per_row);
    s.scale = reinterpret_cast<float *>(base + ws.off_scale);
    const int64_t per_wg = kSearchThreads / 16;
    hipLaunchKernelGGL(rq_wsearch_kernel, dim3((unsigned) ((s.segments + per_wg - 1) / per_wg)), dim3(kSearchThreads), 0,
                       st, s);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int) e;

    EncodeArgs c;
    c.x = src;
    c.ld = ld;
    c.K = (int) K;
    c.per_row = per_row;
    c.groups = wgroup != 0;
    c.scale = s.scale;
    c.blocks = reinterpret_cast<rq_block_w4a4 *>(blocks_dev);
    c.len_field = len_field;
    hipLaunchKernelGGL(rq_wencode_kernel, dim3((unsigned) N), dim3(256), 0, st, c);
    return (int) hipGetLastError();
}

int rq_w4a4_dequantize(int type, const void *blocks_dev, int64_t rows, int64_t K, int64_t n_rot, float *out_dev,
                       int64_t ldo, rq_stream_t stream) {
    if (!blocks_dev || !out_dev) return RQ_E_ARGUMENT;
    if (type < RQ_TYPE_W4A4 || type > RQ_TYPE_A4H) return RQ_E_UNSUPPORTED;
    if (K <= 0 || K % RQ_BLOCK_CODES != 0 || K > RQ_MAX_K || rows < 0 || rows > 0x7fffffff) return RQ_E_UNSUPPORTED;
    if (ldo < K || (ldo * 4) % 16 != 0 || (reinterpret_cast<uintptr_t>(out_dev) & 15) != 0) return RQ_E_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(blocks_dev) & 15) != 0) return RQ_E_ARGUMENT;
    if (rows == 0) return 0;
    DequantArgs a;
    memset(&a, 0, sizeof a);
    a.blocks = reinterpret_cast<const rq_block_w4a4 *>(blocks_dev);
    a.K = (int) K;
    a.act = type == RQ_TYPE_A4 || type == RQ_TYPE_A4H;
    a.rotate = type == RQ_TYPE_W4A4H || type == RQ_TYPE_A4H;
    a.out = out_dev;
    a.ldo = ldo;
    int p = 1, m = 1;
    if (a.rotate) {
        if (n_rot <= 0 || K % n_rot != 0 || !factor(n_rot, p, m)) return RQ_E_ARGUMENT;
        a.n_rot = (int) n_rot;
        a.m = m;
        a.scale = 1.0f / sqrtf((float) n_rot);
    }
    hipStream_t st = (hipStream_t) stream;
    switch (p) {
        case 1:   return (int) launch_dequant<1>(a, rows, st);
        case 12:  return (int) launch_dequant<12>(a, rows, st);
        case 20:  return (int) launch_dequant<20>(a, rows, st);
        case 44:  return (int) launch_dequant<44>(a, rows, st);
        case 60:  return (int) launch_dequant<60>(a, rows, st);
        case 68:  return (int) launch_dequant<68>(a, rows, st);
        case 72:  return (int) launch_dequant<72>(a, rows, st);
        case 84:  return (int) launch_dequant<84>(a, rows, st);
        case 104: return (int) launch_dequant<104>(a, rows, st);
        case 108: return (int) launch_dequant<108>(a, rows, st);
        default:  return RQ_E_UNSUPPORTED;
    }
}

}  // extern "C"
