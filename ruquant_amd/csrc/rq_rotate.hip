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

__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fminf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

template <int P>
__global__ void __launch_bounds__(kRT) rq_rotate_slab_kernel(const RotQuantArgs a, int slabs) {
    extern __shared__ __align__(16) float buf[];

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

    const int t = blockIdx.x / slabs, slab = blockIdx.x - t * slabs;
    const int K = a.K, m = a.m, ng = K / kGroup;
    const int lm = __ffs(m) - 1;
    const int wave = tid >> 6, lane = tid & 63;

    const float *xr = a.x + (int64_t) t * a.ldx;
    load_row<kRT>(buf, xr, K, tid);
    __syncthreads();
    fwht_row(buf, K, lm, tid, kRT);

    float *out = a.out_f32 + (int64_t) t * a.ldo;
    float *lh = a.lohi + (size_t) t * ng * 2;
    float rmax = 0.0f;   // widest range this wavefront has produced

    if constexpr (P == 1) {
        // no Paley stage: the slab is a share of the row's runs of 64
        const int runs = K >> 6;
        for (int r = slab * (kRT / 64) + wave; r < runs; r += slabs * (kRT / 64)) {
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
        // wave-items = (rotation block, slice of four output chunks) for this slab's 64 columns; a wavefront takes a
        // contiguous block of items so that it stays in one slice's straight-line code where it can
        const int n_rb = K / a.n_rot;
        const int n_items = n_rb * (P / 4);
        const int per_wave = (n_items + kRT / 64 - 1) / (kRT / 64);
        const int pm = m + (m >> 4);
        for (int it = 0; it < per_wave; ++it) {
            const int wi = wave * per_wave + it;
            if (wi >= n_items) break;
            const int s = wi / n_rb, rb = wi - s * n_rb;
            const int b0 = rb * a.n_rot + 64 * slab + lane;
            const float *src = buf + padi(b0);
            float col[P];
#pragma unroll
            for (int i = 0; i < P; ++i) col[i] = src[i * pm];
            float res[4];
            paley_pick<P>(s, col, res);
#pragma unroll
            for (int o = 0; o < 4; ++o) {
                const int idx = b0 + (4 * s + o) * m;
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
    // slot (slab, wave) of the token's partial maxima; slots nobody owns are written as zero by slab 0
    if (lane == 0) a.rpart[(size_t) t * kRangeParts + slab * (kRT / 64) + wave] = rmax;
    if (slab == 0 && tid >= slabs * (kRT / 64) && tid < kRangeParts) a.rpart[(size_t) t * kRangeParts + tid] = 0.0f;
}

template <int P>
hipError_t launch_slab(const RotQuantArgs &a, hipStream_t stream) {
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&rq_rotate_slab_kernel<P>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 64);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    // one slab per 64 columns of a chunk; without a Paley stage, a few workgroups share the row's runs
    int slabs = P > 1 ? a.m / 64 : (a.K >= 4096 ? 4 : 1);
    if (slabs * (kRT / 64) > kRangeParts) return launch_rotate_quant(a, stream);   // more slabs than range slots
    const int zero_blocks = (int) ((a.zero_ints + (int64_t) kRT * 4 - 1) / ((int64_t) kRT * 4));
    RotQuantArgs b = a;
    b.token_blocks = a.M * slabs;
    const size_t lds = (size_t) (a.K + (a.K >> 4) + 1) * sizeof(float);
    hipLaunchKernelGGL((rq_rotate_slab_kernel<P>), dim3(b.token_blocks + zero_blocks), dim3(kRT), lds, stream, b, slabs);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_rotate_stats(const RotQuantArgs &a, hipStream_t stream) {
    // The slab kernel needs whole groups per (chunk, slab): chunks that are a multiple of 64 long. Everything else,
    // and unrotated activations (ranges only), goes through the one-workgroup-per-token kernel.
    if (!a.rotate || (a.m & 63) != 0 || a.M > 16) return launch_rotate_quant(a, stream);
    switch (a.p) {
        case 1:  return launch_slab<1>(a, stream);
        case 12: return launch_slab<12>(a, stream);
        case 20: return launch_slab<20>(a, stream);
        case 68: return launch_slab<68>(a, stream);
        default: return launch_rotate_quant(a, stream);
    }
}

}  // namespace rq
