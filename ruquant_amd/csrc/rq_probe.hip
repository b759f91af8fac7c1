// Machine-peak probes for gfx950 (librq_probe.so), launched through rq_probe() and timed by the caller (bench.py captures a
// batch of launches in a HIP graph and brackets it with events, exactly as it times the operator).
//
// They answer the questions the operator's kernels are judged against:
//   * how fast a plain kernel streams a given number of bytes from HBM (the ceiling of the GEMV),
//   * how fast the matrix pipe runs v_mfma_i32_16x16x64_i8, v_mfma_i32_32x32x32_i8 and v_mfma_f32_32x32x64_f8f6f4 (fp8
//     and fp6 operands) alone (the ceilings of the GEMMs),
//   * whether vector-ALU instructions overlap with MFMAs: in one wavefront, and between two wavefronts that share
//     a SIMD, one issuing only MFMAs and the other only VALU (the per-group integer fold of the W4A4 format is VALU
//     work beside every MFMA),
//   * what an (almost) empty kernel costs per launch inside a graph (the floor of a two-kernel decode op).
// The method follows the reference's rig/membench/stream_bench.hip and rig/bench_valu.cu: dependent chains per
// register so that nothing can be optimized away, independent chains across registers so that issue, not latency,
// is measured.
#include "rq_common.h"

#include "../../include/rq_probe.h"

namespace rq {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

__global__ void __launch_bounds__(256) probe_empty_kernel(int *sink) { (void) sink; }

// Streaming read: workgroup b takes chunks b, b + grid, ... of U KiB-per-wavefront loads (U x 4 KiB per workgroup);
// all U loads of a thread are in flight before the first is consumed. Loads are non-temporal, like the GEMV's.
template <int U>
__global__ void __launch_bounds__(256) probe_stream_kernel(const v4u *__restrict__ p, int64_t chunks, int *sink) {
    unsigned acc = 0;
    for (int64_t c = blockIdx.x; c < chunks; c += gridDim.x) {
        const v4u *q = p + (c * U) * 256 + threadIdx.x;
        v4u v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(q + u * 256);
#pragma unroll
        for (int u = 0; u < U; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x9e3779b9u) sink[0] = 1;   // the probe buffer holds small integers: never true
}

#define RQ_VALU8(OP)                                                                                   \
    asm volatile(OP " %0, %8, %0\n\t" OP " %1, %8, %1\n\t" OP " %2, %8, %2\n\t" OP " %3, %8, %3\n\t"   \
                 OP " %4, %8, %4\n\t" OP " %5, %8, %5\n\t" OP " %6, %8, %6\n\t" OP " %7, %8, %7"       \
                 : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3), "+v"(x4), "+v"(x5), "+v"(x6), "+v"(x7)      \
                 : "v"(y))
// eight dependent chains of v_fma_f32 (x = y * y + x)
#define RQ_FMA8()                                                                                              \
    asm volatile("v_fma_f32 %0, %8, %8, %0\n\tv_fma_f32 %1, %8, %8, %1\n\tv_fma_f32 %2, %8, %8, %2\n\t"          \
                 "v_fma_f32 %3, %8, %8, %3\n\tv_fma_f32 %4, %8, %8, %4\n\tv_fma_f32 %5, %8, %8, %5\n\t"          \
                 "v_fma_f32 %6, %8, %8, %6\n\tv_fma_f32 %7, %8, %8, %7"                                          \
                 : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3), "+v"(x4), "+v"(x5), "+v"(x6), "+v"(x7)              \
                 : "v"(y))
#define RQ_VALU8_OF(OPK)                                  \
    do {                                                  \
        if (OPK == 0) RQ_VALU8("v_add_u32");              \
        if (OPK == 1) RQ_VALU8("v_ashrrev_i32");          \
        if (OPK == 2) RQ_VALU8("v_mul_i32_i24");          \
        if (OPK == 3) RQ_VALU8("v_dot8c_i32_i4");         \
        if (OPK == 4) RQ_FMA8();                          \
        if (OPK == 5) RQ_VALU8("v_add_f32");              \
    } while (0)

// Four independent accumulators of one MFMA form. MK: 0 v_mfma_i32_16x16x64_i8, 1 v_mfma_i32_32x32x32_i8,
// 2 v_mfma_f32_32x32x64_f8f6f4 with fp8 (E4M3) operands, 3 the same with fp6 (E2M3) operands
template <int MK>
struct Mfma;
template <>
struct Mfma<0> {
    v4i c[4] = {};
    __device__ __forceinline__ void step(const v8i &a, const v8i &b, int r) {
        c[r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{ a[0], a[1], a[2], a[3] }, v4i{ b[0], b[1], b[2], b[3] }, c[r], 0, 0, 0);
    }
    __device__ __forceinline__ int sum() const { return c[0][0] + c[1][1] + c[2][2] + c[3][3]; }
};
template <>
struct Mfma<1> {
    v16i c[4] = {};
    __device__ __forceinline__ void step(const v8i &a, const v8i &b, int r) {
        c[r] = __builtin_amdgcn_mfma_i32_32x32x32_i8(v4i{ a[0], a[1], a[2], a[3] }, v4i{ b[0], b[1], b[2], b[3] }, c[r], 0, 0, 0);
    }
    __device__ __forceinline__ int sum() const { return c[0][0] + c[1][1] + c[2][2] + c[3][3]; }
};
template <>
struct Mfma<2> {
    v16f c[4] = {};
    __device__ __forceinline__ void step(const v8i &a, const v8i &b, int r) {
        c[r] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c[r], 0, 0, 0, 0, 0, 0);
    }
    __device__ __forceinline__ int sum() const { return (int) (c[0][0] + c[1][1] + c[2][2] + c[3][3]); }
};
template <>
struct Mfma<3> {
    v16f c[4] = {};
    __device__ __forceinline__ void step(const v8i &a, const v8i &b, int r) {
        c[r] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c[r], 2, 2, 0, 0, 0, 0);
    }
    __device__ __forceinline__ int sum() const { return (int) (c[0][0] + c[1][1] + c[2][2] + c[3][3]); }
};

// role of a wavefront: bit 0 = issues MFMAs, bit 1 = issues VALU. Wavefronts w and w + 4 of a workgroup share a SIMD
// (the hardware deals a workgroup's wavefronts to the four SIMDs in turn; `simd_of` records where each one ran so
// that the caller can check it).
//   SAME  = true : every wavefront interleaves 1 MFMA with NV VALU instructions (roles ignored)
//   SAME  = false: wavefronts 0..3 take role_lo, wavefronts 4..7 role_hi
// OPK: 0 = v_add_u32, 1 = v_ashrrev_i32, 2 = v_mul_i32_i24, 3 = v_dot8c_i32_i4, 4 = v_fma_f32 (eight chains of
// dependent ones), 5 = v_add_f32
template <bool SAME, int NV, int OPK, int MK>
__global__ void __launch_bounds__(512) probe_mix_kernel(int mfma_iters, int valu_iters, int role_lo, int role_hi,
                                                        int *sink, int *simd_of) {
    // operand bits that are small finite values in every format
    v8i a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = ((int) threadIdx.x * 0x01010101 + i) & 0x0b2cb2cb;
        b[i] = ((int) threadIdx.x * 0x00010203 + 7 * i) & 0x0b2cb2cb;
    }
    Mfma<MK> m;
    int x0 = threadIdx.x, x1 = 1, x2 = 2, x3 = 3, x4 = 4, x5 = 5, x6 = 6, x7 = 7, y = threadIdx.x * 3 + 1;
    const int wave = threadIdx.x >> 6;
    if (simd_of != nullptr && blockIdx.x == 0 && (threadIdx.x & 63) == 0) {
        // HW_REG_HW_ID (4), bits 5:4 = SIMD id
        simd_of[wave] = (int) __builtin_amdgcn_s_getreg((2 - 1) << 11 | 4 << 6 | 4);
    }
    if (SAME) {
        for (int it = 0; it < mfma_iters; ++it) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                m.step(a, b, r & 3);
                if (NV >= 8) RQ_VALU8_OF(OPK);
                if (NV >= 16) RQ_VALU8_OF(OPK);
            }
        }
    } else {
        const int role = wave < 4 ? role_lo : role_hi;
        if (role & 1) {
            for (int it = 0; it < mfma_iters; ++it) {
#pragma unroll
                for (int r = 0; r < 16; ++r) m.step(a, b, r & 3);
            }
        }
        if (role & 2) {
            for (int it = 0; it < valu_iters; ++it) {
#pragma unroll
                for (int r = 0; r < 16; ++r) RQ_VALU8_OF(OPK);
            }
        }
    }
    if (m.sum() + x0 + x1 + x2 + x3 + x4 + x5 + x6 + x7 == 0x7fffffff) sink[0] = 1;
}

template <int OPK, int MK>
hipError_t launch_mix(int sub, int grid, int block, int mi, int vi, int *sink, int *simd_of, hipStream_t s) {
    switch (sub) {
        case 0:   // all wavefronts: MFMA only
            hipLaunchKernelGGL((probe_mix_kernel<false, 0, OPK, MK>), dim3(grid), dim3(block), 0, s, mi, vi, 1, 1, sink, simd_of);
            break;
        case 1:   // all wavefronts: VALU only
            hipLaunchKernelGGL((probe_mix_kernel<false, 0, OPK, MK>), dim3(grid), dim3(block), 0, s, mi, vi, 2, 2, sink, simd_of);
            break;
        case 2:   // wavefronts 0..3 MFMA, 4..7 VALU: one of each on every SIMD
            hipLaunchKernelGGL((probe_mix_kernel<false, 0, OPK, MK>), dim3(grid), dim3(block), 0, s, mi, vi, 1, 2, sink, simd_of);
            break;
        case 3:   // wavefronts 0..3 MFMA, 4..7 idle
            hipLaunchKernelGGL((probe_mix_kernel<false, 0, OPK, MK>), dim3(grid), dim3(block), 0, s, mi, vi, 1, 0, sink, simd_of);
            break;
        case 4:   // wavefronts 0..3 idle, 4..7 VALU
            hipLaunchKernelGGL((probe_mix_kernel<false, 0, OPK, MK>), dim3(grid), dim3(block), 0, s, mi, vi, 0, 2, sink, simd_of);
            break;
        case 5:   // one wavefront: 1 MFMA + 8 VALU, interleaved
            hipLaunchKernelGGL((probe_mix_kernel<true, 8, OPK, MK>), dim3(grid), dim3(block), 0, s, mi, vi, 3, 3, sink, simd_of);
            break;
        case 6:   // one wavefront: 1 MFMA + 16 VALU, interleaved
            hipLaunchKernelGGL((probe_mix_kernel<true, 16, OPK, MK>), dim3(grid), dim3(block), 0, s, mi, vi, 3, 3, sink, simd_of);
            break;
        case 7:   // every wavefront: its MFMAs first, then its VALU work (no interleaving inside a wavefront)
            hipLaunchKernelGGL((probe_mix_kernel<false, 0, OPK, MK>), dim3(grid), dim3(block), 0, s, mi, vi, 3, 3, sink, simd_of);
            break;
        default:
            return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace
}  // namespace rq

using namespace rq;

extern "C" int rq_probe(int kind, int64_t a0, int64_t a1, int64_t a2, int64_t a3, void *buf, size_t bytes,
                        void *stream) {
    hipStream_t s = (hipStream_t) stream;
    if (!buf || bytes < 4096 || (reinterpret_cast<uintptr_t>(buf) & 255) != 0) return RQ_E_ARGUMENT;
    int *sink = reinterpret_cast<int *>(buf);   // never written (the conditions above are never true)
    switch (kind) {
        case RQ_PROBE_EMPTY: {
            if (a0 < 1 || a0 > 65536) return RQ_E_ARGUMENT;
            hipLaunchKernelGGL(probe_empty_kernel, dim3((unsigned) a0), dim3(256), 0, s, sink);
            return (int) hipGetLastError();
        }
        case RQ_PROBE_STREAM: {
            // a0 = bytes to read, a1 = 16-byte loads in flight per thread, a2 = workgroups (0: one per chunk)
            const int64_t U = a1;
            if (U != 4 && U != 5 && U != 8 && U != 10 && U != 16 && U != 20) return RQ_E_ARGUMENT;
            const int64_t chunk = U * 4096;
            if (a0 < chunk || a0 % chunk != 0 || (size_t) a0 > bytes) return RQ_E_ARGUMENT;
            const int64_t chunks = a0 / chunk;
            const int64_t grid = a2 > 0 ? a2 : chunks;
            if (grid > (1 << 24)) return RQ_E_ARGUMENT;
            const v4u *p = reinterpret_cast<const v4u *>(buf);
            int *snk = sink;
            switch (U) {
                case 4:  hipLaunchKernelGGL(probe_stream_kernel<4>, dim3((unsigned) grid), dim3(256), 0, s, p, chunks, snk); break;
                case 5:  hipLaunchKernelGGL(probe_stream_kernel<5>, dim3((unsigned) grid), dim3(256), 0, s, p, chunks, snk); break;
                case 8:  hipLaunchKernelGGL(probe_stream_kernel<8>, dim3((unsigned) grid), dim3(256), 0, s, p, chunks, snk); break;
                case 10: hipLaunchKernelGGL(probe_stream_kernel<10>, dim3((unsigned) grid), dim3(256), 0, s, p, chunks, snk); break;
                case 16: hipLaunchKernelGGL(probe_stream_kernel<16>, dim3((unsigned) grid), dim3(256), 0, s, p, chunks, snk); break;
                default: hipLaunchKernelGGL(probe_stream_kernel<20>, dim3((unsigned) grid), dim3(256), 0, s, p, chunks, snk); break;
            }
            return (int) hipGetLastError();
        }
        case RQ_PROBE_MIX: {
            // a0 = sub-kind | VALU instruction << 8, a1 = workgroups, a2 = MFMA iterations (16 MFMAs each),
            // a3 = VALU iterations (128 instructions each). Workgroups are 512 threads (two wavefronts per SIMD), or
            // 256 threads for the one-wavefront-per-SIMD interleaved forms (sub-kinds 5 and 6 with bit 16 set).
            const int sub = (int) (a0 & 0xFF), opk = (int) ((a0 >> 8) & 0xFF), mk = (int) ((a0 >> 20) & 0xF);
            const int block = (a0 >> 16) & 1 ? 256 : 512;
            if (a1 < 1 || a1 > 65536 || a2 < 0 || a3 < 0 || a2 > (1 << 24) || a3 > (1 << 24)) return RQ_E_ARGUMENT;
            int *simd_of = bytes >= 8192 ? sink + 1024 : nullptr;   // 8 ints at byte 4096
#define RQ_MIX(O, M) return (int) launch_mix<O, M>(sub, (int) a1, block, (int) a2, (int) a3, sink, simd_of, s)
            // every VALU instruction beside the int8 16x16x64 form; the other MFMA forms beside v_add_u32 and v_fma_f32
            if (mk == 0) {
                switch (opk) {
                    case 0: RQ_MIX(0, 0);
                    case 1: RQ_MIX(1, 0);
                    case 2: RQ_MIX(2, 0);
                    case 3: RQ_MIX(3, 0);
                    case 4: RQ_MIX(4, 0);
                    case 5: RQ_MIX(5, 0);
                    default: return RQ_E_ARGUMENT;
                }
            }
            if (opk != 0 && opk != 4) return RQ_E_ARGUMENT;
            switch (mk) {
                case 1: if (opk == 0) RQ_MIX(0, 1); else RQ_MIX(4, 1);
                case 2: if (opk == 0) RQ_MIX(0, 2); else RQ_MIX(4, 2);
                case 3: if (opk == 0) RQ_MIX(0, 3); else RQ_MIX(4, 3);
                default: return RQ_E_ARGUMENT;
            }
#undef RQ_MIX
        }
        default:
            return RQ_E_ARGUMENT;
    }
}
