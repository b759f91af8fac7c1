// extern "C" layer of the gfx950 W4A4 / W4A4H MUL_MAT library: argument checks, clip / rotation-length
// resolution, workspace carving and the choice between the GEMV and the MFMA GEMM.
#include "rq_common.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <unordered_map>

// Workspace of rq_w4a4_mul_mat_static: one array per GPU, part of the code object, so that callers which cannot
// allocate device memory (HIP graph capture, serving loops) need none. In host code the array's name is only a handle
// for hipGetSymbolAddress; every use goes through the per-device address that static_scratch() keeps.
static __device__ __align__(256) unsigned char scratch[RQ_STATIC_SCRATCH_BYTES];

namespace rq {

// same search as the reference's ggml_rq_hadamard_factor (reference patch lines 2419-2430): smallest p first
bool hadamard_factor(int64_t n, int &p, int &m) {
    for (int cand = 1; cand <= 128 && cand <= n; ++cand) {
        if (cand > 1) {
            if (cand % 4 != 0 || (cand - 1) % 4 != 3) continue;
            bool prime = cand - 1 >= 2;
            for (int d = 2; d * d <= cand - 1; ++d) {
                if ((cand - 1) % d == 0) {
                    prime = false;
                    break;
                }
            }
            if (!prime) continue;
        }
        if (n % cand != 0) continue;
        const int64_t rest = n / cand;
        if (rest & (rest - 1)) continue;
        p = cand;
        m = (int) rest;
        return true;
    }
    return false;
}

namespace {

// Environment switches are read once per process, as the reference's function-local statics do
// (reference patch lines 2590-2600, 2623-2631).
struct Env {
    float clip[2];   // RQ_ACT_CLIP, RQ_ACT_CLIP_H (falls back to the former); -1 = unset
    int   act_group;
    int   decode_fused;   // one token: the single-launch kernel. RQ_DECODE_FUSED=0 (a debug switch) sends one token
                          // down the rotation kernel + GEMV that serves two and three
    int   gemm_fp6;       // wide batches: the fp6 MFMA kernel on the weight's fp6 plane. RQ_GEMM_FP6=0 leaves the plane
                          // out of prepared weights (0.75 bytes per weight) and runs the int8 MFMA kernel instead
    Env() {
        const char *e = getenv("RQ_ACT_CLIP");
        const char *eh = getenv("RQ_ACT_CLIP_H");
        clip[0] = e ? (float) atof(e) : -1.0f;
        clip[1] = eh ? (float) atof(eh) : clip[0];
        const char *g = getenv("RQ_ACT_GROUP");
        const int v = g ? atoi(g) : 64;
        act_group = v == 128 || v == 256 ? v : 64;
        const char *df = getenv("RQ_DECODE_FUSED");
        decode_fused = df ? atoi(df) != 0 : 1;
        const char *f6 = getenv("RQ_GEMM_FP6");
        gemm_fp6 = f6 ? atoi(f6) != 0 : 1;
    }
};

const Env &env() {
    static const Env e;
    return e;
}

}  // namespace

bool gemm_fp6_enabled() { return env().gemm_fp6 != 0; }

namespace {

// Which prepared weights carry weight multipliers, for the weights this process has prepared: what the wide-batch
// launcher chooses its kernel by. Only a hint: both kernels are right for every tensor (one is slow on tensors with
// multipliers, the other a few percent slower on tensors without), so an address the table does not know, or knows
// from a buffer that has since been reused, costs time at most.
std::mutex g_notes_mutex;
std::unordered_map<const void *, bool> g_notes;

// reads the prepared weight's flag word back (first use synchronizes anyway); under graph capture nothing is noted
void note_multipliers(const void *prepared, const PreparedLayout &L, hipStream_t stream) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    bool known = false, has = false;
    if (hipStreamIsCapturing(stream, &st) == hipSuccess && st == hipStreamCaptureStatusNone) {
        int32_t word = 0;
        if (hipMemcpyAsync(&word, reinterpret_cast<const uint8_t *>(prepared) + L.off_flags, sizeof word, hipMemcpyDeviceToHost, stream) == hipSuccess &&
            hipStreamSynchronize(stream) == hipSuccess) {
            known = true;
            has = (word & 1) != 0;
        }
    }
    std::lock_guard<std::mutex> lock(g_notes_mutex);
    if (known) g_notes[prepared] = has;
    else g_notes.erase(prepared);
}

bool multipliers_noted(const void *prepared) {
    std::lock_guard<std::mutex> lock(g_notes_mutex);
    const auto it = g_notes.find(prepared);
    return it != g_notes.end() && it->second;
}

}  // namespace


namespace {

// Device address of `scratch` on the current device, resolved once per device (each GPU holds its own copy of the
// array at its own address). Returns null with *err set when the runtime refuses.
constexpr int kMaxDevices = 64;
void *static_scratch(hipError_t *err) {
    static std::mutex mu;
    static void *ptr[kMaxDevices] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess && (dev < 0 || dev >= kMaxDevices)) e = hipErrorInvalidDevice;
    if (e != hipSuccess) {
        *err = e;
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (!ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            *err = e != hipSuccess ? e : hipErrorInvalidSymbol;
            return nullptr;
        }
        ptr[dev] = p;
    }
    *err = hipSuccess;
    return ptr[dev];
}

bool is_w_type(int type) { return type == RQ_TYPE_W4A4 || type == RQ_TYPE_W4A4H; }

bool shape_ok(int type, int64_t K, int64_t N, int64_t M) {
    if (!is_w_type(type)) return false;
    if (K <= 0 || K % RQ_BLOCK_CODES != 0 || K > RQ_MAX_K) return false;
    if (N <= 0 || N > (int64_t) 1 << 24) return false;
    if (M < 0 || M > (int64_t) 1 << 24) return false;
    return true;
}

// rotation parameters of one call; returns false where the reference aborts (reference patch lines 2612-2620)
bool rotation_of(int type, int64_t K, int64_t n_rot, int &p, int &m) {
    p = 1;
    m = 1;
    if (type != RQ_TYPE_W4A4H) return true;
    if (n_rot <= 0 || n_rot > K || K % n_rot != 0) return false;
    return hadamard_factor(n_rot, p, m);
}

// Measured crossovers: up to four tokens the dot-product GEMV, from five the skinny MFMA kernel, from 65 the tiled
// MFMA GEMM. (Four tokens, K = 5120, whole call on the GEMV against the skinny kernel: N = 1024 9.1 against 11.4 us,
// N = 5120 11.8 against 12.3, N = 8192 and 17408 the same, N = 34816 26.2 against 25.5: the GEMV's activation side is
// one launch, the skinny kernel's two. Five tokens: 13.7 against 12.3 us at N = 5120, 22.7 against 18.0 at N = 17408.
// The choice depends on the token count only, so that a quantized activation can be shared between weights.)
enum Path { kPathGemv, kPathSkinny, kPathGemm };
constexpr int kGemvMax = 4;
Path path_of(int64_t M) {
    if (M > kSkinnyTokens) return kPathGemm;
    return M <= kGemvMax ? kPathGemv : kPathSkinny;
}

int run_products(int type, int n, const void *const *prepared, int64_t K, const int64_t *N, const float *x,
                 int64_t ldx, int64_t M, float *const *y, const int64_t *ldy, float clip, int64_t n_rot, void *ws,
                 size_t ws_bytes, hipStream_t stream, int stages = 3) {
    if (n < 1 || n > 3 || !prepared || !N || !y || !ldy || !x || !ws) return RQ_E_ARGUMENT;
    int64_t Nmax = 0;
    for (int i = 0; i < n; ++i) {
        if (!shape_ok(type, K, N[i], M)) return RQ_E_UNSUPPORTED;
        if (!prepared[i] || !y[i] || ldy[i] < N[i]) return RQ_E_ARGUMENT;
        if ((reinterpret_cast<uintptr_t>(prepared[i]) & 255) != 0) return RQ_E_WORKSPACE;
        if (N[i] > Nmax) Nmax = N[i];
    }
    if (!(clip > 0.0f) || !isfinite(clip)) return RQ_E_ARGUMENT;
    if (ldx < K || (ldx * 4) % 16 != 0 || (reinterpret_cast<uintptr_t>(x) & 15) != 0) return RQ_E_ARGUMENT;
    int p, m;
    if (!rotation_of(type, K, n_rot, p, m)) return RQ_E_ARGUMENT;
    if (M == 0) return 0;

    // The streaming kernels serve all the weights of a fused call in one launch when the workspace has split-K cells
    // for all their rows (rq_w4a4_workspace_bytes with N = the padded sum); with cells for the largest weight only,
    // the products are launched one after the other. Everything else in the workspace does not depend on N.
    int64_t Nsum = 0;
    for (int i = 0; i < n; ++i) Nsum += (N[i] + kPanelRows - 1) / kPanelRows * kPanelRows;
    WorkspaceLayout W = workspace_layout(K, Nmax, M);
    bool one_launch = false;
    if (n > 1) {
        const WorkspaceLayout Wsum = workspace_layout(K, Nsum, M);
        if (ws_bytes >= Wsum.bytes_min) {
            W = Wsum;
            one_launch = true;
        }
    }
    const int64_t Ncells = one_launch ? Nsum : Nmax;
    if (ws_bytes < W.bytes_min || (reinterpret_cast<uintptr_t>(ws) & 255) != 0) return RQ_E_WORKSPACE;
    const bool have_slabs = ws_bytes >= W.bytes;   // (fp6 GEMM: room to cut leftover tiles along K)
    uint8_t *wsb = reinterpret_cast<uint8_t *>(ws);

    // Activation groups of 128 / 256 (RQ_ACT_GROUP) change where the per-group floor falls. The GEMV and the skinny
    // kernel (single-plane form) fold at that granularity over the same token ranges as with groups of 64 (K = 5120,
    // N = 17408, groups of 128: four tokens 19.6 us on the GEMV, nine 18.3 us on the skinny kernel); beyond 64 tokens
    // the narrow-tile MFMA kernel does (a format variant, not a tuned path).
    const int G = env().act_group;
    if (M == 1 && env().decode_fused && decode_takes((int) K, type == RQ_TYPE_W4A4H, p, m, G)) {
        // one token: rotation, quantizer, product and epilogue in one launch, all weights of a fused call included
        if (!(stages & 2)) return 0;
        DecodeArgs d;
        memset(&d, 0, sizeof d);
        d.w.n = n;
        for (int i = 0; i < n; ++i) {
            d.w.prepared[i] = reinterpret_cast<const uint8_t *>(prepared[i]);
            d.w.L[i] = prepared_layout(K, N[i]);
            d.w.y[i] = y[i];
            d.w.ldy[i] = ldy[i];
        }
        d.x = x;
        d.K = (int) K;
        d.rotate = type == RQ_TYPE_W4A4H;
        d.n_rot = (int) (d.rotate ? n_rot : K);
        d.p = p;
        d.m = m;
        d.scale = 1.0f / sqrtf((float) d.n_rot);
        d.clip = clip;
        d.compute_units = device_compute_units();
        return (int) launch_decode(d, stream);
    }
    const Path path = path_of(M);
    const bool gemm = path != kPathGemv;   // the int8 digit planes feed both MFMA kernels
    RotQuantArgs q;
    memset(&q, 0, sizeof q);
    q.x = x;
    q.ldx = ldx;
    q.M = (int) M;
    q.K = (int) K;
    q.rotate = type == RQ_TYPE_W4A4H;
    q.n_rot = (int) (q.rotate ? n_rot : K);
    q.p = p;
    q.m = m;
    q.scale = 1.0f / sqrtf((float) q.n_rot);
    q.clip = clip;
    q.G = G;   // (the GEMV path takes ranges per run of 64 whatever G is, and folds them itself: set below)
    // Skinny batches with a long Paley stage: one workgroup per token would leave most of the chip idle for tens of
    // microseconds, so the rotation runs spread over workgroups (ranges out) and a second small kernel quantizes.
    // (up to 40 tokens: from there on the one-workgroup-per-token kernel has enough tokens to fill the chip: K = 17408,
    // 64 tokens: 17.9 us against 21.2 us)
    // (the second kernel reads ranges per run of 64: activation groups of 64 only)
    const bool two_step = path == kPathSkinny && G == kGroup && q.rotate && p >= 44 && (m & 63) == 0 && M <= kTwoStepTokens;
    q.mode = gemm && !two_step ? kActI8 : kActStats;
    q.u = reinterpret_cast<float *>(wsb + W.off_u);
    q.act = reinterpret_cast<uint32_t *>(wsb + W.off_i8);
    // token stride of the digit planes: the GEMM pads to its tile; the skinny kernel wants them dense (a padded
    // plane would put all of its reads on the few L2 channels that the used 256 bytes of every 2 KB map to)
    const int act_mp = path == kPathSkinny ? (int) ((M + 15) / 16 * 16) : (int) W.Mp;
    q.Mp = act_mp;
    // the skinny path: one plane of q - z and the multipliers beside it (half the activation bytes per group, which
    // count against the weight bytes a compute unit can have in flight)
    const bool single = path == kPathSkinny;
    const bool fp6 = path == kPathGemm && gemm_fp6_enabled();
    q.single = fp6 ? 2 : single;
    q.m4 = reinterpret_cast<float *>(wsb + W.off_i8 + act6_plane_bytes((int) (K / kGroup), W.Mp));
    q.mvals = reinterpret_cast<uint8_t *>(wsb + W.off_i8) + (size_t) (K / kGroup) * act_mp * 64;
    const float *gemv_x = x;      // what the GEMV quantizes from: the rotated rows, or x itself for W4A4
    int64_t gemv_ldx = ldx;
    if (!gemm) q.G = kGroup;
    if (!gemm || two_step) {
        q.lohi = reinterpret_cast<float *>(wsb + W.off_lohi);
        q.rpart = reinterpret_cast<float *>(wsb + W.off_rpart);
        if (q.rotate) {
            q.out_f32 = reinterpret_cast<float *>(wsb + W.off_act);
            q.ldo = K;
            gemv_x = q.out_f32;
            gemv_ldx = K;
        }
    }
    if (!gemm) {
        q.zero_ptr = reinterpret_cast<int32_t *>(wsb + W.off_tot);
        // only the token slots this call can touch: [min(M, 8)][padded rows] cells of two ints
        const int64_t slots = M < kGemvTokens ? M : kGemvTokens;
        q.zero_ints = 2 * slots * (int64_t) ((Ncells + kPanelRows - 1) / kPanelRows * kPanelRows);
    } else if (path == kPathSkinny) {
        q.zero_ptr = reinterpret_cast<int32_t *>(wsb + W.off_tot);
        q.zero_ints = 2 * M * (int64_t) ((Ncells + kPanelRows - 1) / kPanelRows * kPanelRows);
    } else if (fp6) {
        // the arrival counters of the tiles the fp6 GEMM cuts along K
        q.zero_ptr = reinterpret_cast<int32_t *>(wsb + W.off_tot);
        q.zero_ints = (int64_t) (kGemm6CounterBytes / sizeof(int32_t));
    }
    hipError_t e = hipSuccess;
    if (stages & 1) {
        e = q.mode == kActI8 ? launch_rotate_quant(q, stream) : launch_rotate_stats(q, stream);
        if (e != hipSuccess) return (int) e;
        if (two_step) {
            e = launch_quantize_digits(q, stream);
            if (e != hipSuccess) return (int) e;
        }
    }
    if (!(stages & 2)) return 0;

    // launches: one for all weights, or one per weight
    const int n_launch = one_launch && path != kPathGemm ? 1 : n;
    for (int l = 0; l < n_launch; ++l) {
        FusedWeights fw;
        memset(&fw, 0, sizeof fw);
        fw.n = n_launch == 1 ? n : 1;
        for (int j = 0; j < fw.n; ++j) {
            const int i = n_launch == 1 ? j : l;
            fw.prepared[j] = reinterpret_cast<const uint8_t *>(prepared[i]);
            fw.L[j] = prepared_layout(K, N[i]);
            fw.y[j] = y[i];
            fw.ldy[j] = ldy[i];
        }
        if (path == kPathSkinny) {
            SkinnyArgs g;
            g.w = fw;
            g.act8 = wsb + W.off_i8;
            g.mvals = single ? q.mvals : nullptr;
            g.u = q.u;
            g.M = (int) M;
            g.Mp = act_mp;
            g.runs_per_group = G / kGroup;
            g.tot = reinterpret_cast<int32_t *>(wsb + W.off_tot);
            g.panel0 = 0;
            g.panels = 0;
            e = launch_skinny(g, stream);
            if (e != hipSuccess) return (int) e;
        } else if (gemm) {
            GemmArgs g;
            g.prepared = fw.prepared[0];
            g.L = fw.L[0];
            g.act8 = wsb + W.off_i8;
            g.u = q.u;
            g.y = fw.y[0];
            g.ldy = fw.ldy[0];
            g.M = (int) M;
            g.Mp = (int) W.Mp;
            g.groups_per_fold = G / kGroup;
            g.cells = have_slabs ? wsb + W.off_tot : nullptr;
            g.weight_multipliers = multipliers_noted(fw.prepared[0]);
            e = fp6 ? launch_gemm6(g, stream) : launch_gemm(g, stream);
            if (e != hipSuccess) return (int) e;
        } else {
            for (int c = 0; c < W.chunks; ++c) {
                GemvArgs g;
                g.w = fw;
                for (int j = 0; j < fw.n; ++j) g.w.y[j] = fw.y[j] + (int64_t) c * kGemvTokens * fw.ldy[j];
                g.x = gemv_x + (int64_t) c * kGemvTokens * gemv_ldx;
                g.ldx = gemv_ldx;
                g.lohi = q.lohi + (size_t) c * kGemvTokens * fw.L[0].ng * 2;
                g.rpart = q.rpart + (size_t) c * kGemvTokens * kRangeParts;
                g.T = (int) (M - (int64_t) c * kGemvTokens < kGemvTokens ? M - (int64_t) c * kGemvTokens : kGemvTokens);
                g.gf = G / kGroup;
                g.tot = reinterpret_cast<int32_t *>(wsb + W.off_tot);
                e = launch_gemv(g, stream);
                if (e != hipSuccess) return (int) e;
            }
        }
    }
    return 0;
}

}  // namespace

int device_compute_units() {
    static std::mutex mu;
    static int cus[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    std::lock_guard<std::mutex> lock(mu);
    if (cus[dev] == 0) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
        cus[dev] = v;
    }
    return cus[dev];
}

}  // namespace rq

using namespace rq;

extern "C" {

int rq_w4a4_abi_version(void) { return RQ_ABI_VERSION; }

int rq_w4a4_hadamard_factor(int64_t n, int *p, int *m) {
    int pp = 0, mm = 0;
    if (n <= 0 || !hadamard_factor(n, pp, mm)) return 0;
    if (p) *p = pp;
    if (m) *m = mm;
    return 1;
}

int rq_w4a4_act_group(void) { return env().act_group; }

int rq_w4a4_weight_group(const void *host_block0) {
    if (!host_block0) return 0;
    uint32_t sum = 0;
    memcpy(&sum, reinterpret_cast<const char *>(host_block0) + 4, sizeof sum);
    if ((sum >> 29) == 3u) return 64;
    if ((sum >> 30) == 1u) return 256;
    return 0;
}

int rq_w4a4_supported(int type, int64_t K, int64_t N, int64_t M, int64_t ldx_bytes, int64_t ldy_bytes) {
    if (!shape_ok(type, K, N, M)) return 0;
    if (ldx_bytes % 16 != 0 || ldx_bytes < K * 4) return 0;
    if (ldy_bytes % 4 != 0 || ldy_bytes < N * 4) return 0;
    if (type == RQ_TYPE_W4A4H) {
        int p, m;
        if (!hadamard_factor(K, p, m)) return 0;  // the whole-row rotation must exist (reference line 1986)
    }
    return 1;
}

float rq_w4a4_resolve_clip(const void *host_block0, int type) {
    float tensor_clip = 0.0f;
    if (host_block0) memcpy(&tensor_clip, reinterpret_cast<const char *>(host_block0) + 12, sizeof tensor_clip);
    const float e = env().clip[type == RQ_TYPE_W4A4H || type == RQ_TYPE_A4H ? 1 : 0];
    return e > 0.0f ? e : tensor_clip > 0.0f ? tensor_clip : 1.0f;
}

int64_t rq_w4a4_tensor_rot(const void *host_block0, int type, int64_t K) {
    if (type != RQ_TYPE_W4A4H && type != RQ_TYPE_A4H) return 0;
    if (!host_block0) return -1;
    int32_t n = 0;
    memcpy(&n, reinterpret_cast<const char *>(host_block0) + 8, sizeof n);
    int p, m;
    if (n <= 0 || K % n != 0 || !hadamard_factor(n, p, m)) return -1;
    return n;
}

size_t rq_w4a4_prepared_bytes(int64_t K, int64_t N) {
    if (K <= 0 || K % RQ_BLOCK_CODES != 0 || K > RQ_MAX_K || N <= 0) return 0;
    return prepared_layout(K, N).bytes;
}

int rq_w4a4_prepare(const void *w_blocks_dev, int64_t K, int64_t N, void *prepared_dev, size_t prepared_bytes,
                    rq_stream_t stream) {
    if (!w_blocks_dev || !prepared_dev) return RQ_E_ARGUMENT;
    if (K <= 0 || K % RQ_BLOCK_CODES != 0 || K > RQ_MAX_K || N <= 0 || N > (int64_t) 1 << 24) return RQ_E_UNSUPPORTED;
    const PreparedLayout L = prepared_layout(K, N);
    if (prepared_bytes < L.bytes || (reinterpret_cast<uintptr_t>(prepared_dev) & 255) != 0) return RQ_E_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(w_blocks_dev) & 15) != 0) return RQ_E_ARGUMENT;
    // first use of a weight on this device: also the place for set-up that must not happen under graph capture
    hipError_t e = init_rotate_quant_kernels();
    if (e == hipSuccess) e = init_rotate_slab_kernels();
    if (e == hipSuccess) e = init_decode_kernels();
    if (e == hipSuccess) static_scratch(&e);   // this device's address of the static workspace
    device_compute_units();
    if (e != hipSuccess) return (int) e;
    e = launch_prepare(w_blocks_dev, L, reinterpret_cast<uint8_t *>(prepared_dev), (hipStream_t) stream);
    if (e == hipSuccess) note_multipliers(prepared_dev, L, (hipStream_t) stream);
    return (int) e;
}

size_t rq_w4a4_plane6_bytes(int64_t K, int64_t N) {
    if (K <= 0 || K % RQ_BLOCK_CODES != 0 || K > RQ_MAX_K || N <= 0 || !gemm_fp6_enabled()) return 0;
    const PreparedLayout L = prepared_layout(K, N);
    return L.bytes - L.off_w6;
}

size_t rq_w4a4_inplace_staging_bytes(int64_t K, int64_t N) {
    if (K <= 0 || K % RQ_BLOCK_CODES != 0 || K > RQ_MAX_K || N <= 0) return 0;
    const PreparedLayout L = prepared_layout(K, N);
    // the least, plus room for chunks of 32 panels (fewer launches)
    return align_up(inplace_staging_min(L) + (size_t) 31 * kPanelRows * (L.ng / 4) * RQ_BLOCK_BYTES, 256);
}

int rq_w4a4_prepare_inplace(void *w_blocks_dev, int64_t K, int64_t N, void *plane6_dev, size_t plane6_bytes,
                            void *staging_dev, size_t staging_bytes, rq_stream_t stream) {
    if (!w_blocks_dev || !staging_dev) return RQ_E_ARGUMENT;
    if (K <= 0 || K % RQ_BLOCK_CODES != 0 || K > RQ_MAX_K || N <= 0 || N > (int64_t) 1 << 24) return RQ_E_UNSUPPORTED;
    const PreparedLayout L = prepared_layout(K, N);
    // the sections up to the flag word must fit where the blocks are
    if (L.off_flags + kFlagRegionBytes > (size_t) N * (size_t) (K / RQ_BLOCK_CODES) * RQ_BLOCK_BYTES) return RQ_E_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(w_blocks_dev) & 255) != 0 || (reinterpret_cast<uintptr_t>(staging_dev) & 255) != 0) return RQ_E_WORKSPACE;
    if (staging_bytes < inplace_staging_min(L)) return RQ_E_WORKSPACE;
    if (gemm_fp6_enabled()) {
        // wide batches read the fp6 plane: a weight without one cannot be served
        if (!plane6_dev) return RQ_E_ARGUMENT;
        if (plane6_bytes < L.bytes - L.off_w6 || (reinterpret_cast<uintptr_t>(plane6_dev) & 255) != 0) return RQ_E_WORKSPACE;
    }
    hipError_t e = init_rotate_quant_kernels();
    if (e == hipSuccess) e = init_rotate_slab_kernels();
    if (e == hipSuccess) e = init_decode_kernels();
    if (e == hipSuccess) static_scratch(&e);
    device_compute_units();
    if (e != hipSuccess) return (int) e;
    e = launch_prepare_inplace(w_blocks_dev, L, gemm_fp6_enabled() ? reinterpret_cast<uint8_t *>(plane6_dev) : nullptr,
                               reinterpret_cast<uint8_t *>(staging_dev), staging_bytes, (hipStream_t) stream);
    if (e == hipSuccess) note_multipliers(w_blocks_dev, L, (hipStream_t) stream);
    return (int) e;
}

size_t rq_w4a4_workspace_bytes(int type, int64_t K, int64_t N, int64_t M) {
    if (!shape_ok(type, K, N, M)) return 0;
    return workspace_layout(K, N, M < 1 ? 1 : M).bytes;
}

int rq_w4a4_mul_mat(int type, const void *prepared_dev, int64_t K, int64_t N, const float *x_dev, int64_t ldx,
                    int64_t M, float *y_dev, int64_t ldy, float clip, int64_t n_rot, void *workspace_dev,
                    size_t workspace_bytes, rq_stream_t stream) {
    return run_products(type, 1, &prepared_dev, K, &N, x_dev, ldx, M, &y_dev, &ldy, clip, n_rot, workspace_dev,
                        workspace_bytes, (hipStream_t) stream);
}

int rq_w4a4_mul_mat_static(int type, const void *prepared_dev, int64_t K, int64_t N, const float *x_dev, int64_t ldx,
                           int64_t M, float *y_dev, int64_t ldy, float clip, int64_t n_rot, rq_stream_t stream) {
    if (!shape_ok(type, K, N, M)) return RQ_E_UNSUPPORTED;
    if (workspace_layout(K, N, M < 1 ? 1 : M).bytes_min > (size_t) RQ_STATIC_SCRATCH_BYTES) return RQ_E_LIMIT;
    hipError_t e = hipSuccess;
    void *ws = static_scratch(&e);   // resolved by rq_w4a4_prepare on this device; here only looked up
    if (!ws) return (int) e;
    return run_products(type, 1, &prepared_dev, K, &N, x_dev, ldx, M, &y_dev, &ldy, clip, n_rot, ws,
                        (size_t) RQ_STATIC_SCRATCH_BYTES, (hipStream_t) stream);
}

int rq_w4a4_mul_mat_stages(int type, const void *prepared_dev, int64_t K, int64_t N, const float *x_dev, int64_t ldx,
                           int64_t M, float *y_dev, int64_t ldy, float clip, int64_t n_rot, void *workspace_dev,
                           size_t workspace_bytes, rq_stream_t stream, int stages) {
    if (stages < 1 || stages > 3) return RQ_E_ARGUMENT;
    return run_products(type, 1, &prepared_dev, K, &N, x_dev, ldx, M, &y_dev, &ldy, clip, n_rot, workspace_dev,
                        workspace_bytes, (hipStream_t) stream, stages);
}

int rq_w4a4_stage_mask(int type, int64_t K, int64_t M, int64_t n_rot) {
    if (!is_w_type(type) || K <= 0 || K % RQ_BLOCK_CODES != 0 || K > RQ_MAX_K || M < 1) return 0;
    int p, m;
    if (!rotation_of(type, K, n_rot, p, m)) return 0;
    // one token that the single-launch kernel takes: everything happens in stage 2
    if (M == 1 && env().decode_fused && decode_takes((int) K, type == RQ_TYPE_W4A4H, p, m, env().act_group)) return 2;
    return 3;
}

int rq_w4a4_mul_mat_fused(int type, int n, const void *const *prepared_dev, int64_t K, const int64_t *N,
                          const float *x_dev, int64_t ldx, int64_t M, float *const *y_dev, const int64_t *ldy,
                          float clip, int64_t n_rot, void *workspace_dev, size_t workspace_bytes,
                          rq_stream_t stream) {
    return run_products(type, n, prepared_dev, K, N, x_dev, ldx, M, y_dev, ldy, clip, n_rot, workspace_dev,
                        workspace_bytes, (hipStream_t) stream);
}

int rq_w4a4_hadamard(const float *x_dev, int64_t ldx, int64_t M, int64_t K, int64_t n_rot, float *out_dev,
                     int64_t ldo, rq_stream_t stream) {
    if (!x_dev || !out_dev) return RQ_E_ARGUMENT;
    if (K <= 0 || K % 4 != 0 || K > RQ_MAX_K || M < 0) return RQ_E_UNSUPPORTED;
    if (ldx < K || ldo < K || (ldx * 4) % 16 != 0 || (ldo * 4) % 16 != 0) return RQ_E_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(x_dev) & 15) != 0 || (reinterpret_cast<uintptr_t>(out_dev) & 15) != 0) return RQ_E_ARGUMENT;
    int p, m;
    if (!rotation_of(RQ_TYPE_W4A4H, K, n_rot, p, m)) return RQ_E_ARGUMENT;
    if (M == 0) return 0;
    RotQuantArgs q;
    memset(&q, 0, sizeof q);
    q.x = x_dev;
    q.ldx = ldx;
    q.M = (int) M;
    q.K = (int) K;
    q.rotate = 1;
    q.n_rot = (int) n_rot;
    q.p = p;
    q.m = m;
    q.scale = 1.0f / sqrtf((float) n_rot);
    q.clip = 1.0f;
    q.G = kGroup;
    q.mode = kActRotateOnly;
    q.out_f32 = out_dev;
    q.ldo = ldo;
    return (int) launch_rotate_quant(q, (hipStream_t) stream);
}

int rq_w4a4_quantize_act(int type, const float *x_dev, int64_t ldx, int64_t M, int64_t K, float clip, int64_t n_rot,
                         void *blocks_dev, rq_stream_t stream) {
    if (!x_dev || !blocks_dev) return RQ_E_ARGUMENT;
    if (type != RQ_TYPE_A4 && type != RQ_TYPE_A4H) return RQ_E_UNSUPPORTED;
    if (K <= 0 || K % RQ_BLOCK_CODES != 0 || K > RQ_MAX_K || M < 0) return RQ_E_UNSUPPORTED;
    if (!(clip > 0.0f) || !isfinite(clip)) return RQ_E_ARGUMENT;
    if (ldx < K || (ldx * 4) % 16 != 0 || (reinterpret_cast<uintptr_t>(x_dev) & 15) != 0) return RQ_E_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(blocks_dev) & 15) != 0) return RQ_E_ARGUMENT;
    const bool had = type == RQ_TYPE_A4H;
    int p, m;
    if (!rotation_of(had ? RQ_TYPE_W4A4H : RQ_TYPE_W4A4, K, n_rot, p, m)) return RQ_E_ARGUMENT;
    if (M == 0) return 0;
    RotQuantArgs q;
    memset(&q, 0, sizeof q);
    q.x = x_dev;
    q.ldx = ldx;
    q.M = (int) M;
    q.K = (int) K;
    q.rotate = had;
    q.n_rot = (int) (had ? n_rot : K);
    q.p = p;
    q.m = m;
    q.scale = 1.0f / sqrtf((float) q.n_rot);
    q.clip = clip;
    q.G = env().act_group;
    q.mode = kActBlocks;
    q.blocks = blocks_dev;
    q.len_field = (int32_t) (had ? n_rot : K);
    q.u = nullptr;  // the token unit goes into the block headers
    return (int) launch_rotate_quant(q, (hipStream_t) stream);
}

}  // extern "C"
