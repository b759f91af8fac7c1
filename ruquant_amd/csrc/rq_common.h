// Shared definitions of the gfx950 W4A4 / W4A4H MUL_MAT library: memory layouts and launch-side helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/rq_w4a4.h"

namespace rq {

constexpr int kGroup      = 64;   // activation group: one zero point and one multiplier per 64 inputs
constexpr int kPanelRows  = 64;   // weight rows per panel: one wavefront lane per row on the GEMV path
constexpr int kTermShift  = 4;    // RQ_TERM_SHIFT (reference patch line 39)
constexpr int kGemvTokens = 8;    // tokens per GEMV pass; the activation slot stride of the int4 layout
constexpr int kGemmTokens = 128;  // token tile of the MFMA GEMM; int8 activations are padded to it
constexpr int kRangeParts = 32;    // partial maxima of a token's group ranges handed from the activation kernel to the GEMV
constexpr int kSkinnyTokens = 64;   // most tokens of one pass of the skinny MFMA kernel
constexpr int kTwoStepTokens = 40;   // long Paley stages: most tokens whose rotation is spread over several workgroups each
constexpr int kGemvMaxTokens = 64;  // workspaces of up to this many tokens hold the fp32 form too (the GEMV takes up to 4
                                    // tokens whatever the activation group; the skinny path's two-step activation
                                    // side, 5 .. 40 tokens, uses the fp32 rows as an intermediate)

// ---------------------------------------------------------------------------------------------------
// Prepared weight (written once by rq_w4a4_prepare, read by every product kernel).
//
//   codes : n_panels x ng x 2 halves x 64 rows x 16 bytes. Row r of panel P, group g (inputs 64g..64g+63),
//           half h (inputs 32h..32h+31 of the group) is the 16 bytes at
//           (((P * ng + g) * 2 + h) * 64 + r) * 16: four code words in the tensor's own nibble order.
//           A wavefront with lane = row reads one group of its 64 rows as two fully coalesced 1 KiB loads;
//           an MFMA tile of 16 rows reads 256-byte runs.
//   s_w   : n_panels x 64 floats (rows past N are zero).
//   kmul  : n_panels x ng x 64 bytes, the integer weight multiplier of (row, group): 1 for legacy headers.
//   flags : one int32; bit 0 set when any multiplier differs from 1 (kernels branch on it, uniformly). At byte 8 of
//           the section: the device address of the fp6 plane below (0: none), which the fp6 GEMM reads from there.
//   w6    : (unless RQ_GEMM_FP6=0) the same codes once more as fp6 (E2M3) MFMA fragments for wide token batches:
//           n_rtiles x ng x 8 fragments x 1536 bytes. Fragment f of row tile R (rows 256 R + 32 f ..), group g:
//           lane l = row % 32 + 32 * half holds inputs 64 g + 32 half .. + 31 as 32 six-bit values (sign, then the
//           magnitude 0 .. 8: as fp6 the value is code / 8), value j in bits 6j .. 6j+5 of the lane's 24 bytes; bytes
//           0 .. 15 of lane l sit at l * 16, bytes 16 .. 23 at 1024 + l * 8. Rows past N are zero. A weight prepared in
//           place (rq_w4a4_prepare_inplace) keeps the sections above in the tensor's own buffer and this plane in a
//           buffer of its own.
// ---------------------------------------------------------------------------------------------------
constexpr int kFrag6 = 1536;      // bytes of one 32 x 64 fp6 MFMA fragment
constexpr int kRowTile6 = 256;    // rows of one tile of the fp6 plane

// The flag region of a prepared weight: int 0 = the flag word (bit 0: some weight multiplier differs from 1), ints 2-3 =
// the device address of the fp6 plane; behind these 256 bytes, kFlagReplicas copies of the flag word, one per 64-byte
// line, for the one-token kernel, whose 2048 stream wavefronts would otherwise all read the one line.
constexpr int kFlagReplicas = 32;
constexpr size_t kFlagRegionBytes = 256 + 64 * kFlagReplicas;

struct PreparedLayout {
    int64_t K, N;
    int     ng;        // K / 64
    int     n_panels;  // ceil(N / 64)
    int     n_rtiles;  // ceil(N / 256)
    size_t  off_codes, off_sw, off_kmul, off_flags, off_w6, bytes;   // off_w6 == 0: no fp6 plane
};

// whether prepared weights carry the fp6 plane and wide batches use the fp6 MFMA kernel (RQ_GEMM_FP6, default on;
// read once per process)
bool gemm_fp6_enabled();

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

inline PreparedLayout prepared_layout(int64_t K, int64_t N) {
    PreparedLayout L;
    L.K = K;
    L.N = N;
    L.ng = (int) (K / kGroup);
    L.n_panels = (int) ((N + kPanelRows - 1) / kPanelRows);
    L.n_rtiles = (int) ((N + kRowTile6 - 1) / kRowTile6);
    size_t off = 0;
    L.off_codes = off;
    off = align_up(off + (size_t) L.n_panels * L.ng * 2048, 256);
    L.off_sw = off;
    off = align_up(off + (size_t) L.n_panels * kPanelRows * sizeof(float), 256);
    L.off_kmul = off;
    off = align_up(off + (size_t) L.n_panels * L.ng * kPanelRows, 256);
    L.off_flags = off;
    off = align_up(off + kFlagRegionBytes, 256);
    L.off_w6 = 0;
    if (gemm_fp6_enabled()) {
        L.off_w6 = off;
        off = align_up(off + (size_t) L.n_rtiles * L.ng * 8 * kFrag6, 256);
    }
    L.bytes = off;
    return L;
}

// bytes of the fp6 activation plane of Mp tokens (a multiple of 32); the multipliers follow it as [ng][Mp] floats
inline size_t act6_plane_bytes(int ng, int64_t Mp) { return (size_t) ng * (size_t) (Mp / 32) * kFrag6; }

// ---------------------------------------------------------------------------------------------------
// Workspace of one rq_w4a4_mul_mat call.
//
//   u      : Mp floats, the token units (GEMM path; the GEMV derives them itself).
//   act    : GEMV path (M <= 4): the rotated activations as fp32 rows [M][K] followed by the clipped group
//            ranges [M][ng][2] (lo, hi) and [M][32] partial maxima of hi - lo; every GEMV workgroup quantizes
//            the K slice it consumes itself.
//            MFMA paths: two int8 digit planes of m (q - z), [g][digit][quarter][Mp][16 bytes], in the byte order
//            the weight unpack produces (for M <= 64 they follow the fp32 form, which the skinny path may use as
//            an intermediate). The fp6 GEMM (M >= 65) takes one plane of q - z as fp6 MFMA fragments instead,
//            [g][Mp / 32][1536 bytes] (lane = token % 32 + 32 * half, as in the weight plane), followed by the
//            group multipliers as floats 4 m, [g][Mp].
//   cells  : split-K cells [8 or 64 tokens][n_panels * 64], 64 bits each: arrival count above bit 48, exact sum
//            below.
// ---------------------------------------------------------------------------------------------------
constexpr int kPlanUnits = 256;   // compute units the fp6 GEMM's launch plan counts with (MI355X)
constexpr size_t kGemm6CounterBytes = kPlanUnits * sizeof(int32_t);
constexpr size_t kGemm6ScratchBytes = kGemm6CounterBytes + (size_t) kPlanUnits * 256 * 128 * sizeof(int32_t);

struct WorkspaceLayout {
    int64_t Mp;       // tokens padded to the GEMM tile
    int     chunks;   // ceil(M / 8)
    size_t  off_u, off_act, off_lohi, off_rpart, off_i8, off_tot, bytes;
    size_t  tot_ints;   // ints of the split-K cells at off_tot (two per cell)
    size_t  bytes_min;  // what a call needs at the least: `bytes` without the slabs of the fp6 GEMM's K slices (a
                        // workspace between the two runs every tile whole)
};

inline WorkspaceLayout workspace_layout(int64_t K, int64_t N, int64_t M) {
    WorkspaceLayout W;
    const int ng = (int) (K / kGroup);
    const int n_panels = (int) ((N + kPanelRows - 1) / kPanelRows);
    W.Mp = (M + kGemmTokens - 1) / kGemmTokens * kGemmTokens;
    W.chunks = (int) ((M + kGemvTokens - 1) / kGemvTokens);
    size_t off = 0;
    W.off_u = off;
    off = align_up(off + (size_t) W.Mp * sizeof(float), 256);
    const size_t rows = (size_t) M * K * sizeof(float);          // GEMV form (only taken for small M)
    const size_t lohi = (size_t) M * ng * 2 * sizeof(float);
    const size_t act_i8 = (size_t) ng * W.Mp * 128;              // GEMM form
    const bool small = M <= kGemvMaxTokens;
    W.off_act = off;
    W.off_lohi = off + align_up(rows, 256);
    const size_t rpart = (size_t) M * kRangeParts * sizeof(float);
    W.off_rpart = W.off_lohi + align_up(lohi, 256);
    const size_t gemv_form = align_up(rows, 256) + align_up(lohi, 256) + align_up(rpart, 256);
    // small batches may use both forms in one call (rotation with ranges first, digit planes from those)
    W.off_i8 = small ? off + gemv_form : off;
    off = align_up(off + (small ? gemv_form + act_i8 : act_i8), 256);
    W.tot_ints = (size_t) 2 * (M <= kGemvTokens ? kGemvTokens : kSkinnyTokens) * n_panels * kPanelRows;
    W.off_tot = off;
    off = align_up(off + W.tot_ints * sizeof(int32_t), 256);
    W.bytes_min = off;
    if (M > kSkinnyTokens && gemm_fp6_enabled() && kGemm6ScratchBytes > W.tot_ints * sizeof(int32_t)) {
        // the fp6 GEMM's arrival counters and slabs for the tiles it cuts along K: never more than kPlanUnits slices
        // (a constant, so that the workspace grows monotonically with the token count)
        off = align_up(W.off_tot + kGemm6ScratchBytes, 256);
    }
    W.bytes = off;
    return W;
}

// Output forms of the rotate + quantize kernel.
enum ActMode : int {
    kActRotateOnly = 0,  // fp32 rotated rows (rq_w4a4_hadamard)
    kActBlocks     = 1,  // the reference's A4 / A4H block rows (rq_w4a4_quantize_act)
    kActStats      = 2,  // fp32 (rotated) rows + clipped group ranges for the GEMV, which quantizes its own slice
    kActI8         = 3,  // two int8 digits of m (q - z) for the MFMA GEMM
};

struct RotQuantArgs {
    const float *x;      // M rows, stride ldx floats
    int64_t      ldx;
    int          M, K;
    int          rotate; // 0: quantize x as is (W4A4); 1: rotate blocks of n_rot first (W4A4H)
    int          n_rot, p, m;
    float        scale;  // 1 / sqrtf(n_rot), computed on the host exactly as the reference does
    float        clip;
    int          G;      // activation group: 64, or 128 / 256 under RQ_ACT_GROUP (one-workgroup kernel, blocks and digits)
    int          mode;
    // outputs
    float       *out_f32;  int64_t ldo;   // kActRotateOnly, kActStats (may be null when rotate == 0)
    float       *lohi;                    // kActStats: [M][K / 64][2]
    float       *rpart;                   // kActStats: [M][kRangeParts] partial maxima of hi - lo (max of them = R)
    void        *blocks;                  // kActBlocks
    int32_t      len_field;               // kActBlocks: pad[1] of the activation blocks (K or n_rot)
    float       *u;
    uint32_t    *act;                     // kActI8
    // kActI8, single-plane form for the skinny kernel (single == 1): one int8 plane of q - z
    // [g][quarter][Mp][16 bytes] at `act`, and the group multipliers m as bytes [g][Mp] at `mvals`.
    // single == 2: the fp6 fragment plane of q - z at `act` and the multipliers as floats 4 m, [g][Mp], at `m4`
    int          single;
    uint8_t     *mvals;
    float       *m4;
    int          Mp;                      // kActI8: padded token count (rows M..Mp-1 are zero filled)
    // split-K scratch to clear (blocks past the token blocks do it)
    int32_t     *zero_ptr;
    int64_t      zero_ints;
    int          token_blocks;            // number of leading blocks that process tokens
};

hipError_t launch_rotate_quant(const RotQuantArgs &a, hipStream_t stream);

// Activation side of the GEMV path: like launch_rotate_quant with mode kActStats, but spreads one token over
// several workgroups when the rotation allows it (decode latency).
hipError_t launch_rotate_stats(const RotQuantArgs &a, hipStream_t stream);
// per-device set-up of the activation kernels (their dynamic LDS limit); done at first use of a weight, which the
// caller keeps outside graph capture
hipError_t init_rotate_quant_kernels();
hipError_t init_rotate_slab_kernels();
// digit planes (kActI8 form) from the outputs of launch_rotate_stats: rows in out_f32, ranges in lohi / rpart
hipError_t launch_quantize_digits(const RotQuantArgs &a, hipStream_t stream);

// Up to three weights of one K served by one launch of a streaming product kernel (q / k / v, gate / up: reference
// lines 2371-2380). The launch sees one list of panels; panel p belongs to weight w with first[w] <= p < first[w + 1].
constexpr int kMaxFused = 3;
struct WeightSet {
    const uint8_t *codes[kMaxFused];
    const float   *s_w[kMaxFused];
    const uint8_t *kmul[kMaxFused];
    const int32_t *flags[kMaxFused];
    float         *y[kMaxFused];
    int64_t        ldy[kMaxFused];
    int64_t        N[kMaxFused];
    int            first[kMaxFused + 1];   // unused slots hold the total, so no panel selects them
    int            ng;
};

struct FusedWeights {
    int             n;
    const uint8_t  *prepared[kMaxFused];
    PreparedLayout  L[kMaxFused];
    float          *y[kMaxFused];
    int64_t         ldy[kMaxFused];
};

inline WeightSet make_weight_set(const FusedWeights &f) {
    WeightSet w;
    int first = 0;
    for (int i = 0; i < kMaxFused; ++i) {
        const int k = i < f.n ? i : f.n - 1;   // unused slots repeat the last weight (never selected)
        const uint8_t *p = f.prepared[k];
        w.codes[i] = p + f.L[k].off_codes;
        w.s_w[i] = reinterpret_cast<const float *>(p + f.L[k].off_sw);
        w.kmul[i] = p + f.L[k].off_kmul;
        w.flags[i] = reinterpret_cast<const int32_t *>(p + f.L[k].off_flags);
        w.y[i] = f.y[k];
        w.ldy[i] = f.ldy[k];
        w.N[i] = f.L[k].N;
        w.first[i] = first;
        if (i < f.n) first += f.L[i].n_panels;
    }
    w.first[kMaxFused] = first;
    w.ng = f.L[0].ng;
    return w;
}

struct GemvArgs {
    FusedWeights    w;      // y: first token row of this chunk
    const float    *x;      // (rotated) activations of this chunk's first token
    int64_t         ldx;    // row stride in floats
    const float    *lohi;   // clipped group ranges of this chunk's first token, [T][ng][2]
    const float    *rpart;  // partial range maxima of this chunk's first token, [T][kRangeParts]
    int             T;      // 1..4 tokens
    int             gf;     // runs of 64 per activation group: 1, or 2 / 4 under RQ_ACT_GROUP
    int32_t        *tot;    // split-K cells (zero on entry, left zero)
};
hipError_t launch_gemv(const GemvArgs &a, hipStream_t stream);
int gemv_ksplit(int n_panels, int ng);

struct GemmArgs {
    const uint8_t  *prepared;
    PreparedLayout  L;
    const uint8_t  *act8;   // [g][digit][quarter][Mp][16]
    const float    *u;      // [Mp]
    float          *y;
    int64_t         ldy;
    int             M, Mp;
    int             groups_per_fold;   // 1; 2 or 4 when the activation groups are 128 or 256 wide
    void           *cells;             // fp6 form: arrival counters (zero on entry, left zero) and slabs of the tiles cut along K
    bool            weight_multipliers = false;   // fp6 form: the host has seen this weight's flag for multipliers set
};
hipError_t launch_gemm(const GemmArgs &a, hipStream_t stream);
// the fp6 form: act8 = the fp6 fragment plane with the multipliers behind it; the weight needs the fp6 plane
hipError_t launch_gemm6(const GemmArgs &a, hipStream_t stream);
// How a launch of the fp6 form is cut: n_whole tiles (256 rows x 128 tokens) run whole, the rest in `parts` slices of
// K each, which meet in cell_bytes of workspace: kGemm6CounterBytes of arrival counters (one int per cut tile: zero on
// entry, left zero), then one slab of partial totals per slice (needs no clearing).

struct Gemm6Plan {
    int    n_tiles, n_whole, parts;
    size_t cell_bytes;
};
Gemm6Plan gemm6_plan(int64_t N, int64_t M, int ng, int groups_per_fold);

// up to 64 tokens: MFMA arithmetic on a GEMV-shaped weight stream; same operands as the GEMM plus the split-K cells
struct SkinnyArgs {
    FusedWeights    w;
    const uint8_t  *act8;   // [g][digit][quarter][Mp][16], or [g][quarter][Mp][16] with mvals (single plane)
    const uint8_t  *mvals;  // null: two digit planes
    const float    *u;      // [Mp]
    int             M, Mp;
    int             runs_per_group;   // runs of 64 per activation group: 1, or 2 / 4 with RQ_ACT_GROUP = 128 / 256 (single plane only)
    int32_t        *tot;    // split-K cells [M][panels of all weights * 64], 64 bits each
    // a sub-range of the (single) weight's panels, whole K per workgroup, any number of 32-token blocks: the tail of
    // a GEMM launch (rq_gemm.hip). panels == 0: all panels, planned by skinny_plan.
    int             panel0, panels;
};
hipError_t launch_skinny(const SkinnyArgs &a, hipStream_t stream);
struct SkinnyPlan {
    int main_panels;   // leading panels that run as one whole-K workgroup each
    int tail_split;    // K slices (workgroups) per remaining panel
};
SkinnyPlan skinny_plan(int n_panels, int ng, int M, int nz, int runs_per_group = 1);

// One token, one launch (rq_decode.hip): every workgroup rotates and quantizes the token for itself behind its share of
// the weight stream; rows are dealt in quads, whole K per workgroup, so no sums cross workgroups.
constexpr int kDecodeCells = 512;   // most rows of one workgroup: its LDS cells (one per row)
struct DecodeArgs {
    FusedWeights    w;
    const float    *x;        // the token's row
    int             K, rotate, n_rot, p, m;
    float           scale, clip;
    int             compute_units;   // of the device (0: unknown)
};
hipError_t launch_decode(const DecodeArgs &a, hipStream_t stream);
hipError_t init_decode_kernels();
bool decode_takes(int K, int rotate, int p, int m, int act_group);

// Compute units of the current device, read once per device (hipDeviceAttributeMultiprocessorCount); 256 when the
// runtime will not say. The launch plans count rounds of the chip with it.
int device_compute_units();
// XCDs (accelerator dies, each with its own L2) that workgroups are dealt to round robin: 8 on MI355X. Used only to
// place workgroups that share operands on one L2; a different count costs locality, never correctness.
constexpr int kXcds = 8;

hipError_t launch_prepare(const void *blocks, const PreparedLayout &L, uint8_t *prepared, hipStream_t stream);
// in place: `blocks` becomes the prepared sections up to the flags (L.off_flags + 256 bytes, which must fit the
// tensor), the fp6 plane goes to plane6 (may be null); staging: inplace_staging_min(L) bytes at the least
hipError_t launch_prepare_inplace(void *blocks, const PreparedLayout &L, uint8_t *plane6, uint8_t *staging,
                                  size_t staging_bytes, hipStream_t stream);
inline size_t inplace_side_bytes(const PreparedLayout &L) {
    return align_up((size_t) L.n_panels * kPanelRows * sizeof(float), 256) +
           align_up((size_t) L.n_panels * L.ng * kPanelRows, 256) + 256;
}
inline size_t inplace_staging_min(const PreparedLayout &L) {
    return inplace_side_bytes(L) + (size_t) kPanelRows * (L.ng / 4) * RQ_BLOCK_BYTES;
}

bool hadamard_factor(int64_t n, int &p, int &m);

}  // namespace rq
