// Host-side tools for the on-disk form of W4A4 / W4A4H tensors: the packers the reference's converter uses to build
// blocks from codes, scales and weight multipliers, the two header writers that set what the kernels read from
// block 0, and the plain weight dequantizer. No GPU work; they live in the library so that a host written in any
// language gets the same bytes.
#include "../../include/rq_w4a4.h"

#include <string.h>

namespace {

// element 8w+j of a block in bits [4j+3:4j] of qs[w], two's-complement int4 (reference patch lines 26-37)
inline int code_of(uint32_t word, int j) { return (int) (((word >> (4 * j)) & 0xF) ^ 8) - 8; }

// the reference's RQ_W_MULT_G (patch lines 40-43): multiplier of 64-wide group g of a block
inline int weight_mult(int32_t sum, int g) {
    const uint32_t s = (uint32_t) sum;
    if ((s >> 29) == 3) return (int) ((s >> (4 * g)) & 0xF);
    if ((s >> 30) == 1) return (int) (s & 0xF);
    return 1;
}

}  // namespace

extern "C" {

// src/gptq.rs:210-231 (`pack`)
int rq_w4a4_pack(const int8_t *codes, const float *scales, int64_t N, int64_t K, void *blocks) {
    if (!codes || !scales || !blocks) return RQ_E_ARGUMENT;
    if (N < 0 || K <= 0 || K % RQ_BLOCK_CODES != 0) return RQ_E_UNSUPPORTED;
    const int64_t nb = K / RQ_BLOCK_CODES;
    rq_block_w4a4 *out = reinterpret_cast<rq_block_w4a4 *>(blocks);
    for (int64_t r = 0; r < N; ++r) {
        const int8_t *c = codes + r * K;
        int32_t sum = 0;
        for (int64_t i = 0; i < K; ++i) sum += c[i];
        for (int64_t b = 0; b < nb; ++b) {
            rq_block_w4a4 &blk = out[r * nb + b];
            blk.d = scales[r];
            blk.sum = sum;
            blk.pad[0] = (int32_t) K;
            blk.pad[1] = 0;
            for (int w = 0; w < 32; ++w) {
                uint32_t word = 0;
                for (int j = 0; j < 8; ++j) word |= ((uint32_t) c[b * RQ_BLOCK_CODES + 8 * w + j] & 0xF) << (4 * j);
                blk.qs[w] = word;
            }
        }
    }
    return 0;
}

// src/gptq.rs:193-207 (`pack_groups`): one multiplier per block (groups of 256) or four (groups of 64)
int rq_w4a4_pack_groups(const int8_t *codes, const float *units, const uint8_t *mults, int mults_per_block, int64_t N,
                        int64_t K, void *blocks) {
    if (!mults || (mults_per_block != 1 && mults_per_block != 4)) return RQ_E_ARGUMENT;
    const int rc = rq_w4a4_pack(codes, units, N, K, blocks);
    if (rc != 0) return rc;
    const int64_t n_blocks = N * (K / RQ_BLOCK_CODES);
    rq_block_w4a4 *out = reinterpret_cast<rq_block_w4a4 *>(blocks);
    for (int64_t b = 0; b < n_blocks; ++b) {
        const uint8_t *m = mults + b * mults_per_block;
        int32_t v;
        if (mults_per_block == 1) {
            v = (int32_t) (1u << 30 | m[0]);
        } else {
            uint32_t a = 3u << 29;
            for (int g = 0; g < 4; ++g) a |= (uint32_t) m[g] << (4 * g);
            v = (int32_t) a;
        }
        out[b].sum = v;
    }
    return 0;
}

// src/convert.rs:876-878 (`ruquant setclip`): pad[1] of every block; 0 clears it
void rq_w4a4_set_clip(void *blocks, int64_t n_blocks, float clip) {
    rq_block_w4a4 *b = reinterpret_cast<rq_block_w4a4 *>(blocks);
    for (int64_t i = 0; i < n_blocks; ++i) memcpy(&b[i].pad[1], &clip, 4);
}

// src/convert.rs:99-101 (`set_rot_len`): the Hadamard length a W4A4H tensor's kernels read, pad[0] of every block
void rq_w4a4_set_rot_len(void *blocks, int64_t n_blocks, int32_t n) {
    rq_block_w4a4 *b = reinterpret_cast<rq_block_w4a4 *>(blocks);
    for (int64_t i = 0; i < n_blocks; ++i) b[i].pad[0] = n;
}

// dequantize_row_w4a4 (reference patch lines 2738-2742): y = code * ((float) k_g * d), rows of K values
int rq_w4a4_dequantize_rows(const void *blocks, int64_t N, int64_t K, float *out) {
    if (!blocks || !out) return RQ_E_ARGUMENT;
    if (N < 0 || K <= 0 || K % RQ_BLOCK_CODES != 0) return RQ_E_UNSUPPORTED;
    const rq_block_w4a4 *in = reinterpret_cast<const rq_block_w4a4 *>(blocks);
    const int64_t n_blocks = N * (K / RQ_BLOCK_CODES);
    for (int64_t b = 0; b < n_blocks; ++b) {
        for (int w = 0; w < 32; ++w) {
            const float scale = (float) weight_mult(in[b].sum, w / 8) * in[b].d;
            for (int j = 0; j < 8; ++j) out[b * RQ_BLOCK_CODES + 8 * w + j] = (float) code_of(in[b].qs[w], j) * scale;
        }
    }
    return 0;
}

}  // extern "C"
