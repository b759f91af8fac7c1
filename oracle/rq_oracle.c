/*
 * CPU oracle for the ruquant W4A4 / W4A4H MUL_MAT path: see rq_oracle.h.
 * TEST INFRASTRUCTURE ONLY: never linked into or called from the shipped HIP library.
 *
 * Pinned against: the known answers of the compiled reference (hashes of Hadamard outputs, activation
 * blocks and vec_dot results at K = 256 .. 17408, three clips), closed forms (all-zero row,
 * non-negative row), H H^T = I, the dense +-1 matrix product on small integers, and brute-force integer
 * dot products. The W4A4 weight dequantizer is pinned by the assertion the reference's own test makes about
 * ggml's to_float (src/gptq.rs:313-319: code * (multiplier * unit), both multiplier encodings). The weight-side
 * quantizer (rqo_quantize_row_w*) has no reference-made vector; it is pinned by the reference's second statement of
 * the same row search and code rule (int4_scale and code, src/gptq.rs:13-38, restated from the Rust text and
 * compared bit for bit), by the minimum property of the chosen ratio in exact rational arithmetic, by what the
 * reference's test asserts about weight groups (src/gptq.rs:303-311) and by round trips through the dequantizers
 * (tests/test_oracle_weight_quant.py). The activation dequantizers (rqo_dequantize_row_a) have no reference-made
 * vector either; they are pinned by the reference's second statement of quantize-then-dequantize for grouped
 * activations (fake_quant_groups, src/hessian.rs:70-92), restated from the Rust text: codes, zero points and
 * multipliers must agree exactly, the values bit for bit under the C line's association (q - z) * (m * u) and
 * within one unit in the last place under the Rust line's ((q - z) * m) * u; plus the rotation round trip for A4H
 * (tests/test_oracle_act_dequant.py).
 *
 * Build: gcc -O3 -ffp-contract=off (no -ffast-math).
 */
#include "rq_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdatomic.h>
#include <stdlib.h>
#include <string.h>

#define BLK 256          /* codes per block, QK_W4A4 (P:38) */
#define TERM_SHIFT 4     /* RQ_TERM_SHIFT (P:39) */
#define AG_MAX 255       /* RQ_AG_M (P:2487) */

/* ------------------------------------------------------------------ factorization and Paley matrix */

static int is_prime(int q) {
    if (q < 2) return 0;
    for (int d = 2; d * d <= q; ++d) {
        if (q % d == 0) return 0;
    }
    return 1;
}

/* P:2419-2430: the smallest admissible p wins. */
int rqo_hadamard_factor(int64_t n, int *p, int *m) {
    for (int cand = 1; cand <= 128 && cand <= n; ++cand) {
        const int paley_ok = cand % 4 == 0 && is_prime(cand - 1) && (cand - 1) % 4 == 3;
        if (cand > 1 && !paley_ok) continue;
        if (n % cand) continue;
        const int64_t rest = n / cand;
        if (rest & (rest - 1)) continue;
        *p = cand;
        *m = (int) rest;
        return 1;
    }
    return 0;
}

/* P:2433-2448: A = I + S; S has a zero diagonal, first row +1, first column -1, and the quadratic
 * character of (j - i) mod q elsewhere, q = p - 1. */
void rqo_paley(int p, int8_t *A) {
    const int q = p - 1;
    int8_t chi[128];
    chi[0] = 0;
    for (int r = 1; r < q; ++r) chi[r] = -1;
    for (int r = 1; r < q; ++r) chi[(r * r) % q] = 1;
    for (int i = 0; i < p; ++i) {
        for (int j = 0; j < p; ++j) {
            int s;
            if (i == 0) {
                s = j ? 1 : 0;
            } else if (j == 0) {
                s = -1;
            } else {
                s = chi[(((j - i) % q) + q) % q];
            }
            A[i * p + j] = (int8_t) (s + (i == j));
        }
    }
}

/* P:2450-2485. Order of operations is the contract:
 *  1. per chunk of m: butterflies with stride 1, 2, 4, ...; lower index <- a + b, upper <- a - b;
 *  2. per column j across the p chunks: out[a] = ((0 +- c0) +- c1) ... +- c_{p-1}, i ascending;
 *  3. every element times 1/sqrtf(n). */
void rqo_hadamard(float *x, int64_t n, int transpose) {
    int p, m;
    if (!rqo_hadamard_factor(n, &p, &m)) abort();
    for (int c = 0; c < p; ++c) {
        float *v = x + (int64_t) c * m;
        for (int h = 1; h < m; h *= 2) {
            for (int base = 0; base < m; base += 2 * h) {
                for (int k = base; k < base + h; ++k) {
                    const float lo = v[k], up = v[k + h];
                    v[k]     = lo + up;
                    v[k + h] = lo - up;
                }
            }
        }
    }
    if (p > 1) {
        static _Thread_local int8_t A[128 * 128];
        float col[128];
        rqo_paley(p, A);
        for (int j = 0; j < m; ++j) {
            for (int i = 0; i < p; ++i) col[i] = x[(int64_t) i * m + j];
            for (int a = 0; a < p; ++a) {
                float acc = 0.0f;
                for (int i = 0; i < p; ++i) {
                    const int8_t sign = transpose ? A[a * p + i] : A[i * p + a];
                    acc = sign > 0 ? acc + col[i] : acc - col[i];
                }
                x[(int64_t) a * m + j] = acc;
            }
        }
    }
    const float scale = 1.0f / sqrtf((float) n);
    for (int64_t i = 0; i < n; ++i) x[i] *= scale;
}

/* ------------------------------------------------------------------ clip / rotation-length resolution */

float rqo_resolve_clip(float env_clip, float tensor_clip) {
    /* P:2598-2599: environment first, then the tensor's header, then 1 */
    if (env_clip > 0.0f) return env_clip;
    if (tensor_clip > 0.0f) return tensor_clip;
    return 1.0f;
}

float rqo_env_clip(int hadamard) {
    const char *plain = getenv("RQ_ACT_CLIP");
    const char *had   = getenv("RQ_ACT_CLIP_H");
    const float e0 = plain ? (float) atof(plain) : -1.0f;
    const float e1 = had ? (float) atof(had) : e0;
    return hadamard ? e1 : e0;
}

float rqo_tensor_clip(const void *blocks) {
    float c;
    memcpy(&c, &((const rqo_block *) blocks)->pad[1], sizeof c);
    return c;
}

int64_t rqo_rot_check(int32_t n, int64_t k) {
    int p, m;
    if (n <= 0 || k % n != 0 || !rqo_hadamard_factor(n, &p, &m)) return -1;
    return n;
}

/* ------------------------------------------------------------------ activation quantizer */

static inline float clampf(float v, float lo, float hi) {
    return fminf(fmaxf(v, lo), hi);
}

/* P:2639-2679. Per group g: range [min(x,0), max(x,0)] * clip; R = widest range over the token
 * (2 if all zero); u = R / 3825; m_g = clamp(ceil((range_g * 255) / R), 1, 255); inv = 1 / (m_g * u);
 * z_g = clamp(rint(-lo_g * inv), 0, 15); q = clamp(rint(x * inv) + z_g, 0, 15); code = q - 8. */
void rqo_quantize_row_a(const float *x, rqo_block *y, int64_t k, float clip, int G) {
    if (k % BLK) abort();
    const int lsub = G == 64 ? 2 : G == 128 ? 1 : 0;
    const int64_t ng = k / G, nb = k / BLK;
    float *lo = (float *) malloc((size_t) ng * 2 * sizeof(float));
    float *hi = lo + ng;
    float R = 0.0f;
    for (int64_t g = 0; g < ng; ++g) {
        float mn = 0.0f, mx = 0.0f;
        for (int i = 0; i < G; ++i) {
            mn = fminf(mn, x[g * G + i]);
            mx = fmaxf(mx, x[g * G + i]);
        }
        lo[g] = mn * clip;
        hi[g] = mx * clip;
        R = fmaxf(R, hi[g] - lo[g]);
    }
    if (R == 0.0f) R = 2.0f;
    const float u = R / (15.0f * AG_MAX);
    for (int64_t b = 0; b < nb; ++b) {
        y[b].d = u;
        y[b].sum = lsub << 16;
        y[b].pad[0] = 0;
        y[b].pad[1] = (int32_t) k;
    }
    const int per_block = BLK / G;
    for (int64_t g = 0; g < ng; ++g) {
        const float range = hi[g] - lo[g];
        const int mult = (int) clampf(ceilf((range * (float) AG_MAX) / R), 1.0f, (float) AG_MAX);
        const float inv = 1.0f / ((float) mult * u);
        const float zf = clampf(rintf(-lo[g] * inv), 0.0f, 15.0f);
        rqo_block *blk = &y[g / per_block];
        const int sg = (int) (g % per_block);
        blk->sum |= (int32_t) zf << (4 * sg);
        blk->pad[0] = (int32_t) ((uint32_t) blk->pad[0] | ((uint32_t) mult << (8 * sg)));
        const float *xg = x + g * G;
        for (int w = 0; w < G / 8; ++w) {
            uint32_t word = 0;
            for (int j = 0; j < 8; ++j) {
                const float q = clampf(rintf(xg[8 * w + j] * inv) + zf, 0.0f, 15.0f);
                word |= (uint32_t) (((int) q - 8) & 0xF) << (4 * j);
            }
            blk->qs[sg * (G / 8) + w] = word;
        }
    }
    free(lo);
}

void rqo_quantize_row_a4h(const float *x, rqo_block *y, int64_t k, float clip, int64_t n_rot, int G) {
    if (n_rot <= 0 || k % n_rot) abort();
    float *t = (float *) malloc((size_t) k * sizeof(float));
    memcpy(t, x, (size_t) k * sizeof(float));
    for (int64_t off = 0; off < k; off += n_rot) rqo_hadamard(t + off, n_rot, 0);
    rqo_quantize_row_a(t, y, k, clip, G);
    for (int64_t b = 0; b < k / BLK; ++b) y[b].pad[1] = (int32_t) n_rot;
    free(t);
}

/* ------------------------------------------------------------------ vec_dot */

static inline int32_t nibble(uint32_t word, int j) {
    return (int32_t) (((word >> (4 * j)) & 0xF) << 28) >> 28;
}

/* weight multiplier of 64-wide group g of a block (P:40-43) */
static inline int32_t w_mult(int32_t sum, int g) {
    const uint32_t s = (uint32_t) sum;
    if ((s >> 29) == 3u) return (int32_t) ((s >> (4 * g)) & 0xF);
    if ((s >> 30) == 1u) return (int32_t) (s & 0xF);
    return 1;
}

/* P:148-177. total = sum over activation groups of (k * m * (acc + (8 - z) * colsum)) >> 4, then
 * y = ((float(total) * 16) * u) * s_w. */
void rqo_vec_dot(int64_t n, float *s, const rqo_block *w, const rqo_block *a) {
    const int64_t nb = n / BLK;
    int32_t total = 0;
    for (int64_t b = 0; b < nb; ++b) {
        const int lsub = (a[b].sum >> 16) & 3;
        const int words = (BLK / 8) >> lsub;
        for (int sg = 0; sg < (1 << lsub); ++sg) {
            int32_t acc = 0, colsum = 0;
            for (int wi = sg * words; wi < (sg + 1) * words; ++wi) {
                const uint32_t ww = w[b].qs[wi], aw = a[b].qs[wi];
                for (int j = 0; j < 8; ++j) {
                    const int32_t cw = nibble(ww, j);
                    acc += cw * nibble(aw, j);
                    colsum += cw;
                }
            }
            const int32_t z = (a[b].sum >> (4 * sg)) & 0xF;
            const int32_t mult = (int32_t) (((uint32_t) a[b].pad[0] >> (8 * sg)) & 0xFF);
            const int32_t kw = w_mult(w[b].sum, sg << (2 - lsub));
            total += (kw * mult * (acc + (8 - z) * colsum)) >> TERM_SHIFT;
        }
    }
    *s = (((float) total * (float) (1 << TERM_SHIFT)) * a[0].d) * w[0].d;
}

/* ------------------------------------------------------------------ weight-side quantizer (test weights) */

/* P:2505-2524: scale = amax * ratio / 7, ratio = 1 - 0.025 r for r = 0..12, least squared rounding error. */
static float scale_search(const float *x, int64_t n) {
    float amax = 0.0f;
    for (int64_t i = 0; i < n; ++i) amax = fmaxf(amax, fabsf(x[i]));
    if (!(amax > 0.0f)) return 0.0f;
    float best = 0.0f;
    double best_err = INFINITY;
    for (int r = 0; r < 13; ++r) {
        const float s = amax * (1.0f - 0.025f * r) / 7.0f;
        double err = 0.0;
        for (int64_t i = 0; i < n; ++i) {
            const float q = clampf(rintf(x[i] / s), -8.0f, 7.0f);
            const double e = (double) (q * s) - (double) x[i];
            err += e * e;
        }
        if (err < best_err) {
            best_err = err;
            best = s;
        }
    }
    return best;
}

static void pack_row(rqo_block *y, const int8_t *codes, int64_t k, float d, int32_t sum) {
    for (int64_t b = 0; b < k / BLK; ++b) {
        y[b].d = d;
        y[b].sum = sum;
        y[b].pad[0] = (int32_t) k;
        y[b].pad[1] = 0;
        for (int w = 0; w < BLK / 8; ++w) {
            uint32_t word = 0;
            for (int j = 0; j < 8; ++j) word |= (uint32_t) (codes[b * BLK + 8 * w + j] & 0xF) << (4 * j);
            y[b].qs[w] = word;
        }
    }
}

/* P:2540-2580 */
void rqo_quantize_row_w(const float *x, rqo_block *y, int64_t k, int wgroup) {
    if (k % BLK) abort();
    int8_t *codes = (int8_t *) malloc((size_t) k);
    if (!wgroup) {
        const float s = scale_search(x, k);
        int32_t sum = 0;
        for (int64_t i = 0; i < k; ++i) {
            codes[i] = s > 0.0f ? (int8_t) clampf(rintf(x[i] / s), -8.0f, 7.0f) : 0;
            sum += codes[i];
        }
        pack_row(y, codes, k, s, sum);
        free(codes);
        return;
    }
    const int gs = wgroup == 64 ? 64 : BLK;
    const int ng = (int) (k / gs);
    float *sg = (float *) malloc((size_t) ng * sizeof(float));
    int32_t *kg = (int32_t *) malloc((size_t) ng * sizeof(int32_t));
    float smax = 0.0f;
    for (int g = 0; g < ng; ++g) {
        sg[g] = scale_search(x + (int64_t) g * gs, gs);
        smax = fmaxf(smax, sg[g]);
    }
    const float unit = smax / 15.0f;
    for (int g = 0; g < ng; ++g) {
        kg[g] = unit > 0.0f ? (int32_t) clampf(rintf(sg[g] / unit), 1.0f, 15.0f) : 1;
        const float s = (float) kg[g] * unit;
        for (int i = 0; i < gs; ++i) {
            const float v = x[(int64_t) g * gs + i];
            codes[(int64_t) g * gs + i] = s > 0.0f ? (int8_t) clampf(rintf(v / s), -8.0f, 7.0f) : 0;
        }
    }
    pack_row(y, codes, k, unit, 0);
    for (int64_t b = 0; b < k / BLK; ++b) {
        y[b].sum = gs == BLK ? (int32_t) (1u << 30 | (uint32_t) kg[b])
                             : (int32_t) (3u << 29 | (uint32_t) kg[4 * b] | (uint32_t) kg[4 * b + 1] << 4 |
                                          (uint32_t) kg[4 * b + 2] << 8 | (uint32_t) kg[4 * b + 3] << 12);
    }
    free(kg);
    free(sg);
    free(codes);
}

/* P:2701-2710: the stored row is Q(W H); pad[0] carries the rotation length */
void rqo_quantize_row_w4a4h(const float *x, rqo_block *y, int64_t k, int64_t n_rot, int wgroup) {
    float *t = (float *) malloc((size_t) k * sizeof(float));
    memcpy(t, x, (size_t) k * sizeof(float));
    for (int64_t off = 0; off < k; off += n_rot) rqo_hadamard(t + off, n_rot, 0);
    rqo_quantize_row_w(t, y, k, wgroup);
    for (int64_t b = 0; b < k / BLK; ++b) y[b].pad[0] = (int32_t) n_rot;
    free(t);
}

static void unrotate(const rqo_block *x, float *y, int64_t k, int which) {
    for (int64_t off = 0; off < k;) {
        const int64_t n = x[off / BLK].pad[which];
        if (n <= 0 || off + n > k) abort();
        rqo_hadamard(y + off, n, 1);
        off += n;
    }
}

/* P:2738-2742, P:2766-2769 */
void rqo_dequantize_row_w(const rqo_block *x, float *y, int64_t k, int hadamard) {
    for (int64_t b = 0; b < k / BLK; ++b) {
        for (int w = 0; w < BLK / 8; ++w) {
            for (int j = 0; j < 8; ++j) {
                y[b * BLK + 8 * w + j] = nibble(x[b].qs[w], j) * ((float) w_mult(x[b].sum, w / 8) * x[b].d);
            }
        }
    }
    if (hadamard) unrotate(x, y, k, 0);
}

/* P:2744-2753, P:2771-2774 */
void rqo_dequantize_row_a(const rqo_block *x, float *y, int64_t k, int hadamard) {
    for (int64_t b = 0; b < k / BLK; ++b) {
        const int lsub = (x[b].sum >> 16) & 3;
        for (int w = 0; w < BLK / 8; ++w) {
            const int sg = (8 * w) >> (8 - lsub);
            const int z = (x[b].sum >> (4 * sg)) & 0xF;
            const int mult = (int) (((uint32_t) x[b].pad[0] >> (8 * sg)) & 0xFF);
            for (int j = 0; j < 8; ++j) {
                y[b * BLK + 8 * w + j] = (nibble(x[b].qs[w], j) + 8 - z) * ((float) mult * x[b].d);
            }
        }
    }
    if (hadamard) unrotate(x, y, k, 1);
}

/* ------------------------------------------------------------------ MUL_MAT (P:92-132, P:71-82) */

typedef struct {
    int type, G, n_threads;
    const rqo_block *w;
    int64_t K, N, M, ldx, ldy, n_rot;
    const float *x;
    float *y;
    float clip;
    rqo_block *act;            /* M rows of K/256 blocks */
    pthread_barrier_t barrier;
    atomic_long next_chunk;
} mm_job;

typedef struct {
    mm_job *job;
    int ith;
} mm_arg;

enum { ROW_CHUNK = 16 };

static void *mm_worker(void *p) {
    mm_arg *arg = (mm_arg *) p;
    mm_job *jb = arg->job;
    const int64_t nb = jb->K / BLK;
    /* phase 1: tokens striped over the threads */
    for (int64_t t = arg->ith; t < jb->M; t += jb->n_threads) {
        const float *xr = jb->x + t * jb->ldx;
        rqo_block *ar = jb->act + t * nb;
        if (jb->type == RQO_TYPE_W4A4H) {
            rqo_quantize_row_a4h(xr, ar, jb->K, jb->clip, jb->n_rot, jb->G);
        } else {
            rqo_quantize_row_a(xr, ar, jb->K, jb->clip, jb->G);
        }
    }
    pthread_barrier_wait(&jb->barrier);
    /* phase 2: chunks of weight rows, all tokens per chunk, handed out by a shared counter */
    const int64_t n_chunks = (jb->N + ROW_CHUNK - 1) / ROW_CHUNK;
    for (;;) {
        const int64_t c = atomic_fetch_add(&jb->next_chunk, 1);
        if (c >= n_chunks) break;
        const int64_t r0 = c * ROW_CHUNK;
        const int64_t r1 = r0 + ROW_CHUNK < jb->N ? r0 + ROW_CHUNK : jb->N;
        for (int64_t t = 0; t < jb->M; ++t) {
            for (int64_t r = r0; r < r1; ++r) {
                rqo_vec_dot(jb->K, jb->y + t * jb->ldy + r, jb->w + r * nb, jb->act + t * nb);
            }
        }
    }
    return NULL;
}

int rqo_mul_mat(int type, const void *w_blocks, int64_t K, int64_t N, const float *x, int64_t ldx, int64_t M,
                float *y, int64_t ldy, float clip, int64_t n_rot, int G, int n_threads) {
    if ((type != RQO_TYPE_W4A4 && type != RQO_TYPE_W4A4H) || K <= 0 || K % BLK || N <= 0 || M < 0) return -1;
    if (G != 64 && G != 128 && G != 256) return -1;
    if (type == RQO_TYPE_W4A4H && rqo_rot_check((int32_t) n_rot, K) < 0) return -1;
    if (M == 0) return 0;
    if (n_threads < 1) n_threads = 1;
    if (n_threads > 256) n_threads = 256;
    mm_job jb;
    jb.type = type; jb.G = G; jb.n_threads = n_threads;
    jb.w = (const rqo_block *) w_blocks;
    jb.K = K; jb.N = N; jb.M = M; jb.ldx = ldx; jb.ldy = ldy; jb.n_rot = n_rot;
    jb.x = x; jb.y = y; jb.clip = clip;
    jb.act = (rqo_block *) malloc((size_t) M * (size_t) (K / BLK) * sizeof(rqo_block));
    if (!jb.act) return -1;
    pthread_barrier_init(&jb.barrier, NULL, (unsigned) n_threads);
    atomic_init(&jb.next_chunk, 0);
    pthread_t tid[256];
    mm_arg args[256];
    for (int i = 0; i < n_threads; ++i) {
        args[i].job = &jb;
        args[i].ith = i;
        if (i > 0) pthread_create(&tid[i], NULL, mm_worker, &args[i]);
    }
    mm_worker(&args[0]);
    for (int i = 1; i < n_threads; ++i) pthread_join(tid[i], NULL);
    pthread_barrier_destroy(&jb.barrier);
    free(jb.act);
    return 0;
}
