/*
 * bkv_oracle.c -- CPU restatement of Breccia's paged-KV reference arithmetic.
 *
 * THIS IS TEST INFRASTRUCTURE.  It is the checker the HIP path is compared
 * against (tests, the smoke check, and the CPU-baseline leg of the benchmark).
 * Nothing in the shipped library links, loads or calls it.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference tree).  Scalar, single-threaded, f64 accumulation -- the same
 * shape as the reference's own CPU path -- plus one OpenMP driver used only
 * to report a multi-core baseline.
 *
 * Parity status of each function (what independent evidence pins it):
 *   bkvo_f32_to_f16_bits / bkvo_to_f16   pinned: reference KATs + exhaustive
 *                                        sweep against the F16C hardware convert
 *                                        and numpy.float16 (two documented
 *                                        deviations: |x|<2^-14 -> 0, NaN -> inf)
 *   bkvo_f16_bits_to_f32                 pinned: numpy.float16 on all 65536 codes
 *   bkvo_to_q8_0                         pinned: reference bound test (LCG fixture),
 *                                        zero blocks, grid/bound invariants
 *   bkvo_elem_index / append / gather    pinned: reference layout recipe (33 cells
 *                                        x 512 elements) + permutation round trips
 *   bkvo_attend                          pinned: torch float64 SDPA, independent
 *                                        numpy softmax, closed forms
 *   bkvo_pool_keys                       pinned: composition of the pinned norm and rotary with
 *                                        a mean that closed forms fix (constant blocks, one
 *                                        non-zero row) and a numpy float32 statement
 *   bkvo_rmsnorm / bkvo_rope_table /     pinned: reference KATs (ops/cpu.rs:373-421: constant row,
 *   bkvo_rope_apply                      identity at position 0, NEOX pairing one-hot),
 *                                        independent numpy float64 statements, rotation
 *                                        invariants (pair norms kept, angles add)
 *   bkvo_indexer_score / bkvo_topk_blocks pinned: reference KATs (qsa/cpu.rs:517-536: ties to the
 *                                        lower block, own block appended once, dead blocks
 *                                        never selected), the reference's LCG score recipes
 *                                        (tests/qsa_topk.rs:87-122) against numpy lexsort,
 *                                        numpy float64 statement of the score
 *   bkvo_to_i8h / append_i8 / gather_i8  NOT IN THE REFERENCE (int8 K+V with an f16
 *                                        scale): parity unpinned against the
 *                                        reference; pinned only by closed-form
 *                                        bounds and round-trip invariants
 *   bkvo_page_copy / bkvo_swap_*         NOT IN THE REFERENCE: byte moves, pinned by
 *                                        memcmp invariants
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define BKVO_Q8_BLOCK 32 /* crates/breccia-kernels/src/qsa/mod.rs:324 (Q8_BLOCK_ELEMS) */

static inline uint32_t f32_bits(float x) {
    uint32_t b;
    memcpy(&b, &x, 4);
    return b;
}
static inline float bits_f32(uint32_t b) {
    float x;
    memcpy(&x, &b, 4);
    return x;
}

/* ---------------------------------------------------------------------------
 * f16 storage rule.
 * Follows crates/breccia-kernels/src/qsa/cpu.rs:23-53 (to_f16) and its GLSL twin
 * crates/breccia-kernels/shaders/f16_storage.glsl:26-55.
 *   zero keeps its sign; exponent > 15 (inf and NaN too) -> signed inf;
 *   exponent < -14 -> signed zero (no subnormals, even where RNE would round up
 *   to 2^-14); otherwise round-to-nearest-even on the 13 dropped bits, with the
 *   carry able to bump the exponent (and overflow to inf).
 * ------------------------------------------------------------------------- */
uint16_t bkvo_f32_to_f16_bits(float x) {
    const uint32_t b = f32_bits(x);
    const uint16_t sign = (uint16_t)((b >> 16) & 0x8000u);
    const uint32_t mag = b & 0x7fffffffu;
    if (mag == 0) return sign;
    int e = (int)(mag >> 23) - 127;
    if (e > 15) return (uint16_t)(sign | 0x7c00u);
    if (e < -14) return sign;
    uint32_t sig = (mag & 0x007fffffu) | 0x00800000u; /* 24-bit significand */
    uint32_t keep = sig >> 13;                        /* 11 bits incl. leading 1 */
    const uint32_t drop = sig & 0x1fffu;
    if (drop > 0x1000u || (drop == 0x1000u && (keep & 1u))) keep += 1;
    if (keep >= 0x800u) {
        keep >>= 1;
        e += 1;
        if (e > 15) return (uint16_t)(sign | 0x7c00u);
    }
    return (uint16_t)(sign | ((uint32_t)(e + 15) << 10) | (keep & 0x3ffu));
}

/* Load rule, crates/breccia-kernels/shaders/f16_storage.glsl:58-69:
 * exponent field 0 -> signed zero (subnormal codes are flushed), 31 -> inf/NaN
 * passthrough, else exact. */
float bkvo_f16_bits_to_f32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu;
    const uint32_t m = h & 0x3ffu;
    if (e == 0) return bits_f32(sign);
    if (e == 31) return bits_f32(sign | 0x7f800000u | (m << 13));
    return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

/* f32 -> f16 -> f32 round trip = cpu.rs:23-53 as a value map. */
float bkvo_to_f16(float x) { return bkvo_f16_bits_to_f32(bkvo_f32_to_f16_bits(x)); }

void bkvo_f32_to_f16_bits_n(const float *x, size_t n, uint16_t *out) {
    for (size_t i = 0; i < n; ++i) out[i] = bkvo_f32_to_f16_bits(x[i]);
}
void bkvo_f16_bits_to_f32_n(const uint16_t *h, size_t n, float *out) {
    for (size_t i = 0; i < n; ++i) out[i] = bkvo_f16_bits_to_f32(h[i]);
}

/* Count disagreements between bkvo_f32_to_f16_bits and a caller-supplied table of
 * expected codes over the bit patterns [first, first+count).  Used by the
 * exhaustive sweep test, which supplies F16C / numpy results as `expect`. */
uint64_t bkvo_f16_sweep_mismatches(uint32_t first, uint64_t count, const uint16_t *expect,
                                   int apply_documented_deviations) {
    uint64_t bad = 0;
    for (uint64_t i = 0; i < count; ++i) {
        const uint32_t b = first + (uint32_t)i;
        uint16_t want = expect[i];
        if (apply_documented_deviations) {
            const uint32_t mag = b & 0x7fffffffu;
            const uint16_t sign = (uint16_t)((b >> 16) & 0x8000u);
            if (mag < 0x38800000u) want = sign;                    /* |x| < 2^-14 -> 0 */
            else if (mag > 0x7f800000u) want = (uint16_t)(sign | 0x7c00u); /* NaN -> inf */
        }
        if (bkvo_f32_to_f16_bits(bits_f32(b)) != want) ++bad;
    }
    return bad;
}

/* ---------------------------------------------------------------------------
 * q8_0 of a V row, crates/breccia-kernels/src/qsa/cpu.rs:65-82 and the store in
 * crates/breccia-kernels/shaders/qsa_kv_append.comp:113-132:
 *   per 32 values: amax = max|v|; scale = amax>0 ? amax/127 : 1 (f32 divide);
 *   q = round_half_away(clamp(v/scale, -127, 127)); dequantised value q*scale.
 * `deq`, `q`, `scales` may each be NULL.
 * ------------------------------------------------------------------------- */
void bkvo_to_q8_0(const float *x, size_t n, float *deq, int8_t *q, float *scales) {
    for (size_t b0 = 0; b0 + BKVO_Q8_BLOCK <= n; b0 += BKVO_Q8_BLOCK) {
        float amax = 0.0f;
        for (int i = 0; i < BKVO_Q8_BLOCK; ++i) {
            const float a = fabsf(x[b0 + i]);
            if (a > amax) amax = a;
        }
        const float scale = amax > 0.0f ? amax / 127.0f : 1.0f;
        if (scales) scales[b0 / BKVO_Q8_BLOCK] = scale;
        for (int i = 0; i < BKVO_Q8_BLOCK; ++i) {
            float t = x[b0 + i] / scale;
            if (t < -127.0f) t = -127.0f;
            if (t > 127.0f) t = 127.0f;
            const float r = roundf(t); /* half away from zero, like Rust f32::round */
            if (q) q[b0 + i] = (int8_t)r;
            if (deq) deq[b0 + i] = r * scale;
        }
    }
}

/* int8 with an f16 scale (34 B per 32 values) -- NOT in the reference; the rule is
 * the q8_0 rule with the scale passed through the cache's f16 encoding:
 *   s32 = amax/127; sh = to_f16(s32), raised to 2^-14 when 0 < amax and the f16
 *   rule would flush it; amax == 0 -> sh = 1;  q = round_half_away(clamp(v/sh));
 *   dequantised value q*sh (f32). */
void bkvo_to_i8h(const float *x, size_t n, float *deq, int8_t *q, uint16_t *scale_bits) {
    for (size_t b0 = 0; b0 + BKVO_Q8_BLOCK <= n; b0 += BKVO_Q8_BLOCK) {
        float amax = 0.0f;
        for (int i = 0; i < BKVO_Q8_BLOCK; ++i) {
            const float a = fabsf(x[b0 + i]);
            if (a > amax) amax = a;
        }
        uint16_t hb;
        if (amax > 0.0f) {
            hb = bkvo_f32_to_f16_bits(amax / 127.0f);
            if ((hb & 0x7fffu) == 0) hb = 0x0400u; /* smallest normal, 2^-14 */
        } else {
            hb = 0x3c00u; /* 1.0 */
        }
        const float sh = bkvo_f16_bits_to_f32(hb);
        if (scale_bits) scale_bits[b0 / BKVO_Q8_BLOCK] = hb;
        for (int i = 0; i < BKVO_Q8_BLOCK; ++i) {
            float t = x[b0 + i] / sh;
            if (!(t >= -127.0f)) t = -127.0f; /* also catches NaN from inf/inf */
            if (t > 127.0f) t = 127.0f;
            const float r = roundf(t);
            if (q) q[b0 + i] = (int8_t)r;
            if (deq) deq[b0 + i] = r * sh;
        }
    }
}

/* ---------------------------------------------------------------------------
 * Pool addressing, crates/breccia-kernels/src/qsa/mod.rs:24-28 and
 * crates/breccia-kernels/shaders/qsa_kv_append.comp:150-153:
 *   row  = (phys_page*n_kv + kvh)*page_cells + cell%page_cells
 *   elem = row*head_dim + d          (f16 pools; u32 word = elem/2, low half even)
 * ------------------------------------------------------------------------- */
typedef struct {
    int32_t n_kv;
    int32_t head_dim;
    int32_t page_cells;
} bkvo_geom;

size_t bkvo_row_index(const bkvo_geom *g, int32_t phys_page, int32_t kvh, int32_t in_page) {
    return ((size_t)phys_page * (size_t)g->n_kv + (size_t)kvh) * (size_t)g->page_cells +
           (size_t)in_page;
}
size_t bkvo_elem_index(const bkvo_geom *g, int32_t phys_page, int32_t kvh, int32_t in_page,
                       int32_t d) {
    return bkvo_row_index(g, phys_page, kvh, in_page) * (size_t)g->head_dim + (size_t)d;
}

/* Append T rows at cells pos0..pos0+T through the block table.
 * k, v: f32 [T][n_kv][head_dim] (qsa_kv_append.comp:155).  Pools: arrays of f16
 * codes in the layout above.  Reference: qsa/mod.rs:1107-1156 (host range check),
 * qsa_kv_append.comp:137-161 (store), qsa/cpu.rs:422-428 (oracle append).
 * Returns 0, or -1 if pos0+T exceeds capacity_cells (qsa/mod.rs:1108-1116). */
int bkvo_append_f16(const bkvo_geom *g, uint16_t *k_pool, uint16_t *v_pool,
                    const int32_t *block_table, int64_t capacity_cells, int64_t pos0, int64_t T,
                    const float *k, const float *v) {
    if (pos0 < 0 || T < 0 || pos0 + T > capacity_cells) return -1;
    const size_t rowlen = (size_t)g->n_kv * (size_t)g->head_dim;
    for (int64_t t = 0; t < T; ++t) {
        const int64_t cell = pos0 + t;
        const int32_t phys = block_table[cell / g->page_cells];
        const int32_t in_page = (int32_t)(cell % g->page_cells);
        for (int32_t kvh = 0; kvh < g->n_kv; ++kvh) {
            const size_t dst = bkvo_elem_index(g, phys, kvh, in_page, 0);
            const size_t src = (size_t)t * rowlen + (size_t)kvh * (size_t)g->head_dim;
            for (int32_t d = 0; d < g->head_dim; ++d) {
                k_pool[dst + d] = bkvo_f32_to_f16_bits(k[src + d]);
                v_pool[dst + d] = bkvo_f32_to_f16_bits(v[src + d]);
            }
        }
    }
    return 0;
}

/* Reference q8_0-V layout: K stays f16; V row = head_dim/32 blocks of 9 u32 words,
 * word 0 = f32 scale bits, words 1..8 = 32 x i8, element j in byte j%4 of word
 * 1+j/4 (qsa_kv_append.comp:38-44, :87-132).  V is quantised from the f32 input. */
int bkvo_append_q8v(const bkvo_geom *g, uint16_t *k_pool, uint32_t *v_pool_words,
                    const int32_t *block_table, int64_t capacity_cells, int64_t pos0, int64_t T,
                    const float *k, const float *v) {
    if (pos0 < 0 || T < 0 || pos0 + T > capacity_cells) return -1;
    if (g->head_dim % BKVO_Q8_BLOCK) return -2;
    const int32_t blocks = g->head_dim / BKVO_Q8_BLOCK;
    const size_t rowlen = (size_t)g->n_kv * (size_t)g->head_dim;
    int8_t q[BKVO_Q8_BLOCK];
    float scale;
    for (int64_t t = 0; t < T; ++t) {
        const int64_t cell = pos0 + t;
        const int32_t phys = block_table[cell / g->page_cells];
        const int32_t in_page = (int32_t)(cell % g->page_cells);
        for (int32_t kvh = 0; kvh < g->n_kv; ++kvh) {
            const size_t row = bkvo_row_index(g, phys, kvh, in_page);
            const size_t src = (size_t)t * rowlen + (size_t)kvh * (size_t)g->head_dim;
            for (int32_t d = 0; d < g->head_dim; ++d)
                k_pool[row * (size_t)g->head_dim + d] = bkvo_f32_to_f16_bits(k[src + d]);
            for (int32_t b = 0; b < blocks; ++b) {
                bkvo_to_q8_0(v + src + (size_t)b * BKVO_Q8_BLOCK, BKVO_Q8_BLOCK, NULL, q, &scale);
                uint32_t *w = v_pool_words + (row * (size_t)blocks + (size_t)b) * 9u;
                w[0] = f32_bits(scale);
                for (int j = 0; j < 8; ++j) {
                    uint32_t packed = 0;
                    for (int i = 0; i < 4; ++i)
                        packed |= ((uint32_t)(uint8_t)q[j * 4 + i]) << (8 * i);
                    w[1 + j] = packed;
                }
            }
        }
    }
    return 0;
}

/* int8 K+V with f16 scales (NOT in the reference).  Row layout, both pools:
 *   [head_dim x i8][head_dim/32 x f16 scale]  = head_dim + head_dim/16 bytes
 * (272 B for head_dim 256; 34 B per 32 values), rows addressed like the f16 pool. */
size_t bkvo_i8_row_bytes(const bkvo_geom *g) {
    return (size_t)g->head_dim + (size_t)(g->head_dim / BKVO_Q8_BLOCK) * 2u;
}
int bkvo_append_i8(const bkvo_geom *g, uint8_t *k_pool, uint8_t *v_pool,
                   const int32_t *block_table, int64_t capacity_cells, int64_t pos0, int64_t T,
                   const float *k, const float *v) {
    if (pos0 < 0 || T < 0 || pos0 + T > capacity_cells) return -1;
    if (g->head_dim % BKVO_Q8_BLOCK) return -2;
    const size_t rb = bkvo_i8_row_bytes(g);
    const size_t rowlen = (size_t)g->n_kv * (size_t)g->head_dim;
    const int32_t blocks = g->head_dim / BKVO_Q8_BLOCK;
    for (int64_t t = 0; t < T; ++t) {
        const int64_t cell = pos0 + t;
        const int32_t phys = block_table[cell / g->page_cells];
        const int32_t in_page = (int32_t)(cell % g->page_cells);
        for (int32_t kvh = 0; kvh < g->n_kv; ++kvh) {
            const size_t row = bkvo_row_index(g, phys, kvh, in_page);
            const size_t src = (size_t)t * rowlen + (size_t)kvh * (size_t)g->head_dim;
            for (int which = 0; which < 2; ++which) {
                uint8_t *dst = (which ? v_pool : k_pool) + row * rb;
                const float *x = (which ? v : k) + src;
                uint16_t sc[64];
                bkvo_to_i8h(x, (size_t)g->head_dim, NULL, (int8_t *)dst, sc);
                memcpy(dst + g->head_dim, sc, (size_t)blocks * 2u);
            }
        }
    }
    return 0;
}

/* Gather cells [cell0, cell0+n) of a block-tabled sequence into the flat
 * [cell][kvh][d] f32 arrays cpu::attend consumes (qsa/cpu.rs:219-222 indexing).
 * `layout`: 0 = f16 K and V; 1 = f16 K + reference q8_0 V; 2 = int8+f16-scale K and V.
 * Load rules: f16_storage.glsl:58-80, qsa_attn_apply.comp:70-77 (i8 * f32 scale). */
int bkvo_gather(const bkvo_geom *g, int layout, const void *k_pool, const void *v_pool,
                const int32_t *block_table, int64_t cell0, int64_t n, float *k_out, float *v_out) {
    const int32_t hd = g->head_dim;
    const int32_t blocks = hd / BKVO_Q8_BLOCK;
    const size_t rb8 = bkvo_i8_row_bytes(g);
    for (int64_t i = 0; i < n; ++i) {
        const int64_t cell = cell0 + i;
        const int32_t phys = block_table[cell / g->page_cells];
        const int32_t in_page = (int32_t)(cell % g->page_cells);
        for (int32_t kvh = 0; kvh < g->n_kv; ++kvh) {
            const size_t row = bkvo_row_index(g, phys, kvh, in_page);
            float *ko = k_out + ((size_t)i * (size_t)g->n_kv + (size_t)kvh) * (size_t)hd;
            float *vo = v_out + ((size_t)i * (size_t)g->n_kv + (size_t)kvh) * (size_t)hd;
            if (layout == 0 || layout == 1) {
                const uint16_t *kp = (const uint16_t *)k_pool + row * (size_t)hd;
                for (int32_t d = 0; d < hd; ++d) ko[d] = bkvo_f16_bits_to_f32(kp[d]);
            }
            if (layout == 0) {
                const uint16_t *vp = (const uint16_t *)v_pool + row * (size_t)hd;
                for (int32_t d = 0; d < hd; ++d) vo[d] = bkvo_f16_bits_to_f32(vp[d]);
            } else if (layout == 1) {
                const uint32_t *w = (const uint32_t *)v_pool + row * (size_t)blocks * 9u;
                for (int32_t b = 0; b < blocks; ++b) {
                    const float scale = bits_f32(w[b * 9]);
                    for (int j = 0; j < BKVO_Q8_BLOCK; ++j) {
                        const int8_t qv = (int8_t)((w[b * 9 + 1 + j / 4] >> (8 * (j % 4))) & 0xffu);
                        vo[b * BKVO_Q8_BLOCK + j] = (float)qv * scale;
                    }
                }
            } else if (layout == 2) {
                for (int which = 0; which < 2; ++which) {
                    const uint8_t *rowp = (const uint8_t *)(which ? v_pool : k_pool) + row * rb8;
                    float *o = which ? vo : ko;
                    for (int32_t d = 0; d < hd; ++d) {
                        uint16_t sb;
                        memcpy(&sb, rowp + hd + (d / BKVO_Q8_BLOCK) * 2, 2);
                        o[d] = (float)(int8_t)rowp[d] * bkvo_f16_bits_to_f32(sb);
                    }
                }
            } else {
                return -1;
            }
        }
    }
    return 0;
}

/* ---------------------------------------------------------------------------
 * Attention.  crates/breccia-kernels/src/qsa/cpu.rs:84-91 (sigmoid), :197-246
 * (attend).  q f32 [n_head][hd]; k, v flat f32 [cell][n_kv][hd] already in cache
 * precision; cells walked in list order, entries > pos skipped; kvh = h*n_kv/n_head;
 * logits, softmax and the V sum in f64; out = f32(acc * sigmoid(gate)).  gate NULL
 * = ungated (the factor is omitted).  No live cell -> zeros.
 * ------------------------------------------------------------------------- */
static double sigmoid64(double x) {
    if (x >= 0.0) return 1.0 / (1.0 + exp(-x));
    const double e = exp(x);
    return e / (1.0 + e);
}

static void attend_one_head(const float *q, const float *k, const float *v, const uint32_t *cells,
                            size_t n_cells, int64_t pos, int32_t h, int32_t n_head, int32_t n_kv,
                            int32_t hd, const float *gate, float *out, double *logits) {
    const double scale = 1.0 / sqrt((double)hd);
    const int32_t kvh = (int32_t)(((int64_t)h * n_kv) / n_head);
    const size_t stride = (size_t)n_kv * (size_t)hd;
    const float *qh = q + (size_t)h * (size_t)hd;
    size_t live = 0;
    double mx = -INFINITY;
    for (size_t i = 0; i < n_cells; ++i) {
        const int64_t c = (int64_t)cells[i];
        if (c > pos) continue;
        const float *kr = k + (size_t)c * stride + (size_t)kvh * (size_t)hd;
        double dot = 0.0;
        for (int32_t d = 0; d < hd; ++d) dot += (double)qh[d] * (double)kr[d];
        const double l = dot * scale;
        logits[live++] = l;
        if (l > mx) mx = l;
    }
    double sum = 0.0;
    for (size_t i = 0; i < live; ++i) {
        logits[i] = exp(logits[i] - mx);
        sum += logits[i];
    }
    double acc[1024];
    for (int32_t d = 0; d < hd; ++d) acc[d] = 0.0;
    size_t j = 0;
    for (size_t i = 0; i < n_cells; ++i) {
        const int64_t c = (int64_t)cells[i];
        if (c > pos) continue;
        const double p = logits[j++] / sum;
        const float *vr = v + (size_t)c * stride + (size_t)kvh * (size_t)hd;
        for (int32_t d = 0; d < hd; ++d) acc[d] += p * (double)vr[d];
    }
    for (int32_t d = 0; d < hd; ++d) {
        const double gte = gate ? sigmoid64((double)gate[(size_t)h * (size_t)hd + d]) : 1.0;
        out[(size_t)h * (size_t)hd + d] = (float)(acc[d] * gte);
    }
}

/* threads <= 1: the reference's scalar single-threaded shape.  threads > 1: heads
 * dealt to an OpenMP team (baseline reporting only; same per-head arithmetic). */
int bkvo_attend(const float *q, const float *k, const float *v, const uint32_t *cells,
                size_t n_cells, int64_t pos, int32_t n_head, int32_t n_kv, int32_t hd,
                const float *gate, float *out, int threads) {
    if (hd > 1024 || hd <= 0 || n_head <= 0 || n_kv <= 0) return -1;
#ifdef _OPENMP
    if (threads > 1) {
        int fail = 0;
#pragma omp parallel for num_threads(threads) schedule(dynamic, 1)
        for (int32_t h = 0; h < n_head; ++h) {
            double *logits = (double *)malloc((n_cells ? n_cells : 1) * sizeof(double));
            if (!logits) {
                fail = 1;
                continue;
            }
            attend_one_head(q, k, v, cells, n_cells, pos, h, n_head, n_kv, hd, gate, out, logits);
            free(logits);
        }
        return fail ? -2 : 0;
    }
#else
    (void)threads;
#endif
    double *logits = (double *)malloc((n_cells ? n_cells : 1) * sizeof(double));
    if (!logits) return -2;
    for (int32_t h = 0; h < n_head; ++h)
        attend_one_head(q, k, v, cells, n_cells, pos, h, n_head, n_kv, hd, gate, out, logits);
    free(logits);
    return 0;
}

/* Probabilities of one head (for the reference's 1e-6 probability bar,
 * crates/breccia-kernels/tests/attn_conformance.rs:1148-1151); same walk as above. */
int bkvo_attend_probs(const float *q, const float *k, const uint32_t *cells, size_t n_cells,
                      int64_t pos, int32_t h, int32_t n_head, int32_t n_kv, int32_t hd,
                      double *probs_out, size_t *n_live) {
    const double scale = 1.0 / sqrt((double)hd);
    const int32_t kvh = (int32_t)(((int64_t)h * n_kv) / n_head);
    const size_t stride = (size_t)n_kv * (size_t)hd;
    size_t live = 0;
    double mx = -INFINITY, sum = 0.0;
    for (size_t i = 0; i < n_cells; ++i) {
        const int64_t c = (int64_t)cells[i];
        if (c > pos) continue;
        double dot = 0.0;
        for (int32_t d = 0; d < hd; ++d)
            dot += (double)q[(size_t)h * hd + d] * (double)k[(size_t)c * stride + (size_t)kvh * hd + d];
        probs_out[live] = dot * scale;
        if (probs_out[live] > mx) mx = probs_out[live];
        ++live;
    }
    for (size_t i = 0; i < live; ++i) {
        probs_out[i] = exp(probs_out[i] - mx);
        sum += probs_out[i];
    }
    for (size_t i = 0; i < live; ++i) probs_out[i] /= sum;
    *n_live = live;
    return 0;
}

/* Block ids -> cell list, crates/breccia-kernels/src/qsa/cpu.rs:249-257. */
size_t bkvo_cells_of(const uint32_t *blocks, size_t n_blocks, uint32_t idx_block, uint32_t *out) {
    size_t n = 0;
    for (size_t i = 0; i < n_blocks; ++i)
        for (uint32_t k = 0; k < idx_block; ++k) out[n++] = blocks[i] * idx_block + k;
    return n;
}

/* Dense selection, crates/breccia-kernels/shaders/qsa_topk.comp:78-95: blocks
 * 0..min(n_blocks, own+1) ascending (own = pos/idx_block, n_blocks = n_kv_after /
 * idx_block), then `own` itself when the tail block is incomplete. */
size_t bkvo_dense_ids(int64_t pos, int64_t n_kv_after, uint32_t idx_block, uint32_t *out) {
    const int64_t own = pos / idx_block;
    const int64_t n_blocks = n_kv_after / idx_block;
    const int64_t lim = n_blocks < own + 1 ? n_blocks : own + 1;
    size_t n = 0;
    for (int64_t b = 0; b < lim; ++b) out[n++] = (uint32_t)b;
    if (own >= n_blocks) out[n++] = (uint32_t)own;
    return n;
}

/* ---- block selection (the indexer's score and the top-k over it) -------------------
 * qsa/cpu.rs:93-123: score[b] = (1/sqrt(idx_dim)) * sum_h relu(q_h . pooled_b), f64,
 * sums in index order; -inf for a block that starts after the query's position. */
void bkvo_indexer_score(const float *q, const float *pooled, size_t n_blocks, int64_t pos,
                        size_t idx_n_head, size_t idx_dim, size_t idx_block, double *out) {
    const double scale = 1.0 / sqrt((double)idx_dim);
    for (size_t b = 0; b < n_blocks; ++b) {
        if ((int64_t)(b * idx_block) > pos) {
            out[b] = -INFINITY;
            continue;
        }
        double acc = 0.0;
        for (size_t h = 0; h < idx_n_head; ++h) {
            double dot = 0.0;
            for (size_t d = 0; d < idx_dim; ++d)
                dot += (double)q[h * idx_dim + d] * (double)pooled[b * idx_dim + d];
            acc += (dot > 0.0 ? dot : 0.0) * scale;
        }
        out[b] = acc;
    }
}

static const double *topk_scores_for_sort;
static int topk_order(const void *pa, const void *pb) {
    const uint32_t a = *(const uint32_t *)pa, b = *(const uint32_t *)pb;
    const double sa = topk_scores_for_sort[a], sb = topk_scores_for_sort[b];
    if (sa > sb) return -1;
    if (sa < sb) return 1;
    return a < b ? -1 : (a > b ? 1 : 0);
}

/* qsa/cpu.rs:125-152: blocks by descending score, ties to the lower index, non-finite
 * scores dropped, the first k kept, then the query's own block when the selection missed
 * it (own < 0: no own block).  Returns the list length; out holds up to k + 1 ids.
 * Not re-entrant (qsort has no context argument). */
size_t bkvo_topk_blocks(const double *scores, size_t n, size_t k, int64_t own, uint32_t *out) {
    uint32_t *order = (uint32_t *)malloc((n ? n : 1) * sizeof(uint32_t));
    size_t live = 0;
    for (size_t i = 0; i < n; ++i)
        if (isfinite(scores[i])) order[live++] = (uint32_t)i;
    topk_scores_for_sort = scores;
    qsort(order, live, sizeof(uint32_t), topk_order);
    size_t count = live < k ? live : k;
    memcpy(out, order, count * sizeof(uint32_t));
    free(order);
    if (own >= 0) {
        int present = 0;
        for (size_t i = 0; i < count; ++i) present |= out[i] == (uint32_t)own;
        if (!present) out[count++] = (uint32_t)own;
    }
    return count;
}

/* ---- K preparation ahead of the append (Qsa::k_norm + Qsa::rope_k) ---------------
 * crates/breccia-kernels/src/ops/cpu.rs:52-88: row-wise RMSNorm, f64 throughout,
 * sequential sum, y = (f32)(x * inv * w) with inv = 1/sqrt(ss/cols + eps); row r uses
 * gamma slice r % wgroups; wgroups == 0 means no gamma. */
void bkvo_rmsnorm(const float *x, size_t rows, size_t cols, size_t wgroups, const float *gamma,
                  float eps, float *out) {
    for (size_t r = 0; r < rows; ++r) {
        const float *xr = x + r * cols;
        double ss = 0.0;
        for (size_t i = 0; i < cols; ++i) {
            const double v = (double)xr[i];
            ss += v * v;
        }
        const double inv = 1.0 / sqrt(ss / (double)cols + (double)eps);
        const float *g = wgroups ? gamma + (r % wgroups) * cols : NULL;
        for (size_t i = 0; i < cols; ++i) {
            const double w = g ? (double)g[i] : 1.0;
            out[r * cols + i] = (float)((double)xr[i] * inv * w);
        }
    }
}

/* ops/cpu.rs:103-119: table[p][i] = (cos, sin)(p * freq_base^(-2i/n_rot)), f64 then f32. */
void bkvo_rope_table(double freq_base, size_t n_rot, size_t max_pos, float *out) {
    const size_t half = n_rot / 2;
    for (size_t p = 0; p < max_pos; ++p)
        for (size_t i = 0; i < half; ++i) {
            const double inv = pow(freq_base, -2.0 * (double)i / (double)n_rot);
            const double ang = (double)p * inv;
            out[(p * half + i) * 2] = (float)cos(ang);
            out[(p * half + i) * 2 + 1] = (float)sin(ang);
        }
}

/* ops/cpu.rs:121-154 (rope_apply at :124): partial NEOX-paired rotary.  out[j] = x[j]*c - x[j+half]*s,
 * out[j+half] = x[j]*s + x[j+half]*c for j < half = n_rot/2, f64 products and sums, cast
 * to f32; dims [n_rot, head_dim) copied; the position is clamped into the table. */
void bkvo_rope_apply(const float *x, size_t rows, size_t head_dim, size_t n_rot, const float *table,
                     size_t max_pos, const int32_t *positions, float *out) {
    const size_t half = n_rot / 2;
    for (size_t r = 0; r < rows; ++r) {
        const float *xr = x + r * head_dim;
        float *o = out + r * head_dim;
        int64_t pc = positions[r];
        if (pc < 0) pc = 0;
        if (pc > (int64_t)max_pos - 1) pc = (int64_t)max_pos - 1;
        const size_t p = (size_t)pc;
        for (size_t j = 0; j < half; ++j) {
            const double a = (double)xr[j], b = (double)xr[j + half];
            const double c = (double)table[(p * half + j) * 2];
            const double sn = (double)table[(p * half + j) * 2 + 1];
            o[j] = (float)(a * c - b * sn);
            o[j + half] = (float)(a * sn + b * c);
        }
        for (size_t j = n_rot; j < head_dim; ++j) o[j] = xr[j];
    }
}

/* qsa/cpu.rs:154-185: pooled indexer keys.  pooled[b] = rope(rmsnorm(mean(raw[4b..4b+3])),
 * position 4b): the mean accumulates raw/idx_block in f32 in cell order, the norm uses one
 * gamma of idx_dim values, the rotary reads the table row of the block's first cell. */
void bkvo_pool_keys(const float *raw, size_t cells, const float *gamma, const float *table,
                    size_t max_pos, size_t idx_dim, size_t idx_block, size_t n_rot, float eps,
                    float *out) {
    const size_t n_blocks = cells / idx_block;
    float *mean = (float *)malloc(idx_dim * sizeof(float));
    float *normed = (float *)malloc(idx_dim * sizeof(float));
    for (size_t b = 0; b < n_blocks; ++b) {
        for (size_t d = 0; d < idx_dim; ++d) mean[d] = 0.0f;
        for (size_t k = 0; k < idx_block; ++k)
            for (size_t d = 0; d < idx_dim; ++d)
                mean[d] += raw[(b * idx_block + k) * idx_dim + d] / (float)idx_block;
        bkvo_rmsnorm(mean, 1, idx_dim, 1, gamma, eps, normed);
        const int32_t pos = (int32_t)(b * idx_block);
        bkvo_rope_apply(normed, 1, idx_dim, n_rot, table, max_pos, &pos, out + b * idx_dim);
    }
    free(mean);
    free(normed);
}

/* ---------------------------------------------------------------------------
 * Byte moves (no reference code; nearest reference primitives are buffer copies,
 * crates/breccia-kernels/src/dispatch_batch.rs:1130-1150 and gemv.rs:1023-1071).
 * A "page" of one layer is `bytes_per_page` contiguous bytes at page*bytes_per_page.
 * ------------------------------------------------------------------------- */
void bkvo_page_copy(uint8_t *pool, size_t bytes_per_page, const int32_t *src_dst_pairs,
                    size_t n_pairs) {
    for (size_t i = 0; i < n_pairs; ++i)
        memmove(pool + (size_t)src_dst_pairs[2 * i + 1] * bytes_per_page,
                pool + (size_t)src_dst_pairs[2 * i] * bytes_per_page, bytes_per_page);
}
void bkvo_swap_out(const uint8_t *pool, size_t bytes_per_page, const int32_t *pages, size_t n,
                   uint8_t *host, size_t host_stride, size_t host_offset) {
    for (size_t i = 0; i < n; ++i)
        memcpy(host + i * host_stride + host_offset, pool + (size_t)pages[i] * bytes_per_page,
               bytes_per_page);
}
void bkvo_swap_in(uint8_t *pool, size_t bytes_per_page, const int32_t *pages, size_t n,
                  const uint8_t *host, size_t host_stride, size_t host_offset) {
    for (size_t i = 0; i < n; ++i)
        memcpy(pool + (size_t)pages[i] * bytes_per_page, host + i * host_stride + host_offset,
               bytes_per_page);
}

/* ---------------------------------------------------------------------------
 * The reference tests' input generator, crates/breccia-kernels/tests/
 * attn_conformance.rs:110-124: s = seed|1; per value four LCG steps
 * s = s*6364136223846793005 + 1442695040888963407, acc += f32(s>>33)/f32(2^31-1)
 * (which is 2147483648.0f), value = (acc - 1)*1.732.  All IEEE f32.
 * ------------------------------------------------------------------------- */
void bkvo_normalish(uint64_t seed, size_t n, float *out) {
    uint64_t s = seed | 1u;
    const float denom = (float)(0xffffffffu >> 1);
    for (size_t i = 0; i < n; ++i) {
        float acc = 0.0f;
        for (int r = 0; r < 4; ++r) {
            s = s * 6364136223846793005ull + 1442695040888963407ull;
            acc += (float)(s >> 33) / denom;
        }
        out[i] = (acc - 1.0f) * 1.732f;
    }
}

/* The q8_0 bound test's fixture, crates/breccia-kernels/src/qsa/mod.rs:2078-2084. */
void bkvo_q8_fixture(float *out, size_t n) {
    uint64_t s = 12345u;
    for (size_t i = 0; i < n; ++i) {
        s = s * 6364136223846793005ull + 1u;
        out[i] = ((float)(s >> 40) / (float)(1ull << 24) - 0.5f) * 8.0f;
    }
}

int bkvo_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
