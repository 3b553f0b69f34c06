/*
 * CPU oracle for the NVFP4 weight x activation path.  TEST INFRASTRUCTURE ONLY: the product
 * (the HIP library and its host wrapper) never links, imports or calls this file; tests, the
 * smoke check and the bench's CPU-baseline leg do.
 *
 * What pins each function (none of these checks retypes the formula under test):
 *   orc_e2m1            closed form over 16 codes; the table at cpu_nvfp4.rs:52
 *   orc_ue4m3           the reference-held vector converter/tests/fixtures/fp8-e4m3fn-lut.tsv
 *                       (torch float8_e4m3fn bits, codes 0..126), monotonic ladder
 *   orc_scale_rule/lut  0x7F reads 448*gs (cpu_nvfp4.rs:545-548)
 *   orc_dequant*        decode of engine/tests/fixtures/synthetic-v2/synthetic-v2.cnq against the
 *                       LCG source it was made from (error <= one scale step, sign kept)
 *   orc_quantize_ceil   byte-exact regeneration of the six NVFP4 tensors of synthetic-v2.cnq and
 *                       their global scales from the LCG source (converter/src/main.rs:2552-2672)
 *   orc_gemv            gamma bound against an independent f64 dot; scalar == AVX2 bits for every
 *                       scale byte and thread count; brute force on tiny shapes; the torch golden
 *                       engine/tests/fixtures/glm5/moe/dense-y.f32 through orc_ffn_clamped
 *   orc_expert_ffn      fused == staged bits; f64 end to end
 *   orc_router_topk     brute force (sort) on small E; crafted ties
 *   orc_argmax_ref      numpy argmax on tie-free data; crafted ties for the tie rule
 *   orc_moe_layer       composition of the above, checked against a staged evaluation
 * The Rust original cannot be compiled here (no rustc), so there is no oracle/_ref.
 *
 * Build: see oracle/Makefile (-O2 -mavx2 -ffp-contract=off: no FMA contraction anywhere, the
 * reference rounds every operation on its own, cpu_nvfp4.rs:22-31).
 */
#include "nvfp4_oracle.h"
#include <immintrin.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ format */

static const float MAG8[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};

/* cnq.rs:1241-1245: magnitude table on the low 3 bits, bit 3 negates (code 8 is -0.0) */
float orc_e2m1(uint32_t nibble) {
    float v = MAG8[nibble & 7u];
    return (nibble & 8u) ? -v : v;
}

/* cnq.rs:1287-1295: e = bits 6..3, m = bits 2..0, bit 7 ignored; e == 0 is the subnormal ladder */
float orc_ue4m3(uint32_t byte) {
    uint32_t e = (byte >> 3) & 15u, m = byte & 7u;
    if (e == 0) return (float)m * 1.953125e-3f;
    return (1.0f + (float)m / 8.0f) * ldexpf(1.0f, (int)e - 7);
}

/* cpu_nvfp4.rs:88-96 (residency.rs:126-137): only the exact byte 0x7F is rewritten */
uint8_t orc_scale_rule(uint8_t byte) { return byte == 0x7F ? 0x7E : byte; }

/* cpu_nvfp4.rs:98-105 */
void orc_scale_lut(float gs, float lut[256]) {
    for (int b = 0; b < 256; b++) lut[b] = orc_ue4m3(orc_scale_rule((uint8_t)b)) * gs;
}

size_t orc_byte_len(size_t rows, size_t cols) { return rows * (cols / NVFP4_BLOCK_VALUES) * NVFP4_BLOCK_BYTES; }

static void dequant_with(const uint8_t* blocks, size_t n_blocks, const float lut[256], float* out) {
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t* blk = blocks + b * NVFP4_BLOCK_BYTES;
        for (int idx = 0; idx < 64; idx++) {
            float s = lut[blk[idx >> 4]];
            uint32_t byte = blk[4 + (idx >> 1)];
            uint32_t nib = (idx & 1) ? (byte >> 4) : (byte & 15u);
            out[b * 64 + idx] = orc_e2m1(nib) * s;
        }
    }
}

/* cnq.rs:1298-1308: w = e2m1(nib) * (ue4m3(sc) * gs), two roundings in that order */
void orc_dequant_raw(const uint8_t* blocks, size_t n_blocks, float gs, float* out) {
    float lut[256];
    for (int b = 0; b < 256; b++) lut[b] = orc_ue4m3((uint32_t)b) * gs;
    dequant_with(blocks, n_blocks, lut, out);
}

void orc_dequant(const uint8_t* blocks, size_t n_blocks, float gs, float* out) {
    float lut[256];
    orc_scale_lut(gs, lut);
    dequant_with(blocks, n_blocks, lut, out);
}

/* ------------------------------------------------------------------ encoder (ceil) */

/* converter/src/main.rs:141-169: smallest ue4m3 value >= v, as its byte */
uint32_t orc_encode_ue4m3_ceil(float v) {
    if (v <= 0.0f) return 0;
    if (v != v) return 0x7F; /* NaN never reaches the encoder (amax of finite weights); refuse loudly */
    int e0 = (int)floorf(log2f(v)) + 7;
    uint32_t e = (uint32_t)(e0 < 0 ? 0 : (e0 > 15 ? 15 : e0));
    for (;;) {
        if (e == 0) {
            float c = ceilf(v * 512.0f);
            uint32_t m = c >= 4294967296.0f ? 0xFFFFFFFFu : (uint32_t)c;
            if (m <= 7) return m;
            e = 1;
            continue;
        }
        float unit = ldexpf(1.0f, (int)e - 7);
        float mf = ceilf((v / unit - 1.0f) * 8.0f);
        /* Rust `as i32` saturates */
        int m = mf >= 2147483648.0f ? 2147483647 : (mf <= -2147483648.0f ? (-2147483647 - 1) : (int)mf);
        if (m < 0) return e << 3;
        if (m <= 7) return (e << 3) | (uint32_t)m;
        if (e >= 15) return (15u << 3) | 7u;
        e += 1;
    }
}

/* converter/src/main.rs:404-410: bump while the decoded byte is still below raw */
static uint32_t encode_subblock_ceil(float raw) {
    uint32_t stored = orc_encode_ue4m3_ceil(raw);
    while (stored < 0x7F && orc_ue4m3(stored) < raw) stored++;
    return stored;
}

/* converter/src/main.rs:111-119: number of midpoints <= m */
static uint32_t e2m1_index(float m) {
    static const float MID[7] = {0.25f, 0.75f, 1.25f, 1.75f, 2.5f, 3.5f, 5.0f};
    uint32_t n = 0;
    for (int i = 0; i < 7; i++) n += (m >= MID[i]);
    return n;
}

/* converter/src/main.rs:550-664, ScalesMode::Ceil, no diag weights, no byte cap */
float orc_quantize_ceil(const float* values, size_t n, uint8_t* out) {
    size_t n_sub = n / 16;
    float* raw = (float*)malloc(n_sub * sizeof(float));
    float max_scale = 0.0f;
    for (size_t i = 0; i < n_sub; i++) {
        float mx = 0.0f;
        for (int j = 0; j < 16; j++) {
            float a = fabsf(values[i * 16 + j]);
            if (a > mx) mx = a; /* f32::max semantics for non-NaN input */
        }
        raw[i] = mx / 6.0f;
        if (raw[i] > max_scale) max_scale = raw[i];
    }
    float global = max_scale > 0.0f ? max_scale / 448.0f : 1.0f;
    for (size_t b = 0; b < n / 64; b++) {
        uint8_t* blk = out + b * NVFP4_BLOCK_BYTES;
        memset(blk, 0, NVFP4_BLOCK_BYTES);
        for (int sb = 0; sb < 4; sb++) {
            float r = raw[b * 4 + sb] / global;
            uint32_t stored = encode_subblock_ceil(r);
            blk[sb] = (uint8_t)stored;
            float dec = orc_ue4m3(stored) * global;
            float inv = 1.0f / dec;
            for (int j = 0; j < 16; j++) {
                float v = values[b * 64 + sb * 16 + j];
                uint32_t nib = e2m1_index(fabsf(v) * inv) | ((uint32_t)(v < 0.0f) << 3);
                int idx = sb * 16 + j;
                blk[4 + idx / 2] |= (uint8_t)(nib << (4 * (idx % 2)));
            }
        }
    }
    free(raw);
    return global;
}

/* ------------------------------------------------------------------ the CPU GEMV */

/* cpu_nvfp4.rs:181-197: per 16 values, the 8 even ones first, then the 8 odd ones */
static size_t lane_pos(size_t j) {
    size_t k = j & 15;
    return (j & ~(size_t)15) | ((k & 1) == 0 ? (k >> 1) : 8 + (k >> 1));
}

static float* permute_x(const float* x, size_t tokens, size_t cols) {
    float* xp = (float*)malloc(tokens * cols * sizeof(float));
    for (size_t t = 0; t < tokens; t++)
        for (size_t j = 0; j < cols; j++) xp[t * cols + lane_pos(j)] = x[t * cols + j];
    return xp;
}

/* cpu_nvfp4.rs:205-235.  nt tokens (<= 4) starting at t0 against one weight row. */
static void row_scalar(const uint8_t* row, const float lut[256], const float* xp, size_t cols, size_t t0,
                       int nt, float* out) {
    float acc[4][8];
    memset(acc, 0, sizeof acc);
    size_t nb = cols / 64;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t* blk = row + b * NVFP4_BLOCK_BYTES;
        for (int sb = 0; sb < 4; sb++) {
            float s = lut[blk[sb]];
            const uint8_t* codes = blk + 4 + sb * 8;
            float lo[8], hi[8];
            for (int l = 0; l < 8; l++) {
                lo[l] = orc_e2m1(codes[l] & 15u);
                hi[l] = orc_e2m1(codes[l] >> 4);
            }
            size_t base = b * 64 + (size_t)sb * 16;
            for (int t = 0; t < nt; t++) {
                const float* xv = xp + (t0 + t) * cols + base;
                for (int l = 0; l < 8; l++) {
                    float p = lo[l] * xv[l] + hi[l] * xv[8 + l];
                    acc[t][l] = acc[t][l] + p * s;
                }
            }
        }
    }
    for (int t = 0; t < nt; t++) {
        float r = 0.0f;
        for (int l = 0; l < 8; l++) r += acc[t][l];
        out[t] = r;
    }
}

/* cpu_nvfp4.rs:237-287: the same operations eight lanes at a time */
__attribute__((target("avx2"))) static void row_avx2(const uint8_t* row, const float lut[256], const float* xp,
                                                     size_t cols, size_t t0, int nt, float* out) {
    const __m256 mag = _mm256_loadu_ps(MAG8);
    const __m256i m15 = _mm256_set1_epi32(15), m8 = _mm256_set1_epi32(8);
    __m256 acc[4] = {_mm256_setzero_ps(), _mm256_setzero_ps(), _mm256_setzero_ps(), _mm256_setzero_ps()};
    size_t nb = cols / 64;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t* blk = row + b * NVFP4_BLOCK_BYTES;
        for (int sb = 0; sb < 4; sb++) {
            __m256 s = _mm256_set1_ps(lut[blk[sb]]);
            __m256i by = _mm256_cvtepu8_epi32(_mm_loadl_epi64((const __m128i*)(blk + 4 + sb * 8)));
            __m256i nl = _mm256_and_si256(by, m15), nh = _mm256_srli_epi32(by, 4);
            __m256 sl = _mm256_castsi256_ps(_mm256_slli_epi32(_mm256_and_si256(nl, m8), 28));
            __m256 sh = _mm256_castsi256_ps(_mm256_slli_epi32(_mm256_and_si256(nh, m8), 28));
            __m256 wl = _mm256_xor_ps(_mm256_permutevar8x32_ps(mag, nl), sl);
            __m256 wh = _mm256_xor_ps(_mm256_permutevar8x32_ps(mag, nh), sh);
            size_t base = b * 64 + (size_t)sb * 16;
            for (int t = 0; t < nt; t++) {
                const float* xv = xp + (t0 + t) * cols + base;
                __m256 p = _mm256_add_ps(_mm256_mul_ps(wl, _mm256_loadu_ps(xv)), _mm256_mul_ps(wh, _mm256_loadu_ps(xv + 8)));
                acc[t] = _mm256_add_ps(acc[t], _mm256_mul_ps(p, s));
            }
        }
    }
    for (int t = 0; t < nt; t++) {
        float lanes[8];
        _mm256_storeu_ps(lanes, acc[t]);
        float r = 0.0f;
        for (int l = 0; l < 8; l++) r += lanes[l];
        out[t] = r;
    }
}

static void row_dot(int path, const uint8_t* row, const float lut[256], const float* xp, size_t cols, size_t t0,
                    int nt, float* out) {
    if (path == 1) row_avx2(row, lut, xp, cols, t0, nt, out);
    else row_scalar(row, lut, xp, cols, t0, nt, out);
}

/* cpu_nvfp4.rs:330-345: rows r0..r1 against every token, tokens in tiles of 4 */
static void rows_into(int path, const uint8_t* w, size_t rows, size_t cols, const float lut[256], const float* xp,
                      size_t tokens, size_t r0, size_t r1, float* out) {
    size_t rb = cols / 64 * NVFP4_BLOCK_BYTES;
    float tmp[4];
    for (size_t r = r0; r < r1; r++) {
        for (size_t t0 = 0; t0 < tokens; t0 += 4) {
            int nt = (int)(tokens - t0 < 4 ? tokens - t0 : 4);
            row_dot(path, w + r * rb, lut, xp, cols, t0, nt, tmp);
            for (int t = 0; t < nt; t++) out[(t0 + t) * rows + r] = tmp[t];
        }
    }
}

static int shape_ok(size_t cols) { return cols != 0 && cols % NVFP4_BLOCK_VALUES == 0; }

static int clamp_threads(int threads, size_t limit) {
    if (threads < 1) threads = 1;
    if (limit < 1) limit = 1;
    return (size_t)threads > limit ? (int)limit : threads;
}

/* cpu_nvfp4.rs:349-373: rows n*w/k .. n*(w+1)/k to worker w */
int orc_gemv(const uint8_t* w, size_t rows, size_t cols, float gs, const float* x, size_t tokens, float* y,
             int threads, int path) {
    if (!shape_ok(cols)) return -1;
    float lut[256];
    orc_scale_lut(gs, lut);
    float* xp = permute_x(x, tokens, cols);
    int k = clamp_threads(threads, rows);
#pragma omp parallel for num_threads(k) schedule(static, 1)
    for (int wk = 0; wk < k; wk++)
        rows_into(path, w, rows, cols, lut, xp, tokens, rows * (size_t)wk / (size_t)k, rows * (size_t)(wk + 1) / (size_t)k, y);
    free(xp);
    return 0;
}

float orc_silu_mul(float g, float u) { return (g / (1.0f + expf(-g))) * u; }

/* glm5_moe.rs:141-154 */
static float swiglu_clamp(float g, float u, float l) {
    if (g > l) g = l;
    if (u > l) u = l;
    else if (u < -l) u = -l;
    return (g / (1.0f + expf(-g))) * u;
}

/* cpu_nvfp4.rs:378-427 (limit <= 0) and glm5_moe.rs:271-278 (limit > 0).  The reference's fused
 * form writes h in lane order and reads it with the down rows; that is the same arithmetic as
 * gemv + activation + gemv (its own test holds them bit-identical), which is what runs here. */
int orc_ffn_clamped(const uint8_t* gate, float gs_g, const uint8_t* up, float gs_u, const uint8_t* down, float gs_d,
                    size_t hidden, size_t inter, float limit, const float* x, size_t tokens, float* y, int threads,
                    int path) {
    if (!shape_ok(hidden) || !shape_ok(inter)) return -1;
    float* g = (float*)malloc(tokens * inter * sizeof(float));
    float* u = (float*)malloc(tokens * inter * sizeof(float));
    orc_gemv(gate, inter, hidden, gs_g, x, tokens, g, threads, path);
    orc_gemv(up, inter, hidden, gs_u, x, tokens, u, threads, path);
    for (size_t i = 0; i < tokens * inter; i++) g[i] = limit > 0.0f ? swiglu_clamp(g[i], u[i], limit) : orc_silu_mul(g[i], u[i]);
    orc_gemv(down, hidden, inter, gs_d, g, tokens, y, threads, path);
    free(g);
    free(u);
    return 0;
}

int orc_expert_ffn(const uint8_t* gate, float gs_g, const uint8_t* up, float gs_u, const uint8_t* down, float gs_d,
                   size_t hidden, size_t inter, const float* x, size_t tokens, float* y, int threads, int path) {
    return orc_ffn_clamped(gate, gs_g, up, gs_u, down, gs_d, hidden, inter, 0.0f, x, tokens, y, threads, path);
}

/* cpu_nvfp4.rs:491-514: the engine's f32 scale, then everything in f64 */
void orc_gemv_f64(const uint8_t* w, size_t rows, size_t cols, float gs, const float* x, size_t tokens, int rule,
                  double* y, double* sum_abs) {
    size_t nb = cols / 64, rb = nb * NVFP4_BLOCK_BYTES;
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)rows; r++) {
        const uint8_t* row = w + (size_t)r * rb;
        for (size_t t = 0; t < tokens; t++) {
            double s1 = 0.0, s2 = 0.0;
            for (size_t b = 0; b < nb; b++) {
                const uint8_t* blk = row + b * NVFP4_BLOCK_BYTES;
                for (int idx = 0; idx < 64; idx++) {
                    uint8_t sc = blk[idx / 16];
                    if (rule) sc = orc_scale_rule(sc);
                    float s = orc_ue4m3(sc) * gs;
                    uint32_t nib = (blk[4 + idx / 2] >> (4 * (idx % 2))) & 15u;
                    double p = (double)orc_e2m1(nib) * (double)s * (double)x[t * cols + b * 64 + idx];
                    s1 += p;
                    s2 += fabs(p);
                }
            }
            y[t * rows + (size_t)r] = s1;
            if (sum_abs) sum_abs[t * rows + (size_t)r] = s2;
        }
    }
}

/* cpu_nvfp4.rs:516-520: gamma_n, n = K/16 + 10, u = 2^-24 */
double orc_gamma(size_t cols) {
    double nu = (double)(cols / 16 + 10) * ldexp(1.0, -24);
    return nu / (1.0 - nu);
}

/* ------------------------------------------------------------------ small kernels */

void orc_silu_mul_combo(const float* h1, size_t combos, size_t inter, float* h2) {
    for (size_t c = 0; c < combos; c++)
        for (size_t j = 0; j < inter; j++) h2[c * inter + j] = orc_silu_mul(h1[c * 2 * inter + j], h1[c * 2 * inter + inter + j]);
}

void orc_acc_combo(const float* x, const float* rw, size_t tokens, size_t topk, size_t hidden, float* y) {
    for (size_t t = 0; t < tokens; t++)
        for (size_t c = 0; c < hidden; c++) {
            float acc = 0.0f;
            for (size_t j = 0; j < topk; j++) acc += rw[t * topk + j] * x[(t * topk + j) * hidden + c];
            y[t * hidden + c] += acc;
        }
}

/* kernels.rs:3109-3184.  The device kernel reduces max and sum with a halving tree over E slots
 * (E a power of two there); the same tree is kept so that the denominator's rounding matches. */
static float tree_reduce(float* red, size_t n, int is_max) {
    for (size_t st = n / 2; st > 0; st >>= 1)
        for (size_t e = 0; e < st; e++) red[e] = is_max ? fmaxf(red[e], red[e + st]) : red[e] + red[e + st];
    return red[0];
}

void orc_router_topk(const float* logits, size_t tokens, size_t experts, size_t topk, int32_t* ids, float* wts) {
    float* p = (float*)malloc(experts * sizeof(float));
    float* red = (float*)malloc(experts * sizeof(float));
    for (size_t t = 0; t < tokens; t++) {
        const float* l = logits + t * experts;
        memcpy(red, l, experts * sizeof(float));
        float mx = tree_reduce(red, experts, 1);
        for (size_t e = 0; e < experts; e++) p[e] = red[e] = expf(l[e] - mx);
        float den = tree_reduce(red, experts, 0);
        for (size_t e = 0; e < experts; e++) p[e] = p[e] / den;
        float sum = 0.0f;
        for (size_t j = 0; j < topk; j++) {
            float best = p[0];
            for (size_t e = 1; e < experts; e++) best = fmaxf(best, p[e]);
            size_t pick = 0;
            while (p[pick] != best) pick++; /* lowest index holding the maximum */
            ids[t * topk + j] = (int32_t)pick;
            wts[t * topk + j] = p[pick];
            sum += p[pick];
            p[pick] = -1.0f;
        }
        for (size_t j = 0; j < topk; j++) wts[t * topk + j] = wts[t * topk + j] / sum;
    }
    free(p);
    free(red);
}

/* kernels.rs:4238-4260 */
int32_t orc_argmax_ref(const float* logits, size_t n) {
    float rb[1024];
    int32_t ri[1024];
    for (size_t t = 0; t < 1024; t++) {
        float best = -3.0e38f;
        int32_t bi = 0;
        for (size_t i = t; i < n; i += 1024)
            if (logits[i] > best) {
                best = logits[i];
                bi = (int32_t)i;
            }
        rb[t] = best;
        ri[t] = bi;
    }
    for (size_t st = 512; st > 0; st >>= 1)
        for (size_t t = 0; t < st; t++)
            if (rb[t + st] > rb[t]) {
                rb[t] = rb[t + st];
                ri[t] = ri[t + st];
            }
    return ri[0];
}

/* gen.rs:4168-4534 without the shared expert and staging: route, per-combo gate|up GEMV on the
 * token's x (x_div = topk), SwiGLU, per-combo down GEMV, weighted sum in pick order into y (y is
 * overwritten: it starts from zero here). */
int orc_moe_layer(const uint8_t* gate_up, float gs_gu, const uint8_t* down, float gs_dn, size_t experts, size_t hidden,
                  size_t inter, const float* x, const float* logits, size_t tokens, size_t topk, int32_t* ids,
                  float* wts, float* y, int threads, int path) {
    if (!shape_ok(hidden) || !shape_ok(inter)) return -1;
    orc_router_topk(logits, tokens, experts, topk, ids, wts);
    size_t gu_bytes = orc_byte_len(2 * inter, hidden), dn_bytes = orc_byte_len(hidden, inter);
    size_t combos = tokens * topk;
    float* h1 = (float*)malloc(combos * 2 * inter * sizeof(float));
    float* h2 = (float*)malloc(combos * inter * sizeof(float));
    float* eo = (float*)malloc(combos * hidden * sizeof(float));
    for (size_t c = 0; c < combos; c++) {
        size_t e = (size_t)ids[c];
        orc_gemv(gate_up + e * gu_bytes, 2 * inter, hidden, gs_gu, x + (c / topk) * hidden, 1, h1 + c * 2 * inter, threads, path);
    }
    orc_silu_mul_combo(h1, combos, inter, h2);
    for (size_t c = 0; c < combos; c++) {
        size_t e = (size_t)ids[c];
        orc_gemv(down + e * dn_bytes, hidden, inter, gs_dn, h2 + c * inter, 1, eo + c * hidden, threads, path);
    }
    memset(y, 0, tokens * hidden * sizeof(float));
    orc_acc_combo(eo, wts, tokens, topk, hidden, y);
    free(h1);
    free(h2);
    free(eo);
    return 0;
}

/* kernels.rs:67-71 */
uint16_t orc_f32_to_bf16(float v) {
    uint32_t x;
    memcpy(&x, &v, 4);
    x += 0x7FFFu + ((x >> 16) & 1u);
    return (uint16_t)(x >> 16);
}

float orc_bf16_to_f32(uint16_t b) {
    uint32_t x = (uint32_t)b << 16;
    float v;
    memcpy(&v, &x, 4);
    return v;
}
