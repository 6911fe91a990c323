// TEST INFRASTRUCTURE — CPU oracle for the batched quantized decode path (see qw_oracle.h for what pins it).
// Plain C; build with oracle/Makefile. Every function names the reference text it restates.
#include "qw_oracle.h"
#include "iq3s_grid.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

// ---------------------------------------------------------------- scalars
// Reference: src/ggml_dq.c:6-19 (h2f through _Float16, bf2f by shifting); written with integer arithmetic here so
// that a compiler without _Float16 builds it.
float qwo_h2f(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 31u, man = h & 1023u, u;
    if (exp == 0) {
        if (man == 0) u = sign;
        else { // subnormal: normalise
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 1024u));
            u = sign | (uint32_t)(127 - 15 - e) << 23 | (man & 1023u) << 13;
        }
    } else if (exp == 31) u = sign | 0x7f800000u | man << 13;
    else u = sign | (exp + 112u) << 23 | man << 13;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

uint16_t qwo_f2h(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    u &= 0x7fffffffu;
    if (u >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (u > 0x7f800000u ? 0x200u : 0)); // inf / nan
    if (u >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);                                   // rounds to inf (>= 65520)
    if (u < 0x33000001u) return (uint16_t)sign;                                                // <= 2^-25 rounds to zero
    int e = (int)(u >> 23) - 127;
    uint32_t man = (u & 0x7fffffu) | 0x800000u;
    int shift = e < -14 ? 13 + (-14 - e) : 13; // subnormal results lose more bits
    uint32_t half = man >> shift, rem = man & ((1u << shift) - 1), mid = 1u << (shift - 1);
    if (rem > mid || (rem == mid && (half & 1))) half++;
    if (e < -14) return (uint16_t)(sign | half); // carries into the exponent field by itself when it rounds up to 2^-14
    return (uint16_t)(sign | (((uint32_t)(e + 15) << 10) + (half - 0x400u)));
}

float qwo_bf2f(uint16_t h) {
    const uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | p[1] << 8); }

// ---------------------------------------------------------------- formats (src/gguf.c:15-25)
int qwo_block_values(int type) {
    switch (type) {
    case 0: case 1: case 30: return 1;
    case 8: case 20: return 32;
    case 12: case 13: case 14: case 21: case 23: return 256;
    default: return 0;
    }
}
int qwo_block_bytes(int type) {
    switch (type) {
    case 0: return 4;
    case 1: case 30: return 2;
    case 8: return 34;
    case 20: return 18;
    case 12: return 144;
    case 13: return 176;
    case 14: return 210;
    case 21: return 110;
    case 23: return 136;
    default: return 0;
    }
}
size_t qwo_row_bytes(int type, int K) { return qwo_block_values(type) ? (size_t)K / (size_t)qwo_block_values(type) * (size_t)qwo_block_bytes(type) : 0; }
bool qwo_dq_ok(int type) { return qwo_block_values(type) != 0; }
const uint32_t *qwo_iq3s_table(void) { return qwo_iq3s_grid; }

// Q8_0, 34 bytes: d, qs[32] (src/ggml_dq.c:34-37)
static void dq_q8_0(const uint8_t *b, float *y) {
    const float d = qwo_h2f(rd16(b));
    for (int j = 0; j < 32; j++) y[j] = (float)(int8_t)b[2 + j] * d;
}

// IQ3_S, 110 bytes: d @0, qs[64] @2, qh[8] @66, signs[32] @74, scales[4] @106 (kernels/moe_iq.metal:102-118,
// written in the per-block style of src/ggml_dq.c)
static void dq_iq3_s(const uint8_t *b, float *y) {
    const float d = qwo_h2f(rd16(b));
    const uint8_t *qs = b + 2, *qh = b + 66, *signs = b + 74, *sc = b + 106;
    for (int ib = 0; ib < 8; ib++) {
        const float db = d * (float)(1 + 2 * ((sc[ib / 2] >> (4 * (ib % 2))) & 15));
        for (int l = 0; l < 4; l++) {
            const uint32_t g1 = qwo_iq3s_grid[qs[8 * ib + 2 * l] | ((qh[ib] << (8 - 2 * l)) & 256)];
            const uint32_t g2 = qwo_iq3s_grid[qs[8 * ib + 2 * l + 1] | ((qh[ib] << (7 - 2 * l)) & 256)];
            const uint32_t s = signs[4 * ib + l];
            for (int j = 0; j < 4; j++) {
                y[32 * ib + 8 * l + j] = db * (float)((g1 >> (8 * j)) & 255) * ((s & (1u << j)) ? -1.0f : 1.0f);
                y[32 * ib + 8 * l + 4 + j] = db * (float)((g2 >> (8 * j)) & 255) * ((s & (1u << (j + 4))) ? -1.0f : 1.0f);
            }
        }
    }
}

// The K-quant and 4-bit codebook formats, written as "value at position i of the block" (the reference walks each
// block with running pointers, src/ggml_dq.c:39-118; the arithmetic per value is the same and in the same order).
static const int8_t iq4nl_values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

// 6-bit scale and minimum of sub-block j (0..7) from the 12 packed bytes of Q4_K / Q5_K (src/ggml_dq.c:24-32):
// j < 4: low six bits of bytes j and j + 4; j >= 4: a nibble of byte j + 4 with the top two bits of byte j - 4 / j.
static void k4_scale_min(const uint8_t *p, int j, int *sc, int *mn) {
    if (j < 4) {
        *sc = p[j] & 63;
        *mn = p[j + 4] & 63;
    } else {
        *sc = (p[j + 4] & 15) | (p[j - 4] >> 6 << 4);
        *mn = (p[j + 4] >> 4) | (p[j] >> 6 << 4);
    }
}

// Q4_K, 144 bytes: d @0, dmin @2, scales[12] @4, qs[128] @16. Values 64 g .. 64 g + 31 are the low nibbles of
// qs[32 g ..], values 64 g + 32 .. 64 g + 63 the high nibbles (src/ggml_dq.c:39-54).
static float q4_k_value(const uint8_t *b, int i) {
    int sc, mn;
    k4_scale_min(b + 4, i >> 5, &sc, &mn);
    const uint8_t byte = b[16 + 32 * (i >> 6) + (i & 31)];
    const int q = (i & 32) ? byte >> 4 : byte & 15;
    const float ds = qwo_h2f(rd16(b)) * (float)sc, ms = qwo_h2f(rd16(b + 2)) * (float)mn;
    return ds * (float)q - ms;
}

// Q5_K, 176 bytes: d, dmin, scales[12] @4, qh[32] @16, qs[128] @48. As Q4_K with a fifth bit: bit (i >> 5) of
// qh[i & 31] (src/ggml_dq.c:56-75).
static float q5_k_value(const uint8_t *b, int i) {
    int sc, mn;
    k4_scale_min(b + 4, i >> 5, &sc, &mn);
    const uint8_t byte = b[48 + 32 * (i >> 6) + (i & 31)];
    const int q = ((i & 32) ? byte >> 4 : byte & 15) + ((b[16 + (i & 31)] >> (i >> 5) & 1) ? 16 : 0);
    const float ds = qwo_h2f(rd16(b)) * (float)sc, ms = qwo_h2f(rd16(b + 2)) * (float)mn;
    return ds * (float)q - ms;
}

// Q6_K, 210 bytes: ql[128] @0, qh[64] @128, int8 scales[16] @192, d @208. Half h = i >> 7; inside a half, quarter
// c = (i >> 5) & 3 and l = i & 31: low four bits from ql[64 h + 32 (c & 1) + l] (high nibble when c >= 2), top two
// bits from bits 2 c, 2 c + 1 of qh[32 h + l]; scale index 8 h + 2 c + l / 16 (src/ggml_dq.c:77-98).
static float q6_k_value(const uint8_t *b, int i) {
    const int h = i >> 7, c = (i >> 5) & 3, l = i & 31;
    const uint8_t lo = b[64 * h + 32 * (c & 1) + l];
    const int q = (int)(((c & 2) ? lo >> 4 : lo & 15) | ((b[128 + 32 * h + l] >> (2 * c) & 3) << 4)) - 32;
    const int sc = (int8_t)b[192 + 8 * h + 2 * c + l / 16];
    return qwo_h2f(rd16(b + 208)) * (float)sc * (float)q;
}

// IQ4_NL, 18 bytes: d, qs[16]: value j < 16 from the low nibble of qs[j], value j + 16 from the high nibble,
// through the 16-entry codebook (src/ggml_dq.c:100-107).
static float iq4_nl_value(const uint8_t *b, int i) {
    const uint8_t byte = b[2 + (i & 15)];
    return qwo_h2f(rd16(b)) * (float)iq4nl_values[(i & 16) ? byte >> 4 : byte & 15];
}

// IQ4_XS, 136 bytes: d @0, scales_h (u16) @2, scales_l[4] @4, qs[128] @8. Sub-block s = i >> 5 has the six-bit
// scale (nibble s of scales_l | two bits of scales_h << 4) - 32, and the nibble layout of IQ4_NL (src/ggml_dq.c:109-124).
static float iq4_xs_value(const uint8_t *b, int i) {
    const int s = i >> 5, j = i & 31;
    const int ls = ((b[4 + s / 2] >> (4 * (s & 1))) & 15) | ((rd16(b + 2) >> (2 * s) & 3) << 4);
    const uint8_t byte = b[8 + 16 * s + (j & 15)];
    const float dl = qwo_h2f(rd16(b)) * (float)(ls - 32);
    return dl * (float)iq4nl_values[(j & 16) ? byte >> 4 : byte & 15];
}

bool qwo_dq_row(int type, const void *src, float *dst, int K) {
    const uint8_t *s = src;
    switch (type) {
    case 0: memcpy(dst, src, (size_t)K * 4); return true;
    case 1: for (int i = 0; i < K; i++) dst[i] = qwo_h2f(rd16(s + 2 * i)); return true;
    case 30: for (int i = 0; i < K; i++) dst[i] = qwo_bf2f(rd16(s + 2 * i)); return true;
    case 12: for (int i = 0; i < K; i++) dst[i] = q4_k_value(s + 144 * (i >> 8), i & 255); return true;
    case 13: for (int i = 0; i < K; i++) dst[i] = q5_k_value(s + 176 * (i >> 8), i & 255); return true;
    case 14: for (int i = 0; i < K; i++) dst[i] = q6_k_value(s + 210 * (i >> 8), i & 255); return true;
    case 20: for (int i = 0; i < K; i++) dst[i] = iq4_nl_value(s + 18 * (i >> 5), i & 31); return true;
    case 23: for (int i = 0; i < K; i++) dst[i] = iq4_xs_value(s + 136 * (i >> 8), i & 255); return true;
    case 8: for (int i = 0; i < K / 32; i++) dq_q8_0(s + 34 * i, dst + 32 * i); return true;
    case 21: for (int i = 0; i < K / 256; i++) dq_iq3_s(s + 110 * i, dst + 256 * i); return true;
    default: return false;
    }
}

// ---------------------------------------------------------------- second formulation: 16-value units + pre-signed table
void qwo_tab_iq3ss(uint16_t *tab) { // kernels/moe_gg.metal:495-500
    for (uint32_t i = 0; i < 8192; i++)
        for (uint32_t j = 0; j < 4; j++) {
            const uint16_t g = qwo_f2h((float)((qwo_iq3s_grid[i & 511] >> (8 * j)) & 255));
            tab[4 * i + j] = (i >> (9 + j)) & 1 ? (uint16_t)(g | 0x8000u) : g;
        }
}

static uint16_t *tab_iq3ss(void) {
    static uint16_t *t;
    if (!t) {
        uint16_t *n = malloc(8192 * 4 * sizeof *n);
        qwo_tab_iq3ss(n);
        t = n;
    }
    return t;
}

// unit u of a row -> 16 values (kernels/moe_gg.metal:321-334 for IQ3_S, :396-407 for Q8_0); value = d * w
static void unit_iq3_s(const uint8_t *row, uint32_t u, const uint16_t *tab, float *y) {
    const uint8_t *b = row + (u >> 4) * 110;
    const uint32_t ib = (u >> 1) & 7, hh = u & 1;
    const uint32_t q0 = rd16(b + 2 + 8 * ib + 4 * hh), q1 = rd16(b + 4 + 8 * ib + 4 * hh);
    const uint32_t qh = (uint32_t)b[66 + ib] >> (4 * hh), sg = rd16(b + 74 + 4 * ib + 2 * hh);
    const float d = qwo_h2f(rd16(b)) * (float)(1 + 2 * ((b[106 + ib / 2] >> (4 * (ib & 1))) & 15));
    const uint32_t idx[4] = {(q0 & 255) | ((qh << 8) & 256) | ((sg & 15) << 9), (q0 >> 8) | ((qh << 7) & 256) | (((sg >> 4) & 15) << 9),
                             (q1 & 255) | ((qh << 6) & 256) | (((sg >> 8) & 15) << 9), (q1 >> 8) | ((qh << 5) & 256) | ((sg >> 12) << 9)};
    for (int i = 0; i < 4; i++)
        for (int j = 0; j < 4; j++) y[4 * i + j] = d * qwo_h2f(tab[4 * idx[i] + j]);
}

static void unit_q8_0(const uint8_t *row, uint32_t u, float *y) {
    const uint8_t *b = row + (u >> 1) * 34;
    const float d = qwo_h2f(rd16(b));
    const uint8_t *q = b + 2 + 16 * (u & 1);
    for (int i = 0; i < 16; i++) y[i] = d * qwo_h2f(qwo_f2h((float)(int8_t)q[i]));
}

bool qwo_dq_row_tab(int type, const void *src, float *dst, int K) {
    if (type != 8 && type != 21) return false;
    const uint16_t *tab = type == 21 ? tab_iq3ss() : NULL;
    for (uint32_t u = 0; u < (uint32_t)K / 16; u++) {
        if (type == 21) unit_iq3_s(src, u, tab, dst + 16 * u);
        else unit_q8_0(src, u, dst + 16 * u);
    }
    return true;
}

// ---------------------------------------------------------------- threads
int qwo_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
static int nthreads(int want) {
    const int m = qwo_max_threads();
    return want <= 0 || want > m ? m : want;
}

// ---------------------------------------------------------------- dense matvec (kernels/qmv_gg.metal:17-39)
void qwo_qmv_f32(int type, const uint8_t *W, int N, int K, const uint16_t *x, int nb, int xstride, float *y, int ystride,
                 int threads) {
    const size_t rb = qwo_row_bytes(type, K);
    float *xf = malloc(sizeof(float) * (size_t)nb * (size_t)K);
    for (int b = 0; b < nb; b++)
        for (int k = 0; k < K; k++) xf[(size_t)b * K + k] = qwo_h2f(x[(size_t)b * xstride + k]);
    const int nt = nthreads(threads);
#pragma omp parallel num_threads(nt)
    {
        float *w = malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(static)
        for (int r = 0; r < N; r++) {
            qwo_dq_row(type, W + (size_t)r * rb, w, K);
            for (int b = 0; b < nb; b++) {
                const float *xb = xf + (size_t)b * K;
                float acc = 0;
                for (int k = 0; k < K; k++) acc += w[k] * xb[k];
                y[(size_t)b * ystride + r] = acc;
            }
        }
        free(w);
    }
    free(xf);
}

void qwo_qmv_f64(int type, const uint8_t *W, int N, int K, const uint16_t *x, int nb, int xstride, double *y, int ystride,
                 int threads) {
    const size_t rb = qwo_row_bytes(type, K);
    const int nt = nthreads(threads);
#pragma omp parallel num_threads(nt)
    {
        float *w = malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(static)
        for (int r = 0; r < N; r++) {
            qwo_dq_row(type, W + (size_t)r * rb, w, K);
            for (int b = 0; b < nb; b++) {
                double acc = 0;
                for (int k = 0; k < K; k++) acc += (double)w[k] * (double)qwo_h2f(x[(size_t)b * xstride + k]);
                y[(size_t)b * ystride + r] = acc;
            }
        }
        free(w);
    }
}

// ---------------------------------------------------------------- router (kernels/moe_gg.metal:25-41)
void qwo_router(int wfmt, const uint16_t *Wr, const uint16_t *Wsg, const uint16_t *x, int nb, int D, int E, float *logits) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r <= E; r++) {
        const uint16_t *w = r < E ? Wr + (size_t)r * D : Wsg;
        for (int t = 0; t < nb; t++) {
            double acc = 0;
            for (int k = 0; k < D; k++) acc += (double)(wfmt == 30 ? qwo_bf2f(w[k]) : qwo_h2f(w[k])) * (double)qwo_h2f(x[(size_t)t * D + k]);
            logits[(size_t)t * (E + 1) + r] = (float)acc;
        }
    }
}

// ---------------------------------------------------------------- selection (kernels/moe_gg.metal:123-189)
size_t qwo_sel_bytes(int gnb, int topk) {
    const size_t gu = (size_t)gnb * (size_t)topk;
    return 4 + 4 * gu + 4 * gu + gu * (size_t)gnb + 4 * (size_t)gnb * (size_t)(topk + 1);
}

// Repeated argmax, strict '>' so that equal values keep the lowest index (kernels/moe_gg.metal:136-147;
// bench/moe_decode.c:139-148 is the same rule written as a scan). pk receives the picked logits.
static void topk_row(const float *lg, int E, int topk, uint32_t *ids, float *pk) {
    char *used = calloc((size_t)E, 1);
    for (int k = 0; k < topk; k++) {
        int bi = -1;
        for (int e = 0; e < E; e++)
            if (!used[e] && (bi < 0 || lg[e] > lg[bi])) bi = e;
        used[bi] = 1;
        ids[k] = (uint32_t)bi;
        if (pk) pk[k] = lg[bi];
    }
    free(used);
}

void qwo_topk(const float *logits, int nbr, int E, int topk, uint32_t *ids) {
    for (int t = 0; t < nbr; t++) topk_row(logits + (size_t)t * (E + 1), E, topk, ids + (size_t)t * topk, NULL);
}

void qwo_select(const float *logits, int nbr, int E, int topk, int gnb, void *sel) {
    const size_t gu = (size_t)gnb * (size_t)topk;
    uint8_t *base = sel;
    memset(base, 0, qwo_sel_bytes(gnb, topk));
    uint32_t *U = (uint32_t *)base, *ue = U + 1, *mask = ue + gu;
    uint8_t *slot = (uint8_t *)(mask + gu);
    float *w = (float *)(slot + gu * (size_t)gnb);
    uint32_t *ids = malloc(sizeof *ids * (size_t)nbr * (size_t)topk);
    float *pk = malloc(sizeof *pk * (size_t)topk);
    for (int t = 0; t < nbr; t++) {
        const float *lg = logits + (size_t)t * (E + 1);
        topk_row(lg, E, topk, ids + (size_t)t * topk, pk);
        // softmax over the picked logits only, max (= rank 0) subtracted, summed in rank order (:151-154)
        float sm = 0;
        for (int k = 0; k < topk; k++) sm += expf(pk[k] - pk[0]);
        for (int k = 0; k < topk; k++) w[(size_t)t * (topk + 1) + k] = expf(pk[k] - pk[0]) / sm;
        w[(size_t)t * (topk + 1) + topk] = 1.0f / (1.0f + expf(-lg[E])); // shared-expert gate (:155)
    }
    // dedupe in order of first appearance over the flat index t * topk + k (:112, :156-188; the simple O(n^2) form is
    // kernels/moe_decode.metal:439-454)
    uint32_t nu = 0;
    for (int p = 0; p < nbr * topk; p++) {
        uint32_t u = 0;
        while (u < nu && ue[u] != ids[p]) u++;
        if (u == nu) ue[nu++] = ids[p];
        mask[u] |= 1u << (p / topk);
        slot[(size_t)u * gnb + (size_t)(p / topk)] = (uint8_t)(p % topk);
    }
    *U = nu;
    free(ids);
    free(pk);
}

// ---------------------------------------------------------------- MoE layer
static float silu_mul_f(float g, float up) { return g / (1.0f + expf(-g)) * up; } // kernels/moe_gg.metal:571, 628

void qwo_moe_layer_f32(const qwo_moe_weights *m, const float *logits, const uint16_t *x, int nb, int gnb, uint16_t *out,
                       float *Hout, void *selout, int threads) {
    const int D = m->D, I = m->I, E = m->E, K = m->topk;
    const size_t gu = (size_t)gnb * (size_t)K;
    void *sel = malloc(qwo_sel_bytes(gnb, K));
    qwo_select(logits, nb, E, K, gnb, sel);
    const uint32_t U = *(uint32_t *)sel, *ue = (uint32_t *)sel + 1, *mask = ue + gu;
    const uint8_t *slot = (const uint8_t *)(mask + gu);
    const float *w = (const float *)(slot + gu * (size_t)gnb);
    float *xf = malloc(sizeof(float) * (size_t)nb * D);
    for (size_t i = 0; i < (size_t)nb * D; i++) xf[i] = qwo_h2f(x[i]);
    float *H = calloc((size_t)nb * (K + 1) * I, sizeof(float));   // [nb][K+1][I], float (src/engine.c:157)
    float *Pg = calloc((size_t)nb * K * D, sizeof(float));         // [nb][K][D]
    float *Psh = calloc((size_t)nb * D, sizeof(float));            // [nb][D]
    const size_t rgu = qwo_row_bytes(m->fgu, D), rd = qwo_row_bytes(m->fd, I);
    const int nt = nthreads(threads);
    // gate/up + SwiGLU: unit of work = (u, j); u == U is the shared expert (all tokens) (kernels/moe_gg.metal:563-573, 600-631)
#pragma omp parallel num_threads(nt)
    {
        float *wg = malloc(sizeof(float) * (size_t)D), *wu = malloc(sizeof(float) * (size_t)D);
#pragma omp for schedule(static)
        for (long q = 0; q < (long)(U + 1) * I; q++) {
            const uint32_t u = (uint32_t)(q / I);
            const int j = (int)(q % I);
            const bool sh = u == U;
            if (sh) {
                qwo_dq_row(m->fsg, m->Wsg + (size_t)j * qwo_row_bytes(m->fsg, D), wg, D);
                qwo_dq_row(m->fsu, m->Wsu + (size_t)j * qwo_row_bytes(m->fsu, D), wu, D);
            } else {
                qwo_dq_row(m->fgu, m->Wg + ((size_t)ue[u] * I + j) * rgu, wg, D);
                qwo_dq_row(m->fgu, m->Wu + ((size_t)ue[u] * I + j) * rgu, wu, D);
            }
            for (int t = 0; t < nb; t++) {
                if (!sh && !((mask[u] >> t) & 1)) continue;
                float g = 0, up = 0;
                for (int k = 0; k < D; k++) {
                    g += wg[k] * xf[(size_t)t * D + k];
                    up += wu[k] * xf[(size_t)t * D + k];
                }
                const int s = sh ? K : slot[(size_t)u * gnb + t];
                H[((size_t)t * (K + 1) + s) * I + j] = silu_mul_f(g, up);
            }
        }
        free(wg);
        free(wu);
    }
    // down (kernels/moe_gg.metal:606-617 shared, :639-652 routed)
#pragma omp parallel num_threads(nt)
    {
        float *wd = malloc(sizeof(float) * (size_t)I);
#pragma omp for schedule(static)
        for (long q = 0; q < (long)(U + 1) * D; q++) {
            const uint32_t u = (uint32_t)(q / D);
            const int r = (int)(q % D);
            const bool sh = u == U;
            if (sh) qwo_dq_row(m->fsd, m->Wsd + (size_t)r * qwo_row_bytes(m->fsd, I), wd, I);
            else qwo_dq_row(m->fd, m->Wd + ((size_t)ue[u] * D + r) * rd, wd, I);
            for (int t = 0; t < nb; t++) {
                if (!sh && !((mask[u] >> t) & 1)) continue;
                const int s = sh ? K : slot[(size_t)u * gnb + t];
                const float *h = H + ((size_t)t * (K + 1) + s) * I;
                float acc = 0;
                for (int k = 0; k < I; k++) acc += wd[k] * h[k];
                if (sh) Psh[(size_t)t * D + r] = acc;
                else Pg[((size_t)t * K + s) * D + r] = acc;
            }
        }
        free(wd);
    }
    // combine in rank order, then the shared expert (kernels/moe_gg.metal:655-663)
    for (int t = 0; t < nb; t++)
        for (int r = 0; r < D; r++) {
            float o = 0;
            for (int s = 0; s < K; s++) o += w[(size_t)t * (K + 1) + s] * Pg[((size_t)t * K + s) * D + r];
            o += w[(size_t)t * (K + 1) + K] * Psh[(size_t)t * D + r];
            out[(size_t)t * D + r] = qwo_f2h(o);
        }
    if (Hout) memcpy(Hout, H, sizeof(float) * (size_t)nb * (K + 1) * I);
    if (selout) memcpy(selout, sel, qwo_sel_bytes(gnb, K));
    free(sel); free(xf); free(H); free(Pg); free(Psh);
}

// Everything in double from the exact dequantized weights (the method of tools/moe_ref.py:72-83).
void qwo_moe_layer_f64(const qwo_moe_weights *m, const float *logits, const uint16_t *x, int nb, double *out, int threads) {
    const int D = m->D, I = m->I, E = m->E, K = m->topk;
    uint32_t *ids = malloc(sizeof *ids * (size_t)nb * K);
    qwo_topk(logits, nb, E, K, ids);
    double *wt = malloc(sizeof(double) * (size_t)nb * (K + 1));
    for (int t = 0; t < nb; t++) {
        const float *lg = logits + (size_t)t * (E + 1);
        double sm = 0, mx = lg[ids[(size_t)t * K]];
        for (int k = 0; k < K; k++) sm += exp((double)lg[ids[(size_t)t * K + k]] - mx);
        for (int k = 0; k < K; k++) wt[(size_t)t * (K + 1) + k] = exp((double)lg[ids[(size_t)t * K + k]] - mx) / sm;
        wt[(size_t)t * (K + 1) + K] = 1.0 / (1.0 + exp(-(double)lg[E]));
    }
    const size_t rgu = qwo_row_bytes(m->fgu, D), rd = qwo_row_bytes(m->fd, I);
    double *H = calloc((size_t)nb * (K + 1) * I, sizeof(double));
    const int nt = nthreads(threads);
#pragma omp parallel num_threads(nt)
    {
        float *wg = malloc(sizeof(float) * (size_t)D), *wu = malloc(sizeof(float) * (size_t)D);
#pragma omp for schedule(static)
        for (long q = 0; q < (long)nb * (K + 1) * I; q++) {
            const int t = (int)(q / ((long)(K + 1) * I)), s = (int)(q / I % (K + 1)), j = (int)(q % I);
            if (s == K) {
                qwo_dq_row(m->fsg, m->Wsg + (size_t)j * qwo_row_bytes(m->fsg, D), wg, D);
                qwo_dq_row(m->fsu, m->Wsu + (size_t)j * qwo_row_bytes(m->fsu, D), wu, D);
            } else {
                const size_t e = ids[(size_t)t * K + s];
                qwo_dq_row(m->fgu, m->Wg + (e * I + j) * rgu, wg, D);
                qwo_dq_row(m->fgu, m->Wu + (e * I + j) * rgu, wu, D);
            }
            double g = 0, up = 0;
            for (int k = 0; k < D; k++) {
                const double xv = qwo_h2f(x[(size_t)t * D + k]);
                g += wg[k] * xv;
                up += wu[k] * xv;
            }
            H[q] = g / (1.0 + exp(-g)) * up;
        }
        free(wg);
        free(wu);
    }
#pragma omp parallel num_threads(nt)
    {
        float *wd = malloc(sizeof(float) * (size_t)I);
#pragma omp for schedule(static)
        for (long q = 0; q < (long)nb * D; q++) {
            const int t = (int)(q / D), r = (int)(q % D);
            double o = 0;
            for (int s = 0; s <= K; s++) {
                if (s == K) qwo_dq_row(m->fsd, m->Wsd + (size_t)r * qwo_row_bytes(m->fsd, I), wd, I);
                else qwo_dq_row(m->fd, m->Wd + ((size_t)ids[(size_t)t * K + s] * D + r) * rd, wd, I);
                const double *h = H + ((size_t)t * (K + 1) + s) * I;
                double acc = 0;
                for (int k = 0; k < I; k++) acc += wd[k] * h[k];
                o += wt[(size_t)t * (K + 1) + s] * acc;
            }
            out[q] = o;
        }
        free(wd);
    }
    free(ids); free(wt); free(H);
}

// ---------------------------------------------------------------- ragged packing (kernels/moe_prefill.metal:15-93)
int qwo_moe_pack(const uint32_t *ids, int P, int E, int tm, uint32_t *counts, uint32_t *offs, uint32_t *pos_of,
                 uint32_t *tiles, int max_tiles) {
    memset(counts, 0, sizeof *counts * (size_t)E);
    for (int p = 0; p < P; p++) counts[ids[p]]++;                 // moe_count
    uint32_t run = 0;
    int nt = 0;
    for (int e = 0; e < E; e++) {                                 // moe_plan: exclusive scans of rows and of tiles
        offs[e] = run;
        for (uint32_t a = run; a < run + counts[e]; a += (uint32_t)tm) {
            if (nt < max_tiles) {
                tiles[4 * nt] = (uint32_t)e;
                tiles[4 * nt + 1] = a;
                tiles[4 * nt + 2] = a + (uint32_t)tm < run + counts[e] ? a + (uint32_t)tm : run + counts[e];
                tiles[4 * nt + 3] = 0;
            }
            nt++;
        }
        run += counts[e];
    }
    for (int t = nt; t < max_tiles; t++) tiles[4 * t] = tiles[4 * t + 1] = tiles[4 * t + 2] = tiles[4 * t + 3] = 0;
    uint32_t *cur = malloc(sizeof *cur * (size_t)E);
    memcpy(cur, offs, sizeof *cur * (size_t)E);
    for (int p = 0; p < P; p++) pos_of[p] = cur[ids[p]]++;        // moe_scatter's cursor, taken in flat order
    free(cur);
    return nt;
}

// ---------------------------------------------------------------- hyper-connection (kernels/hyper_gg.metal:94-233, tools/hc_ref.py:60-70)
void qwo_hyper_gg(int D, int HC, int LR, int NB, int apply, const float *h, const uint16_t *out_f16, const float *inj, const float *w,
                  const uint16_t *Wd_bf16, const uint16_t *Wi_bf16, const uint16_t *Wu_bf16, double *h_out, double *x, double *inj_out) {
    const size_t HCD = (size_t)HC * D;
    double *y = malloc(sizeof(double) * HCD), *sx = malloc(sizeof(double) * (size_t)LR);
    for (int t = 0; t < NB; t++) {
        double *h1 = h_out + (size_t)t * HCD;
        for (int s = 0; s < HC; s++) {
            double js = 0;
            if (apply) { // kernels/hyper_gg.metal:47-51: the column sum over the streams' partial sums
                double a = 0;
                for (int q = 0; q < HC; q++) a += inj[((size_t)t * HC + q) * HC + s];
                js = 2.0 / (1.0 + exp(-a / HC));
            }
            double ss = 0;
            for (int j = 0; j < D; j++) {
                const double v = (double)h[(size_t)t * HCD + (size_t)s * D + j] + (apply ? (double)qwo_h2f(out_f16[(size_t)t * D + j]) * js : 0.0);
                h1[(size_t)s * D + j] = v;
                ss += v * v;
            }
            const double r = 1.0 / sqrt(ss / D + 1e-6);
            for (int j = 0; j < D; j++) y[(size_t)s * D + j] = h1[(size_t)s * D + j] * r * (double)w[(size_t)s * D + j];
        }
#pragma omp parallel for
        for (int r = 0; r < LR; r++) {
            double d = 0;
            for (size_t c = 0; c < HCD; c++) d += (double)qwo_bf2f(Wd_bf16[(size_t)r * HCD + c]) * y[c];
            sx[r] = (d / HC) / (1.0 + exp(-d / HC));
        }
#pragma omp parallel for
        for (int j = 0; j < D; j++) {
            double m = 0;
            for (int s = 0; s < HC; s++) {
                const uint16_t *row = Wu_bf16 + ((size_t)s * D + j) * LR;
                double u = 0;
                for (int r = 0; r < LR; r++) u += (double)qwo_bf2f(row[r]) * sx[r];
                m += y[(size_t)s * D + j] / (1.0 + exp(-u));
            }
            x[(size_t)t * D + j] = m / HC;
        }
        if (Wi_bf16 && inj_out)
            for (int s = 0; s < HC; s++)
                for (int q = 0; q < HC; q++) {
                    double a = 0;
                    for (int j = 0; j < D; j++) a += (double)qwo_bf2f(Wi_bf16[(size_t)q * HCD + (size_t)s * D + j]) * y[(size_t)s * D + j];
                    inj_out[((size_t)t * HC + s) * HC + q] = a;
                }
    }
    free(y);
    free(sx);
}
