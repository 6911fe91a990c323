// Block decoders of the other GGUF formats for the matrix cores: Q4_K (12), Q5_K (13), Q6_K (14), IQ4_NL (20),
// IQ4_XS (23), binary16 (1) and bfloat16 (30) rows. Arithmetic of every format: src/ggml_dq.c:39-143 of the reference.
//
// Every format is cut into "steps": the K-values one matrix instruction consumes (32, or 16 for Q6_K whose scales
// cover 16 values). In a step lane group kg (lane >> 4) supplies 8 (or 4) integer-valued weights of row lane & 15 as
// binary16 — exact, they are small integers — and the step's result is multiplied by the step's scale in float:
//     acc += scale * (x . q) - min * sum(x)        (the last term for Q4_K / Q5_K only)
// so that no product of a scale and an integer is ever rounded to binary16. Which K-values a lane supplies differs
// by format (4-bit codebook bytes hold values j and j + 16); xfrag() of the format fetches the matching activations.
//
// A decoder holds the raw dwords of one block that its lane group needs (r[NR]); load() fills them from the block's
// first byte, so the same object works in "quad" order (lanes 4 r .. 4 r + 3 load row r: 4 lanes read neighbouring
// bytes) followed by pull(), and directly in matrix-core lane order.
#pragma once
#include "qw_common.hip.h"

typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef uint32_t __attribute__((aligned(2))) u1a2;

#define QW_KQ_TAB 256 // entries of the 4-bit codebook table: byte -> (value of low nibble, value of high nibble) as binary16

__device__ __forceinline__ f4 qw_mfma16(h4 a, h4 b, f4 c) { return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0); }
__device__ __forceinline__ f4 qw_mfma_bf(bf8 a, bf8 b, f4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }

// Activations of up to 16 tokens in LDS: xf[c * 16 + m] = the 8 binary16 values k = 8 c .. 8 c + 7 of token m;
// xs[c32 * 16 + m] = float sum of the 32 values of chunk c32 of token m.
struct qw_afrag_kq {
    const u4 *xf;
    const float *xs;
    uint32_t m, kg;
    __device__ __forceinline__ h8 at8(uint32_t k) const { return __builtin_bit_cast(h8, xf[(k >> 3) * 16 + m]); }
    __device__ __forceinline__ h4 at4(uint32_t k) const { return __builtin_bit_cast(h4, ((const u2 *)xf)[((k >> 3) * 16 + m) * 2 + ((k >> 2) & 1)]); }
    __device__ __forceinline__ f4 sum32(uint32_t k) const { return *(const f4 *)(xs + (k >> 5) * 16 + 4 * kg); } // tokens 4 kg .. 4 kg + 3
};

__constant__ const int8_t qw_iq4nl_values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
__device__ __forceinline__ void qw_kq_tab_build(uint32_t *tab) {
    for (uint32_t i = threadIdx.x; i < QW_KQ_TAB; i += blockDim.x) {
        const _Float16 lo = (_Float16)(float)qw_iq4nl_values[i & 15], hi = (_Float16)(float)qw_iq4nl_values[i >> 4];
        tab[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | (uint32_t)__builtin_bit_cast(uint16_t, hi) << 16;
    }
}

// Four bytes (each < 256) to four binary16 integers minus bias: bytes b0 b1 -> first pair, b2 b3 -> second pair.
__device__ __forceinline__ u2 qw_bytes_h4(uint32_t v, float bias) {
    const h2 b = {(_Float16)(1024.0f + bias), (_Float16)(1024.0f + bias)};
    u2 r;
    r.x = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u)) - b);
    r.y = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u)) - b);
    return r;
}
__device__ __forceinline__ h8 qw_bytes_h8(uint32_t lo, uint32_t hi, float bias) {
    const u2 a = qw_bytes_h4(lo, bias), b = qw_bytes_h4(hi, bias);
    return __builtin_bit_cast(h8, u4{a.x, a.y, b.x, b.y});
}

// Six-bit scale and minimum j of the 12 packed bytes of Q4_K / Q5_K held in three dwords (src/ggml_dq.c:24-32).
template <int J> __device__ __forceinline__ void qw_k4_scale_min(const uint32_t *s, uint32_t &sc, uint32_t &mn) {
    auto byte = [&](int i) { return (s[i >> 2] >> (8 * (i & 3))) & 255u; };
    if constexpr (J < 4) {
        sc = byte(J) & 63;
        mn = byte(J + 4) & 63;
    } else {
        sc = (byte(J + 4) & 15) | (byte(J - 4) >> 6 << 4);
        mn = (byte(J + 4) >> 4) | (byte(J) >> 6 << 4);
    }
}

template <int F> struct qw_kq;

// ---------------------------------------------------------------- Q4_K: 144 bytes, d @0, dmin @2, scales[12] @4, qs[128] @16
// Step S = sub-block S (32 values): lane group kg supplies values 32 S + 8 kg .. + 8 = the low (S even) or high
// (S odd) nibbles of qs[32 (S / 2) + 8 kg .. + 8].
template <> struct qw_kq<12> {
    static constexpr uint32_t BLK_K = 256, BLK_B = 144, NR = 12, STEPS = 8, KSTEP = 32;
    static constexpr bool HAS_MIN = true;
    typedef h8 W;
    uint32_t r[NR];
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t kg) {
        const u4 h = *(const u4 *)p;
        r[0] = h.x, r[1] = h.y, r[2] = h.z, r[3] = h.w;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const u2 q = *(const u2 *)(p + 16 + 32 * j + 8 * kg);
            r[4 + 2 * j] = q.x, r[5 + 2 * j] = q.y;
        }
    }
    template <int S> __device__ __forceinline__ void dec(const uint32_t *, uint32_t, W &w, float &a, float &c) const {
        constexpr int sh = 4 * (S & 1);
        w = qw_bytes_h8((r[4 + 2 * (S >> 1)] >> sh) & 0x0f0f0f0fu, (r[5 + 2 * (S >> 1)] >> sh) & 0x0f0f0f0fu, 0.0f);
        uint32_t sc, mn;
        qw_k4_scale_min<S>(r + 1, sc, mn);
        a = qw_h2f((uint16_t)r[0]) * (float)sc;
        c = qw_h2f((uint16_t)(r[0] >> 16)) * (float)mn;
    }
    template <int S> static __device__ __forceinline__ uint32_t pos(uint32_t kg, uint32_t i) { return 32 * S + 8 * kg + i; }
    template <int S, class AFK> static __device__ __forceinline__ h8 xfrag(const AFK &af, uint32_t kb, uint32_t kg) { return af.at8(kb + 32 * S + 8 * kg); }
};

// ---------------------------------------------------------------- Q5_K: 176 bytes, d, dmin, scales[12] @4, qh[32] @16, qs[128] @48
// As Q4_K; the fifth bit of value 32 S + l is bit S of qh[l].
template <> struct qw_kq<13> {
    static constexpr uint32_t BLK_K = 256, BLK_B = 176, NR = 14, STEPS = 8, KSTEP = 32;
    static constexpr bool HAS_MIN = true;
    typedef h8 W;
    uint32_t r[NR];
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t kg) {
        const u4 h = *(const u4 *)p;
        r[0] = h.x, r[1] = h.y, r[2] = h.z, r[3] = h.w;
        const u2 qh = *(const u2 *)(p + 16 + 8 * kg);
        r[4] = qh.x, r[5] = qh.y;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const u2 q = *(const u2 *)(p + 48 + 32 * j + 8 * kg);
            r[6 + 2 * j] = q.x, r[7 + 2 * j] = q.y;
        }
    }
    template <int S> __device__ __forceinline__ void dec(const uint32_t *, uint32_t, W &w, float &a, float &c) const {
        constexpr int sh = 4 * (S & 1);
        const uint32_t lo = ((r[6 + 2 * (S >> 1)] >> sh) & 0x0f0f0f0fu) | (((r[4] >> S) & 0x01010101u) << 4);
        const uint32_t hi = ((r[7 + 2 * (S >> 1)] >> sh) & 0x0f0f0f0fu) | (((r[5] >> S) & 0x01010101u) << 4);
        w = qw_bytes_h8(lo, hi, 0.0f);
        uint32_t sc, mn;
        qw_k4_scale_min<S>(r + 1, sc, mn);
        a = qw_h2f((uint16_t)r[0]) * (float)sc;
        c = qw_h2f((uint16_t)(r[0] >> 16)) * (float)mn;
    }
    template <int S> static __device__ __forceinline__ uint32_t pos(uint32_t kg, uint32_t i) { return 32 * S + 8 * kg + i; }
    template <int S, class AFK> static __device__ __forceinline__ h8 xfrag(const AFK &af, uint32_t kb, uint32_t kg) { return af.at8(kb + 32 * S + 8 * kg); }
};

// ---------------------------------------------------------------- Q6_K: 210 bytes, ql[128] @0, qh[64] @128, int8 scales[16] @192, d @208
// Step G = scale group G (16 values): half h = G >> 3, quarter c = (G >> 1) & 3, l0 = 16 (G & 1); lane group kg
// supplies l = l0 + 4 kg .. + 4: low nibbles (c < 2) or high nibbles of ql[64 h + 32 (c & 1) + l], bits 2 c, 2 c + 1
// of qh[32 h + l], minus 32. Blocks are only 2-byte aligned.
template <> struct qw_kq<14> {
    static constexpr uint32_t BLK_K = 256, BLK_B = 210, NR = 17, STEPS = 16, KSTEP = 16;
    static constexpr bool HAS_MIN = false;
    typedef h4 W;
    uint32_t r[NR]; // ql: r[(2 h + (c & 1)) * 2 + (G & 1)], qh: r[8 + 2 h + (G & 1)], scales r[12..15], d r[16]
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t kg) {
#pragma unroll
        for (int i = 0; i < 8; i++) r[i] = *(const u1a2 *)(p + 64 * (i >> 2) + 32 * ((i >> 1) & 1) + 16 * (i & 1) + 4 * kg);
#pragma unroll
        for (int i = 0; i < 4; i++) r[8 + i] = *(const u1a2 *)(p + 128 + 32 * (i >> 1) + 16 * (i & 1) + 4 * kg);
#pragma unroll
        for (int i = 0; i < 4; i++) r[12 + i] = *(const u1a2 *)(p + 192 + 4 * i);
        r[16] = *(const uint16_t *)(p + 208);
    }
    template <int G> __device__ __forceinline__ void dec(const uint32_t *, uint32_t, W &w, float &a, float &c) const {
        constexpr int h = G >> 3, q4 = (G >> 1) & 3, g1 = G & 1;
        const uint32_t q = ((r[(2 * h + (q4 & 1)) * 2 + g1] >> (4 * (q4 >> 1))) & 0x0f0f0f0fu) | (((r[8 + 2 * h + g1] >> (2 * q4)) & 0x03030303u) << 4);
        w = __builtin_bit_cast(h4, qw_bytes_h4(q, 32.0f));
        constexpr int si = 8 * h + 2 * q4 + g1;
        const int sc = (int)(int8_t)(r[12 + (si >> 2)] >> (8 * (si & 3)));
        a = qw_h2f((uint16_t)r[16]) * (float)sc;
        c = 0.0f;
    }
    template <int G> static __device__ __forceinline__ uint32_t pos(uint32_t kg, uint32_t i) { return 16 * G + 4 * kg + i; }
    template <int G, class AFK> static __device__ __forceinline__ h4 xfrag(const AFK &af, uint32_t kb, uint32_t kg) { return af.at4(kb + 16 * G + 4 * kg); }
};

// ---------------------------------------------------------------- the 4-bit codebook formats
// A block of 32 values is 16 bytes: byte j holds value j (low nibble) and value j + 16 (high nibble). Lane group kg
// takes bytes 4 kg .. 4 kg + 3: values 4 kg + i and 16 + 4 kg + i, one table read per byte giving both.
__device__ __forceinline__ h8 qw_iq4_bytes(const uint32_t *tab, uint32_t q) {
    const uint32_t t0 = tab[q & 255], t1 = tab[(q >> 8) & 255], t2 = tab[(q >> 16) & 255], t3 = tab[q >> 24];
    u4 raw; // low-nibble values of the four bytes, then the high-nibble values
    raw[0] = __builtin_amdgcn_perm(t1, t0, 0x05040100u);
    raw[1] = __builtin_amdgcn_perm(t3, t2, 0x05040100u);
    raw[2] = __builtin_amdgcn_perm(t1, t0, 0x07060302u);
    raw[3] = __builtin_amdgcn_perm(t3, t2, 0x07060302u);
    return __builtin_bit_cast(h8, raw);
}
template <class AFK> __device__ __forceinline__ h8 qw_iq4_xfrag(const AFK &af, uint32_t k32, uint32_t kg) { // x[4 kg .. + 4], x[16 + 4 kg .. + 4] of a 32-block
    const h4 a = af.at4(k32 + 4 * kg), b = af.at4(k32 + 16 + 4 * kg);
    return h8{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
}
__device__ __forceinline__ uint32_t qw_iq4_pos(uint32_t kg, uint32_t i) { return (i < 4 ? 0 : 12) + 4 * kg + i; }

// IQ4_XS: 136 bytes, d @0, scales_h (u16) @2, scales_l[4] @4, qs[128] @8; step S = sub-block S, scale
// (nibble S of scales_l | bits 2 S, 2 S + 1 of scales_h << 4) - 32.
template <> struct qw_kq<23> {
    static constexpr uint32_t BLK_K = 256, BLK_B = 136, NR = 10, STEPS = 8, KSTEP = 32;
    static constexpr bool HAS_MIN = false;
    typedef h8 W;
    uint32_t r[NR];
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t kg) {
        const u2 h = *(const u2 *)p;
        r[0] = h.x, r[1] = h.y;
#pragma unroll
        for (int s = 0; s < 8; s++) r[2 + s] = *(const uint32_t *)(p + 8 + 16 * s + 4 * kg);
    }
    template <int S> __device__ __forceinline__ void dec(const uint32_t *tab, uint32_t, W &w, float &a, float &c) const {
        w = qw_iq4_bytes(tab, r[2 + S]);
        const int ls = (int)(((r[1] >> (4 * S)) & 15) | (((r[0] >> (16 + 2 * S)) & 3) << 4));
        a = qw_h2f((uint16_t)r[0]) * (float)(ls - 32);
        c = 0.0f;
    }
    template <int S> static __device__ __forceinline__ uint32_t pos(uint32_t kg, uint32_t i) { return 32 * S + qw_iq4_pos(kg, i); }
    template <int S, class AFK> static __device__ __forceinline__ h8 xfrag(const AFK &af, uint32_t kb, uint32_t kg) { return qw_iq4_xfrag(af, kb + 32 * S, kg); }
};

// IQ4_NL: 18 bytes, d @0, qs[16] @2 (2-byte aligned); one step.
template <> struct qw_kq<20> {
    static constexpr uint32_t BLK_K = 32, BLK_B = 18, NR = 2, STEPS = 1, KSTEP = 32;
    static constexpr bool HAS_MIN = false;
    typedef h8 W;
    uint32_t r[NR];
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t kg) {
        r[0] = *(const uint16_t *)p;
        r[1] = *(const u1a2 *)(p + 2 + 4 * kg);
    }
    template <int S> __device__ __forceinline__ void dec(const uint32_t *tab, uint32_t, W &w, float &a, float &c) const {
        w = qw_iq4_bytes(tab, r[1]);
        a = qw_h2f((uint16_t)r[0]);
        c = 0.0f;
    }
    template <int S> static __device__ __forceinline__ uint32_t pos(uint32_t kg, uint32_t i) { return qw_iq4_pos(kg, i); }
    template <int S, class AFK> static __device__ __forceinline__ h8 xfrag(const AFK &af, uint32_t kb, uint32_t kg) { return qw_iq4_xfrag(af, kb, kg); }
};

// ---------------------------------------------------------------- plain rows: 32 values a step, 8 consecutive values a lane group
template <> struct qw_kq<1> { // binary16
    static constexpr uint32_t BLK_K = 32, BLK_B = 64, NR = 4, STEPS = 1, KSTEP = 32;
    static constexpr bool HAS_MIN = false;
    typedef h8 W;
    uint32_t r[NR];
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t kg) {
        const u4 v = *(const u4 *)(p + 16 * kg);
        r[0] = v.x, r[1] = v.y, r[2] = v.z, r[3] = v.w;
    }
    template <int S> __device__ __forceinline__ void dec(const uint32_t *, uint32_t, W &w, float &a, float &c) const {
        w = __builtin_bit_cast(h8, u4{r[0], r[1], r[2], r[3]});
        a = 1.0f;
        c = 0.0f;
    }
    template <int S> static __device__ __forceinline__ uint32_t pos(uint32_t kg, uint32_t i) { return 8 * kg + i; }
    template <int S, class AFK> static __device__ __forceinline__ h8 xfrag(const AFK &af, uint32_t kb, uint32_t kg) { return af.at8(kb + 8 * kg); }
};

// bfloat16 weights go to the bfloat16 matrix instruction unchanged; the binary16 activations are split there into two
// bfloat16 values (upper 8 significant bits, then the remaining 3, both exact), one instruction each.
template <> struct qw_kq<30> {
    static constexpr uint32_t BLK_K = 32, BLK_B = 64, NR = 4, STEPS = 1, KSTEP = 32;
    static constexpr bool HAS_MIN = false;
    typedef bf8 W;
    uint32_t r[NR];
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t kg) {
        const u4 v = *(const u4 *)(p + 16 * kg);
        r[0] = v.x, r[1] = v.y, r[2] = v.z, r[3] = v.w;
    }
    template <int S> __device__ __forceinline__ void dec(const uint32_t *, uint32_t, W &w, float &a, float &c) const {
        w = __builtin_bit_cast(bf8, u4{r[0], r[1], r[2], r[3]});
        a = 1.0f;
        c = 0.0f;
    }
    template <int S> static __device__ __forceinline__ uint32_t pos(uint32_t kg, uint32_t i) { return 8 * kg + i; }
    template <int S, class AFK> static __device__ __forceinline__ h8 xfrag(const AFK &af, uint32_t kb, uint32_t kg) { return af.at8(kb + 8 * kg); }
};
__device__ __forceinline__ float qw_w2f(_Float16 v) { return (float)v; }
__device__ __forceinline__ float qw_w2f(__bf16 v) { return (float)v; }

// x (8 binary16 values) = hi + lo in bfloat16
__device__ __forceinline__ void qw_split_bf(h8 x, bf8 &hi, bf8 &lo) {
    u4 rh, rl;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float f0 = (float)x[2 * i], f1 = (float)x[2 * i + 1];
        const uint32_t b0 = __builtin_bit_cast(uint32_t, f0) & 0xffff0000u, b1 = __builtin_bit_cast(uint32_t, f1) & 0xffff0000u;
        const float l0 = f0 - __builtin_bit_cast(float, b0), l1 = f1 - __builtin_bit_cast(float, b1);
        rh[i] = (b0 >> 16) | b1;
        rl[i] = (__builtin_bit_cast(uint32_t, l0) >> 16) | (__builtin_bit_cast(uint32_t, l1) & 0xffff0000u);
    }
    hi = __builtin_bit_cast(bf8, rh);
    lo = __builtin_bit_cast(bf8, rl);
}

// One step of a block into the accumulator (tokens 4 kg .. 4 kg + 3 of row lane & 15).
template <int F, int S> __device__ __forceinline__ void qw_kq_step(const qw_kq<F> &b, const uint32_t *tab, const qw_afrag_kq &af, uint32_t kb, uint32_t kg, f4 &acc) {
    typename qw_kq<F>::W w;
    float a, c;
    b.template dec<S>(tab, kg, w, a, c);
    const auto x = qw_kq<F>::template xfrag<S>(af, kb, kg);
    f4 sub = {0, 0, 0, 0};
    if constexpr (F == 30) {
        bf8 xh, xl;
        qw_split_bf(x, xh, xl);
        sub = qw_mfma_bf(xh, w, sub);
        sub = qw_mfma_bf(xl, w, sub);
    } else if constexpr (qw_kq<F>::KSTEP == 16) sub = qw_mfma16(x, w, sub);
    else sub = qw_mfma(x, w, sub);
    if constexpr (F == 1 || F == 30) acc += sub;
    else acc += a * sub;
    if constexpr (qw_kq<F>::HAS_MIN) acc -= c * af.sum32(kb + 32 * S);
}
template <int F, int S = 0> __device__ __forceinline__ void qw_kq_block(const qw_kq<F> &b, const uint32_t *tab, const qw_afrag_kq &af, uint32_t kb, uint32_t kg, f4 &acc) {
    if constexpr (S < (int)qw_kq<F>::STEPS) {
        qw_kq_step<F, S>(b, tab, af, kb, kg, acc);
        qw_kq_block<F, S + 1>(b, tab, af, kb, kg, acc);
    }
}

// The values of a block as the reference computes them (scale * integer - min, in float), scattered to y[position].
template <int F, int S = 0> __device__ __forceinline__ void qw_kq_values(const qw_kq<F> &b, const uint32_t *tab, uint32_t kg, float *y) {
    if constexpr (S < (int)qw_kq<F>::STEPS) {
        typename qw_kq<F>::W w;
        float a, c;
        b.template dec<S>(tab, kg, w, a, c);
        constexpr int NV = qw_kq<F>::KSTEP / 4;
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const float v = qw_w2f(w[i]);
            y[qw_kq<F>::template pos<S>(kg, i)] = (F == 1 || F == 30) ? v : a * v - c;
        }
        qw_kq_values<F, S + 1>(b, tab, kg, y);
    }
}

// IQ4_NL rows for the MoE kernels (the interface of qw_chunk<8, NB>): NB blocks of 18 bytes, loaded in quad order
// (lane & 3 takes bytes 4 kl .. 4 kl + 3 of qs), pulled to matrix-core lane order. "lut" is the 256-entry byte table
// of qw_kq_tab_build. Operand A of a block: x[4 kg .. + 4] and x[16 + 4 kg .. + 4], the values the lane's four bytes hold.
template <int NB> struct qw_chunk<20, NB> {
    static constexpr uint32_t BLK_K = 32, BLK_B = 18;
    static constexpr int DEPTH = 3; // blocks are small: two chunks ahead keep enough bytes in flight
    uint32_t q[NB];
    uint16_t d[NB];
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t kl) {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            q[b] = *(const u1a2 *)(p + 18 * b + 2 + 4 * kl);
            d[b] = *(const uint16_t *)(p + 18 * b);
        }
    }
    __device__ __forceinline__ void transpose() {
        const uint32_t src4 = qw_pull_addr();
#pragma unroll
        for (int b = 0; b < NB; b++) {
            q[b] = qw_pull(q[b], src4);
            d[b] = (uint16_t)qw_pull(d[b], src4);
        }
    }
    static __device__ __forceinline__ h8 join(h4 a, h4 b) { return h8{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]}; }
    template <class AF> __device__ __forceinline__ void mac(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const h8 w = qw_iq4_bytes((const uint32_t *)lut, q[b]);
            const uint32_t kb = k0 + 32 * b + 4 * kg;
            f4 sub = {0, 0, 0, 0};
            sub = qw_mfma(join(af.hi4(kb), af.hi4(kb + 16)), w, sub);
            if (AF::has_lo) sub = qw_mfma(join(af.lo4(kb), af.lo4(kb + 16)), w, sub);
            acc += qw_h2f(d[b]) * sub;
        }
    }
    template <class AF> __device__ __forceinline__ void mac_lean(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const { mac(lut, af, k0, kg, acc); }
    template <class AF> __device__ __forceinline__ void mac_half(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const { mac(lut, af, k0, kg, acc); }
    // NG groups of 16 activation rows (binary16, one plane, global memory) against the same decoded weights
    template <int NG> __device__ __forceinline__ void mac_groups(const u2 *lut, const uint16_t *const (&rows)[NG], uint32_t k0, uint32_t kg, f4 (&acc)[NG]) const {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const h8 w = qw_iq4_bytes((const uint32_t *)lut, q[b]);
            const uint32_t kb = k0 + 32 * b + 4 * kg;
#pragma unroll
            for (int g = 0; g < NG; g++) {
                f4 sub = {0, 0, 0, 0};
                sub = qw_mfma(join(*(const h4 *)(rows[g] + kb), *(const h4 *)(rows[g] + kb + 16)), w, sub);
                acc[g] += qw_h2f(d[b]) * sub;
            }
        }
    }
    template <class AF> __device__ __forceinline__ void mac_gather(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const uint32_t kb = k0 + 32 * b + 4 * kg;
            h8 xh = {}, xl = {};
            if (af.on) {
                xh = join(*(const h4 *)(af.rowhi + kb), *(const h4 *)(af.rowhi + kb + 16));
                xl = join(*(const h4 *)(af.rowlo + kb), *(const h4 *)(af.rowlo + kb + 16));
            }
            const h8 w = qw_iq4_bytes((const uint32_t *)lut, q[b]);
            f4 sub = {0, 0, 0, 0};
            sub = qw_mfma(xh, w, sub);
            sub = qw_mfma(xl, w, sub);
            acc += qw_h2f(d[b]) * sub;
        }
    }
};

// The same rows from their tile-major copy (layout: QW_F_PACKED_NL in qw_kargs.h): one chunk = ten blocks of the 16
// rows of a tile, already in matrix-core lane order. BLK_B is the bytes of a block of all 16 rows, so that
// NB * BLK_B is the chunk's size as for the other chunk types.
typedef u4 __attribute__((aligned(4))) u4a4;
template <> struct qw_chunk<QW_F_PACKED_NL, 10> {
    static constexpr uint32_t BLK_K = 32, BLK_B = 288;
    static constexpr int DEPTH = 2; // (one chunk ahead: the reference model's down launch 46.0 -> 44.8 us at 16 tokens)
    uint32_t q[10], dd[5];
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t lane) {
        const u4 a = *(const u4 *)(p + 16 * lane), b = *(const u4 *)(p + 1024 + 16 * lane);
        const u2 c = *(const u2 *)(p + 2048 + 8 * lane);
        const uint8_t *ds = p + 2560 + 20 * (lane & 15);
        const u4 d0 = *(const u4a4 *)ds;
        q[0] = a.x, q[1] = a.y, q[2] = a.z, q[3] = a.w, q[4] = b.x, q[5] = b.y, q[6] = b.z, q[7] = b.w, q[8] = c.x, q[9] = c.y;
        dd[0] = d0.x, dd[1] = d0.y, dd[2] = d0.z, dd[3] = d0.w, dd[4] = *(const uint32_t *)(ds + 16);
    }
    __device__ __forceinline__ void transpose() {}
    __device__ __forceinline__ float scale(int b) const { return qw_h2f((uint16_t)(dd[b >> 1] >> (16 * (b & 1)))); }
    template <class AF> __device__ __forceinline__ void mac(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const {
#pragma unroll
        for (int b = 0; b < 10; b++) {
            const h8 w = qw_iq4_bytes((const uint32_t *)lut, q[b]);
            const uint32_t kb = k0 + 32 * b + 4 * kg;
            f4 sub = {0, 0, 0, 0};
            sub = qw_mfma(qw_chunk<20, 1>::join(af.hi4(kb), af.hi4(kb + 16)), w, sub);
            if (AF::has_lo) sub = qw_mfma(qw_chunk<20, 1>::join(af.lo4(kb), af.lo4(kb + 16)), w, sub);
            acc += scale(b) * sub;
        }
    }
    template <class AF> __device__ __forceinline__ void mac_half(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const { mac(lut, af, k0, kg, acc); }
    // operand A gathered from the two H planes in global memory by the lanes whose token is in use
    template <class AF> __device__ __forceinline__ void mac_gather(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const {
#pragma unroll
        for (int b = 0; b < 10; b++) {
            const uint32_t kb = k0 + 32 * b + 4 * kg;
            h8 xh = {}, xl = {};
            if (af.on) {
                xh = qw_chunk<20, 1>::join(*(const h4 *)(af.rowhi + kb), *(const h4 *)(af.rowhi + kb + 16));
                xl = qw_chunk<20, 1>::join(*(const h4 *)(af.rowlo + kb), *(const h4 *)(af.rowlo + kb + 16));
            }
            const h8 w = qw_iq4_bytes((const uint32_t *)lut, q[b]);
            f4 sub = {0, 0, 0, 0};
            sub = qw_mfma(xh, w, sub);
            sub = qw_mfma(xl, w, sub);
            acc += scale(b) * sub;
        }
    }
};

// NB blocks of one row for the task pipeline: loaded in quad order, pulled to matrix-core lane order.
template <int F, int NB> struct qw_chunk_kq {
    static constexpr uint32_t BLK_K = qw_kq<F>::BLK_K, BLK_B = qw_kq<F>::BLK_B;
    static constexpr int DEPTH = qw_kq<F>::NR * NB <= 20 ? 3 : 2; // chunks in flight ahead of the arithmetic
    qw_kq<F> b[NB];
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t kl) {
#pragma unroll
        for (int i = 0; i < NB; i++) b[i].load(p + BLK_B * i, kl);
    }
    __device__ __forceinline__ void transpose() {
        const uint32_t src4 = qw_pull_addr();
#pragma unroll
        for (int i = 0; i < NB; i++)
#pragma unroll
            for (uint32_t j = 0; j < qw_kq<F>::NR; j++) b[i].r[j] = qw_pull(b[i].r[j], src4);
    }
    __device__ __forceinline__ void mac(const uint32_t *tab, const qw_afrag_kq &af, uint32_t k0, uint32_t kg, f4 &acc) const {
#pragma unroll
        for (int i = 0; i < NB; i++) qw_kq_block<F>(b[i], tab, af, k0 + BLK_K * i, kg, acc);
    }
};

// The tile-major copy of Q6_K rows (QW_F_PACKED_Q6 in qw_kargs.h): the decoder's seventeen dwords arrive in matrix-core
// lane order by five coalesced loads a block (three of 16 bytes a lane, the row's scales, its d), and nothing moves
// between lanes. p is the wave-uniform address of the chunk's first slab, the second argument the lane. The arithmetic
// is qw_kq<14>'s, so the results are those of the GGUF rows bit for bit.
template <int NB> struct qw_chunk_kq<QW_F_PACKED_Q6, NB> {
    static constexpr uint32_t BLK_K = 256, BLK_B = QW_Q6_SLAB_BYTES;
    static constexpr int DEPTH = 3; // (two chunks ahead: a 131072-row matrix at one token 44.4 us, with one ahead 46.3)
    qw_kq<14> b[NB];
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t lane) {
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const uint8_t *sl = p + QW_Q6_SLAB_BYTES * i;
#pragma unroll
            for (int pl = 0; pl < 3; pl++) {
                const u4 v = *(const u4 *)(sl + 1024 * pl + 16 * lane);
                b[i].r[4 * pl] = v[0], b[i].r[4 * pl + 1] = v[1], b[i].r[4 * pl + 2] = v[2], b[i].r[4 * pl + 3] = v[3];
            }
            const u4 sc = *(const u4 *)(sl + 3072 + 16 * (lane & 15));
            b[i].r[12] = sc[0], b[i].r[13] = sc[1], b[i].r[14] = sc[2], b[i].r[15] = sc[3];
            b[i].r[16] = *(const uint16_t *)(sl + 3328 + 2 * (lane & 15));
        }
    }
    __device__ __forceinline__ void transpose() {}
    __device__ __forceinline__ void mac(const uint32_t *tab, const qw_afrag_kq &af, uint32_t k0, uint32_t kg, f4 &acc) const {
#pragma unroll
        for (int i = 0; i < NB; i++) qw_kq_block<14>(b[i], tab, af, k0 + BLK_K * i, kg, acc);
    }
};

// ---------------------------------------------------------------- the same decoders in the MoE kernels' chunk interface
// qw_chunk<F, NB> for Q4_K, Q5_K, Q6_K and IQ4_XS rows (kernels/moe_gg.metal:336-395 of the reference takes them for
// the routed experts too): GGUF-order rows loaded in quad order, operand A from any of the fragment providers (one plane
// or hi + lo). "lut" is the 256-entry byte table of qw_kq_tab_build (read by IQ4_XS only). The minimum term of Q4_K and
// Q5_K needs the sum of the step's 32 activations per token: one more matrix instruction against a fragment of ones
// delivers it in the accumulator's own layout, whatever the provider. Built for coverage of the formats, not tuned.
template <class AF, bool LO> struct qw_kq_plane { // one plane of a provider, in the at8 / at4 interface of xfrag
    const AF &af;
    __device__ __forceinline__ h8 at8(uint32_t k) const {
        if constexpr (LO) return af.lo(k);
        else return af.hi(k);
    }
    __device__ __forceinline__ h4 at4(uint32_t k) const {
        if constexpr (LO) return af.lo4(k);
        else return af.hi4(k);
    }
};
template <int F, int S, class AF> __device__ __forceinline__ void qw_kq_step_af(const qw_kq<F> &b, const uint32_t *tab, const AF &af, uint32_t kb, uint32_t kg, f4 &acc) {
    typename qw_kq<F>::W w;
    float a, c;
    b.template dec<S>(tab, kg, w, a, c);
    const qw_kq_plane<AF, false> ph = {af};
    const qw_kq_plane<AF, true> pl = {af};
    const auto xh = qw_kq<F>::template xfrag<S>(ph, kb, kg);
    f4 sub = {0, 0, 0, 0};
    if constexpr (qw_kq<F>::KSTEP == 16) {
        sub = qw_mfma16(xh, w, sub);
        if (AF::has_lo) sub = qw_mfma16(qw_kq<F>::template xfrag<S>(pl, kb, kg), w, sub);
    } else {
        sub = qw_mfma(xh, w, sub);
        if (AF::has_lo) sub = qw_mfma(qw_kq<F>::template xfrag<S>(pl, kb, kg), w, sub);
        if constexpr (qw_kq<F>::HAS_MIN) {
            const _Float16 o = (_Float16)1.0f;
            const h8 ones = {o, o, o, o, o, o, o, o};
            f4 xs = {0, 0, 0, 0};
            xs = qw_mfma(xh, ones, xs);
            if (AF::has_lo) xs = qw_mfma(qw_kq<F>::template xfrag<S>(pl, kb, kg), ones, xs);
            acc -= c * xs;
        }
    }
    acc += a * sub;
}
template <int F, class AF, int S = 0> __device__ __forceinline__ void qw_kq_block_af(const qw_kq<F> &b, const uint32_t *tab, const AF &af, uint32_t kb, uint32_t kg, f4 &acc) {
    if constexpr (S < (int)qw_kq<F>::STEPS) {
        qw_kq_step_af<F, S>(b, tab, af, kb, kg, acc);
        qw_kq_block_af<F, AF, S + 1>(b, tab, af, kb, kg, acc);
    }
}
template <int F, int NB> struct qw_chunk_kqa : qw_chunk_kq<F, NB> {
    template <class AF> __device__ __forceinline__ void mac(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const {
#pragma unroll
        for (int i = 0; i < NB; i++) qw_kq_block_af<F>(this->b[i], (const uint32_t *)lut, af, k0 + qw_kq<F>::BLK_K * i, kg, acc);
    }
    template <class AF> __device__ __forceinline__ void mac_lean(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const { mac(lut, af, k0, kg, acc); }
    template <class AF> __device__ __forceinline__ void mac_half(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const { mac(lut, af, k0, kg, acc); }
    // operand A from the two H planes in global memory, read by the lanes whose token is in use
    template <class AF> __device__ __forceinline__ void mac_gather(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const {
        const qw_afrag_glb<true> g = {af.on ? af.rowhi : nullptr, af.on ? af.rowlo : nullptr};
        mac(lut, g, k0, kg, acc);
    }
};
template <int NB> struct qw_chunk<12, NB> : qw_chunk_kqa<12, NB> {};
template <int NB> struct qw_chunk<13, NB> : qw_chunk_kqa<13, NB> {};
template <int NB> struct qw_chunk<14, NB> : qw_chunk_kqa<14, NB> {};
template <int NB> struct qw_chunk<23, NB> : qw_chunk_kqa<23, NB> {};
