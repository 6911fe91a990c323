// Device-side building blocks for the quantized decode kernels (gfx950, wave64).
//
// Matrix-core formulation used by every weight-streaming kernel here: one wave owns a tile of 16 weight rows
// and up to 16 token columns and issues v_mfma_f32_16x16x32_f16 with the ACTIVATIONS as operand A (M = token)
// and the decoded WEIGHTS as operand B (N = weight row):
//     lane l:  n = l & 15 (weight row in the tile),  kg = l >> 4 (which 8 of the 32 k-values of a step)
//     A: lane supplies x[token = n][8 k-values of group kg]      B: lane supplies w[row n][8 k-values of group kg]
//     D: lane receives out[token 4*kg + i][row n], i = 0..3
// so a lane's four results belong to the row whose bytes that lane decodes, and the per-block scale of that row
// is already in the lane's registers.
// Global loads use another lane order: lane l loads the bytes of (row l >> 2, k-group l & 3), so that the four lanes
// of a quad read adjacent addresses and the cache sees one access per quad instead of one per lane. The registers
// are then moved to the matrix-core order above with ds_bpermute (a transpose of the 16 x 4 lane grid). The decoded weights are small integers (exact in binary16); products and
// sums are accumulated in binary32 by the matrix core; the binary16 block scale d multiplies the binary32
// partial sum afterwards. A token's result never depends on the other token columns.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "qw_kargs.h"
#define QW_CODES_QUAL __constant__ const
#include "iq3s_codes.h"

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));
// GGUF blocks are only 2-byte aligned (110- and 34-byte blocks); the hardware takes unaligned wide loads.
typedef u4 __attribute__((aligned(2))) u4a2;
typedef u2 __attribute__((aligned(2))) u2a2;

#define QW_LUT_ENTRIES 8192
#define QW_LUT_BYTES (QW_LUT_ENTRIES * 8)

__device__ __forceinline__ float qw_h2f(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
__device__ __forceinline__ uint16_t qw_f2h(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }
__device__ __forceinline__ float qw_bf2f(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }

// One pre-signed table entry: index = codebook entry (9 bits) | sign nibble << 9; four binary16 values, value j =
// magnitude j of the codebook entry with the sign taken from bit j of the nibble (the reference builds the same
// table in kernels/moe_gg.metal:495-500).
__device__ __forceinline__ u2 qw_lut_entry(uint32_t i) {
    const uint32_t code = qw_iq3s_codes[i & 511];
    uint32_t h[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int mag = 2 * (int)((code >> (3 * j)) & 7) + 1;
        h[j] = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)mag) | (((i >> (9 + j)) & 1) << 15);
    }
    u2 r;
    r.x = h[0] | h[1] << 16;
    r.y = h[2] | h[3] << 16;
    return r;
}

// Where entry i of the reference's index order (codebook entry | sign nibble << 9) lives in this library's copy of
// the table: slot = qs byte << 5 | ninth index bit << 4 | sign nibble. A slot's byte address is then made of two
// whole bytes (high byte = the qs byte as loaded, low byte = (nibble | bit << 4) << 3), which one byte-permute
// instruction assembles.
__device__ __forceinline__ uint32_t qw_lut_slot(uint32_t i) { return ((i & 255) << 5) | (((i >> 8) & 1) << 4) | (i >> 9); }

// Fill the 64 KB table in LDS; every thread of the workgroup takes part. Caller synchronises afterwards.
__device__ __forceinline__ void qw_lut_build(u2 *lut) {
    for (uint32_t i = threadIdx.x; i < QW_LUT_ENTRIES; i += blockDim.x) lut[qw_lut_slot(i)] = qw_lut_entry(i);
}

__device__ __forceinline__ f4 qw_mfma(h8 a, h8 b, f4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }

// ---------------------------------------------------------------- IQ3_S (110-byte block of 256 values)
// Bytes: d @0 (binary16), qs[64] @2, qh[8] @66, signs[32] @74, scales[4] @106 (kernels/moe_iq.metal:102-118).
// Lane group kg decodes the 64 values [64 kg, 64 kg + 64) of a block — sub-blocks 2 kg and 2 kg + 1 — whose
// bytes are contiguous: qs[16 kg .. +16), signs[8 kg .. +8), qh[2 kg .. +2), scales[kg]. In step j (0..7) the lane
// supplies values 64 kg + 8 j .. + 8. The sub-block factor 1 + 2 s is multiplied into the binary16 integers
// (|value| <= 15 * 31, exact); the block scale d multiplies the binary32 sum of the eight steps.
struct qw_iq3_slice {
    u4 qs;
    u2 sg;
    uint32_t qh, sc;
    float d;
};

__device__ __forceinline__ qw_iq3_slice qw_iq3_load(const uint8_t *blk, uint32_t kg) {
    qw_iq3_slice s;
    s.qs = *(const u4a2 *)(blk + 2 + 16 * kg);
    s.sg = *(const u2a2 *)(blk + 74 + 8 * kg);
    s.qh = *(const uint16_t *)(blk + 66 + 2 * kg);
    s.sc = blk[106 + kg];
    s.d = qw_h2f(*(const uint16_t *)blk);
    return s;
}

// Pull a register from the lane that loaded this lane's (row, k-group): source lane = 4 * n + kg.
__device__ __forceinline__ uint32_t qw_pull(uint32_t v, uint32_t src4) { return (uint32_t)__builtin_amdgcn_ds_bpermute((int)src4, (int)v); }
__device__ __forceinline__ uint32_t qw_pull_addr() {
    const uint32_t l = threadIdx.x & 63;
    return 4 * (4 * (l & 15) + (l >> 4));
}
__device__ __forceinline__ void qw_iq3_transpose(qw_iq3_slice &s, uint32_t src4) {
#pragma unroll
    for (int i = 0; i < 4; i++) s.qs[i] = qw_pull(s.qs[i], src4);
    s.sg.x = qw_pull(s.sg.x, src4);
    s.sg.y = qw_pull(s.sg.y, src4);
    const uint32_t m = qw_pull(s.qh | (s.sc << 16), src4);
    s.qh = m & 0xffff;
    s.sc = m >> 16;
    s.d = __builtin_bit_cast(float, qw_pull(__builtin_bit_cast(uint32_t, s.d), src4));
}

// Low address bytes of the sixteen table reads of a slice: p[2 t] holds, byte j, (nibble | ninth bit << 4) << 3 of
// read 2 j of sub-block t, p[2 t + 1] the same for read 2 j + 1. The eight qh bits of a sub-block are spread to bit 4
// of eight bytes by two 24-bit multiplications (no two partial products that can both be set meet at a kept bit).
struct qw_iq3_keys {
    uint32_t p[4];
};
__device__ __forceinline__ qw_iq3_keys qw_iq3_prep(const qw_iq3_slice &s) {
    qw_iq3_keys k;
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const uint32_t S = s.sg[t], H = s.qh >> (8 * t);
        const uint32_t he = __umul24(H & 0x55u, 0x410410u); // bit 8 j + 4 = qh bit 2 j
        const uint32_t ho = __umul24(H & 0xaau, 0x208208u); // bit 8 j + 4 = qh bit 2 j + 1
        k.p[2 * t] = ((he & 0x10101010u) | (S & 0x0f0f0f0fu)) << 3;
        k.p[2 * t + 1] = ((ho & 0x10101010u) | ((S >> 4) & 0x0f0f0f0fu)) << 3;
    }
    return k;
}
// Byte addresses (relative to the table) of the two reads of step J: high byte = qs byte, low byte from the keys.
template <int J> __device__ __forceinline__ void qw_iq3_addr(const qw_iq3_slice &s, const qw_iq3_keys &k, uint32_t &a0, uint32_t &a1) {
    constexpr uint32_t t = J / 4, j = J % 4, qb = 2 * (J % 2);
    a0 = __builtin_amdgcn_perm(s.qs[J / 2], k.p[2 * t], 0x0c0c0000u | ((4 + qb) << 8) | j);
    a1 = __builtin_amdgcn_perm(s.qs[J / 2], k.p[2 * t + 1], 0x0c0c0000u | ((5 + qb) << 8) | j);
}
__device__ __forceinline__ u2 qw_lut_at(const u2 *lut, uint32_t byteaddr) { return *(const u2 *)((const uint8_t *)lut + byteaddr); }
// The binary16 sub-block factor 1 + 2 s of sub-block t of a slice, in both halves.
__device__ __forceinline__ h2 qw_iq3_factor(const qw_iq3_slice &s, int t) {
    const _Float16 f = (_Float16)(uint16_t)(1 + 2 * ((s.sc >> (4 * t)) & 15));
    return h2{f, f};
}

// The eight binary16 values of step J, already multiplied by the sub-block factor.
template <int J> __device__ __forceinline__ h8 qw_iq3_step(const qw_iq3_slice &s, const u2 *lut) {
    const qw_iq3_keys k = qw_iq3_prep(s);
    uint32_t a0, a1;
    qw_iq3_addr<J>(s, k, a0, a1);
    const u2 w0 = qw_lut_at(lut, a0), w1 = qw_lut_at(lut, a1);
    const h2 ff = qw_iq3_factor(s, J / 4);
    u4 raw = {w0.x, w0.y, w1.x, w1.y};
#pragma unroll
    for (int i = 0; i < 4; i++) raw[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, (uint32_t)raw[i]) * ff);
    return __builtin_bit_cast(h8, raw);
}

// ---------------------------------------------------------------- Q8_0 (34-byte block of 32 values)
// Bytes: d @0, qs[32] int8 @2 (src/ggml_dq.c:34-37). Lane group kg decodes values [8 kg, 8 kg + 8) of a block.
// int8 -> binary16 without conversions: (q ^ 0x80) placed under the exponent byte 0x64 is 1024 + q + 128 exactly.
__device__ __forceinline__ h8 qw_q8_cvt(u2 q) {
    const uint32_t a = q.x ^ 0x80808080u, b = q.y ^ 0x80808080u;
    const h2 bias = {(_Float16)1152.0f, (_Float16)1152.0f};
    u4 raw;
    raw[0] = __builtin_amdgcn_perm(0x64646464u, a, 0x04010400u); // bytes: a0, 0x64, a1, 0x64
    raw[1] = __builtin_amdgcn_perm(0x64646464u, a, 0x04030402u);
    raw[2] = __builtin_amdgcn_perm(0x64646464u, b, 0x04010400u);
    raw[3] = __builtin_amdgcn_perm(0x64646464u, b, 0x04030402u);
#pragma unroll
    for (int i = 0; i < 4; i++) raw[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, (uint32_t)raw[i]) - bias);
    return __builtin_bit_cast(h8, raw);
}

// ---------------------------------------------------------------- result stores of the streaming kernels
// Loads and stores share one counter of outstanding operations on this hardware, and stores may complete out of order
// with respect to loads; once the compiler has seen a store it therefore no longer waits for "all but the youngest N
// loads" but for everything in flight, which empties the prefetch queue. The few result stores at the end of a tile are
// issued as assembly that this bookkeeping does not see. That is safe in the direction that matters: an outstanding
// store only makes the hardware counter larger than the number of outstanding loads, so "at most N outstanding" still
// implies that all but the N youngest loads have returned. A store reads its data registers when it is issued, and it
// has completed when the kernel ends, which is when its readers start. INVARIANT for every user: what is stored this way
// is never read back from memory inside the same kernel (the compiler would not wait for the store before such a read).
// (the default cache policy: the same stores marked nontemporal or of device scope made the step 1.2 % and 0.4 % slower)
__device__ __forceinline__ void qw_store_u16(uint16_t *p, uint16_t v) { asm volatile("global_store_short %0, %1, off" : : "v"(p), "v"((uint32_t)v) : "memory"); }
__device__ __forceinline__ void qw_store_f32(float *p, float v) { asm volatile("global_store_dword %0, %1, off" : : "v"(p), "v"(v) : "memory"); }

// ---------------------------------------------------------------- data handed between workgroups of one launch
// The eight XCDs of the device have an L2 each, coherent with one another only at the boundaries of a kernel. What one
// workgroup writes and another reads inside one launch therefore goes around those caches: stores and loads of device
// ("agent") scope (cache policy sc1), which the hardware carries out at the memory side. No fences: a release fence
// writes back a whole L2 and an acquire fence drops one (tens of microseconds per hand-over). A store of device scope
// that its wave has waited for (s_waitcnt) is visible to every load of device scope issued after it.
__device__ __forceinline__ void qw_st_coh(uint32_t *p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint32_t qw_ld_coh(const uint32_t *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// Seven 16-byte loads of device scope, issued together and awaited (every outstanding memory operation of the wave is):
// one statement, so that the compiler never touches a destination register before the wait.
__device__ __forceinline__ void qw_ld_coh7(u4 (&v)[7], const u4 *const (&p)[7]) {
    asm volatile("global_load_dwordx4 %0, %7, off sc1\n\t"
                 "global_load_dwordx4 %1, %8, off sc1\n\t"
                 "global_load_dwordx4 %2, %9, off sc1\n\t"
                 "global_load_dwordx4 %3, %10, off sc1\n\t"
                 "global_load_dwordx4 %4, %11, off sc1\n\t"
                 "global_load_dwordx4 %5, %12, off sc1\n\t"
                 "global_load_dwordx4 %6, %13, off sc1\n\t"
                 "s_waitcnt vmcnt(0)"
                 : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6])
                 : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6])
                 : "memory");
}

// Synchronisation words of a launch whose workgroups wait for one another (QW_SYNC_BYTES of device memory owned by
// the backend, zero between launches except the generation). Such a launch has at most one workgroup per compute unit,
// so all of them are resident at once and a wait ends as soon as the others arrive; every wait is bounded all the same
// (limit = number of polls): a workgroup that gives up sets the error word, everybody winds down without waiting
// again, and the host fails the batch.
//   word 0: generation, raised by one by the workgroup that completes a barrier     word 32: arrivals at the top level
//   word 64 + 32 g: arrivals of group g (workgroup index & 7: one XCD)              word 352: error
enum { QW_SYNC_GEN = 0, QW_SYNC_TOP = 32, QW_SYNC_GROUP = 64, QW_SYNC_ERR = QW_SYNC_ERR_WORD };
__device__ __forceinline__ uint32_t qw_sync_add(uint32_t *p) { return __hip_atomic_fetch_add(p, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// One thread per workgroup calls this, after a __syncthreads() behind which every thread of the workgroup has waited
// for its own stores. gen0: the generation read when the launch began (no barrier can complete before every workgroup
// has read it); k: number of this barrier in the launch, from 1; G: workgroups of the launch. The last to arrive clears
// the counters for the next use and only then raises the generation. False: the wait gave up.
__device__ __forceinline__ bool qw_grid_barrier(uint32_t *sync, uint32_t gen0, uint32_t k, uint32_t G, uint32_t limit) {
    const uint32_t g = blockIdx.x & 7, per = (G + 7 - g) >> 3, groups = G < 8 ? G : 8;
    if (qw_sync_add(sync + QW_SYNC_GROUP + 32 * g) + 1 == per) {
        qw_st_coh(sync + QW_SYNC_GROUP + 32 * g, 0);
        __builtin_amdgcn_s_waitcnt(0); // cleared before anybody can be released into a later barrier
        if (qw_sync_add(sync + QW_SYNC_TOP) + 1 == groups) {
            qw_st_coh(sync + QW_SYNC_TOP, 0);
            __builtin_amdgcn_s_waitcnt(0);
            qw_st_coh(sync + QW_SYNC_GEN, gen0 + k);
        }
    }
    for (uint32_t spins = 0; qw_ld_coh(sync + QW_SYNC_GEN) - gen0 < k; spins++) {
        if (spins >= limit || ((spins & 63) == 63 && qw_ld_coh(sync + QW_SYNC_ERR))) {
            qw_st_coh(sync + QW_SYNC_ERR, 1);
            return false;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    return true;
}

// ---------------------------------------------------------------- activation fragment providers (operand A)
// Fragment order in LDS: chunk c (8 consecutive k-values) of token m lives at xf[c * 16 + m], 16 bytes, so that the
// 16 lanes of a k-group read 256 contiguous bytes. Tokens >= nb are stored as zeros.
struct qw_afrag_lds {
    const u4 *xf;
    uint32_t m;
    static constexpr bool has_lo = false;
    __device__ __forceinline__ h8 hi(uint32_t koff) const { return __builtin_bit_cast(h8, xf[(koff >> 3) * 16 + m]); }
    __device__ __forceinline__ h8 lo(uint32_t) const { return h8{}; }
    __device__ __forceinline__ h4 hi4(uint32_t koff) const { return __builtin_bit_cast(h4, ((const u2 *)xf)[((koff >> 3) * 16 + m) * 2 + ((koff >> 2) & 1)]); } // koff a multiple of 4
    __device__ __forceinline__ h4 lo4(uint32_t) const { return h4{}; }
};

// Two planes (hi + lo) staged the same way.
struct qw_afrag_lds2 {
    const u4 *hi_, *lo_;
    uint32_t m;
    static constexpr bool has_lo = true;
    __device__ __forceinline__ h8 hi(uint32_t koff) const { return __builtin_bit_cast(h8, hi_[(koff >> 3) * 16 + m]); }
    __device__ __forceinline__ h8 lo(uint32_t koff) const { return __builtin_bit_cast(h8, lo_[(koff >> 3) * 16 + m]); }
    // four values (koff a multiple of 4): one half of a 16-byte unit
    __device__ __forceinline__ h4 hi4(uint32_t koff) const { return __builtin_bit_cast(h4, ((const u2 *)hi_)[((koff >> 3) * 16 + m) * 2 + ((koff >> 2) & 1)]); }
    __device__ __forceinline__ h4 lo4(uint32_t koff) const { return __builtin_bit_cast(h4, ((const u2 *)lo_)[((koff >> 3) * 16 + m) * 2 + ((koff >> 2) & 1)]); }
};

// Every workgroup of a launch copies the same bytes: each starts at a different place (a rotation by its index), so
// that at any moment the workgroups ask different memory channels instead of all the same one.
// qw_stage_x_issue: direct global-to-LDS loads of the token columns in use, plain zero stores for the others; the
// caller runs qw_lds_arrive() and a barrier before the fragments are read.
__device__ __forceinline__ void qw_load_to_lds(const u4 *src_lane, u4 *dst_wave);
__device__ __forceinline__ void qw_lds_arrive();
// part, nparts: the calling wave is number `part` of the `nparts` waves that do the copy (default: all of the workgroup).
__device__ __forceinline__ void qw_stage_x_issue(u4 *xf, const uint16_t *x, uint32_t xstride, uint32_t K, uint32_t nb, uint32_t part = ~0u, uint32_t nparts = 0) {
    const uint32_t n = (K >> 3) * 16, rot = (blockIdx.x * 320u) % n, lane = threadIdx.x & 63; // n and rot are multiples of 64
    if (part == ~0u) part = threadIdx.x >> 6, nparts = blockDim.x >> 6;
    for (uint32_t i0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)part) * 64; i0 < n; i0 += 64 * nparts) {
        const uint32_t base = i0 + rot < n ? i0 + rot : i0 + rot - n, i = base + lane, c = i >> 4, m = i & 15;
        if (m < nb) qw_load_to_lds((const u4 *)(x + (size_t)m * xstride + 8 * c), xf + base);
        else xf[i] = u4{0, 0, 0, 0};
    }
}
__device__ __forceinline__ void qw_stage_x(u4 *xf, const uint16_t *x, uint32_t xstride, uint32_t K, uint32_t nb) {
    qw_stage_x_issue(xf, x, xstride, K, nb);
    qw_lds_arrive();
}

// Straight from global memory: row pointers of binary16 planes; a null row contributes zeros.
template <bool LO> struct qw_afrag_glb {
    const uint16_t *rowhi, *rowlo;
    static constexpr bool has_lo = LO;
    __device__ __forceinline__ h8 hi(uint32_t koff) const { return rowhi ? *(const h8 *)(rowhi + koff) : h8{}; }
    __device__ __forceinline__ h8 lo(uint32_t koff) const { return rowlo ? *(const h8 *)(rowlo + koff) : h8{}; }
    __device__ __forceinline__ h4 hi4(uint32_t koff) const { return rowhi ? *(const h4 *)(rowhi + koff) : h4{}; } // four values
    __device__ __forceinline__ h4 lo4(uint32_t koff) const { return rowlo ? *(const h4 *)(rowlo + koff) : h4{}; }
};

// One token's row of both planes staged in LDS as [hi I halves][lo I halves].
struct qw_afrag_ldsrow {
    const uint16_t *row;
    uint32_t I;
    static constexpr bool has_lo = true;
    __device__ __forceinline__ h8 hi(uint32_t koff) const { return *(const h8 *)(row + koff); }
    __device__ __forceinline__ h8 lo(uint32_t koff) const { return *(const h8 *)(row + I + koff); }
};

// Rows of the two H planes in global memory, read only by the lanes whose token column is in use ("on"): four
// fragments per plane at a time inside one predicated region, into registers the caller keeps (and has zeroed once),
// so that a lane that is off neither reads memory nor costs the address unit anything.
struct qw_afrag_gather {
    const uint16_t *rowhi, *rowlo;
    bool on;
    h8 (&hi)[4];
    h8 (&lo)[4];
    static constexpr bool has_lo = true;
    static constexpr bool stacked = false; // (true: both planes of a token in one operand A, the provider of the down launch by token shares)
    __device__ __forceinline__ void fetch4(uint32_t koff, uint32_t kstep) const {
        if (on) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                hi[i] = *(const h8 *)(rowhi + koff + i * kstep);
                lo[i] = *(const h8 *)(rowlo + koff + i * kstep);
            }
        }
    }
};

// A provider that holds its fragments in registers (member x[], declared `indexed`) is read by position, the others by
// K offset: idx is a constant wherever the loops around the call are unrolled, so x[idx] is a register, not an address.
template <class T, class = void> struct qw_is_indexed : std::false_type {};
template <class T> struct qw_is_indexed<T, std::void_t<decltype(T::indexed)>> : std::true_type {};
template <class AF> __device__ __forceinline__ h8 qw_af_hi(const AF &af, int idx, uint32_t koff) {
    if constexpr (qw_is_indexed<AF>::value) return af.x[idx];
    else return af.hi(koff);
}

// ---------------------------------------------------------------- chunks: the unit of prefetch
// A chunk is NB consecutive blocks of one weight row, held in registers by the lane that decodes them. Kernels keep
// DEPTH chunks per wave (two or three): while one is decoded and multiplied, the loads of the next one or two are in
// flight. With 12 waves per compute unit and 3.5 to 7 KB per wave in flight this covers the HBM latency; more in flight
// than that slows the device-wide streams down (see qw_chunk<QW_F_PACKED, NB>).
template <int F, int NB> struct qw_chunk;

template <int NB> struct qw_chunk<21, NB> {
    static constexpr uint32_t BLK_K = 256, BLK_B = 110;
    static constexpr int DEPTH = 3; // chunk buffers of the task pipeline (8 registers per block and buffer)
    qw_iq3_slice s[NB];
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t kg) {
#pragma unroll
        for (int b = 0; b < NB; b++) s[b] = qw_iq3_load(p + 110 * b, kg);
    }
    // All sixteen table reads of one block, issued together.
    __device__ __forceinline__ void lookups(int b, const u2 *lut, u2 (&w)[16]) const {
        const qw_iq3_keys k = qw_iq3_prep(s[b]);
        uint32_t i[16];
        qw_iq3_addr<0>(s[b], k, i[0], i[1]);
        qw_iq3_addr<1>(s[b], k, i[2], i[3]);
        qw_iq3_addr<2>(s[b], k, i[4], i[5]);
        qw_iq3_addr<3>(s[b], k, i[6], i[7]);
        qw_iq3_addr<4>(s[b], k, i[8], i[9]);
        qw_iq3_addr<5>(s[b], k, i[10], i[11]);
        qw_iq3_addr<6>(s[b], k, i[12], i[13]);
        qw_iq3_addr<7>(s[b], k, i[14], i[15]);
#pragma unroll
        for (int j = 0; j < 16; j++) {
            w[j] = qw_lut_at(lut, i[j]);
        }
    }
    // acc += this chunk's contribution; k0 = k-offset of the chunk's first value. Software pipeline over the blocks:
    // the table reads of block b + 1 and the activation fragments of block b are in flight while block b - 1's
    // matrix instructions run; two accumulators keep consecutive matrix instructions independent.
    // Loaded in quad order (load() was called with the row and k-group of lane >> 2, lane & 3): bring every block
    // to the matrix-core lane order.
    __device__ __forceinline__ void transpose() {
        const uint32_t src4 = qw_pull_addr();
#pragma unroll
        for (int b = 0; b < NB; b++) qw_iq3_transpose(s[b], src4);
    }
    template <class AF> __device__ __forceinline__ void mac(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const {
        u2 w[2][16];
        lookups(0, lut, w[0]);
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const uint32_t kb = k0 + 256 * b + 64 * kg;
            h8 xh[8], xl[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                xh[j] = af.hi(kb + 8 * j);
                if (AF::has_lo) xl[j] = af.lo(kb + 8 * j);
            }
            if (b + 1 < NB) lookups(b + 1, lut, w[(b + 1) & 1]);
            const h2 ff0 = qw_iq3_factor(s[b], 0), ff1 = qw_iq3_factor(s[b], 1);
            f4 sub0 = {0, 0, 0, 0}, sub1 = {0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const h2 ff = j < 4 ? ff0 : ff1;
                const u2 w0 = w[b & 1][2 * j], w1 = w[b & 1][2 * j + 1];
                u4 raw = {w0.x, w0.y, w1.x, w1.y};
#pragma unroll
                for (int i = 0; i < 4; i++) raw[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, (uint32_t)raw[i]) * ff);
                const h8 wv = __builtin_bit_cast(h8, raw);
                if (AF::has_lo) {
                    sub0 = qw_mfma(xh[j], wv, sub0);
                    sub1 = qw_mfma(xl[j], wv, sub1);
                } else if (j & 1) sub1 = qw_mfma(xh[j], wv, sub1);
                else sub0 = qw_mfma(xh[j], wv, sub0);
            }
            acc += s[b].d * (sub0 + sub1);
        }
    }
    // The same arithmetic without the cross-block pipeline (fewer registers; for kernels that run more waves).
    template <class AF> __device__ __forceinline__ void mac_lean(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const uint32_t kb = k0 + 256 * b + 64 * kg;
            u2 w[16];
            lookups(b, lut, w);
            h8 xh[8], xl[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                xh[j] = qw_af_hi(af, 8 * b + j, kb + 8 * j);
                if (AF::has_lo) xl[j] = af.lo(kb + 8 * j);
            }
            block_mfma(b, w, xh, xl, AF::has_lo, acc);
        }
    }
    // The VALU form of the same product, for NT <= 4 tokens (the GEMV the matrix-core form is measured against):
    // the lane's 64 values of a block times the same 64 activations of every token, by two-element dot
    // instructions into one binary32 sum per token; the caller adds the four k-group lanes of a row afterwards.
    template <int NT> __device__ __forceinline__ void dot_valu(const u2 *lut, const u4 *xf, uint32_t k0, uint32_t kg, float (&acc)[NT]) const {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const uint32_t kb = k0 + 256 * b + 64 * kg;
            u2 w[16];
            lookups(b, lut, w);
            const h2 ff0 = qw_iq3_factor(s[b], 0), ff1 = qw_iq3_factor(s[b], 1);
            float sub[NT];
#pragma unroll
            for (int t = 0; t < NT; t++) sub[t] = 0;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const h2 ff = j < 4 ? ff0 : ff1;
                u4 raw = {w[2 * j].x, w[2 * j].y, w[2 * j + 1].x, w[2 * j + 1].y};
#pragma unroll
                for (int i = 0; i < 4; i++) raw[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, (uint32_t)raw[i]) * ff);
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const u4 xv = xf[((kb + 8 * j) >> 3) * 16 + t]; // token t's 8 values: the same address in all 16 row lanes (broadcast)
#pragma unroll
                    for (int i = 0; i < 4; i++) sub[t] = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, (uint32_t)raw[i]), __builtin_bit_cast(h2, (uint32_t)xv[i]), sub[t], false);
                }
            }
#pragma unroll
            for (int t = 0; t < NT; t++) acc[t] += s[b].d * sub[t];
        }
    }
    // NG groups of 16 activation rows against the same decoded weights (the grouped product over packed rows):
    // rows[g] is the lane's row of group g in global memory; every group has its own accumulator.
    template <int NG> __device__ __forceinline__ void mac_groups(const u2 *lut, const uint16_t *const (&rows)[NG], uint32_t k0, uint32_t kg, f4 (&acc)[NG]) const {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const uint32_t kb = k0 + 256 * b + 64 * kg;
            u2 w[16];
            lookups(b, lut, w);
            const h2 ff0 = qw_iq3_factor(s[b], 0), ff1 = qw_iq3_factor(s[b], 1);
            f4 sub[NG];
#pragma unroll
            for (int g = 0; g < NG; g++) sub[g] = f4{0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const h2 ff = j < 4 ? ff0 : ff1;
                u4 raw = {w[2 * j].x, w[2 * j].y, w[2 * j + 1].x, w[2 * j + 1].y};
#pragma unroll
                for (int i = 0; i < 4; i++) raw[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, (uint32_t)raw[i]) * ff);
                const h8 wv = __builtin_bit_cast(h8, raw);
#pragma unroll
                for (int g = 0; g < NG; g++) sub[g] = qw_mfma(*(const h8 *)(rows[g] + kb + 8 * j), wv, sub[g]);
            }
#pragma unroll
            for (int g = 0; g < NG; g++) acc[g] += s[b].d * sub[g];
        }
    }
    // The same arithmetic with operand A gathered from global memory four steps at a time (qw_afrag_gather).
    template <class AF> __device__ __forceinline__ void mac_gather(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const uint32_t kb = k0 + 256 * b + 64 * kg;
            u2 w[16];
            lookups(b, lut, w);
            const h2 ff0 = qw_iq3_factor(s[b], 0), ff1 = qw_iq3_factor(s[b], 1);
            f4 sub0 = {0, 0, 0, 0}, sub1 = {0, 0, 0, 0};
#pragma unroll
            for (int half = 0; half < 2; half++) {
                af.fetch4(kb + 32 * half, 8);
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const int j = 4 * half + jj;
                    const h2 ff = half ? ff1 : ff0;
                    u4 raw = {w[2 * j].x, w[2 * j].y, w[2 * j + 1].x, w[2 * j + 1].y};
#pragma unroll
                    for (int i = 0; i < 4; i++) raw[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, (uint32_t)raw[i]) * ff);
                    const h8 wv = __builtin_bit_cast(h8, raw);
                    sub0 = qw_mfma(af.hi[jj], wv, sub0);
                    if constexpr (!AF::stacked) sub1 = qw_mfma(af.lo[jj], wv, sub1);
                }
            }
            if constexpr (AF::stacked) {
                // operand A rows 0 .. 3 held the hi plane, rows 4 .. 7 the lo plane of the same tokens: the lo sums lie
                // in the lanes 16 further (k-group 1). Each output row depends on its own operand A row only, so both
                // sums have the bits the two instructions above would give; only lanes 0 .. 15 hold a result.
                // (The elements are copied to scalars first: __builtin_bit_cast applied to a vector element directly read
                // element 0 whatever the index.)
                const int from = (int)(((threadIdx.x & 63) + 16) & 63) * 4;
                const float a0 = sub0[0], a1 = sub0[1], a2 = sub0[2], a3 = sub0[3];
                sub1 = f4{__builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(from, __builtin_bit_cast(int, a0))), __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(from, __builtin_bit_cast(int, a1))),
                          __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(from, __builtin_bit_cast(int, a2))), __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(from, __builtin_bit_cast(int, a3)))};
            }
            acc += s[b].d * (sub0 + sub1);
        }
    }
    // mac_lean with the operand-A fragments of four steps in registers at a time instead of eight (two planes cost
    // 32 registers instead of 64): for kernels whose operand A has a lo plane.
    template <class AF> __device__ __forceinline__ void mac_half(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const uint32_t kb = k0 + 256 * b + 64 * kg;
            u2 w[16];
            lookups(b, lut, w);
            const h2 ff0 = qw_iq3_factor(s[b], 0), ff1 = qw_iq3_factor(s[b], 1);
            f4 sub0 = {0, 0, 0, 0}, sub1 = {0, 0, 0, 0};
#pragma unroll
            for (int half = 0; half < 2; half++) {
                h8 xh[4], xl[4];
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    xh[jj] = af.hi(kb + 32 * half + 8 * jj);
                    if (AF::has_lo) xl[jj] = af.lo(kb + 32 * half + 8 * jj);
                }
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const int j = 4 * half + jj;
                    const h2 ff = half ? ff1 : ff0;
                    u4 raw = {w[2 * j].x, w[2 * j].y, w[2 * j + 1].x, w[2 * j + 1].y};
#pragma unroll
                    for (int i = 0; i < 4; i++) raw[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, (uint32_t)raw[i]) * ff);
                    const h8 wv = __builtin_bit_cast(h8, raw);
                    if (AF::has_lo) {
                        sub0 = qw_mfma(xh[jj], wv, sub0);
                        sub1 = qw_mfma(xl[jj], wv, sub1);
                    } else if (j & 1) sub1 = qw_mfma(xh[jj], wv, sub1);
                    else sub0 = qw_mfma(xh[jj], wv, sub0);
                }
            }
            acc += s[b].d * (sub0 + sub1);
        }
    }
    // One block's table values times two operand-A fragment sets (hi, lo), accumulated the way mac() does.
    __device__ __forceinline__ void block_mfma(int b, const u2 (&w)[16], const h8 (&xh)[8], const h8 (&xl)[8], bool lo, f4 &acc) const {
        const h2 ff0 = qw_iq3_factor(s[b], 0), ff1 = qw_iq3_factor(s[b], 1);
        f4 sub0 = {0, 0, 0, 0}, sub1 = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const h2 ff = j < 4 ? ff0 : ff1;
            u4 raw = {w[2 * j].x, w[2 * j].y, w[2 * j + 1].x, w[2 * j + 1].y};
#pragma unroll
            for (int i = 0; i < 4; i++) raw[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, (uint32_t)raw[i]) * ff);
            const h8 wv = __builtin_bit_cast(h8, raw);
            if (lo) {
                sub0 = qw_mfma(xh[j], wv, sub0);
                sub1 = qw_mfma(xl[j], wv, sub1);
            } else if (j & 1) sub1 = qw_mfma(xh[j], wv, sub1);
            else sub0 = qw_mfma(xh[j], wv, sub0);
        }
        acc += s[b].d * (sub0 + sub1);
    }
};

// Packed IQ3_S (see qwk_pack_args): the slab already lies in matrix-core lane order; three coalesced loads per block
// and no transpose. p is the (wave-uniform) address of the chunk's first slab, the second argument the lane.
#ifndef QW_PACKED_DEPTH
#define QW_PACKED_DEPTH 2
#endif
template <int NB> struct qw_chunk<QW_F_PACKED, NB> : qw_chunk<21, NB> {
    static constexpr uint32_t BLK_K = 256, BLK_B = QW_SLAB_BYTES;
    // One chunk ahead, not two: with every wave of the device streaming, more loads in flight made the launches slower
    // (24 layers at 16 tokens, ms: 1.80 with two chunks ahead in the routed gate/up and down launches, 1.70 with one, 1.85
    // and 1.95 with three and four in the gate/up launch; the grouped product of the packing path 4 % faster with one;
    // measured again after the queue loop stopped emptying the queue at every turn: two ahead 1.74 against 1.67).
    // QW_PACKED_DEPTH: for working builds that measure this.
    static constexpr int DEPTH = QW_PACKED_DEPTH;
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t lane) {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const uint8_t *sl = p + QW_SLAB_BYTES * b;
            this->s[b].qs = *(const u4 *)(sl + 16 * lane);
            this->s[b].sg = *(const u2 *)(sl + 1024 + 8 * lane);
            this->s[b].qh = *(const uint32_t *)(sl + 1536 + 4 * lane); // qh | scales << 16 | d byte << 24: unpacked in transpose()
        }
    }
    // Nothing moves between lanes except the second byte of d, which the lane 16 further holds.
    __device__ __forceinline__ void transpose() {
        const bool odd = (threadIdx.x >> 4) & 1;
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const uint32_t w = this->s[b].qh, mine = w >> 24, other = (uint32_t)__shfl_xor((int)w, 16) >> 24;
            this->s[b].d = qw_h2f((uint16_t)(odd ? (other | mine << 8) : (mine | other << 8)));
            this->s[b].sc = (w >> 16) & 255;
            this->s[b].qh = w & 0xffff;
        }
    }
};

// QW_F_ABLATE: the same loads and lane moves, no decoding and no matrix instructions (a measurement; see qw_kargs.h).
template <int NB> struct qw_chunk<QW_F_ABLATE, NB> : qw_chunk<QW_F_PACKED, NB> {
    static constexpr uint32_t BLK_K = 256, BLK_B = QW_SLAB_BYTES;
    static constexpr int DEPTH = 2;
    template <class AF> __device__ __forceinline__ void mac_lean(const u2 *, const AF &, uint32_t, uint32_t, f4 &acc) const {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const qw_iq3_slice &s = this->s[b];
            acc[0] += __builtin_bit_cast(float, (s.qs[0] ^ s.qs[1] ^ s.qs[2] ^ s.qs[3] ^ s.sg.x ^ s.sg.y ^ s.qh ^ s.sc) & 0x007fffffu) + s.d;
        }
    }
};

template <int NB> struct qw_chunk<8, NB> {
    static constexpr uint32_t BLK_K = 32, BLK_B = 34;
    static constexpr int DEPTH = 2;
    u2 q[NB];
    uint16_t d[NB];
    __device__ __forceinline__ void load(const uint8_t *p, uint32_t kg) {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            q[b] = *(const u2a2 *)(p + 34 * b + 2 + 8 * kg);
            d[b] = *(const uint16_t *)(p + 34 * b);
        }
    }
    __device__ __forceinline__ void transpose() {
        const uint32_t src4 = qw_pull_addr();
#pragma unroll
        for (int b = 0; b < NB; b++) {
            q[b].x = qw_pull(q[b].x, src4);
            q[b].y = qw_pull(q[b].y, src4);
        }
#pragma unroll
        for (int b = 0; b + 1 < NB; b += 2) { // two scales per pull
            const uint32_t m = qw_pull((uint32_t)d[b] | ((uint32_t)d[b + 1] << 16), src4);
            d[b] = (uint16_t)m;
            d[b + 1] = (uint16_t)(m >> 16);
        }
        if (NB & 1) d[NB - 1] = (uint16_t)qw_pull(d[NB - 1], src4);
    }
    template <class AF> __device__ __forceinline__ void mac_lean(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const { mac(lut, af, k0, kg, acc); }
    template <class AF> __device__ __forceinline__ void mac_half(const u2 *lut, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const { mac(lut, af, k0, kg, acc); }
    template <int NG> __device__ __forceinline__ void mac_groups(const u2 *, const uint16_t *const (&rows)[NG], uint32_t k0, uint32_t kg, f4 (&acc)[NG]) const {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const h8 w = qw_q8_cvt(q[b]);
            const uint32_t kb = k0 + 32 * b + 8 * kg;
#pragma unroll
            for (int g = 0; g < NG; g++) {
                f4 sub = {0, 0, 0, 0};
                sub = qw_mfma(*(const h8 *)(rows[g] + kb), w, sub);
                acc[g] += qw_h2f(d[b]) * sub;
            }
        }
    }
    // operand A gathered four blocks at a time (NB a multiple of 4)
    template <class AF> __device__ __forceinline__ void mac_gather(const u2 *, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const {
        if constexpr (NB % 4 != 0) { // block by block
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const uint32_t kb = k0 + 32 * b + 8 * kg;
                if (af.on) af.hi[0] = *(const h8 *)(af.rowhi + kb), af.lo[0] = *(const h8 *)(af.rowlo + kb);
                f4 sub = {0, 0, 0, 0};
                sub = qw_mfma(af.hi[0], qw_q8_cvt(q[b]), sub);
                sub = qw_mfma(af.lo[0], qw_q8_cvt(q[b]), sub);
                acc += qw_h2f(d[b]) * sub;
            }
            return;
        }
#pragma unroll
        for (int b4 = 0; b4 + 3 < NB; b4 += 4) {
            af.fetch4(k0 + 32 * b4 + 8 * kg, 32);
#pragma unroll
            for (int bb = 0; bb < 4; bb++) {
                const int b = b4 + bb;
                const h8 w = qw_q8_cvt(q[b]);
                f4 sub = {0, 0, 0, 0};
                sub = qw_mfma(af.hi[bb], w, sub);
                sub = qw_mfma(af.lo[bb], w, sub);
                acc += qw_h2f(d[b]) * sub;
            }
        }
    }
    template <class AF> __device__ __forceinline__ void mac(const u2 *, const AF &af, uint32_t k0, uint32_t kg, f4 &acc) const {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const h8 w = qw_q8_cvt(q[b]);
            const uint32_t kb = k0 + 32 * b + 8 * kg;
            f4 sub = {0, 0, 0, 0};
            sub = qw_mfma(qw_af_hi(af, b, kb), w, sub);
            if (AF::has_lo) sub = qw_mfma(af.lo(kb), w, sub);
            acc += qw_h2f(d[b]) * sub;
        }
    }
};

// Two-chunk software pipeline over n items: load(i, chunk&) issues the loads of item i (in quad lane order),
// use(i, chunk&) consumes them after the move to matrix-core lane order.
template <class C, class L, class U> __device__ __forceinline__ void qw_pipeline(uint32_t n, L load, U use) {
    C a, b;
    if (n) load(0u, a);
    uint32_t i = 0;
    while (i < n) {
        if (i + 1 < n) load(i + 1, b);
        a.transpose();
        use(i, a);
        if (++i >= n) break;
        if (i + 1 < n) load(i + 1, a);
        b.transpose();
        use(i, b);
        ++i;
    }
}

// The same pipeline over the tasks w0, w0 + nw, ... < ntasks of one wave, cpr chunks per task, without a division
// per chunk: two cursors step through (task, chunk). rowp(task) is the lane's byte pointer to the task's first
// chunk (chunk c follows at c * cstride bytes); use(task, c, chunk) consumes chunk c of a task. All of ntasks, w0,
// nw and cpr must be wave-uniform.
// ready() is called exactly once by every wave, after the first loads are issued and before anything is consumed:
// the place for the workgroup's set-up and barrier, so that the first memory round trip overlaps them.
template <class C, int DEPTH = C::DEPTH, class R, class U, class S>
__device__ __forceinline__ void qw_task_pipeline(uint32_t ntasks, uint32_t w0, uint32_t nw, uint32_t cpr, uint32_t cstride, uint32_t kl, R rowp, U use, S ready) {
    if (w0 >= ntasks) {
        ready();
        return;
    }
    // DEPTH chunk buffers: the loads run DEPTH - 1 chunks ahead of the arithmetic
    C buf[DEPTH];
    const uint32_t total = ((ntasks - w0 + nw - 1) / nw) * cpr;
    uint32_t li = 0, ui = 0, lt = w0, lc = 0, ut = w0, uc = 0;
    const uint8_t *lrow = rowp(lt);
    auto load = [&](C &x) {
        if (li == total) return;
        ++li;
        x.load(lrow + (size_t)lc * cstride, kl);
        if (++lc == cpr) {
            lc = 0;
            lt += nw;
            if (lt < ntasks) lrow = rowp(lt);
        }
    };
    auto consume = [&](C &x) {
        x.transpose();
        use(ut, uc, x);
        if (++uc == cpr) uc = 0, ut += nw;
        return ++ui == total;
    };
#pragma unroll
    for (int i = 0; i + 1 < DEPTH; i++) load(buf[i]);
    ready();
    for (bool done = false; !done;) {
#pragma unroll
        for (int i = 0; i < DEPTH; i++) {
            if (done) break;
            load(buf[(i + DEPTH - 1) % DEPTH]);
            done = consume(buf[i]);
        }
    }
}


// The streaming form of qw_task_pipeline, for the kernels whose waves each run through several tasks (the routed
// gate/up and down products): same arguments and the same calls of rowp, use and ready, plus spare, which is null or the
// address of 64 KB of readable memory that stays in cache (the lookup table).
template <class C, int DEPTH = C::DEPTH, class R, class U, class S>
__device__ __forceinline__ void qw_task_stream(uint32_t ntasks, uint32_t w0, uint32_t nw, uint32_t cpr, uint32_t cstride, uint32_t kl, R rowp, U use, S ready, const uint8_t *spare = nullptr) {
    if (w0 >= ntasks) {
        ready();
        return;
    }
    // DEPTH chunk buffers: the loads run DEPTH - 1 chunks ahead of the arithmetic
    C buf[DEPTH];
    uint32_t left = ((ntasks - w0 + nw - 1) / nw) * cpr;
    uint32_t lt = w0, lc = 0, ut = w0, uc = 0;
    const uint8_t *lrow = rowp(lt);
    // Every step issues one chunk's loads, whatever happens: once the wave's rows are used up the loads read a row's worth
    // of valid, cached memory that is never consumed (the caller's spare region of at least 64 KB if a row fits in it,
    // else the wave's own first row again). The loop below then has no memory operation under a condition and a fixed
    // trip structure, so the number of loads in flight at each wait is the same on every path and the compiler waits for
    // "all but the youngest DEPTH - 1 chunks" instead of emptying the queue.
    const uint8_t *const past = spare && cpr * cstride <= 65536u ? spare : lrow;
    auto load = [&](C &x) {
        x.load(lrow + (size_t)lc * cstride, kl);
        if (++lc == cpr) {
            lc = 0;
            lt += nw;
            lrow = lt < ntasks ? rowp(lt) : past;
        }
    };
    auto consume = [&](C &x) {
        x.transpose();
        use(ut, uc, x);
        if (++uc == cpr) uc = 0, ut += nw;
    };
#pragma unroll
    for (int i = 0; i + 1 < DEPTH; i++) load(buf[i]);
    ready();
    for (; left >= DEPTH; left -= DEPTH) {
#pragma unroll
        for (int i = 0; i < DEPTH; i++) {
            load(buf[(i + DEPTH - 1) % DEPTH]);
            consume(buf[i]);
        }
    }
#pragma unroll
    for (int i = 0; i + 1 < DEPTH; i++)
        if (left > (uint32_t)i) consume(buf[i]);
}

// The same streaming with the tasks taken from a queue instead of a fixed stride: `first` is the wave's first task,
// next() returns its next one whenever it has asked for all chunks of the current one (any value >= ntasks: none left,
// and none ever again). A workgroup's waves share a counter in LDS behind next(): the hardware serves the older waves of
// a compute unit first, so with a fixed deal the first waves finish their tiles long before the last ones and the unit
// runs its last third with a few waves' loads in flight; from a queue every wave works until the workgroup's tiles are gone.
// Each chunk buffer carries the task and chunk it was loaded for.
template <class C, int DEPTH = C::DEPTH, class N, class R, class U, class S>
__device__ __forceinline__ void qw_task_queue(uint32_t ntasks, uint32_t first, N next, uint32_t cpr, uint32_t cstride, uint32_t kl, R rowp, U use, S ready, const uint8_t *spare = nullptr) {
    if (first >= ntasks) {
        ready();
        return;
    }
    C buf[DEPTH];
    uint32_t btask[DEPTH], bchunk[DEPTH];
    uint32_t lt = first, lc = 0;
    const uint8_t *lrow = rowp(lt);
    // (every step issues one chunk's loads whatever happens, as in qw_task_stream: past the last task they read valid, cached memory)
    const uint8_t *const past = spare && cpr * cstride <= 65536u ? spare : lrow;
    auto load = [&](int i) {
        btask[i] = lt, bchunk[i] = lc;
        buf[i].load(lrow + (size_t)lc * cstride, kl);
        if (++lc == cpr) {
            lc = 0;
            if (lt < ntasks) lt = next();
            lrow = lt < ntasks ? rowp(lt) : past;
        }
    };
#pragma unroll
    for (int i = 0; i + 1 < DEPTH; i++) load(i);
    ready();
    // One phase per chunk buffer, written out instead of an unrolled loop with a flag: the wave leaves from inside a
    // phase, so the only way back to the top is the one on which every load but the last phase's has been waited for,
    // and the youngest chunk stays in flight across the turn (with the flag, the leaving path met the top of the loop
    // and the compiler emptied the queue there on every turn).
    static_assert(DEPTH >= 1 && DEPTH <= 4, "chunk buffers");
    auto phase = [&](auto I) -> bool {
        constexpr int i = decltype(I)::value;
        load((i + DEPTH - 1) % DEPTH);
        if (btask[i] >= ntasks) return false;
        buf[i].transpose();
        use(btask[i], bchunk[i], buf[i]);
        return true;
    };
    for (;;) {
        if (!phase(std::integral_constant<int, 0>{})) break;
        if constexpr (DEPTH > 1) {
            if (!phase(std::integral_constant<int, 1>{})) break;
        }
        if constexpr (DEPTH > 2) {
            if (!phase(std::integral_constant<int, 2>{})) break;
        }
        if constexpr (DEPTH > 3) {
            if (!phase(std::integral_constant<int, 3>{})) break;
        }
    }
}


// Copy the 64 KB pre-signed table from global memory into LDS (all loads first, then the stores).
// Sixty-four 16-byte units from global memory straight into LDS, no register in between: lane l's unit lands at
// dst + 16 l bytes (dst the same in every lane); src is per lane. Completion is counted like any other vector load:
// qw_lds_arrive() before the barrier that publishes the data.
__device__ __forceinline__ void qw_load_to_lds(const u4 *src_lane, u4 *dst_wave) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src_lane, (__attribute__((address_space(3))) void *)dst_wave, 16, 0, 0);
}
__device__ __forceinline__ void qw_lds_arrive() { __builtin_amdgcn_s_waitcnt(0); }

// Issue the copy of the 64 KB table into LDS (direct loads, a wave takes 64 entries at a time). Every workgroup of a
// launch starts at a different place of the table (a rotation by its index), so that at any moment the workgroups
// ask different memory channels. The caller runs qw_lds_arrive() and a barrier before the table is read.
// part, nparts: as in qw_stage_x_issue.
__device__ __forceinline__ void qw_lut_copy_issue(u2 *lut, const u2 *glut, uint32_t part = ~0u, uint32_t nparts = 0) {
    const u4 *src = (const u4 *)glut;
    u4 *dst = (u4 *)lut;
    constexpr uint32_t N = QW_LUT_BYTES / 16;
    const uint32_t rot = blockIdx.x * 320u, lane = threadIdx.x & 63;
    if (part == ~0u) part = threadIdx.x >> 6, nparts = blockDim.x >> 6;
    for (uint32_t i = (uint32_t)__builtin_amdgcn_readfirstlane((int)part) * 64; i < N; i += 64 * nparts) {
        const uint32_t j = (i + rot) & (N - 1); // a multiple of 64, the same in every lane
        qw_load_to_lds(src + j + lane, dst + j);
    }
}
__device__ __forceinline__ void qw_lut_copy(u2 *lut, const u2 *glut) {
    qw_lut_copy_issue(lut, glut);
    qw_lds_arrive();
}

template <class C, class R, class U>
__device__ __forceinline__ void qw_task_pipeline(uint32_t ntasks, uint32_t w0, uint32_t nw, uint32_t cpr, uint32_t cstride, uint32_t kl, R rowp, U use) {
    qw_task_pipeline<C>(ntasks, w0, nw, cpr, cstride, kl, rowp, use, [] {});
}

// ---------------------------------------------------------------- wave-wide maximum of an unsigned key
// DPP row shifts inside each row of 16 lanes, then the two row broadcasts of the gfx9 family; every lane receives
// the result through a read of lane 63.
__device__ __forceinline__ uint32_t qw_wave_max_u32(uint32_t v) {
#define QW_DPP_MAX(ctrl, rmask, bmask) v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, ctrl, rmask, bmask, false)) /* 0: lanes without a source keep v */
    QW_DPP_MAX(0x111, 0xf, 0xf); // row_shr:1
    QW_DPP_MAX(0x112, 0xf, 0xf); // row_shr:2
    QW_DPP_MAX(0x114, 0xf, 0xf); // row_shr:4
    QW_DPP_MAX(0x118, 0xf, 0xf); // row_shr:8  -> lane 15 of each row holds the row maximum
    QW_DPP_MAX(0x142, 0xa, 0xf); // row_bcast:15 into rows 1 and 3
    QW_DPP_MAX(0x143, 0xc, 0xf); // row_bcast:31 into rows 2 and 3 -> lane 63 holds the wave maximum
#undef QW_DPP_MAX
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}
// Order-preserving map float -> uint32 (larger float = larger key); -0.0 is taken as +0.0 so that the two tie.
__device__ __forceinline__ uint32_t qw_fkey(float f) {
    uint32_t b = __builtin_bit_cast(uint32_t, f);
    if (b == 0x80000000u) b = 0;
    return b ^ ((b >> 31) ? 0xffffffffu : 0x80000000u);
}
__device__ __forceinline__ float qw_fkey_inv(uint32_t k) {
    const uint32_t b = k ^ ((k >> 31) ? 0x80000000u : 0xffffffffu);
    return __builtin_bit_cast(float, b);
}
