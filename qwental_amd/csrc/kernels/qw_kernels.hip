// HIP kernels of the quantized decode path for gfx950. One code object; gpu_hip.c loads it and launches these
// entry points by name. Each kernel takes one argument record from qw_kargs.h by value.
//
// Shape of the weight-streaming kernels (dense matvec, gate/up, down): persistent workgroups of 512 or 768 threads, one
// per compute unit (the 64 KB pre-signed table plus the staged activations fill most of the 160 KB LDS). Each wave
// walks 16-row tiles through a register pipeline of chunks: the loads of the next chunk (for some formats the next two)
// are issued before the current one is decoded. In the routed gate/up launch and the down launch by token shares the
// tiles of a workgroup go to its waves from a queue in LDS, elsewhere every wave has its own fixed list.
#include "qw_common.hip.h"
#include "qw_kquants.hip.h"

// The entry points come in groups, QW_IN_PART(k) around each: a build with -DQW_PARTS=<bit mask> holds only the groups
// whose bit is set (experiments that need a few kernels and a short compile); the product build holds all of them, in
// one code object (the same kernels spread over several code objects measured 3 % slower on the 48-layer step).
#ifdef QW_PARTS
#define QW_IN_PART(k) ((QW_PARTS >> (k)) & 1)
#else
#define QW_IN_PART(k) 1
#endif
#ifdef QW_STAMPS // working builds only: time stamps (10 ns units) of thread 0 of every workgroup, 16 words a workgroup, where the host points this
extern "C" __device__ uint32_t *qw_stamp_ptr;
__device__ uint32_t *qw_stamp_ptr;
#if QW_STAMPS == 2 // only the routed gate/up launch: every wave's end (slots 0 .. 11), the workgroup's entry (12) and selection (13)
#define QW_DSTAMP(k) do {} while (0)
#define QW_WSTAMP(k) do { if (qw_stamp_ptr && (threadIdx.x & 63) == 0) qw_stamp_ptr[512 + 16 * blockIdx.x + (k)] = (uint32_t)__builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define QW_DSTAMP(k) do { if (threadIdx.x == 0 && qw_stamp_ptr) qw_stamp_ptr[512 + 16 * blockIdx.x + (k)] = (uint32_t)__builtin_amdgcn_s_memrealtime(); } while (0)
#define QW_WSTAMP(k) do {} while (0)
#endif
#else
#define QW_DSTAMP(k) do {} while (0)
#define QW_WSTAMP(k) do {} while (0)
#endif
#if defined(QW_STAMPS) && QW_STAMPS == 3 // steps of the selection in the routed gate/up launch: 16 stamps a wave, kept in LDS until the launch ends
__shared__ uint32_t qw_sst[12 * 16];
#undef QW_DSTAMP
#define QW_DSTAMP(k) do {} while (0)
#define QW_SSTAMP(k) do { if ((threadIdx.x & 63) == 0) qw_sst[(threadIdx.x >> 6) * 16 + (k)] = (uint32_t)__builtin_amdgcn_s_memrealtime(); } while (0)
#define QW_SDEP(v) asm volatile("" :: "v"(v))
#define QW_SST_FLUSH() do { QW_SSTAMP(15); __syncthreads(); if (qw_stamp_ptr && blockIdx.x < 32 && threadIdx.x < 192) qw_stamp_ptr[512 + 192 * blockIdx.x + threadIdx.x] = qw_sst[threadIdx.x]; } while (0)
#else
#define QW_SSTAMP(k) do {} while (0)
#define QW_SDEP(v) do {} while (0)
#define QW_SST_FLUSH() do {} while (0)
#endif
#if defined(QW_STAMPS) && QW_STAMPS == 4 // steps of the front launch only
#undef QW_DSTAMP
#define QW_DSTAMP(k) do {} while (0)
#define QW_PSTAMP(k) do { if (threadIdx.x == 0 && qw_stamp_ptr) qw_stamp_ptr[512 + 16 * blockIdx.x + (k)] = (uint32_t)__builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define QW_PSTAMP(k) do {} while (0)
#endif
#if defined(QW_STAMPS) && QW_STAMPS == 5 // steps of the hyper-connection's launches (workgroups 0 .. 255 of each)
#undef QW_DSTAMP
#define QW_DSTAMP(k) do {} while (0)
#define QW_HSTAMP(k) do { const uint32_t wg_ = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z); if (threadIdx.x == 0 && qw_stamp_ptr && wg_ < 256) qw_stamp_ptr[512 + 16 * wg_ + (k)] = (uint32_t)__builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define QW_HSTAMP(k) do {} while (0)
#endif
#ifdef QW_STAMPS
#define QW_WG_END_STAMP(k) do { __syncthreads(); QW_DSTAMP(k); } while (0)
#else
#define QW_WG_END_STAMP(k) do {} while (0)
#endif

#define QW_WG 512          // threads per workgroup of the down and front kernels (8 waves)
#define QW_WG_DN 768       // down range kernels: 12 waves
#define QW_WG_GU 768       // gate/up and dense matvec: 12 waves, three per SIMD (a wave issues at most one instruction in ~6 cycles)
#define QW_XF_MAXK 2560    // largest K whose activations are staged in LDS in fragment order (K * 32 bytes)

// wave index in the workgroup, as a scalar (so that task indices and row bases stay in scalar registers)
__device__ __forceinline__ uint32_t qw_wave() { return (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }
__device__ __forceinline__ uint32_t qw_lane() { return threadIdx.x & 63; }
constexpr bool qw_has_lut(int f) { return f == 21 || f == QW_F_PACKED || f == QW_F_ABLATE; } // formats decoded through the LDS table (the ablation copies it too)
__device__ __forceinline__ uint32_t qw_all_tokens(uint32_t nbr) { return nbr >= 32 ? 0xffffffffu : (1u << nbr) - 1; }

// ================================================================ dq_test (kernels/moe_iq.metal:208-217)
// rows x K values to float, decoded with the same step decoders the matrix-core kernels use. Grid: rows x 64.
template <int F> __device__ __forceinline__ void dq_test_body(const qwk_dq_args &a, const u2 *lut) {
    const uint8_t *row = a.W + (size_t)blockIdx.x * a.rowbytes;
    float *y = a.y + (size_t)blockIdx.x * a.K;
    if (F == 21) {
        for (uint32_t i = threadIdx.x; i < a.K / 64; i += blockDim.x) {
            const uint32_t blk = i >> 2, kg = i & 3;
            const qw_iq3_slice s = qw_iq3_load(row + 110 * blk, kg);
            h8 v[8] = {qw_iq3_step<0>(s, lut), qw_iq3_step<1>(s, lut), qw_iq3_step<2>(s, lut), qw_iq3_step<3>(s, lut),
                       qw_iq3_step<4>(s, lut), qw_iq3_step<5>(s, lut), qw_iq3_step<6>(s, lut), qw_iq3_step<7>(s, lut)};
            for (int j = 0; j < 8; j++)
                for (int e = 0; e < 8; e++) y[256 * blk + 64 * kg + 8 * j + e] = s.d * (float)v[j][e];
        }
    } else {
        for (uint32_t i = threadIdx.x; i < a.K / 8; i += blockDim.x) {
            const uint32_t blk = i >> 2, kg = i & 3;
            const uint8_t *b = row + 34 * blk;
            const h8 v = qw_q8_cvt(*(const u2a2 *)(b + 2 + 8 * kg));
            const float d = qw_h2f(*(const uint16_t *)b);
            for (int e = 0; e < 8; e++) y[32 * blk + 8 * kg + e] = d * (float)v[e];
        }
    }
}

#if QW_IN_PART(0)
extern "C" __global__ __launch_bounds__(64) void qwk_dq_test_f21(qwk_dq_args a) {
    __shared__ u2 lut[QW_LUT_ENTRIES];
    qw_lut_build(lut);
    __syncthreads();
    dq_test_body<21>(a, lut);
}
extern "C" __global__ __launch_bounds__(64) void qwk_dq_test_f8(qwk_dq_args a) { dq_test_body<8>(a, nullptr); }
#endif

// The formats of qw_kquants.hip.h: every lane decodes the slice of a block it would supply to the matrix instruction
// and writes the values as the reference computes them (scale * integer - min in float). Grid: rows x 64.
template <int F> __device__ __forceinline__ void dq_test_kq(const qwk_dq_args &a, const uint32_t *tab) {
    const uint8_t *row = a.W + (size_t)blockIdx.x * a.rowbytes;
    float *y = a.y + (size_t)blockIdx.x * a.K;
    for (uint32_t i = threadIdx.x; i < a.K / qw_kq<F>::BLK_K * 4; i += blockDim.x) {
        const uint32_t blk = i >> 2, kg = i & 3;
        qw_kq<F> b;
        b.load(row + (size_t)qw_kq<F>::BLK_B * blk, kg);
        qw_kq_values<F>(b, tab, kg, y + (size_t)qw_kq<F>::BLK_K * blk);
    }
}
#if QW_IN_PART(0)
extern "C" __global__ __launch_bounds__(64) void qwk_dq_test_kq(qwk_dq_args a) {
    __shared__ uint32_t tab[QW_KQ_TAB];
    qw_kq_tab_build(tab);
    __syncthreads();
    switch (a.fmt) {
    case 1: dq_test_kq<1>(a, tab); break;
    case 12: dq_test_kq<12>(a, tab); break;
    case 13: dq_test_kq<13>(a, tab); break;
    case 14: dq_test_kq<14>(a, tab); break;
    case 20: dq_test_kq<20>(a, tab); break;
    case 23: dq_test_kq<23>(a, tab); break;
    case 30: dq_test_kq<30>(a, tab); break;
    }
}
#endif

// ================================================================ lookup-table buffer (kernels/moe_gg.metal:495-515)
// Only the IQ3_S section is produced; the sections of formats without a gfx950 build stay zero. Grid: 32 x 256.
#if QW_IN_PART(0)
extern "C" __global__ void qwk_tab_init(qwk_tab_args a) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < QW_LUT_ENTRIES) ((u2 *)(a.tab + QW_TAB_IQ3SS))[a.slot_order ? qw_lut_slot(i) : i] = qw_lut_entry(i);
}
#endif

// ================================================================ packing of IQ3_S rows (layout: qwk_pack_args)
// One thread per (slab, lane), grid-stride over the slabs; run once per weight matrix, at its first use.
#if QW_IN_PART(0)
extern "C" __global__ __launch_bounds__(256) void qwk_pack_iq3(qwk_pack_args a) {
    const uint64_t nslab = a.ntiles * a.nblk, step = (uint64_t)gridDim.x * (blockDim.x >> 6);
    const uint32_t lane = threadIdx.x & 63, n = lane & 15, kg = lane >> 4;
    for (uint64_t sl = (uint64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6); sl < nslab; sl += step) {
        const uint64_t tile = sl / a.nblk;
        const uint32_t blk = (uint32_t)(sl % a.nblk);
        const uint8_t *row = n < a.split ? a.A + (tile * a.split + n) * a.rowbytes : a.B + (tile * (16 - a.split) + (n - a.split)) * a.rowbytes;
        const uint8_t *src = row + 110 * blk;
        uint8_t *dst = a.dst + sl * QW_SLAB_BYTES;
        *(u4 *)(dst + 16 * lane) = *(const u4a2 *)(src + 2 + 16 * kg);
        *(u2 *)(dst + 1024 + 8 * lane) = *(const u2a2 *)(src + 74 + 8 * kg);
        const uint32_t qh = *(const uint16_t *)(src + 66 + 2 * kg), sc = src[106 + kg], db = src[kg & 1];
        *(uint32_t *)(dst + 1536 + 4 * lane) = qh | sc << 16 | db << 24;
    }
}
#endif

// The tile-major copy of Q6_K rows (layout: QW_F_PACKED_Q6 in qw_kargs.h); a wave per (tile, block). The twelve dwords a
// lane takes are the ones qw_kq<14>::load reads for that lane's row and k-group.
#if QW_IN_PART(0)
extern "C" __global__ __launch_bounds__(256) void qwk_pack_q6(qwk_pack_args a) {
    const uint64_t nslab = a.ntiles * a.nblk, step = (uint64_t)gridDim.x * (blockDim.x >> 6);
    const uint32_t lane = threadIdx.x & 63, n = lane & 15, kg = lane >> 4;
    for (uint64_t sl = (uint64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6); sl < nslab; sl += step) {
        const uint64_t tile = sl / a.nblk;
        const uint8_t *src = a.A + (tile * 16 + n) * a.rowbytes + 210 * (sl % a.nblk);
        uint8_t *dst = a.dst + sl * QW_Q6_SLAB_BYTES;
        uint32_t r[12];
#pragma unroll
        for (int i = 0; i < 8; i++) r[i] = *(const u1a2 *)(src + 64 * (i >> 2) + 32 * ((i >> 1) & 1) + 16 * (i & 1) + 4 * kg);
#pragma unroll
        for (int i = 0; i < 4; i++) r[8 + i] = *(const u1a2 *)(src + 128 + 32 * (i >> 1) + 16 * (i & 1) + 4 * kg);
#pragma unroll
        for (int pl = 0; pl < 3; pl++) *(u4 *)(dst + 1024 * pl + 16 * lane) = u4{r[4 * pl], r[4 * pl + 1], r[4 * pl + 2], r[4 * pl + 3]};
        *(uint32_t *)(dst + 3072 + 16 * n + 4 * kg) = *(const u1a2 *)(src + 192 + 4 * kg); // the row's four lanes write its sixteen scales
        if (kg == 0) *(uint16_t *)(dst + 3328 + 2 * n) = *(const uint16_t *)(src + 208);
    }
}
#endif

// The tile-major copy of IQ4_NL rows (layout: QW_F_PACKED_NL in qw_kargs.h); a wave per (tile, chunk of ten blocks).
#if QW_IN_PART(0)
extern "C" __global__ __launch_bounds__(256) void qwk_pack_nl(qwk_pack_args a) {
    const uint64_t nchunk = a.ntiles * a.nblk, step = (uint64_t)gridDim.x * (blockDim.x >> 6);
    const uint32_t lane = threadIdx.x & 63, n = lane & 15, kg = lane >> 4;
    for (uint64_t ch = (uint64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6); ch < nchunk; ch += step) {
        const uint64_t tile = ch / a.nblk;
        const uint8_t *src = a.A + (tile * 16 + n) * a.rowbytes + 180 * (ch % a.nblk);
        uint8_t *dst = a.dst + ch * QW_NL_CHUNK_BYTES;
        uint32_t q[10];
#pragma unroll
        for (int b = 0; b < 10; b++) q[b] = *(const u1a2 *)(src + 18 * b + 2 + 4 * kg);
        *(u4 *)(dst + 16 * lane) = u4{q[0], q[1], q[2], q[3]};
        *(u4 *)(dst + 1024 + 16 * lane) = u4{q[4], q[5], q[6], q[7]};
        *(u2 *)(dst + 2048 + 8 * lane) = u2{q[8], q[9]};
        if (kg == 0)
#pragma unroll
            for (int b = 0; b < 10; b++) *(uint16_t *)(dst + 2560 + 20 * n + 2 * b) = *(const uint16_t *)(src + 18 * b);
    }
}
#endif

// ================================================================ dense matvec (kernels/qmv_gg.metal:17-39)
// y[b][row] = sum_k W[row][k] x[b][k] for up to 16 activations; the weights are streamed once for all of them.
// Tiles of 16 rows are dealt round-robin to the waves of a persistent grid; a row is CPR chunks of CH blocks.
template <int F, int CH, bool XLDS> __device__ __forceinline__ void qmv_body(const qwk_qmv_args &a, u2 *lut, u4 *xf, f4 *red) {
    typedef qw_chunk<F, CH> C;
    const uint32_t lane = qw_lane(), n = lane & 15, kg = lane >> 4;
    const uint32_t nw = gridDim.x * (blockDim.x >> 6), w0 = qw_wave() * gridDim.x + blockIdx.x /* wave-major: see gu_body */;
    const uint32_t cpr = a.K / (C::BLK_K * CH);
    const uint32_t nl = lane >> 2, kl = lane & 3; // (row, k-group) this lane loads
    auto rowp = [&](uint32_t t) {
        if constexpr (F == QW_F_PACKED) return a.W + (size_t)t * a.rowbytes; // the tile's slabs
        else {
            const uint32_t r = 16 * t + nl;
            return a.W + (size_t)(r < a.N ? r : a.N - 1) * a.rowbytes;
        }
    };
    auto store = [&](uint32_t t, const f4 &acc) {
        const uint32_t r = 16 * t + n;
        if (r < a.N)
#pragma unroll
            for (uint32_t j = 0; j < 4; j++) {
                const uint32_t tok = 4 * kg + j;
                if (tok < a.nb) {
                    if (a.yfloat) ((float *)a.y)[(size_t)tok * a.ystride + r] = acc[j];
                    else ((uint16_t *)a.y)[(size_t)tok * a.ystride + r] = qw_f2h(acc[j]);
                }
            }
    };
    if (qw_has_lut(F)) qw_lut_copy_issue(lut, (const u2 *)a.glut);
    if (XLDS) qw_stage_x_issue(xf, a.x, a.xstride, a.K, a.nb);
    qw_lds_arrive(); // both awaited once
    __syncthreads();
    const qw_afrag_lds afl = {xf, n};
    const qw_afrag_glb<false> afg = {n < a.nb ? a.x + (size_t)n * a.xstride : nullptr, nullptr};
    f4 acc = {0, 0, 0, 0};
    if (a.split > 1) {
        // Few tiles (the projections of one decode step): the chunks of a tile are cut over split waves of one
        // workgroup, so that a row is one memory round trip and not a chain of them; the partial sums are added in
        // part order through LDS. A group is 12 / split tiles; workgroup g takes groups g, g + gridDim.x, ...
        const uint32_t wave = qw_wave(), sp = a.split, tpg = (QW_WG_GU / 64) / sp, part = wave % sp, cpp = cpr / sp;
        const uint32_t ngroups = (a.ntiles + tpg - 1) / tpg;
        for (uint32_t g = blockIdx.x; g < ngroups; g += gridDim.x) {
            const uint32_t t = wave / sp < tpg ? g * tpg + wave / sp : a.ntiles; // waves past a whole number of tiles: none
            acc = f4{0, 0, 0, 0};
            if (t < a.ntiles)
                qw_task_pipeline<C>(1, 0, 1, cpp, CH * C::BLK_B, F == QW_F_PACKED ? lane : kl, [&](uint32_t) { return rowp(t) + (size_t)part * cpp * CH * C::BLK_B; },
                                    [&](uint32_t, uint32_t ci, const C &c) {
                                        if (XLDS) c.mac_lean(lut, afl, (part * cpp + ci) * CH * C::BLK_K, kg, acc);
                                        else c.mac_lean(lut, afg, (part * cpp + ci) * CH * C::BLK_K, kg, acc);
                                    });
            red[wave * 64 + lane] = acc;
            __syncthreads();
            if (part == 0 && t < a.ntiles) {
                f4 sum = red[wave * 64 + lane];
                for (uint32_t q = 1; q < sp; q++) sum += red[(wave + q) * 64 + lane];
                store(t, sum);
            }
            __syncthreads();
        }
        return;
    }
    qw_task_pipeline<C>(a.ntiles, w0, nw, cpr, CH * C::BLK_B, F == QW_F_PACKED ? lane : kl, rowp, [&](uint32_t t, uint32_t ci, const C &c) {
        if (XLDS) c.mac_lean(lut, afl, ci * CH * C::BLK_K, kg, acc);
        else c.mac_lean(lut, afg, ci * CH * C::BLK_K, kg, acc);
        if (ci + 1 != cpr) return;
        store(t, acc);
        acc = f4{0, 0, 0, 0};
    });
}
#define QW_QMV(F, CH, XLDS, SFX)                                                                        \
    extern "C" __global__ __launch_bounds__(QW_WG_GU) void qwk_qmv_f##F##SFX(qwk_qmv_args a) {             \
        __shared__ struct { u2 lut[qw_has_lut(F) ? QW_LUT_ENTRIES : 1]; u4 xf[XLDS ? QW_XF_MAXK * 2 : 1]; f4 red[QW_WG_GU]; } L; /* table first: LDS address 0 */ \
        qmv_body<F, CH, XLDS>(a, L.lut, L.xf, L.red);                                                   \
    }
#if QW_IN_PART(0)
QW_QMV(21, 2, true, _c2) QW_QMV(21, 1, true, _c1) QW_QMV(21, 1, false, _c1g)
QW_QMV(121, 2, true, _c2) QW_QMV(121, 1, true, _c1) // packed IQ3_S: a.rowbytes = bytes of a 16-row tile
#endif

// ---- the other formats, one to four matrices a launch (kernels/qmv_ggm.metal:232-262).
// split == 1: the 16-row tiles of all matrices form one list dealt round-robin to the waves of a persistent grid; a
// wave walks its tiles matrix by matrix, each with the decoder of that matrix's format.
// split > 1 (few tiles: the projections of one decode step): the K range of a tile is cut into split parts, one per
// wave, so that a row is one memory round trip instead of a chain of them; the waves of a tile sit in one workgroup
// and their partial sums are added in part order through LDS (the same order whatever else the launch holds).
#define QW_WG_QMVM 768 // 12 waves: a tile's K range is cut over 1, 2 or 4 of them
template <int F, int NB> struct qmvm_tile {
    typedef qw_chunk_kq<F, NB> C;
    const qwk_qmvm_args &a;
    uint32_t j;
    static constexpr bool TILED = F == QW_F_PACKED_Q6; // a tile-major copy: rowbytes = bytes of a tile, loads in matrix-core lane order
    __device__ __forceinline__ uint32_t kl() const { return TILED ? qw_lane() : qw_lane() & 3; }
    __device__ __forceinline__ const uint8_t *rowp(uint32_t t) const {
        if constexpr (TILED) return a.W[j] + (size_t)t * a.rowbytes[j];
        const uint32_t r = 16 * t + (qw_lane() >> 2);
        return a.W[j] + (size_t)(r < a.N[j] ? r : a.N[j] - 1) * a.rowbytes[j];
    }
    __device__ __forceinline__ void store(uint32_t t, const f4 &acc) const {
        const uint32_t lane = qw_lane(), r = 16 * t + (lane & 15), kg = lane >> 4;
        if (r >= a.N[j]) return;
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) {
            const uint32_t tok = 4 * kg + i;
            if (tok < a.nb) {
                if (a.yfloat) ((float *)a.y[j])[(size_t)tok * a.ystride[j] + r] = acc[i];
                else ((uint16_t *)a.y[j])[(size_t)tok * a.ystride[j] + r] = qw_f2h(acc[i]);
            }
        }
    }
};
template <int F, int NB> __device__ __forceinline__ void qmvm_matrix(const qwk_qmvm_args &a, uint32_t j, const uint32_t *tab, const qw_afrag_kq &af, uint32_t t0, uint32_t nw) {
    typedef qw_chunk_kq<F, NB> C;
    const qmvm_tile<F, NB> T = {a, j};
    const uint32_t lane = qw_lane(), kg = lane >> 4, cpr = a.K / (C::BLK_K * NB);
    f4 acc = {0, 0, 0, 0};
    qw_task_pipeline<C>(a.ntiles[j], t0, nw, cpr, NB * C::BLK_B, T.kl(), [&](uint32_t t) { return T.rowp(t); }, [&](uint32_t t, uint32_t ci, const C &c) {
        c.mac(tab, af, ci * NB * C::BLK_K, kg, acc);
        if (ci + 1 != cpr) return;
        T.store(t, acc);
        acc = f4{0, 0, 0, 0};
    });
}
// Workgroup g0, g0 + ng, ... takes the tile groups of matrix j; wave w does part
// w % split of tile w / split of the group (12 / split tiles a group).
template <int F, int NB> __device__ __forceinline__ void qmvm_matrix_split(const qwk_qmvm_args &a, uint32_t j, const uint32_t *tab, const qw_afrag_kq &af, f4 *red, uint32_t g0, uint32_t ng) {
    typedef qw_chunk_kq<F, NB> C;
    const qmvm_tile<F, NB> T = {a, j};
    const uint32_t lane = qw_lane(), kg = lane >> 4, wave = qw_wave(), sp = a.split, tpg = (QW_WG_QMVM / 64) / sp;
    const uint32_t cpp = a.K / (C::BLK_K * NB) / sp, part = wave % sp; // chunks per part
    const uint32_t ngroups = (a.ntiles[j] + tpg - 1) / tpg;
    for (uint32_t g = g0; g < ngroups; g += ng) {
        const uint32_t t = wave / sp < tpg ? g * tpg + wave / sp : a.ntiles[j]; // waves past a whole number of tiles: none
        f4 acc = {0, 0, 0, 0};
        if (t < a.ntiles[j])
            qw_task_pipeline<C>(1, 0, 1, cpp, NB * C::BLK_B, T.kl(), [&](uint32_t) { return T.rowp(t) + (size_t)part * cpp * NB * C::BLK_B; },
                                [&](uint32_t, uint32_t ci, const C &c) { c.mac(tab, af, (part * cpp + ci) * NB * C::BLK_K, kg, acc); });
        red[wave * 64 + lane] = acc;
        __syncthreads();
        if (part == 0 && t < a.ntiles[j]) {
            f4 sum = red[wave * 64 + lane];
            for (uint32_t q = 1; q < sp; q++) sum += red[(wave + q) * 64 + lane];
            T.store(t, sum);
        }
        __syncthreads();
    }
}
// One part of one tile: the product over chunks [part * cpp, (part + 1) * cpp) of the rows of tile t of matrix j.
template <int F, int NB> __device__ __forceinline__ f4 qmvm_part(const qwk_qmvm_args &a, uint32_t j, const uint32_t *tab, const qw_afrag_kq &af, uint32_t t, uint32_t part) {
    typedef qw_chunk_kq<F, NB> C;
    const qmvm_tile<F, NB> T = {a, j};
    const uint32_t lane = qw_lane(), kg = lane >> 4, cpp = a.K / (C::BLK_K * NB) / a.split;
    f4 acc = {0, 0, 0, 0};
    qw_task_pipeline<C>(1, 0, 1, cpp, NB * C::BLK_B, lane & 3, [&](uint32_t) { return T.rowp(t) + (size_t)part * cpp * NB * C::BLK_B; },
                        [&](uint32_t, uint32_t ci, const C &c) { c.mac(tab, af, (part * cpp + ci) * NB * C::BLK_K, kg, acc); });
    return acc;
}
// The shared expert's gate/up in the other format family with SwiGLU in the same launch (kernels/moe_gg.metal:563-573):
// matrix 0 holds the gate rows, matrix 1 the up rows, each of its own format. A workgroup takes 12 / split / 2 pairs of
// tiles (gate tile t and up tile t side by side), split waves a tile as in qwk_qmvm; the partial sums meet in LDS, and
// the first wave of a gate tile adds up both tiles in part order, applies SwiGLU and stores H's two planes.
// bid of nblk: the workgroup's number among those that do this work (the front launch puts the router's workgroups first).
struct qw_qmvm_lds { u4 xf[QW_KQ_MAXK * 2]; float xs[QW_KQ_MAXK / 2]; uint32_t tab[QW_KQ_TAB]; f4 red[QW_WG_QMVM]; };
__device__ __forceinline__ void qmvm_swiglu_body(const qwk_qmvm_args &a, qw_qmvm_lds &L, uint32_t bid, uint32_t nblk) {
    qw_kq_tab_build(L.tab);
    qw_stage_x(L.xf, a.x, a.xstride, a.K, a.nb);
    __syncthreads();
    if (a.sums) { // sums of 32 activations per token, in index order
        for (uint32_t i = threadIdx.x; i < (a.K >> 5) * 16; i += blockDim.x) {
            const uint32_t c = i >> 4, m = i & 15;
            float sum = 0;
#pragma unroll
            for (uint32_t f = 0; f < 4; f++) {
                const h8 v = __builtin_bit_cast(h8, L.xf[(4 * c + f) * 16 + m]);
#pragma unroll
                for (int e = 0; e < 8; e++) sum += (float)v[e];
            }
            L.xs[i] = sum;
        }
        __syncthreads();
    }
    const uint32_t lane = qw_lane(), n = lane & 15, kg = lane >> 4, wave = qw_wave(), sp = a.split;
    const qw_afrag_kq af = {L.xf, L.xs, n, kg};
    const uint32_t pairs = (QW_WG_QMVM / 64) / sp / 2, slot = wave / sp, part = wave % sp, which = slot & 1, ntiles = a.ntiles[0];
    const uint32_t ngroups = (ntiles + pairs - 1) / pairs;
    for (uint32_t g = bid; g < ngroups; g += nblk) {
        const uint32_t t = slot < 2 * pairs ? g * pairs + slot / 2 : ntiles; // waves past a whole number of pairs: none
        f4 acc = {0, 0, 0, 0};
        if (t < ntiles) {
            switch (a.fmt[which]) { // uniform in a wave
            case 12: acc = qmvm_part<12, 1>(a, which, L.tab, af, t, part); break;
            case 13: acc = qmvm_part<13, 1>(a, which, L.tab, af, t, part); break;
            case 14: acc = qmvm_part<14, 1>(a, which, L.tab, af, t, part); break;
            case 23: acc = qmvm_part<23, 1>(a, which, L.tab, af, t, part); break;
            case 20: acc = qmvm_part<20, 8>(a, which, L.tab, af, t, part); break;
            case 1: acc = qmvm_part<1, 8>(a, which, L.tab, af, t, part); break;
            case 30: acc = qmvm_part<30, 8>(a, which, L.tab, af, t, part); break;
            }
        }
        L.red[wave * 64 + lane] = acc;
        __syncthreads();
        if (part == 0 && which == 0 && t < ntiles) {
            f4 gate = L.red[wave * 64 + lane], up = L.red[(wave + sp) * 64 + lane];
            for (uint32_t q = 1; q < sp; q++) gate += L.red[(wave + q) * 64 + lane], up += L.red[(wave + sp + q) * 64 + lane];
            const uint32_t r = 16 * t + n;
            if (r < a.N[0])
#pragma unroll
                for (uint32_t j = 0; j < 4; j++) {
                    const uint32_t tok = 4 * kg + j;
                    if (tok < a.nb) {
                        const float gv = gate[j], h = gv / (1.0f + __expf(-gv)) * up[j];
                        const _Float16 hi = (_Float16)h, lo = (_Float16)(h - (float)hi);
                        const size_t o = ((size_t)tok * (a.topk + 1) + a.topk) * a.N[0] + r;
                        a.H[o] = __builtin_bit_cast(uint16_t, hi);
                        a.H[o + a.hplane] = __builtin_bit_cast(uint16_t, lo);
                    }
                }
        }
        __syncthreads();
    }
}
#if QW_IN_PART(0)
extern "C" __global__ __launch_bounds__(QW_WG_QMVM) void qwk_qmvm_swiglu(qwk_qmvm_args a) {
    __shared__ qw_qmvm_lds L;
    qmvm_swiglu_body(a, L, blockIdx.x, gridDim.x);
}
#endif

#if QW_IN_PART(0)
extern "C" __global__ __launch_bounds__(QW_WG_QMVM) void qwk_qmvm(qwk_qmvm_args a) {
    __shared__ struct { u4 xf[QW_KQ_MAXK * 2]; float xs[QW_KQ_MAXK / 2]; uint32_t tab[QW_KQ_TAB]; f4 red[QW_WG_QMVM]; } L;
    qw_kq_tab_build(L.tab);
    qw_stage_x(L.xf, a.x, a.xstride, a.K, a.nb);
    __syncthreads();
    if (a.sums) { // sums of 32 activations per token, in index order
        for (uint32_t i = threadIdx.x; i < (a.K >> 5) * 16; i += blockDim.x) {
            const uint32_t c = i >> 4, m = i & 15;
            float sum = 0;
#pragma unroll
            for (uint32_t f = 0; f < 4; f++) {
                const h8 v = __builtin_bit_cast(h8, L.xf[(4 * c + f) * 16 + m]);
#pragma unroll
                for (int e = 0; e < 8; e++) sum += (float)v[e];
            }
            L.xs[i] = sum;
        }
        __syncthreads();
    }
    const uint32_t lane = qw_lane(), nw = gridDim.x * (blockDim.x >> 6), w0 = qw_wave() * gridDim.x + blockIdx.x /* wave-major: see gu_body */;
    const qw_afrag_kq af = {L.xf, L.xs, lane & 15, lane >> 4};
    const bool k256 = a.K % 256 == 0;
    uint32_t toff = 0; // tiles (split == 1) or tile groups (split > 1) of the matrices before j
    for (uint32_t j = 0; j < a.nmat; j++) {
        if (a.split > 1) { // K is a multiple of 256 here
            const uint32_t ng = gridDim.x, g0 = (blockIdx.x + ng - toff % ng) % ng;
            switch (a.fmt[j]) {
            case 12: qmvm_matrix_split<12, 1>(a, j, L.tab, af, L.red, g0, ng); break;
            case 13: qmvm_matrix_split<13, 1>(a, j, L.tab, af, L.red, g0, ng); break;
            case 14: qmvm_matrix_split<14, 1>(a, j, L.tab, af, L.red, g0, ng); break;
            case QW_F_PACKED_Q6: qmvm_matrix_split<QW_F_PACKED_Q6, 1>(a, j, L.tab, af, L.red, g0, ng); break;
            case 23: qmvm_matrix_split<23, 1>(a, j, L.tab, af, L.red, g0, ng); break;
            case 20: qmvm_matrix_split<20, 8>(a, j, L.tab, af, L.red, g0, ng); break;
            case 1: qmvm_matrix_split<1, 8>(a, j, L.tab, af, L.red, g0, ng); break;
            case 30: qmvm_matrix_split<30, 8>(a, j, L.tab, af, L.red, g0, ng); break;
            }
            toff += (a.ntiles[j] + 12 / a.split - 1) / (12 / a.split);
            continue;
        }
        const uint32_t t0 = (w0 + nw - toff % nw) % nw; // first tile of matrix j that falls to this wave
        switch (a.fmt[j]) {
        case 12: qmvm_matrix<12, 1>(a, j, L.tab, af, t0, nw); break;
        case 13: qmvm_matrix<13, 1>(a, j, L.tab, af, t0, nw); break;
        case 14: qmvm_matrix<14, 1>(a, j, L.tab, af, t0, nw); break;
        case QW_F_PACKED_Q6: qmvm_matrix<QW_F_PACKED_Q6, 1>(a, j, L.tab, af, t0, nw); break;
        case 23: qmvm_matrix<23, 1>(a, j, L.tab, af, t0, nw); break;
        case 20: k256 ? qmvm_matrix<20, 8>(a, j, L.tab, af, t0, nw) : qmvm_matrix<20, 1>(a, j, L.tab, af, t0, nw); break;
        case 1: k256 ? qmvm_matrix<1, 8>(a, j, L.tab, af, t0, nw) : qmvm_matrix<1, 1>(a, j, L.tab, af, t0, nw); break;
        case 30: k256 ? qmvm_matrix<30, 8>(a, j, L.tab, af, t0, nw) : qmvm_matrix<30, 1>(a, j, L.tab, af, t0, nw); break;
        }
        toff += a.ntiles[j];
    }
}
#endif

// The VALU GEMV the matrix-core kernels are measured against (1, 2 or 4 activations, K a multiple of 512 up to 2560,
// packed IQ3_S): the same streaming and decoding, v_dot2_f32_f16 instead of the matrix instruction, and a sum over
// the four k-group lanes of a row by two cross-lane adds.
template <int NT> __device__ __forceinline__ void qmv_valu_body(const qwk_qmv_args &a, u2 *lut, u4 *xf) {
    typedef qw_chunk<QW_F_PACKED, 2> C;
    const uint32_t lane = qw_lane(), n = lane & 15, kg = lane >> 4;
    const uint32_t nw = gridDim.x * (blockDim.x >> 6), w0 = blockIdx.x * (blockDim.x >> 6) + qw_wave(), cpr = a.K / 512;
    float acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) acc[t] = 0;
    qw_task_pipeline<C>(a.ntiles, w0, nw, cpr, 2 * C::BLK_B, lane, [&](uint32_t t) { return a.W + (size_t)t * a.rowbytes; },
        [&](uint32_t t, uint32_t ci, const C &c) {
            c.template dot_valu<NT>(lut, xf, ci * 512, kg, acc);
            if (ci + 1 != cpr) return;
            const uint32_t r = 16 * t + n;
#pragma unroll
            for (int tk = 0; tk < NT; tk++) {
                float v = acc[tk];
                v += __shfl_xor(v, 16);
                v += __shfl_xor(v, 32);
                if (kg == 0 && r < a.N && (uint32_t)tk < a.nb) {
                    if (a.yfloat) ((float *)a.y)[(size_t)tk * a.ystride + r] = v;
                    else ((uint16_t *)a.y)[(size_t)tk * a.ystride + r] = qw_f2h(v);
                }
                acc[tk] = 0;
            }
        },
        [&] {
            qw_lut_copy(lut, (const u2 *)a.glut);
            qw_stage_x(xf, a.x, a.xstride, a.K, a.nb);
            __syncthreads();
        });
}
#define QW_QMV_VALU(NT)                                                                                  \
    extern "C" __global__ __launch_bounds__(QW_WG_GU) void qwk_qmv_valu_n##NT(qwk_qmv_args a) {          \
        __shared__ struct { u2 lut[QW_LUT_ENTRIES]; u4 xf[QW_XF_MAXK * 2]; } L;                          \
        qmv_valu_body<NT>(a, L.lut, L.xf);                                                               \
    }
#if QW_IN_PART(0)
QW_QMV_VALU(1) QW_QMV_VALU(2) QW_QMV_VALU(4)
QW_QMV(8, 16, true, _c16) QW_QMV(8, 1, true, _c1) QW_QMV(8, 1, false, _c1g)
#endif

// ================================================================ router (kernels/moe_gg.metal:25-41)
// logits[t][r] = Wr[r] . x[t] in binary32, one wave per row; a token's sum order does not depend on nb: explicit
// fused multiply-adds in index order per lane, then a fixed butterfly. WF: 1 = binary16 weights, 30 = bfloat16.
template <int WF, int NB> __device__ __forceinline__ void router_row(const qwk_router_args &a, uint32_t r, uint32_t lane) {
    const uint16_t *w = r < a.E ? a.Wr + (size_t)r * a.D : a.Wsg;
    float acc[NB];
#pragma unroll
    for (int t = 0; t < NB; t++) acc[t] = 0;
    for (uint32_t c = lane; c < a.D / 8; c += 64) {
        const u4 wv = *(const u4 *)(w + 8 * c);
        h8 xv[NB];
#pragma unroll
        for (int t = 0; t < NB; t++) xv[t] = *(const h8 *)(a.x + (size_t)((uint32_t)t < a.nb ? t : a.nb - 1) * a.D + 8 * c); // all loads first
        float wf[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            wf[2 * i] = WF == 30 ? qw_bf2f((uint16_t)wv[i]) : qw_h2f((uint16_t)wv[i]);
            wf[2 * i + 1] = WF == 30 ? qw_bf2f((uint16_t)(wv[i] >> 16)) : qw_h2f((uint16_t)(wv[i] >> 16));
        }
#pragma unroll
        for (int t = 0; t < NB; t++)
#pragma unroll
            for (int i = 0; i < 8; i++) acc[t] = __builtin_fmaf(wf[i], (float)xv[t][i], acc[t]);
    }
#pragma unroll
    for (int t = 0; t < NB; t++) {
        float v = acc[t];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
        if (lane == 0 && (uint32_t)t < a.nb) a.logits[(size_t)t * (a.E + 1) + r] = v;
    }
}
// The same arithmetic with the activations read from LDS (xs: binary16 [nb][D], copied there by the workgroup).
template <int WF, int NB> __device__ __forceinline__ void router_row_lds(const qwk_router_args &a, const uint16_t *xs, uint32_t r, uint32_t lane) {
    const uint16_t *w = r < a.E ? a.Wr + (size_t)r * a.D : a.Wsg;
    float acc[NB];
#pragma unroll
    for (int t = 0; t < NB; t++) acc[t] = 0;
    for (uint32_t c = lane; c < a.D / 8; c += 64) {
        const u4 wv = *(const u4 *)(w + 8 * c);
        float wf[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            wf[2 * i] = WF == 30 ? qw_bf2f((uint16_t)wv[i]) : qw_h2f((uint16_t)wv[i]);
            wf[2 * i + 1] = WF == 30 ? qw_bf2f((uint16_t)(wv[i] >> 16)) : qw_h2f((uint16_t)(wv[i] >> 16));
        }
#pragma unroll
        for (int t = 0; t < NB; t++) {
            const h8 xv = *(const h8 *)(xs + (size_t)((uint32_t)t < a.nb ? t : a.nb - 1) * a.D + 8 * c);
#pragma unroll
            for (int i = 0; i < 8; i++) acc[t] = __builtin_fmaf(wf[i], (float)xv[i], acc[t]);
        }
    }
#pragma unroll
    for (int t = 0; t < NB; t++) {
        float v = acc[t];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
        if (lane == 0 && (uint32_t)t < a.nb) a.logits[(size_t)t * (a.E + 1) + r] = v;
    }
}
template <int WF> __device__ __forceinline__ void router_rows_lds(const qwk_router_args &a, const uint16_t *xs, uint32_t r, uint32_t lane) {
    if (r > a.E) return;
    if (a.nb <= 1) router_row_lds<WF, 1>(a, xs, r, lane);
    else if (a.nb <= 2) router_row_lds<WF, 2>(a, xs, r, lane);
    else if (a.nb <= 4) router_row_lds<WF, 4>(a, xs, r, lane);
    else if (a.nb <= 8) router_row_lds<WF, 8>(a, xs, r, lane);
    else router_row_lds<WF, 16>(a, xs, r, lane);
}

template <int WF> __device__ __forceinline__ void router_rows(const qwk_router_args &a, uint32_t r, uint32_t lane) {
    if (r > a.E) return;
    if (a.nb <= 1) router_row<WF, 1>(a, r, lane);
    else if (a.nb <= 2) router_row<WF, 2>(a, r, lane);
    else if (a.nb <= 4) router_row<WF, 4>(a, r, lane);
    else if (a.nb <= 8) router_row<WF, 8>(a, r, lane);
    else router_row<WF, 16>(a, r, lane);
}
#if QW_IN_PART(0)
extern "C" __global__ __launch_bounds__(256) void qwk_router_w1(qwk_router_args a) { router_rows<1>(a, blockIdx.x * 4 + qw_wave(), qw_lane()); }
extern "C" __global__ __launch_bounds__(256) void qwk_router_w30(qwk_router_args a) { router_rows<30>(a, blockIdx.x * 4 + qw_wave(), qw_lane()); }
#endif

// ================================================================ selection + dedupe (kernels/moe_gg.metal:123-189)
// Per token (one wave): top-k by repeated maximum with ties to the lowest expert index, softmax over the picked logits
// in rank order, sigmoid of the shared-expert logit; then the nbr * topk picks are deduplicated in order of first
// appearance over the flat index. The unique list, masks and slots are assembled in LDS (qw_sel_cache: a weight kernel
// that makes the selection itself reads them from there) and written to global memory in one pass at the end.
struct qw_sel_cache { // the part of the selection record a weight kernel needs, in LDS
    uint32_t U, ue[256], mask[256];
    uint8_t slot[256 * 16];
    uint32_t qnext; // the workgroup's tile queue (gu_tasks): how many of its tiles have been handed out
};
struct qw_sel_scratch {
    uint32_t ids[256], lead[8], first[1024];
    float w[16 * 17];
};

// PER = E / 64 values per lane, lane l holding experts l * PER .. l * PER + PER - 1 (lowest lane = lowest index).
// T tokens at once (tok0, tok0 + tstep, ...; those >= nbr are skipped): a round is a chain of dependent instructions,
// so two tokens in flight cost about the time of one. Every lane keeps the maximum of its PER keys and the position
// of that maximum; a round takes the wave maximum of those, the lowest lane that holds it, and only that lane
// recomputes its own maximum.
template <int PER, int T>
__device__ __forceinline__ void select_tokens(const float *logits, uint32_t E, uint32_t K, uint32_t tok0, uint32_t tstep, uint32_t nbr, float *w, uint32_t *ids, uint32_t lane) {
    uint32_t k[T][PER], bk[T], bj[T], pk[T];
    bool on[T];
#pragma unroll
    for (int t = 0; t < T; t++) {
        const uint32_t tok = tok0 + t * tstep;
        on[t] = tok < nbr;
        const float *lg = logits + (size_t)(on[t] ? tok : tok0) * (E + 1);
#pragma unroll
        for (int j = 0; j < PER; j++) k[t][j] = qw_fkey(lg[lane * PER + j]);
        pk[t] = 0;
    }
    auto local_max = [&](int t) { // among equals the lower position wins
        bk[t] = k[t][0], bj[t] = 0;
#pragma unroll
        for (int j = 1; j < PER; j++)
            if (k[t][j] > bk[t]) bk[t] = k[t][j], bj[t] = j;
    };
#pragma unroll
    for (int t = 0; t < T; t++) local_max(t);
    for (uint32_t r = 0; r < K; r++) {
#pragma unroll
        for (int t = 0; t < T; t++) {
            const uint32_t m = qw_wave_max_u32(bk[t]);
            const uint32_t L = (uint32_t)__builtin_ctzll(__ballot(bk[t] == m)); // lowest lane among equals
            const uint32_t j = (uint32_t)__builtin_amdgcn_readlane((int)bj[t], (int)L);
            if (lane == 0 && on[t]) ids[(tok0 + t * tstep) * K + r] = L * PER + j;
            if (lane == r) pk[t] = m;
            if (lane == L) {
#pragma unroll
                for (int jj = 0; jj < PER; jj++)
                    if ((uint32_t)jj == j) k[t][jj] = 0; // below every key, -inf included
                local_max(t);
            }
        }
    }
#pragma unroll
    for (int t = 0; t < T; t++) {
        const uint32_t tok = tok0 + t * tstep;
        const float p = qw_fkey_inv(pk[t]), mx = __shfl(p, 0), ex = __expf(p - mx);
        float sm = 0;
        for (uint32_t r = 0; r < K; r++) sm += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ex), (int)r)); // rank order
        if (!on[t]) continue;
        if (lane < K) w[tok * (K + 1) + lane] = ex / sm;
        if (lane == K) w[tok * (K + 1) + K] = 1.0f / (1.0f + __expf(-logits[(size_t)tok * (E + 1) + E]));
    }
}

// The same result without the chain of K dependent wave-wide maxima. Lane l holds experts l, l + 64, ... here (which lane
// holds a key does not matter to this form, and a wave's load is then 256 contiguous bytes). Every lane finds the maximum of its PER keys;
// a value T0 that at least K of the 64 lane maxima reach bounds the answer from below: at least K keys are >= T0, so
// no key below T0 can be picked. The keys >= T0 (K of them, or a few more) are gathered one to a lane, each is ranked among
// them by (key descending, expert ascending) - the order of the repeated maximum with ties to the lowest index - and
// the ranks below K are the picks. T tokens go through together (the steps are chains of LDS and cross-lane
// latencies, so a second token costs little). Returns a bit per token that was NOT done, with nothing written for
// it: more than 64 keys reach T0 (many equal logits) and the caller falls back to select_tokens.
// ws: 144 dwords of LDS scratch per token for this wave. need_w: also the gating weights (softmax over the picked
// logits in rank order, sigmoid of the shared-expert logit).
// issued(): called once the loads of the logits are issued (work that needs no memory: with loads straight into LDS
// outstanding beside them the compiler would wait for everything at the first use of a key).
template <int PER, int T, class H>
__device__ __forceinline__ uint32_t select_tokens_ranked(const float *logits, uint32_t E, uint32_t K, const uint32_t (&tok)[T], const bool (&on)[T], float *w, uint32_t *ids, uint32_t *ws,
                                                        uint32_t lane, bool need_w, H issued) {
    uint32_t k[T][PER], M[T], T0[T], c[T], pos[T][PER];
#pragma unroll
    for (int t = 0; t < T; t++)
#pragma unroll
        for (int j = 0; j < PER; j++) k[t][j] = __builtin_bit_cast(uint32_t, logits[(size_t)tok[t] * (E + 1) + j * 64 + lane]); // (a wave reads 256 contiguous bytes)
    QW_DSTAMP(12);
    QW_SSTAMP(3);
    issued();
    QW_DSTAMP(13);
    QW_SSTAMP(4);
#pragma unroll
    for (int t = 0; t < T; t++) {
        M[t] = 0;
#pragma unroll
        for (int j = 0; j < PER; j++) k[t][j] = qw_fkey(__builtin_bit_cast(float, k[t][j])), M[t] = max(M[t], k[t][j]);
        T0[t] = 0;
    }
    QW_SDEP(M[T - 1]);
    QW_SSTAMP(5);
    // T0: the largest value with bits [lo, 32) such that at least K lane maxima reach it, found bit by bit with a
    // ballot each (scalar work but for the comparison). The upper 16 bits are nearly always enough to leave at most
    // 64 keys; otherwise the lower 16 follow, which makes T0 the K-th largest lane maximum itself.
    // (the tokens of `which` side by side: a step is a chain of vector compare -> scalar count -> scalar select)
    auto refine = [&](uint32_t which, int hi, int lo) {
        for (int b = hi; b >= lo; b--)
#pragma unroll
            for (int t = 0; t < T; t++) {
                const uint32_t cd = T0[t] | (1u << b);
                if (((which >> t) & 1) && (uint32_t)__popcll(__ballot(M[t] >= cd)) >= K) T0[t] = cd;
            }
    };
    // gather the keys >= T0: position = candidates of earlier j, plus those of lower lanes at this j
    auto gather = [&](int t) {
        c[t] = 0;
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const unsigned long long bal = __ballot(k[t][j] >= T0[t]);
            pos[t][j] = c[t] + __builtin_amdgcn_mbcnt_hi((uint32_t)(bal >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)bal, 0));
            c[t] += (uint32_t)__popcll(bal);
        }
    };
    uint32_t fail = 0, more = 0;
    refine((1u << T) - 1, 31, 16);
#pragma unroll
    for (int t = 0; t < T; t++) {
        gather(t);
        if (c[t] > 64) more |= 1u << t;
    }
    if (more) refine(more, 15, 0);
#pragma unroll
    for (int t = 0; t < T; t++) {
        if ((more >> t) & 1) gather(t);
        if (c[t] > 64 || !on[t]) fail |= 1u << t;
    }
    QW_SDEP(pos[T - 1][PER - 1]);
    QW_SSTAMP(6);
#pragma unroll
    for (int t = 0; t < T; t++) {
        if ((fail >> t) & 1) continue;
        u2 *cand = (u2 *)(ws + 144 * t); // (key, expert) of candidate p
#pragma unroll
        for (int j = 0; j < PER; j++)
            if (k[t][j] >= T0[t]) cand[pos[t][j]] = u2{k[t][j], j * 64 + lane};
    }
    uint32_t mk[T], me[T], rank[T];
#pragma unroll
    for (int t = 0; t < T; t++) {
        const u2 mine = ((const u2 *)(ws + 144 * t))[lane];
        // one 64-bit value per candidate whose order is the ranking order; lanes without a candidate hold the least
        mk[t] = lane < c[t] ? mine.x : 0, me[t] = lane < c[t] ? ~mine.y : 0;
        rank[t] = 0;
    }
    QW_SDEP(mk[T - 1]);
    QW_SSTAMP(7);
    // (all tokens against candidate lane l in one step; lanes past a token's own count hold the least value and add nothing)
    uint32_t cm = 0;
#pragma unroll
    for (int t = 0; t < T; t++)
        if (!((fail >> t) & 1)) cm = max(cm, c[t]);
    for (uint32_t q0 = 0; q0 < cm; q0 += 16) // candidates sixteen at a time, read from their lanes
#pragma unroll
        for (uint32_t q = 0; q < 16; q++) {
            if (q >= 8 && q0 + q >= cm) break; // uniform: ten to twelve candidates are the common case
            const uint32_t l = q0 ? (q0 + q) & 63 : q;
#pragma unroll
            for (int t = 0; t < T; t++) {
                const unsigned long long mine = (unsigned long long)mk[t] << 32 | me[t];
                const unsigned long long o = (unsigned long long)(uint32_t)__builtin_amdgcn_readlane((int)mk[t], (int)l) << 32 | (uint32_t)__builtin_amdgcn_readlane((int)me[t], (int)l);
                rank[t] += o > mine;
            }
        }
#pragma unroll
    for (int t = 0; t < T; t++) {
        if ((fail >> t) & 1) continue;
        uint32_t *pkr = ws + 144 * t + 128; // key of rank r
        if (lane < c[t] && rank[t] < K) {
            ids[tok[t] * K + rank[t]] = ~me[t];
            pkr[rank[t]] = mk[t];
        }
    }
    QW_SDEP(rank[T - 1]);
    QW_SSTAMP(8);
    if (!need_w) return fail; // the gating weights are only wanted by the workgroup that writes the record
#pragma unroll
    for (int t = 0; t < T; t++) {
        if ((fail >> t) & 1) continue;
        const float p = qw_fkey_inv(ws[144 * t + 128 + (lane < K ? lane : 0)]);
        const float mx = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, p), 0)), ex = __expf(p - mx);
        float sm = 0;
        for (uint32_t r = 0; r < K; r++) sm += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ex), (int)r)); // rank order
        if (lane < K) w[tok[t] * (K + 1) + lane] = ex / sm;
        if (lane == K) w[tok[t] * (K + 1) + K] = 1.0f / (1.0f + __expf(-logits[(size_t)tok[t] * (E + 1) + E]));
    }
    return fail;
}

// Any E <= 1024: the values live in LDS (v, E floats); lane l scans experts l, l + 64, ...
__device__ __forceinline__ void select_token_any(const float *lg, float *v, uint32_t E, uint32_t K, uint32_t tok, float *w, uint32_t *ids, uint32_t lane) {
    for (uint32_t e = lane; e < E; e += 64) v[e] = lg[e];
    float pk = 0;
    for (uint32_t r = 0; r < K; r++) {
        float bv = -INFINITY;
        uint32_t bi = 0xffffffffu;
        for (uint32_t e = lane; e < E; e += 64) {
            const float x = v[e];
            if (x > bv || bi == 0xffffffffu) { bv = x; bi = e; }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o);
            const uint32_t oi = __shfl_xor(bi, o);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        if (lane == 0) ids[tok * K + r] = bi;
        if (lane == r) pk = bv;
        if ((bi & 63) == lane) v[bi] = -INFINITY; // only the owning lane ever reads this element again
    }
    const float mx = __shfl(pk, 0), ex = __expf(pk - mx);
    float sm = 0;
    for (uint32_t r = 0; r < K; r++) sm += __shfl(ex, r);
    if (lane < K) w[tok * (K + 1) + lane] = ex / sm;
    if (lane == K) w[tok * (K + 1) + K] = 1.0f / (1.0f + __expf(-lg[E]));
}

__device__ __forceinline__ bool qw_select_fast_e(uint32_t E) { return E == 64 || E == 128 || E == 256 || E == 512 || E == 1024; }

// The whole selection by one workgroup (a multiple of 64 threads, at least nbr * topk of them). lgs: LDS scratch, 1024
// floats per wave (288 are used when E is 64 * {1, 2, 4, 8, 16}). c is complete for every thread on return.
// store: this workgroup writes the record; need_w: it wants the gating weights in s.w (store implies it).
// NSTAGE: the workgroup's last NSTAGE waves take no tokens; each of them runs stage(part, NSTAGE) instead, the caller's
// copies into LDS (table, activations). A wave that asks for 128 KB of such copies sits in the issue of those loads for
// 2 to 3 us - the copies go at the rate of the unit's path into LDS - so a wave that did both made its keys that much
// later; the waves with tokens ask for nothing but their logits.
template <uint32_t NSTAGE = 0, class H>
__device__ __forceinline__ void select_all(const qwk_select_args &a, qw_sel_scratch &s, qw_sel_cache &c, float *lgs, bool store, H stage, bool need_w = false) {
    need_w = need_w || store;
    const uint32_t tid = threadIdx.x, nth = blockDim.x, wave = qw_wave(), lane = qw_lane(), nwv = nth >> 6;
    const uint32_t E = a.E, K = a.topk, gnb = a.gnb, GU = gnb * K, UM = a.nbr * K;
    const bool fast = qw_select_fast_e(E);
    const uint32_t tw = nwv - NSTAGE; // the waves that take tokens
    QW_SDEP(E + K + gnb + a.nbr);
    QW_SSTAMP(1);
    // nothing the token loop writes is cleared here (rows of w past the batch only), so no barrier separates the two,
    // and a wave clears its part once it has asked for what it reads
    auto clear = [&] {
        for (uint32_t i = tid; i < E; i += nth) s.first[i] = 0xffffffffu;
        for (uint32_t i = tid; i < GU; i += nth) c.ue[i] = 0, c.mask[i] = 0;
        for (uint32_t i = tid; i < GU * gnb / 4; i += nth) ((uint32_t *)c.slot)[i] = 0;
        if (tid < 8) s.lead[tid] = 0;
        for (uint32_t i = a.nbr * (K + 1) + tid; i < gnb * (K + 1); i += nth) s.w[i] = 0;
        QW_DSTAMP(11);
        QW_SSTAMP(2);
    };
    if (NSTAGE != 0 && wave >= tw) { // (uniform)
        stage(wave - tw, NSTAGE);
        QW_SSTAMP(4);
        clear();
    } else if (fast) { // a wave takes one token, or two when there are more tokens than such waves (lgs gives a wave 288 dwords)
        uint32_t *ws = (uint32_t *)lgs + 288 * wave;
        const uint32_t trot = a.nbr ? blockIdx.x % a.nbr : 0; // the workgroups of a launch read the tokens' logits in different orders
        auto rot = [&](uint32_t tt) { return tt + trot < a.nbr ? tt + trot : tt + trot - a.nbr; };
        const bool pairs = E <= 512; // sixteen keys a lane: one token at a time (registers)
        auto slow = [&](uint32_t tok) { // the repeated maximum
            switch (E) {
            case 64: select_tokens<1, 1>(a.logits, E, K, tok, nwv, a.nbr, s.w, s.ids, lane); break;
            case 128: select_tokens<2, 1>(a.logits, E, K, tok, nwv, a.nbr, s.w, s.ids, lane); break;
            case 256: select_tokens<4, 1>(a.logits, E, K, tok, nwv, a.nbr, s.w, s.ids, lane); break;
            case 512: select_tokens<8, 1>(a.logits, E, K, tok, nwv, a.nbr, s.w, s.ids, lane); break;
            default: select_tokens<16, 1>(a.logits, E, K, tok, nwv, a.nbr, s.w, s.ids, lane); break;
            }
        };
        if (wave < a.nbr) {
            const uint32_t tt = wave;
            const bool two = pairs && tt + tw < a.nbr;
            const uint32_t tk[2] = {rot(tt), two ? rot(tt + tw) : rot(tt)};
            const bool on2[2] = {true, two}, on1[1] = {true};
            const uint32_t t1[1] = {tk[0]};
            uint32_t fail;
            switch (E) {
            case 64: fail = two ? select_tokens_ranked<1, 2>(a.logits, E, K, tk, on2, s.w, s.ids, ws, lane, need_w, clear) : select_tokens_ranked<1, 1>(a.logits, E, K, t1, on1, s.w, s.ids, ws, lane, need_w, clear); break;
            case 128: fail = two ? select_tokens_ranked<2, 2>(a.logits, E, K, tk, on2, s.w, s.ids, ws, lane, need_w, clear) : select_tokens_ranked<2, 1>(a.logits, E, K, t1, on1, s.w, s.ids, ws, lane, need_w, clear); break;
            case 256: fail = two ? select_tokens_ranked<4, 2>(a.logits, E, K, tk, on2, s.w, s.ids, ws, lane, need_w, clear) : select_tokens_ranked<4, 1>(a.logits, E, K, t1, on1, s.w, s.ids, ws, lane, need_w, clear); break;
            case 512: fail = two ? select_tokens_ranked<8, 2>(a.logits, E, K, tk, on2, s.w, s.ids, ws, lane, need_w, clear) : select_tokens_ranked<8, 1>(a.logits, E, K, t1, on1, s.w, s.ids, ws, lane, need_w, clear); break;
            default: fail = select_tokens_ranked<16, 1>(a.logits, E, K, t1, on1, s.w, s.ids, ws, lane, need_w, clear); break;
            }
            for (uint32_t i = 0; i < 2; i++) // more than 64 keys tie at the bound
                if (((fail >> i) & 1) && (i == 0 || two)) slow(tk[i]);
        } else clear();
        // tokens that the first pass does not reach (more than such waves when a lane holds sixteen keys, more than twice as many otherwise)
        for (uint32_t tt = wave + (pairs ? 2 : 1) * tw; tt < a.nbr; tt += tw) {
            const uint32_t t1[1] = {rot(tt)};
            const bool on1[1] = {true};
            if (pairs || select_tokens_ranked<16, 1>(a.logits, E, K, t1, on1, s.w, s.ids, ws, lane, need_w, [] {})) slow(t1[0]);
        }
    } else {
        clear();
        for (uint32_t t = wave; t < a.nbr; t += tw) select_token_any(a.logits + (size_t)t * (E + 1), lgs + (size_t)wave * 1024, E, K, t, s.w, s.ids, lane);
    }
    QW_DSTAMP(15);
    QW_SSTAMP(9);
    __syncthreads();
    QW_SSTAMP(10);
    if (a.nbr == 1) { // one token: its picks are the unique experts, in rank order (what the steps below would leave)
        if (tid < K) c.ue[tid] = s.ids[tid], c.mask[tid] = 1, c.slot[tid * gnb] = (uint8_t)tid;
        if (tid == 0) c.U = K;
        __syncthreads();
    } else {
    if (tid < UM) atomicMin(&s.first[s.ids[tid]], tid); // first flat index of every picked expert
    __syncthreads();
    QW_SSTAMP(11);
    // lead = this pair is its expert's first; every wave leaves the ballot of its leads (UM <= 256: four waves)
    uint32_t f = 0;
    bool lead = false;
    if (tid < UM) {
        f = s.first[s.ids[tid]];
        lead = f == tid;
    }
    if (wave < 4) { // a wave index is uniform, so the ballot is taken by whole waves
        const unsigned long long bal = __ballot(lead);
        if (lane == 0) s.lead[2 * wave] = (uint32_t)bal, s.lead[2 * wave + 1] = (uint32_t)(bal >> 32);
    }
    __syncthreads();
    QW_SSTAMP(12);
    // unique index of a pair = number of leads before its expert's first pair
    if (tid < UM) {
        uint32_t u = 0;
        for (uint32_t w = 0; w < (f >> 6); w++) u += __popc(s.lead[2 * w]) + __popc(s.lead[2 * w + 1]);
        const unsigned long long m = ((unsigned long long)s.lead[2 * (f >> 6) + 1] << 32 | s.lead[2 * (f >> 6)]) & ((1ull << (f & 63)) - 1);
        u += __popcll(m);
        const uint32_t t = tid / K;
        atomicOr(&c.mask[u], 1u << t);
        c.slot[u * gnb + t] = (uint8_t)(tid % K);
        if (lead) c.ue[u] = s.ids[tid];
    }
    if (tid == 0) {
        uint32_t U = 0;
        for (uint32_t w = 0; w < 8; w++) U += __popc(s.lead[w]);
        c.U = U;
    }
    __syncthreads();
    }
    QW_SSTAMP(13);
    if (!store) return;
    // the record, in one pass of dword stores: U | ue[GU] | mask[GU] | slot[GU][gnb] | w[gnb][K + 1]
    uint32_t *out = (uint32_t *)a.sel;
    const uint32_t n_slot = GU * gnb / 4, n_w = gnb * (K + 1), total = 1 + 2 * GU + n_slot + n_w;
    for (uint32_t i = tid; i < total; i += nth) {
        uint32_t v;
        if (i == 0) v = c.U;
        else if (i < 1 + GU) v = c.ue[i - 1];
        else if (i < 1 + 2 * GU) v = c.mask[i - 1 - GU];
        else if (i < 1 + 2 * GU + n_slot) v = ((const uint32_t *)c.slot)[i - 1 - 2 * GU];
        else v = __builtin_bit_cast(uint32_t, s.w[i - 1 - 2 * GU - n_slot]);
        out[i] = v;
    }
    __syncthreads(); // the caller may reuse the scratch
}

#if QW_IN_PART(0)
extern "C" __global__ __launch_bounds__(1024) void qwk_select(qwk_select_args a) {
    __shared__ qw_sel_scratch s;
    __shared__ qw_sel_cache c;
    __shared__ float lgs[16 * 1024];
    select_all(a, s, c, lgs, true, [](uint32_t, uint32_t) {});
}
#endif

// ================================================================ gate/up + SwiGLU (kernels/moe_gg.metal:428-447, 563-573, 600-631)
// A tile holds gate rows j0..j0+7 (n < 8) and up rows j0..j0+7 (n >= 8) of one expert; the up results move over by
// 8 lanes, and H = g / (1 + exp(-g)) * up is stored as binary16 hi + lo planes for the tokens that picked the expert.
__device__ __forceinline__ void qw_sel_load(qw_sel_cache &c, const uint8_t *sel, uint32_t K, uint32_t gnb) {
    const uint32_t GU = gnb * K;
    const uint32_t *ue = (const uint32_t *)(sel + QW_SEL_OFF_UE(gnb, K)), *mask = (const uint32_t *)(sel + QW_SEL_OFF_MASK(gnb, K));
    const uint32_t *slot = (const uint32_t *)(sel + QW_SEL_OFF_SLOT(gnb, K));
    for (uint32_t i = threadIdx.x; i < GU; i += blockDim.x) c.ue[i] = ue[i], c.mask[i] = mask[i];
    for (uint32_t i = threadIdx.x; i < GU * gnb / 4; i += blockDim.x) ((uint32_t *)c.slot)[i] = slot[i];
    if (threadIdx.x == 0) c.U = *(const uint32_t *)sel;
}

// Where the SwiGLU values of a tile go. The plain form: the two planes of H in global memory, for a later launch.
struct qw_h_global {
    uint16_t *H;
    uint32_t hplane;
    // a tile is done: m = the tokens that picked its expert (wave-uniform)
    __device__ __forceinline__ void tile(uint32_t) const {}
    __device__ __forceinline__ void stamp(uint32_t k) const { QW_DSTAMP(k); }
    // column j0 + n of (token, slot): o = its offset in a plane
    __device__ __forceinline__ void put(uint32_t, uint32_t, size_t o, uint16_t hi, uint16_t lo) const {
        // (stores the compiler does not track: nothing in this kernel may read H back from memory)
        qw_store_u16(H + o, hi);
        qw_store_u16(H + o + hplane, lo);
    }
};
// QUEUE: the workgroup's tiles (blockIdx.x, blockIdx.x + gridDim.x, ...) go to its waves from the counter sc->qnext, which
// the caller has set to the number of waves before a barrier (wave w starts with the w-th of them); else wave w0 of nw takes
// tiles w0, w0 + nw, ...
template <int F, int CH, bool QUEUE, class S, class HS>
__device__ __forceinline__ void gu_tasks(const qwk_gu_args &a, const u2 *lut, const u4 *xf, qw_sel_cache *sc, uint32_t w0, uint32_t nw, S ready, HS &hs) {
    typedef qw_chunk<F, CH> C;
    const uint32_t lane = qw_lane(), n = lane & 15, kg = lane >> 4, K = a.topk, gnb = a.gnb;
    const uint32_t U = a.shared ? 1 : sc->U, tpe = a.I / 8, ntasks = U * tpe;
    const uint32_t cpr = a.D / (C::BLK_K * CH);
    const qw_afrag_lds af = {xf, n};
    const uint32_t nl = lane >> 2; // (row, k-group) this lane loads from GGUF rows: (lane >> 2, lane & 3)
    auto rowp = [&](uint32_t task) {
        const uint32_t u = task / tpe, e = a.shared ? 0 : (uint32_t)__builtin_amdgcn_readfirstlane((int)sc->ue[u]); // (wave-uniform: the row base stays in scalar registers)
        if constexpr (F == QW_F_PACKED || F == QW_F_ABLATE) return a.Wg + ((size_t)e * tpe + task % tpe) * a.rowbytes; // the tile's slabs; rowbytes = bytes of a tile
        else return (nl < 8 ? a.Wg : a.Wu) + ((size_t)e * a.I + 8 * (task % tpe) + (nl & 7)) * a.rowbytes;
    };
    f4 acc = {0, 0, 0, 0};
    auto use = [&](uint32_t task, uint32_t ci, const C &c) {
        c.mac_lean(lut, af, ci * CH * C::BLK_K, kg, acc);
        if (ci + 1 != cpr) return;
        const uint32_t u = task / tpe, j0 = 8 * (task % tpe);
        const uint32_t m = (a.shared ? 0xffffffffu : sc->mask[u]) & qw_all_tokens(a.nbr);
        hs.tile(m);
#pragma unroll
        for (uint32_t j = 0; j < 4; j++) {
            const float up = __shfl_xor(acc[j], 8), g = acc[j];
            const uint32_t tok = 4 * kg + j;
            if (n < 8 && ((m >> tok) & 1)) {
                const uint32_t s = a.shared ? K : sc->slot[u * gnb + tok];
                const float h = g / (1.0f + __expf(-g)) * up;
                const _Float16 hi = (_Float16)h, lo = (_Float16)(h - (float)hi);
                const size_t o = ((size_t)tok * (K + 1) + s) * a.I + j0 + n;
                hs.put(m, tok, o, __builtin_bit_cast(uint16_t, hi), __builtin_bit_cast(uint16_t, lo));
            }
        }
        acc = f4{0, 0, 0, 0};
    };
    const uint32_t kl = F == QW_F_PACKED || F == QW_F_ABLATE ? lane : lane & 3;
    const uint8_t *spare = qw_has_lut(F) ? (const uint8_t *)a.glut : nullptr;
    if constexpr (QUEUE) {
        auto next = [&]() -> uint32_t {
            uint32_t j = 0;
            if (lane == 0) j = atomicAdd(&sc->qnext, 1u);
            // (a workgroup's tiles lie gridDim.x tiles apart: neighbouring tiles on one compute unit measured slower, 38.4 -> 40.3 us)
            return blockIdx.x + gridDim.x * (uint32_t)__builtin_amdgcn_readfirstlane((int)j);
        };
        qw_task_queue<C>(ntasks, blockIdx.x + gridDim.x * qw_wave(), next, cpr, CH * C::BLK_B, kl, rowp, use, ready, spare);
    } else qw_task_stream<C>(ntasks, w0, nw, cpr, CH * C::BLK_B, kl, rowp, use, ready, spare);
}

// FGU: routed gate/up format; FSG: shared gate/up format done by the same launch (0 = none).
// Order of the set-up when the record is given: the record first (one memory round trip, one barrier: the row
// addresses depend on it); then every wave issues its first weight loads, and only then the table copy, the activation
// staging and the second barrier follow, overlapping that first round trip to HBM. When the selection is made here,
// the table and the activations are fetched under it instead (direct global-to-LDS loads: no registers are held).
// hs: where the SwiGLU values go (qw_h_global, or the fused launch's LDS buffer). all_w: every workgroup wants the gating
// weights in ss->w, not only the one that writes the record. selected(): called by every thread once the selection
// cache *sc (and ss->w) is complete and published, before any tile is taken; ss may be reused after a barrier of its own.
template <int FGU, int CHGU, int FSG, int CHSG, class HS, class SEL>
__device__ __forceinline__ void gu_body(const qwk_gu_args &a, u2 *lut, u4 *xf, qw_sel_cache *sc, qw_sel_scratch *ss, HS &hs, bool all_w, SEL selected) {
    bool staged = false, tabled = false;
    if (threadIdx.x == 0) sc->qnext = blockDim.x >> 6; // (nothing below writes it; a barrier follows on every path)
    if (threadIdx.x == 0) QW_WSTAMP(12);
    QW_DSTAMP(0);
    QW_SSTAMP(0);
    if constexpr (FGU == QW_F_RT) qw_kq_tab_build((uint32_t *)(lut + (qw_has_lut(FSG) ? QW_LUT_ENTRIES : 0))); // (published by the barriers below)
    if (a.logits) { // the selection, made here by every workgroup
        const qwk_select_args sa = {a.logits, const_cast<uint8_t *>(a.sel), a.nbr, a.E, a.topk, a.gnb};
        if (qw_select_fast_e(a.E)) {
            // The selection's scratch lies behind the staged activations when D leaves room there (D <= 2048), else in
            // their place (they follow in ready()).
            constexpr bool lutp = qw_has_lut(FGU) || qw_has_lut(FSG);
            const bool early = a.D * 2 + (QW_WG_GU / 64) * 288 / 4 <= QW_XF_MAXK * 2;
            // (four of the twelve waves ask for the table and the activations, the others make the selection meanwhile)
            select_all<4>(sa, *ss, *sc, (float *)(early ? xf + a.D * 2 : xf), blockIdx.x == 0, [&](uint32_t part, uint32_t nparts) {
                if (lutp) qw_lut_copy_issue(lut, (const u2 *)a.glut, part, nparts);
                if (early) qw_stage_x_issue(xf, a.x, a.D, a.D, a.nbr, part, nparts);
            }, all_w);
            qw_lds_arrive();
            __syncthreads();
            QW_SSTAMP(14);
            staged = early;
            tabled = true;
        } else { // other expert counts need 1024 floats of scratch per wave: everything lies where x is staged afterwards
            qw_sel_scratch &so = *(qw_sel_scratch *)xf;
            select_all(sa, so, *sc, (float *)(xf + (sizeof(qw_sel_scratch) + 15) / 16), blockIdx.x == 0, [](uint32_t, uint32_t) {}, all_w);
            if (all_w) { // (the caller reads the weights from ss)
                for (uint32_t i = threadIdx.x; i < a.gnb * (a.topk + 1); i += blockDim.x) ss->w[i] = so.w[i];
                __syncthreads();
            }
        }
    } else {
        if (!a.shared) qw_sel_load(*sc, a.sel, a.topk, a.gnb);
        if (all_w) {
            const float *wg = (const float *)(a.sel + QW_SEL_OFF_W(a.gnb, a.topk));
            for (uint32_t i = threadIdx.x; i < a.gnb * (a.topk + 1); i += blockDim.x) ss->w[i] = wg[i];
        }
        __syncthreads();
    }
    selected();
    if (threadIdx.x == 0) QW_WSTAMP(13);
    QW_DSTAMP(1);
    auto ready = [&] {
        if (staged) return;
        staged = true;
        if (!tabled && (qw_has_lut(FGU) || qw_has_lut(FSG))) qw_lut_copy_issue(lut, (const u2 *)a.glut);
        qw_stage_x_issue(xf, a.x, a.D, a.D, a.nbr);
        qw_lds_arrive();
        __syncthreads();
    };
    // Waves are numbered wave-major (wave w of workgroup b is number w * gridDim.x + b), so that when the tiles do not
    // divide evenly the waves with one tile more are spread over all compute units instead of filling the first ones.
    const uint32_t nw = gridDim.x * (blockDim.x >> 6), w0 = qw_wave() * gridDim.x + blockIdx.x;
    if (FSG != 0) {
        if (a.Wsg) { // the shared expert's tiles go to the first waves
            qwk_gu_args sa = a;
            sa.Wg = a.Wsg;
            sa.Wu = a.Wsu;
            sa.rowbytes = a.sg_rowbytes;
            sa.shared = 1;
            gu_tasks<FSG == 0 ? 8 : FSG, CHSG, false>(sa, lut, xf, nullptr, w0, nw, ready, hs);
        }
    }
    // the routed tiles: from the workgroup's queue (a wave that did a shared tile simply takes its next one later)
    if constexpr (FGU == QW_F_RT) { // the other GGUF types, one block a chunk; their byte table lies behind the IQ3_S table
        const u2 *tab = lut + (qw_has_lut(FSG) ? QW_LUT_ENTRIES : 0);
        switch (a.fgu) {
        case 12: gu_tasks<12, 1, true>(a, tab, xf, sc, 0, 0, ready, hs); break;
        case 13: gu_tasks<13, 1, true>(a, tab, xf, sc, 0, 0, ready, hs); break;
        case 14: gu_tasks<14, 1, true>(a, tab, xf, sc, 0, 0, ready, hs); break;
        case 20: gu_tasks<20, 8, true>(a, tab, xf, sc, 0, 0, ready, hs); break;
        case 23: gu_tasks<23, 1, true>(a, tab, xf, sc, 0, 0, ready, hs); break;
        default: break; // (the host launches this kernel for these five only)
        }
    } else gu_tasks<FGU, CHGU, true>(a, lut, xf, sc, 0, 0, ready, hs);
    QW_WSTAMP(qw_wave());
    QW_DSTAMP(2);
}
#define QW_GU(FGU, CHGU, FSG, CHSG, NAME)                                                                 \
    extern "C" __global__ __launch_bounds__(QW_WG_GU) void NAME(qwk_gu_args a) {                             \
        __shared__ struct { u2 lut[((qw_has_lut(FGU) || qw_has_lut(FSG)) ? QW_LUT_ENTRIES : 0) + (FGU == QW_F_RT ? QW_KQ_TAB / 2 : 1)]; u4 xf[QW_XF_MAXK * 2]; qw_sel_cache sc; qw_sel_scratch ss; } L; \
        qw_h_global hs = {a.H, a.hplane};                                                                      \
        gu_body<FGU, CHGU, FSG, CHSG>(a, L.lut, L.xf, &L.sc, &L.ss, hs, false, [] {});                           \
        QW_WG_END_STAMP(10);                                                                                    \
        QW_SST_FLUSH();                                                                                         \
    }
// K = D a multiple of 512: 2 IQ3_S blocks or 16 Q8_0 blocks a chunk; any other K: 1.
#if QW_IN_PART(1)
QW_GU(21, 2, 0, 1, qwk_gu_f21_c2) QW_GU(21, 1, 0, 1, qwk_gu_f21_c1)
QW_GU(8, 16, 0, 1, qwk_gu_f8_c16) QW_GU(8, 1, 0, 1, qwk_gu_f8_c1)
QW_GU(21, 2, 21, 2, qwk_gu_f21_c2_s21_c2) QW_GU(21, 2, 8, 16, qwk_gu_f21_c2_s8_c16)
QW_GU(21, 1, 21, 1, qwk_gu_f21_c1_s21_c1) QW_GU(21, 1, 8, 1, qwk_gu_f21_c1_s8_c1)
QW_GU(8, 16, 8, 16, qwk_gu_f8_c16_s8_c16) QW_GU(8, 16, 21, 2, qwk_gu_f8_c16_s21_c2)
QW_GU(8, 1, 8, 1, qwk_gu_f8_c1_s8_c1) QW_GU(8, 1, 21, 1, qwk_gu_f8_c1_s21_c1)
#endif
// packed IQ3_S routed experts (and shared expert, when it is IQ3_S too)
#if QW_IN_PART(1)
QW_GU(121, 2, 0, 1, qwk_gu_f121_c2) QW_GU(121, 2, 121, 2, qwk_gu_f121_c2_s121_c2) QW_GU(121, 2, 8, 16, qwk_gu_f121_c2_s8_c16)
QW_GU(QW_F_ABLATE, 2, 0, 1, qwk_gu_f122_c2) // measurement: the launch above without its arithmetic
QW_GU(121, 1, 0, 1, qwk_gu_f121_c1) QW_GU(121, 1, 121, 1, qwk_gu_f121_c1_s121_c1) QW_GU(121, 1, 8, 1, qwk_gu_f121_c1_s8_c1)
#endif
// routed rows of the other GGUF types (Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS: kernels/moe_gg.metal:336-395), the type an argument
#if QW_IN_PART(1)
QW_GU(QW_F_RT, 1, 0, 1, qwk_gu_rt) QW_GU(QW_F_RT, 1, 21, 1, qwk_gu_rt_s21_c1) QW_GU(QW_F_RT, 1, 8, 1, qwk_gu_rt_s8_c1)
#endif

// ================================================================ front part of a layer (kernels/moe_gg.metal:534-590)
// Router rows with the activations copied into LDS once per workgroup (8 rows per workgroup) on the first
// a.nrouter workgroups. The workgroups after them do the shared expert's gate/up (the reference computes it in the
// same dispatch, kernels/moe_gg.metal:563-573): a tile of 8 gate + 8 up rows is split by chunk over consecutive
// waves of one workgroup (a chunk each, so that the whole expert takes one memory round trip), the partial sums meet
// in LDS and the wave of chunk 0 adds them in chunk order, applies SwiGLU and stores H[t][topk].
// The selection is not made here: handing it to the last router workgroup through a device-wide counter was measured
// slower than a kernel boundary.
template <int WF> __device__ __forceinline__ void pre_router(const qwk_pre_args &a, u4 *lds) {
    const uint32_t nx = a.r.nb * a.r.D / 8; // 16-byte units of x
    for (uint32_t i = threadIdx.x; i < nx; i += blockDim.x) lds[i] = ((const u4 *)a.r.x)[i];
    __syncthreads();
    router_rows_lds<WF>(a.r, (const uint16_t *)lds, blockIdx.x * (blockDim.x >> 6) + qw_wave(), qw_lane());
}
// Binary16 router on the matrix cores: a workgroup takes 16 router rows (row E is the shared-expert gate vector), its
// waves split K among themselves (256 values = 8 matrix instructions a wave per pass), the partial sums meet in LDS
// and wave 0 adds them in wave order. A token's logits do not depend on the other token columns.
// Eight waves take part whatever the workgroup's size: the split of K and the order of the final sum, hence the bits
// of the logits, are the same in every kernel that holds this router.
// Up to this many tokens the front launch reads operand A straight from memory instead of staging all of x in LDS: a
// wave then reads only the K range it multiplies (8 KB of 64 at sixteen tokens) and no barrier stands before the first
// product — but every lane of an operand reads its own token's row, 64 requests an instruction, which the address unit
// serialises: with 8 or 16 tokens the staged form is 1 to 2 us faster, with one or two the direct one (24 layers at one
// token: 0.638 -> 0.618 ms).
#define QW_PRE_DIRECT_NB 2u
__device__ __forceinline__ void pre_router_mfma(const qwk_router_args &a, u4 *xf, f4 *part) {
    const uint32_t lane = qw_lane(), n = lane & 15, kg = lane >> 4, wave = qw_wave(), nwv = QW_WG / 64;
    const uint32_t row = 16 * blockIdx.x + n;
    const uint16_t *wrow = row < a.E ? (const uint16_t *)a.Wr + (size_t)row * a.D : (const uint16_t *)a.Wsg; // rows past E repeat the gate vector; not stored
    f4 acc = {0, 0, 0, 0};
    u4 w[8];
    uint32_t k0 = wave < nwv ? 256 * wave : a.D; // (waves past the eighth: nothing)
    if (a.nb <= QW_PRE_DIRECT_NB) {
        // lane (n, kg) supplies eight activations of token n per step; token columns past the batch read token 0's row,
        // their results are never stored
        const uint16_t *xrow = a.x + (size_t)(n < a.nb ? n : 0) * a.D;
        u4 xa[8];
        if (k0 < a.D)
#pragma unroll
            for (int j = 0; j < 8; j++) w[j] = *(const u4 *)(wrow + k0 + 32 * j + 8 * kg), xa[j] = *(const u4 *)(xrow + k0 + 32 * j + 8 * kg);
        for (; k0 < a.D; k0 += 256 * nwv) {
#pragma unroll
            for (int j = 0; j < 8; j++) acc = qw_mfma(__builtin_bit_cast(h8, xa[j]), __builtin_bit_cast(h8, w[j]), acc);
            if (k0 + 256 * nwv < a.D)
#pragma unroll
                for (int j = 0; j < 8; j++) w[j] = *(const u4 *)(wrow + k0 + 256 * nwv + 32 * j + 8 * kg), xa[j] = *(const u4 *)(xrow + k0 + 256 * nwv + 32 * j + 8 * kg);
        }
    } else {
        // the first pass's weights are in flight while x is staged
        if (k0 < a.D)
#pragma unroll
            for (int j = 0; j < 8; j++) w[j] = *(const u4 *)(wrow + k0 + 32 * j + 8 * kg);
        qw_stage_x(xf, a.x, a.D, a.D, a.nb);
        __syncthreads();
        for (; k0 < a.D; k0 += 256 * nwv) {
#pragma unroll
            for (int j = 0; j < 8; j++) acc = qw_mfma(__builtin_bit_cast(h8, xf[((k0 + 32 * j + 8 * kg) >> 3) * 16 + n]), __builtin_bit_cast(h8, w[j]), acc);
            if (k0 + 256 * nwv < a.D)
#pragma unroll
                for (int j = 0; j < 8; j++) w[j] = *(const u4 *)(wrow + k0 + 256 * nwv + 32 * j + 8 * kg);
        }
    }
    part[wave * 64 + lane] = acc;
    __syncthreads();
    if (wave != 0) return;
    for (uint32_t i = 1; i < nwv; i++) acc += part[i * 64 + lane];
    if (row <= a.E)
#pragma unroll
        for (uint32_t j = 0; j < 4; j++)
            if (4 * kg + j < a.nb) a.logits[(size_t)(4 * kg + j) * (a.E + 1) + row] = acc[j];
}
// Operand A of one chunk held in registers: the fragments a lane needs for its chunk, asked for together with the chunk's
// weights (read by position: qw_af_hi). BLK_K = 256: a lane's slice of a block is 64 values, eight steps of 8; BLK_K = 32:
// one step a block.
template <int BLK_K, int NB> struct qw_afrag_regs {
    static constexpr int NX = BLK_K == 256 ? 8 * NB : NB;
    static constexpr bool indexed = true, has_lo = false;
    h8 x[NX];
    __device__ __forceinline__ void load(const uint16_t *row, uint32_t k0, uint32_t kg) { // row: this lane's token
#pragma unroll
        for (int i = 0; i < NX; i++) x[i] = *(const h8 *)(row + k0 + (BLK_K == 256 ? 64 * kg + 256 * (i >> 3) + 8 * (i & 7) : 8 * kg + 32 * i));
    }
    __device__ __forceinline__ h8 hi(uint32_t) const { return h8{}; } // (not used: the provider is indexed)
    __device__ __forceinline__ h8 lo(uint32_t) const { return h8{}; }
};
template <int F, int CH> __device__ __forceinline__ void pre_shared(const qwk_pre_args &pa, u2 *lut, u4 *xf, f4 *part) {
    typedef qw_chunk<F, CH> C;
    const qwk_gu_args &a = pa.g;
    const uint32_t lane = qw_lane(), n = lane & 15, kg = lane >> 4, K = a.topk, wave = qw_wave(), nwv = blockDim.x >> 6;
    const uint32_t cpr = a.D / (C::BLK_K * CH), tpw = nwv / cpr; // tiles per workgroup (the host checks cpr <= waves)
    const uint32_t tile = (blockIdx.x - pa.nrouter) * tpw + wave / cpr, ci = wave % cpr;
    const bool on = wave < tpw * cpr && tile < a.I / 8;
    QW_PSTAMP(1);
    C c;
    if (on) {
        if constexpr (F == QW_F_PACKED) c.load(a.Wg + (size_t)tile * a.rowbytes + (size_t)ci * CH * C::BLK_B, lane);
        else c.load(((lane >> 2) < 8 ? a.Wg : a.Wu) + ((size_t)8 * tile + ((lane >> 2) & 7)) * a.rowbytes + (size_t)ci * CH * C::BLK_B, lane & 3);
    }
    f4 acc = {0, 0, 0, 0};
    if (a.nbr <= QW_PRE_DIRECT_NB) {
        // one or two tokens: the chunk's activations straight into registers, the table behind the weights; all awaited
        // once. Token columns past the batch read token 0's row; their results are never stored.
        qw_afrag_regs<C::BLK_K, CH> af;
        if (on) af.load(a.x + (size_t)(n < a.nbr ? n : 0) * a.D, ci * CH * C::BLK_K, kg);
        if (qw_has_lut(F)) {
            qw_lut_copy_issue(lut, (const u2 *)a.glut);
            qw_lds_arrive();
            __syncthreads();
        }
        if (on) {
            c.transpose();
            c.mac_lean(lut, af, ci * CH * C::BLK_K, kg, acc);
            part[wave * 64 + lane] = acc;
        }
    } else {
        // the table and the activations behind the weights, all awaited once: one memory round trip before the barrier
        QW_PSTAMP(2);
        if (qw_has_lut(F)) qw_lut_copy_issue(lut, (const u2 *)a.glut);
        qw_stage_x_issue(xf, a.x, a.D, a.D, a.nbr);
        QW_PSTAMP(3);
        qw_lds_arrive();
        QW_PSTAMP(4);
        __syncthreads();
        QW_PSTAMP(5);
        if (on) {
            c.transpose();
            const qw_afrag_lds af = {xf, n};
            c.mac_lean(lut, af, ci * CH * C::BLK_K, kg, acc);
            part[wave * 64 + lane] = acc;
        }
        QW_PSTAMP(6);
    }
    __syncthreads();
    QW_PSTAMP(7);
    if (!on || ci != 0) return;
    acc = part[wave * 64 + lane];
    for (uint32_t i = 1; i < cpr; i++) acc += part[(wave + i) * 64 + lane]; // chunk order
#pragma unroll
    for (uint32_t j = 0; j < 4; j++) {
        const float up = __shfl_xor(acc[j], 8), g = acc[j];
        const uint32_t tok = 4 * kg + j;
        if (n < 8 && tok < a.nbr) {
            const float h = g / (1.0f + __expf(-g)) * up;
            const _Float16 hi = (_Float16)h, lo = (_Float16)(h - (float)hi);
            const size_t o = ((size_t)tok * (K + 1) + K) * a.I + 8 * tile + n;
            a.H[o] = __builtin_bit_cast(uint16_t, hi);
            a.H[o + a.hplane] = __builtin_bit_cast(uint16_t, lo);
        }
    }
    QW_PSTAMP(8);
}
#define QW_PRE(WF, F, CH, NAME)                                                                          \
    extern "C" __global__ __launch_bounds__(QW_WG) void NAME(qwk_pre_args a) {                           \
        __shared__ struct { u2 lut[qw_has_lut(F) ? QW_LUT_ENTRIES : 1]; u4 xf[QW_XF_MAXK * 2]; f4 part[(QW_WG / 64) * 64]; } L; \
        QW_DSTAMP(3);                                                                                   \
        QW_PSTAMP(0);                                                                                   \
        if (blockIdx.x < a.nrouter) {                                                                   \
            if (WF == 1) pre_router_mfma(a.r, L.xf, L.part);                                            \
            else pre_router<WF>(a, L.xf);                                                               \
            QW_DSTAMP(4);                                                                               \
        }                                                                                               \
        else if (F != 0) { pre_shared<F ? F : 8, CH>(a, L.lut, L.xf, L.part); QW_DSTAMP(5); }            \
    }
#if QW_IN_PART(2)
QW_PRE(1, 0, 1, qwk_pre_w1) QW_PRE(30, 0, 1, qwk_pre_w30)
QW_PRE(1, 121, 2, qwk_pre_w1_s121_c2) QW_PRE(30, 121, 2, qwk_pre_w30_s121_c2) QW_PRE(1, 8, 16, qwk_pre_w1_s8_c16) QW_PRE(30, 8, 16, qwk_pre_w30_s8_c16)
#endif
// The same front launch for a shared expert whose gate/up rows are in the K-quant / IQ4 / plain family: the binary16
// router on the first workgroups, the multi-format product with SwiGLU (qwk_qmvm_swiglu's work) on those after them.
#if QW_IN_PART(2)
extern "C" __global__ __launch_bounds__(QW_WG_QMVM) void qwk_pre_w1_kq(qwk_prekq_args a) {
    __shared__ qw_qmvm_lds L;
    if (blockIdx.x < a.nrouter) pre_router_mfma(a.r, L.xf, L.red);
    else qmvm_swiglu_body(a.m, L, blockIdx.x - a.nrouter, gridDim.x - a.nrouter);
}
#endif

// SwiGLU of the shared expert (kernels/moe_gg.metal:563-573) after a matvec of its gate and up rows in another format
// family: the arithmetic and the two-plane store of pre_shared. One thread per (token, column).
#if QW_IN_PART(2)
extern "C" __global__ __launch_bounds__(256) void qwk_sh_act(qwk_shact_args a) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= a.nb * a.I) return;
    const uint32_t t = i / a.I, j = i % a.I;
    const float g = a.g[i], up = a.u[i], h = g / (1.0f + __expf(-g)) * up;
    const _Float16 hi = (_Float16)h, lo = (_Float16)(h - (float)hi);
    const size_t o = ((size_t)t * (a.topk + 1) + a.topk) * a.I + j;
    a.H[o] = __builtin_bit_cast(uint16_t, hi);
    a.H[o + a.hplane] = __builtin_bit_cast(uint16_t, lo);
}
#endif

// ================================================================ down (kernels/moe_gg.metal:456-483, 606-617, 639-652)
// The shared expert's down projection rides in the same launch: tiles of 16 rows, operand A = H[t][topk] (hi + lo
// planes) of every token straight from global memory. Wave w takes tiles w, w + nw, ...
template <int F, int CH> __device__ __forceinline__ void shared_down_tiles(const qwk_dn_args &a, const u2 *lut, uint32_t w0, uint32_t nw) {
    typedef qw_chunk<F, CH> C;
    const uint32_t lane = qw_lane(), n = lane & 15, kg = lane >> 4, K = a.topk;
    const uint32_t ntiles = a.D / 16, cpr = a.I / (C::BLK_K * CH);
    h8 xhi[4] = {}, xlo[4] = {}; // token columns past the batch stay zero
    const uint16_t *rowhi = a.H + ((size_t)(n < a.snbr ? n : 0) * (K + 1) + K) * a.I;
    const qw_afrag_gather af = {rowhi, rowhi + a.hplane, n < a.snbr, xhi, xlo};
    f4 acc = {0, 0, 0, 0};
    qw_task_pipeline<C>(ntiles, w0, nw, cpr, CH * C::BLK_B, lane & 3,
        [&](uint32_t t) { return a.Wsd + (size_t)(16 * t + (lane >> 2)) * a.sd_rowbytes; },
        [&](uint32_t t, uint32_t ci, const C &c) {
            c.mac_gather(lut, af, ci * CH * C::BLK_K, kg, acc);
            if (ci + 1 != cpr) return;
            const uint32_t r = 16 * t + n;
#pragma unroll
            for (uint32_t j = 0; j < 4; j++)
                if (4 * kg + j < a.snbr) a.Psh[(size_t)(4 * kg + j) * a.D + r] = acc[j];
            acc = f4{0, 0, 0, 0};
        });
}

// Range form (I <= 512). The task list is "virtual experts" x tiles of 16 rows: virtual expert 0 is the shared expert
// when the launch carries one, then the unique routed experts in record order. Every workgroup takes one contiguous
// range of at most D / 16 tasks, which touches at most two experts: their H rows (both planes, only the tokens
// that picked them) are copied into LDS once, in fragment order, and the waves then stream the range's tiles with operand A read
// from LDS. The first weight loads are issued before the table copy, the row copy and the barrier.
constexpr bool qw_tiled(int F) { return F == QW_F_PACKED || F == QW_F_PACKED_NL; } // weights come from a tile-major copy
struct qw_dn_seg { // one expert's part of a workgroup's range (all fields wave-uniform)
    const uint8_t *W;  // the expert's matrix
    float *P;          // Pg or Psh
    uint32_t rowbytes, mask, tile0, ntile, sh; // sh: shared expert (results to P[t][row], every token < nbr)
    uint32_t u;        // routed: index into the record
};
template <int F, int CH, class S> __device__ __forceinline__ void dn_range_run(const qwk_dn_args &a, const u2 *lut, const uint16_t *arows, const qw_dn_seg &g0, const qw_dn_seg &g1,
                                                                                 bool both, const uint8_t *slots0, const uint8_t *slots1, S ready) {
    typedef qw_chunk<F, CH> C;
    const uint32_t lane = qw_lane(), n = lane & 15, kg = lane >> 4, K = a.topk, nwv = blockDim.x >> 6, nl = lane >> 2;
    const uint32_t ntask = g0.ntile + (both ? g1.ntile : 0), cpr = a.I / (C::BLK_K * CH);
    // per lane: where the results of tokens 4 kg .. 4 kg + 3 go in either segment, as float offsets of row 0
    // (token * topk + slot for a routed expert, token for the shared one; 32 bits hold them), ~0 = not picked
    uint32_t off0[4], off1[4];
#pragma unroll
    for (uint32_t j = 0; j < 4; j++) {
        const uint32_t tok = 4 * kg + j;
        off0[j] = !((g0.mask >> tok) & 1) ? ~0u : (g0.sh ? tok : tok * K + slots0[tok]) * a.D;
        off1[j] = !both || !((g1.mask >> tok) & 1) ? ~0u : (g1.sh ? tok : tok * K + slots1[tok]) * a.D;
    }
    f4 acc = {0, 0, 0, 0};
    qw_task_stream<C>(ntask, qw_wave(), nwv, cpr, CH * C::BLK_B, qw_tiled(F) ? lane : lane & 3,
        [&](uint32_t i) {
            // (field by field: a reference chosen between the two records would put them in scratch memory)
            const bool second = i >= g0.ntile;
            const uint8_t *W = second ? g1.W : g0.W;
            const uint32_t tile = second ? g1.tile0 + i - g0.ntile : g0.tile0 + i, rbs = second ? g1.rowbytes : g0.rowbytes;
            if constexpr (qw_tiled(F)) return W + (size_t)tile * rbs; // rowbytes = bytes of a tile
            else return W + (size_t)(16 * tile + nl) * rbs;
        },
        [&](uint32_t i, uint32_t ci, const C &c) {
            const bool second = i >= g0.ntile;
            const u4 *ab = (const u4 *)arows + (second ? 4 * a.I : 0); // fragment order: [plane][8 k-values][token], 16 bytes each
            const qw_afrag_lds2 af = {ab, ab + 2 * a.I, n};
            c.mac_half(lut, af, ci * CH * C::BLK_K, kg, acc);
            if (ci + 1 != cpr) return;
            const uint32_t r = 16 * (second ? g1.tile0 + i - g0.ntile : g0.tile0 + i) + n;
            float *P = second ? g1.P : g0.P;
#pragma unroll
            for (uint32_t j = 0; j < 4; j++) {
                const uint32_t o = second ? off1[j] : off0[j];
                if (o != ~0u) qw_store_f32(P + o + r, acc[j]); // (untracked store: Pg and Psh are never read back in this kernel)
            }
            acc = f4{0, 0, 0, 0};
        },
        ready, qw_has_lut(F) ? (const uint8_t *)a.glut : nullptr);
}
template <int F, int CH, int FSD, int CHSD> __device__ __forceinline__ void dn_range_body(const qwk_dn_args &a, u2 *lut, uint16_t *arows /* [2][16][2][I] */, qw_sel_cache *sc) {
    const uint32_t K = a.topk, gnb = a.gnb, GU = gnb * K, tpe = a.D / 16;
    const bool tp2 = (tpe & (tpe - 1)) == 0; // D = 1024, 2048: shifts instead of divisions
    const uint32_t tsh = (uint32_t)__builtin_ctz(tpe);
    auto div_tpe = [&](uint32_t x) { return tp2 ? x >> tsh : x / tpe; };
    qw_sel_load(*sc, a.sel, K, gnb); // one memory round trip for everything the ranges depend on
    if (qw_has_lut(F) || qw_has_lut(FSD)) qw_lut_copy_issue(lut, (const u2 *)a.glut); // lands in LDS meanwhile; awaited in ready()
    if (F == 20 || FSD == 20 || F == QW_F_PACKED_NL || FSD == QW_F_PACKED_NL) qw_kq_tab_build((uint32_t *)lut); // the byte table of the 4-bit codebook instead
    __syncthreads();
    const uint32_t *ue = sc->ue, *mask = sc->mask;
    const uint8_t *slot = sc->slot;
    uint32_t U = (uint32_t)__builtin_amdgcn_readfirstlane((int)sc->U);
    if (U > GU) U = GU;
    // a shared-expert tile of a wider format counts as several tasks, so that ranges hold about the same bytes
    const uint32_t tb = qw_tiled(F) ? a.rowbytes : 16 * a.rowbytes, stb = qw_tiled(FSD) ? a.sd_rowbytes : 16 * a.sd_rowbytes; // bytes of a tile
    const uint32_t nsh = (FSD != 0 && a.Wsd) ? 1 : 0, shw = nsh ? (stb + tb - 1) / tb : 1, vsh = nsh * shw * tpe;
    const uint32_t V = vsh + U * tpe;
    uint32_t per = (V + gridDim.x - 1) / gridDim.x;
    if (per > tpe) per = tpe;
    for (uint32_t base = blockIdx.x * per; base < V; base += gridDim.x * per) { // one round unless the grid is small
        const uint32_t end = base + per < V ? base + per : V;
        // virtual expert of a position: 0 = shared (positions below vsh), then the routed experts
        const uint32_t v0 = base < vsh ? 0 : nsh + div_tpe(base - vsh), v1 = end - 1 < vsh ? 0 : nsh + div_tpe(end - 1 - vsh);
        auto seg = [&](uint32_t v) {
            qw_dn_seg g;
            g.sh = v < nsh;
            if (g.sh) {
                const uint32_t hi = end < vsh ? end : vsh; // positions [base, hi) -> tiles, rounded so that neighbours meet
                g.tile0 = shw == 1 ? base : (base + shw - 1) / shw;
                g.ntile = (shw == 1 ? hi : (hi + shw - 1) / shw) - g.tile0;
                g.u = 0;
                g.W = a.Wsd, g.P = a.Psh, g.rowbytes = a.sd_rowbytes, g.mask = qw_all_tokens(a.snbr);
            } else {
                const uint32_t first = vsh + (v - nsh) * tpe, lo = first > base ? first : base, hi = first + tpe < end ? first + tpe : end;
                g.u = v - nsh;
                g.tile0 = lo - first;
                g.ntile = hi - lo;
                const uint32_t e = (uint32_t)__builtin_amdgcn_readfirstlane((int)ue[g.u]);
                g.W = a.Wd + (size_t)e * (qw_tiled(F) ? tpe : a.D) * a.rowbytes, g.P = a.P, g.rowbytes = a.rowbytes;
                g.mask = (uint32_t)__builtin_amdgcn_readfirstlane((int)mask[g.u]) & qw_all_tokens(a.nbr);
            }
            return g;
        };
        const qw_dn_seg g0 = seg(v0), g1 = seg(v1);
        const bool both = v1 != v0;
        bool staged = false;
        // Set-up of a round, run by every wave once its first weight loads are in flight: the H rows of the tokens that
        // picked the range's (at most two) experts, both planes, by direct global-to-LDS loads, and the barrier.
        // Fragment order in LDS, [segment][plane][c][token], 16 bytes each (the sixteen lanes of a k-group read 256
        // contiguous bytes): one load instruction fills four c of one plane, lane = (c, token); the lanes of tokens
        // that did not pick the expert stay off and leave their columns as they are (those results are never stored).
        auto ready = [&] {
            if (staged) return;
            staged = true;
            const uint32_t upr = a.I / 8, ncb = upr / 4, ninst = (both ? 2 : 1) * 2 * ncb; // 16-byte units per plane row; instructions
            const uint32_t lane = qw_lane(), t = lane & 15, rows = g0.mask | (both ? g1.mask << 16 : 0), nrows = (uint32_t)__builtin_popcount(rows);
            if (nrows * 2 * upr <= blockDim.x) {
                // few rows (a token or two per expert): one 16-byte unit per thread through a register, the waves
                // of a row finding its bit in the mask by a (mostly scalar) walk
                // (a row of both planes is 2 upr threads: whole waves when I is a multiple of 256, else a wave may span two rows)
                const uint32_t i = threadIdx.x, kl = i / (2 * upr), k = (2 * upr) % 64 == 0 ? (uint32_t)__builtin_amdgcn_readfirstlane((int)kl) : kl, r = i % (2 * upr), pl = r / upr, c = r % upr;
                if (k < nrows) {
                    uint32_t m = rows;
                    for (uint32_t j = 0; j < k; j++) m &= m - 1;
                    const uint32_t bit = (uint32_t)__builtin_ctz(m), sg = bit >> 4, tk = bit & 15;
                    const uint32_t sl = (sg ? g1.sh : g0.sh) ? K : slot[(sg ? g1.u : g0.u) * gnb + tk];
                    ((u4 *)arows)[((sg * 2 + pl) * upr + c) * 16 + tk] = *(const u4 *)(a.H + pl * (size_t)a.hplane + ((size_t)tk * (K + 1) + sl) * a.I + 8 * c);
                }
            } else {
                const uint32_t s0 = g0.sh ? K : slot[g0.u * gnb + t], s1 = !both ? 0 : g1.sh ? K : slot[g1.u * gnb + t]; // result slot of token t
                for (uint32_t q = qw_wave(); q < ninst; q += blockDim.x >> 6) {
                    const uint32_t sg = q / (2 * ncb), r = q % (2 * ncb), pl = r / ncb, cb = r % ncb;
                    const uint32_t m = sg ? g1.mask : g0.mask, sl = sg ? s1 : s0, c = 4 * cb + (lane >> 4);
                    if ((m >> t) & 1)
                        qw_load_to_lds((const u4 *)(a.H + pl * (size_t)a.hplane + ((size_t)t * (K + 1) + sl) * a.I + 8 * c), (u4 *)arows + ((sg * 2 + pl) * upr + 4 * cb) * 16);
                }
            }
            qw_lds_arrive(); // the table's loads too (issued at the start of the kernel)
            __syncthreads();
        };
        // the two segments share one pipeline when their formats agree; a shared expert of another format runs first
        if (FSD != 0 && FSD != F && g0.sh) {
            qw_dn_seg none = g0;
            none.ntile = 0;
            dn_range_run<FSD == 0 ? F : FSD, CHSD>(a, lut, arows, g0, none, false, slot, slot, ready);
            if (both) dn_range_run<F, CH>(a, lut, arows + 32 * a.I, g1, none, false, slot + g1.u * gnb, slot, ready);
        } else {
            dn_range_run<F, CH>(a, lut, arows, g0, g1, both, slot + g0.u * gnb, slot + g1.u * gnb, ready);
        }
        __syncthreads();
    }
}
#define QW_DN_RANGE(F, CH, FSD, CHSD, NAME)                                                       \
    extern "C" __global__ __launch_bounds__(QW_WG_DN) void NAME(qwk_dn_args a) {                  \
        __shared__ struct { u2 lut[(qw_has_lut(F) || qw_has_lut(FSD)) ? QW_LUT_ENTRIES : 1]; uint16_t arows[2 * 16 * 2 * 512]; qw_sel_cache sc; } L; \
        dn_range_body<F, CH, FSD, CHSD>(a, L.lut, L.arows, &L.sc);                                \
    }
// IQ4_NL rows (the reference model's down projections: I = 640, five chunks of 4 blocks a row): no IQ3_S table in LDS,
// so the staged H rows may be 640 wide
#define QW_DN_RANGE_NL(CH, FSD, CHSD, NAME)                                                       \
    extern "C" __global__ __launch_bounds__(QW_WG_DN) void NAME(qwk_dn_args a) {                  \
        __shared__ struct { u2 lut[QW_KQ_TAB / 2]; uint16_t arows[2 * 16 * 2 * 640]; qw_sel_cache sc; } L; \
        dn_range_body<20, CH, FSD, CHSD>(a, L.lut, L.arows, &L.sc);                               \
    }
#if QW_IN_PART(3)
QW_DN_RANGE_NL(4, 0, 1, qwk_dnr_f20_c4) QW_DN_RANGE_NL(4, 20, 4, qwk_dnr_f20_c4_s20_c4) QW_DN_RANGE_NL(4, 8, 4, qwk_dnr_f20_c4_s8_c4)
#endif
#define QW_DN_RANGE_NLP(FSD, CHSD, NAME)                                                          \
    extern "C" __global__ __launch_bounds__(QW_WG_DN) void NAME(qwk_dn_args a) {                  \
        __shared__ struct { u2 lut[QW_KQ_TAB / 2]; uint16_t arows[2 * 16 * 2 * 640]; qw_sel_cache sc; } L; \
        dn_range_body<QW_F_PACKED_NL, 10, FSD, CHSD>(a, L.lut, L.arows, &L.sc);                   \
    }
// the tile-major copy: rows of 320 or 640
#if QW_IN_PART(3)
QW_DN_RANGE_NLP(0, 10, qwk_dnr_f120_c10) QW_DN_RANGE_NLP(QW_F_PACKED_NL, 10, qwk_dnr_f120_c10_s120_c10) QW_DN_RANGE_NLP(8, 4, qwk_dnr_f120_c10_s8_c4)
#endif
// rows of 320 or 640: chunks of ten blocks (a row of 640 in two), 5760 bytes a tile in flight per wave
#if QW_IN_PART(3)
QW_DN_RANGE_NL(10, 0, 1, qwk_dnr_f20_c10) QW_DN_RANGE_NL(10, 20, 10, qwk_dnr_f20_c10_s20_c10) QW_DN_RANGE_NL(10, 8, 4, qwk_dnr_f20_c10_s8_c4)
#endif
// I = 512: a row is one chunk of 2 IQ3_S blocks or four chunks of 4 Q8_0 blocks; I = 256: one IQ3_S block, two Q8_0 chunks
#if QW_IN_PART(3)
QW_DN_RANGE(21, 2, 0, 1, qwk_dnr_f21_c2) QW_DN_RANGE(21, 2, 21, 2, qwk_dnr_f21_c2_s21_c2) QW_DN_RANGE(21, 2, 8, 4, qwk_dnr_f21_c2_s8_c4)
QW_DN_RANGE(21, 1, 0, 1, qwk_dnr_f21_c1) QW_DN_RANGE(21, 1, 21, 1, qwk_dnr_f21_c1_s21_c1) QW_DN_RANGE(21, 1, 8, 4, qwk_dnr_f21_c1_s8_c4)
QW_DN_RANGE(121, 2, 0, 1, qwk_dnr_f121_c2) QW_DN_RANGE(121, 2, 121, 2, qwk_dnr_f121_c2_s121_c2) QW_DN_RANGE(121, 2, 8, 4, qwk_dnr_f121_c2_s8_c4)
QW_DN_RANGE(121, 1, 0, 1, qwk_dnr_f121_c1) QW_DN_RANGE(121, 1, 121, 1, qwk_dnr_f121_c1_s121_c1) QW_DN_RANGE(121, 1, 8, 4, qwk_dnr_f121_c1_s8_c4)
QW_DN_RANGE(8, 4, 0, 1, qwk_dnr_f8_c4) QW_DN_RANGE(8, 4, 8, 4, qwk_dnr_f8_c4_s8_c4) QW_DN_RANGE(8, 4, 21, 2, qwk_dnr_f8_c4_s21_c2) QW_DN_RANGE(8, 4, 21, 1, qwk_dnr_f8_c4_s21_c1)
#endif

// Down + combine in one launch for a few tokens (at most QW_DNC_MAXNB; kernels/moe_gg.metal:639-663 in one pass).
// With one or two tokens the layer is bound by its launches, and the combine is a launch that only adds up what the
// down launch wrote. Here a workgroup owns one tile of 16 output rows: its waves take the shared expert and the unique
// routed experts of the record, one (expert, tile) product each (operand A straight from the H planes, only the lanes
// of tokens that picked the expert read), leave the partial results in LDS by (token, slot), and after one barrier
// sixteen lanes per token add them up in rank order, the shared expert last, exactly as the combine kernel does.
// Pg and Psh are still written, so that the buffers hold what the two separate launches would have left.
template <int F, int CH, class S>
__device__ __forceinline__ f4 dnc_tile(const qwk_dn_args &a, const u2 *lut, const uint8_t *W, uint32_t rowbytes, uint32_t tile, const qw_afrag_gather &af, S ready) {
    typedef qw_chunk<F, CH> C;
    const uint32_t lane = qw_lane(), kg = lane >> 4, cpr = a.I / (C::BLK_K * CH);
    f4 acc = {0, 0, 0, 0};
    qw_task_pipeline<C>(1, 0, 1, cpr, CH * C::BLK_B, qw_tiled(F) ? lane : lane & 3,
        [&](uint32_t) {
            if constexpr (qw_tiled(F)) return W + (size_t)tile * rowbytes; // rowbytes = bytes of a tile
            else return W + (size_t)(16 * tile + (lane >> 2)) * rowbytes;
        },
        [&](uint32_t, uint32_t ci, const C &c) { c.mac_gather(lut, af, ci * CH * C::BLK_K, kg, acc); }, ready);
    return acc;
}
template <int F, int CH, int FSD, int CHSD>
__device__ __forceinline__ void dnc_body(const qwk_dn_args &a, u2 *lut, float *part /* [QW_DNC_MAXNB][topk + 1][16] */, float *wl /* [QW_DNC_MAXNB][topk + 1] */, qw_sel_cache *sc) {
    const uint32_t K = a.topk, gnb = a.gnb, tpe = a.D / 16, tile = blockIdx.x, lane = qw_lane(), n = lane & 15, kg = lane >> 4, nwv = blockDim.x >> 6;
    // The table through registers, asked for first and stored behind the record (published by the barrier of ready()): a
    // copy straight into LDS kept every wave in the issue of its loads for more than a microsecond, between the record and
    // the first weights (which need the record).
    constexpr bool TAB = qw_has_lut(F) || qw_has_lut(FSD);
    constexpr uint32_t TPER = TAB ? (QW_LUT_BYTES / 16 + QW_WG_DN - 1) / QW_WG_DN : 0;
    u4 tabv[TPER ? TPER : 1];
    uint32_t tat[TPER ? TPER : 1];
    if constexpr (TAB) { // (every workgroup starts at another place of the table; the last piece of some threads repeats an earlier one)
#pragma unroll
        for (uint32_t it = 0; it < TPER; it++) {
            uint32_t i = threadIdx.x + it * QW_WG_DN;
            if (i >= QW_LUT_BYTES / 16) i -= QW_WG_DN;
            tat[it] = (i + blockIdx.x * 320u) & (QW_LUT_BYTES / 16 - 1);
            tabv[it] = ((const u4 *)a.glut)[tat[it]];
        }
    }
    qw_sel_load(*sc, a.sel, K, gnb);
    const float *wg = (const float *)(a.sel + QW_SEL_OFF_W(gnb, K));
    for (uint32_t i = threadIdx.x; i < a.nbr * (K + 1); i += blockDim.x) wl[i] = wg[i];
    if (F == QW_F_PACKED_NL || FSD == QW_F_PACKED_NL) qw_kq_tab_build((uint32_t *)lut); // the byte table of the 4-bit codebook instead
    if constexpr (TAB) {
#pragma unroll
        for (uint32_t it = 0; it < TPER; it++) ((u4 *)lut)[tat[it]] = tabv[it];
    }
    __syncthreads();
    uint32_t U = (uint32_t)__builtin_amdgcn_readfirstlane((int)sc->U);
    if (U > gnb * K) U = gnb * K;
    const uint32_t nsh = (FSD != 0 && a.Wsd) ? 1 : 0, V = nsh + U;
    bool staged = false;
    auto ready = [&] { // once per wave, behind its first weight loads
        if (staged) return;
        staged = true;
        __syncthreads();
    };
    for (uint32_t v = qw_wave(); v < V; v += nwv) {
        const bool sh = v < nsh;
        const uint32_t u = sh ? 0 : v - nsh;
        const uint32_t mask = sh ? qw_all_tokens(a.snbr) : (uint32_t)__builtin_amdgcn_readfirstlane((int)sc->mask[u]) & qw_all_tokens(a.nbr);
        const bool on = (mask >> n) & 1; // token n of the batch takes part in this product
        const uint32_t sl = sh || !on ? K : sc->slot[u * gnb + n];
        const uint16_t *rowhi = a.H + ((size_t)(on ? n : 0) * (K + 1) + sl) * a.I;
        h8 xhi[4] = {}, xlo[4] = {}; // the columns of tokens that are off stay zero
        const qw_afrag_gather af = {rowhi, rowhi + a.hplane, on, xhi, xlo};
        f4 acc;
        if (sh) {
            if constexpr (FSD != 0) acc = dnc_tile<FSD, CHSD>(a, lut, a.Wsd, a.sd_rowbytes, tile, af, ready);
            else acc = f4{0, 0, 0, 0};
        } else {
            const uint32_t e = (uint32_t)__builtin_amdgcn_readfirstlane((int)sc->ue[u]);
            acc = dnc_tile<F, CH>(a, lut, a.Wd + (size_t)e * (qw_tiled(F) ? tpe : a.D) * a.rowbytes, a.rowbytes, tile, af, ready);
        }
        const uint32_t r = 16 * tile + n;
#pragma unroll
        for (uint32_t j = 0; j < 4; j++) {
            const uint32_t tok = 4 * kg + j;
            if (tok < QW_DNC_MAXNB && ((mask >> tok) & 1)) {
                const uint32_t s = sh ? K : sc->slot[u * gnb + tok];
                part[(tok * (K + 1) + s) * 16 + n] = acc[j];
                if (sh) a.Psh[(size_t)tok * a.D + r] = acc[j];
                else a.P[((size_t)tok * K + s) * a.D + r] = acc[j];
            }
        }
    }
    ready(); // waves without a product still meet the others at the barrier
    __syncthreads();
    if (threadIdx.x < a.nbr * 16) { // rank order, then the shared expert (qwk_cmb's arithmetic)
        const uint32_t t = threadIdx.x >> 4, i = threadIdx.x & 15, r = 16 * tile + i;
        const float *w = wl + t * (K + 1), *p = part + t * (K + 1) * 16 + i;
        float o = 0;
        for (uint32_t s = 0; s < K; s++) o = __builtin_fmaf(w[s], p[s * 16], o);
        o = __builtin_fmaf(w[K], nsh ? p[K * 16] : a.Psh[(size_t)t * a.D + r], o);
        a.out[(size_t)t * a.D + r] = qw_f2h(o);
    }
}
#define QW_DNC(F, CH, FSD, CHSD, NAME)                                                              \
    extern "C" __global__ __launch_bounds__(QW_WG_DN) void NAME(qwk_dn_args a) {                    \
        __shared__ struct { u2 lut[(qw_has_lut(F) || qw_has_lut(FSD)) ? QW_LUT_ENTRIES : (F == QW_F_PACKED_NL || FSD == QW_F_PACKED_NL) ? QW_KQ_TAB / 2 : 1]; float part[QW_DNC_MAXNB * 17 * 16], wl[QW_DNC_MAXNB * 17]; qw_sel_cache sc; } L; \
        dnc_body<F, CH, FSD, CHSD>(a, L.lut, L.part, L.wl, &L.sc);                                  \
    }
#if QW_IN_PART(4)
QW_DNC(121, 2, 0, 1, qwk_dnc_f121_c2) QW_DNC(121, 2, 121, 2, qwk_dnc_f121_c2_s121_c2) QW_DNC(121, 2, 8, 4, qwk_dnc_f121_c2_s8_c4)
QW_DNC(121, 1, 0, 1, qwk_dnc_f121_c1) QW_DNC(121, 1, 121, 1, qwk_dnc_f121_c1_s121_c1) QW_DNC(121, 1, 8, 4, qwk_dnc_f121_c1_s8_c4)
QW_DNC(8, 4, 0, 1, qwk_dnc_f8_c4) QW_DNC(8, 4, 8, 4, qwk_dnc_f8_c4_s8_c4)
QW_DNC(120, 10, 0, 10, qwk_dnc_f120_c10) QW_DNC(120, 10, 120, 10, qwk_dnc_f120_c10_s120_c10) QW_DNC(120, 10, 8, 4, qwk_dnc_f120_c10_s8_c4) // tile-major IQ4_NL rows of 640
#endif

// Down + combine in one launch for 3 to 16 tokens. The range form above needs a second launch because the products
// that make up one output row are spread over all workgroups. Here a workgroup owns tpw tiles of 16 output rows and a
// quarter of the tokens (four): it stages all H rows of its tokens in LDS once (4 x (topk + 1) rows, both planes),
// lists the unique experts that its tokens picked, and its waves stream those experts' tiles (the shared expert's
// first) through the same pipeline and the same arithmetic as the range form; the partial results meet in LDS by (token,
// slot, row) and are added in rank order, the shared expert last, exactly as the combine kernel does. An expert picked
// by tokens of several quarters is read once per quarter (about 1.15 times the unique experts' bytes at 16 tokens);
// the quarters of a tile group are placed on one XCD so that the repeats hit its L2. Pg and Psh are still written.
struct qw_dnq_lds {
    u4 hrows[2 * 64 * QW_DNQ_ROWS]; // [plane][8 k-values][row], 16 bytes each: row = local token * (topk + 1) + slot
    float part[4 * 11 * 32];        // [local token][slot][row of the group]
    float wl[4 * 11];               // gating weights of the quarter's tokens
    uint32_t ue[QW_DNQ_MAXU], slot4[QW_DNQ_MAXU]; // expert of unique index u; the slot bytes of the quarter's four tokens
    uint16_t mask[QW_DNQ_MAXU], vlist[48];        // token mask of u; the unique indices this quarter needs
    uint32_t U, nv, q[2];
};
// Operand A from the staged rows, in the manner of qw_afrag_gather: lane m < 4 is local token m, its row chosen per
// expert; four fragments per plane at a time inside one predicated region, into registers the caller keeps (and has
// zeroed once), so that the lanes that are off (12 of every 16 at least) cost LDS nothing.
template <uint32_t ROWS> struct qw_afrag_rows {
    const u4 *hi_, *lo_; // this lane's row in the two planes
    bool on;
    h8 (&hi)[4];
    h8 (&lo)[4];
    static constexpr bool has_lo = true;
    static constexpr bool stacked = false;
    __device__ __forceinline__ void place(const u4 *hi0, const u4 *lo0, uint32_t m, uint32_t r, bool picked) {
        on = picked && m < 4, hi_ = hi0 + r, lo_ = lo0 + r; // (read only where on: one of the staged rows then)
    }
    __device__ __forceinline__ void fetch4(uint32_t koff, uint32_t kstep) const {
        if (on) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                hi[i] = __builtin_bit_cast(h8, hi_[((koff + i * kstep) >> 3) * ROWS]);
                lo[i] = __builtin_bit_cast(h8, lo_[((koff + i * kstep) >> 3) * ROWS]);
            }
        }
    }
};
// The same rows with both planes in one operand A: lane m < 4 supplies the hi plane of local token m, lane 4 + m its lo
// plane, so that one matrix instruction does the work of two (a share has at most four tokens: eight of the sixteen
// operand rows are in use instead of four). For the chunk types whose mac_gather knows the stacked form.
template <uint32_t ROWS> struct qw_afrag_rows2 {
    const u4 *hi_, *lo_; // hi_: this lane's row in its plane; lo_ unused
    bool on;
    h8 (&hi)[4];
    h8 (&lo)[4];
    static constexpr bool has_lo = true;
    static constexpr bool stacked = true;
    __device__ __forceinline__ void place(const u4 *hi0, const u4 *lo0, uint32_t m, uint32_t r, bool picked) {
        on = picked && m < 8, hi_ = (m & 4 ? lo0 : hi0) + r;
    }
    __device__ __forceinline__ void fetch4(uint32_t koff, uint32_t kstep) const {
        if (on) {
#pragma unroll
            for (int i = 0; i < 4; i++) hi[i] = __builtin_bit_cast(h8, hi_[((koff + i * kstep) >> 3) * ROWS]);
        }
    }
};
// What dnq_run reads and writes in LDS (the two kernels that hold it lay their LDS out differently).
struct qw_dnq_view {
    const u4 *hrows;       // [plane][8 k-values][row], 16 bytes each, ROWS rows: row = local token * (topk + 1) + slot
    float *part;           // [local token][slot][row of the group]
    const uint32_t *ue, *slot4;
    const uint16_t *mask, *vlist;
    uint32_t *q;           // two counters: the routed tiles handed out (starts at the number of waves: wave w begins with tile w), the shared ones (starts at 0)
};
// The tiles of `nv` experts (shared: the one shared expert) for this workgroup's tpw tiles, dealt to its waves.
template <int F, int CH, bool SHARED, uint32_t ROWS, class S>
__device__ __forceinline__ void dnq_run(const qwk_dn_args &a, const u2 *lut, const qw_dnq_view &L, uint32_t g, uint32_t t0, uint32_t nt, uint32_t nv, S ready) {
    typedef qw_chunk<F, CH> C;
    const uint32_t lane = qw_lane(), n = lane & 15, kg = lane >> 4, K = a.topk, tpe = a.D / 16, tpw = a.tpw, cpr = a.I / (C::BLK_K * CH), rw = 16 * tpw;
    const uint32_t ts = (uint32_t)__builtin_ctz(tpw), tm = tpw - 1; // tpw is a power of two
    const uint32_t m = n; // operand A row of this lane
    f4 acc = {0, 0, 0, 0};
    const u4 *const lo0 = L.hrows + a.I / 8 * ROWS;
    h8 xhi[4] = {}, xlo[4] = {};
    // (tile-major IQ3_S: both planes in one matrix instruction; the Q8_0 form adds the planes inside the accumulator, which one instruction cannot reproduce bit for bit)
    typename std::conditional<F == QW_F_PACKED, qw_afrag_rows2<ROWS>, qw_afrag_rows<ROWS>>::type af = {L.hrows, lo0, false, xhi, xlo};
    auto expert = [&](uint32_t task) { return SHARED ? 0u : (uint32_t)L.vlist[task >> ts]; };
    // the workgroup's tiles go to its waves from a queue (qw_task_queue): a wave that is done takes the next one, and the
    // shared expert's tiles go to the waves that leave the routed ones first
    auto next = [&]() -> uint32_t {
        uint32_t j = 0;
        if (lane == 0) j = atomicAdd(&L.q[SHARED ? 1 : 0], 1u);
        return (uint32_t)__builtin_amdgcn_readfirstlane((int)j);
    };
    qw_task_queue<C>(nv * tpw, SHARED ? next() : qw_wave(), next, cpr, CH * C::BLK_B, qw_tiled(F) ? lane : lane & 3,
        [&](uint32_t task) {
            const uint32_t tile = g * tpw + (task & tm);
            const uint8_t *W = SHARED ? a.Wsd : a.Wd + (size_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)L.ue[expert(task)]) * (qw_tiled(F) ? tpe : a.D) * a.rowbytes;
            const uint32_t rb = SHARED ? a.sd_rowbytes : a.rowbytes;
            if constexpr (qw_tiled(F)) return W + (size_t)tile * rb; // rowbytes = bytes of a tile
            else return W + (size_t)(16 * tile + (lane >> 2)) * rb;
        },
        [&](uint32_t task, uint32_t ci, const C &c) {
            const uint32_t u = expert(task);
            if (ci == 0) { // this lane's operand A row for the task's expert
                const uint32_t tl = m & 3, mk = SHARED ? qw_all_tokens(a.snbr) >> t0 : (uint32_t)L.mask[u] >> t0;
                const uint32_t r = tl * (K + 1) + (SHARED ? K : (L.slot4[u] >> (8 * tl)) & 255);
                af.place(L.hrows, lo0, m, r, tl < nt && ((mk >> tl) & 1));
                // a lane that is off keeps the fragments of an earlier expert: they feed output rows that are never
                // stored (a matrix-core output row depends on its own operand A row only)
            }
            c.mac_gather(lut, af, ci * CH * C::BLK_K, kg, acc);
            if (ci + 1 != cpr) return;
            // lanes of k-group 0 hold local tokens 0 .. 3 of row n
            const uint32_t mk = SHARED ? qw_all_tokens(a.snbr) >> t0 : (uint32_t)L.mask[u] >> t0, col = 16 * (task & tm) + n, r = 16 * (g * tpw + (task & tm)) + n;
            if (kg == 0) {
#pragma unroll
                for (uint32_t j = 0; j < 4; j++) {
                    if (j < nt && ((mk >> j) & 1)) {
                        const uint32_t s = SHARED ? K : (L.slot4[u] >> (8 * j)) & 255;
                        L.part[(j * (K + 1) + s) * rw + col] = acc[j];
                        // (untracked store: the combine below reads L.part, never Pg or Psh of this launch from memory)
                        qw_store_f32(SHARED ? a.Psh + (size_t)(t0 + j) * a.D + r : a.P + ((size_t)(t0 + j) * K + s) * a.D + r, acc[j]);
                    }
                }
            }
            acc = f4{0, 0, 0, 0};
        },
        ready, qw_has_lut(F) ? (const uint8_t *)a.glut : nullptr);
}
template <int F, int CH, int FSD, int CHSD>
__device__ __forceinline__ void dnq_body(const qwk_dn_args &a, u2 *lut, qw_dnq_lds &L) {
    const uint32_t K = a.topk, gnb = a.gnb, tid = threadIdx.x, lane = qw_lane(), nq = a.nq, tpw = a.tpw, rw = 16 * tpw;
    uint32_t GU = gnb * K;
    if (GU > QW_DNQ_MAXU) GU = QW_DNQ_MAXU; // (the host admits topk <= 10: 160 at most)
    // workgroup -> (tile group g, quarter q): the quarters of a group are eight workgroups apart, which puts them on one XCD.
    // The nq quarters (2 or 4) share the tokens evenly: sizes differ by one at most, four at most each.
    const uint32_t hi8 = blockIdx.x >> 3, g = (hi8 / nq) * 8 + (blockIdx.x & 7), q = hi8 % nq;
    const uint32_t base = a.nbr / nq, rem = a.nbr % nq, t0 = q * base + (q < rem ? q : rem);
    uint32_t nt = base + (q < rem ? 1 : 0);
    if (nt > 4) nt = 4; // (the host admits 16 tokens in four quarters, 8 in two)
    QW_DSTAMP(6);
    // Everything is asked for at once, in the order in which it is wanted: the record (U, experts, masks, this quarter's slot
    // bytes and gating weights), every H row of the quarter's tokens (which rows they are does not depend on the record)
    // and the table - all through registers, so that the waits are exact (with loads straight into LDS in flight the
    // compiler waits for everything outstanding). The record goes to LDS as soon as it is there, the waves list the
    // experts and ask for their first tiles; rows and table follow into LDS while those tiles are on their way (ready()).
    // A wave's row load takes 8 rows x 128 bytes (whole cache lines), lanes 0 .. 31 the first 64 bytes of a row, 32 .. 63 the rest.
    constexpr uint32_t NW = QW_WG_DN / 64, RPER = (2 * 6 * 8 + NW - 1) / NW; // 2 planes x 6 row blocks x 8 column blocks at most
    constexpr bool TAB = qw_has_lut(F) || qw_has_lut(FSD);
    constexpr uint32_t TPER = TAB ? (QW_LUT_BYTES / 16 + QW_WG_DN - 1) / QW_WG_DN : 0;
    u4 rowv[RPER], tabv[TPER ? TPER : 1];
    uint32_t at[RPER], tat[TPER ? TPER : 1];
    {
        const uint32_t *ue = (const uint32_t *)(a.sel + QW_SEL_OFF_UE(gnb, K)), *mk = (const uint32_t *)(a.sel + QW_SEL_OFF_MASK(gnb, K));
        const uint8_t *sl = a.sel + QW_SEL_OFF_SLOT(gnb, K);
        const float *wg = (const float *)(a.sel + QW_SEL_OFF_W(gnb, K)) + t0 * (K + 1);
        // (GU <= 160 and nt * (K + 1) <= 44: one element a thread; a thread without one reads element 0)
        const bool rec = tid < GU, hasw = tid < nt * (K + 1);
        const uint32_t ri = rec ? tid : 0;
        const uint32_t r_ue = ue[ri], r_mk = mk[ri], r_U = *(const uint32_t *)a.sel;
        uint32_t r_sl[4];
#pragma unroll
        for (uint32_t j = 0; j < 4; j++) r_sl[j] = sl[ri * gnb + t0 + (j < nt ? j : 0)];
        const float r_w = wg[hasw ? tid : 0];
        const uint32_t upr = a.I / 8, cbs = upr / 8, used = nt * (K + 1), nrb = (used + 7) / 8, nunits = 2 * nrb * cbs, wv = qw_wave();
#pragma unroll
        for (uint32_t it = 0; it < RPER; it++) {
            const uint32_t unit = wv + it * NW, cb = unit % cbs, rest = unit / cbs, rb = rest % nrb, pl = rest / nrb;
            const uint32_t r = 8 * rb + ((lane >> 2) & 7), c = 8 * cb + 4 * (lane >> 5) + (lane & 3);
            const bool on = unit < nunits && r < used;
            at[it] = on ? (pl * upr + c) * QW_DNQ_ROWS + r : ~0u;
            // (a unit that is off reads the first bytes of H: a load under a condition made the compiler keep the whole array in scratch memory)
            rowv[it] = *(const u4 *)(on ? a.H + pl * (size_t)a.hplane + ((size_t)t0 * (K + 1) + r) * a.I + 8 * c : a.H);
        }
        if constexpr (TAB) { // every workgroup starts at another place of the table (as qw_lut_copy_issue); the last piece of some threads repeats an earlier one
#pragma unroll
            for (uint32_t it = 0; it < TPER; it++) {
                uint32_t i = tid + it * QW_WG_DN;
                if (i >= QW_LUT_BYTES / 16) i -= QW_WG_DN;
                tat[it] = (i + blockIdx.x * 320u) & (QW_LUT_BYTES / 16 - 1);
                tabv[it] = ((const u4 *)a.glut)[tat[it]];
            }
        }
        if (rec) {
            uint32_t s4 = 0;
#pragma unroll
            for (uint32_t j = 0; j < 4; j++)
                if (j < nt) s4 |= r_sl[j] << (8 * j);
            L.ue[tid] = r_ue, L.mask[tid] = (uint16_t)r_mk, L.slot4[tid] = s4;
        }
        if (hasw) L.wl[tid] = r_w;
        if (tid == 0) L.U = r_U, L.q[0] = blockDim.x >> 6, L.q[1] = 0;
    }
    __syncthreads();
    QW_DSTAMP(7);
    // the unique experts this quarter's tokens picked, in record order: every wave makes the whole list (all write the
    // same values to the same places), so that none waits for another before it asks for its first weights
    uint32_t nv = 0;
    {
        uint32_t U = L.U;
        if (U > GU) U = GU;
        const uint32_t want = (1u << nt) - 1;
        for (uint32_t u0 = 0; u0 < U; u0 += 64) {
            const uint32_t u = u0 + lane;
            const bool on = u < U && (((uint32_t)L.mask[u] >> t0) & want);
            const unsigned long long bal = __ballot(on);
            const uint32_t at = nv + __builtin_amdgcn_mbcnt_hi((uint32_t)(bal >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)bal, 0));
            if (on && at < 48) L.vlist[at] = (uint16_t)u;
            nv += (uint32_t)__popcll(bal);
        }
        if (nv > 48) nv = 48; // (four tokens of ten experts: 40 at most)
    }
    const uint32_t nsh = (FSD != 0 && a.Wsd) ? 1 : 0;
    bool staged = false;
    auto ready = [&] { // called by every wave once it has asked for its first tile
        if (staged) return;
        staged = true;
#pragma unroll
        for (uint32_t it = 0; it < RPER; it++)
            if (at[it] != ~0u) L.hrows[at[it]] = rowv[it];
        if constexpr (TAB) {
#pragma unroll
            for (uint32_t it = 0; it < TPER; it++) ((u4 *)lut)[tat[it]] = tabv[it];
        }
        __syncthreads();
        QW_DSTAMP(8);
    };
    // the routed experts first; the shared expert's tiles go to the waves that leave the routed ones first
    const qw_dnq_view V = {L.hrows, L.part, L.ue, L.slot4, L.mask, L.vlist, L.q};
    dnq_run<F, CH, false, QW_DNQ_ROWS>(a, lut, V, g, t0, nt, nv, ready);
    if (FSD != 0) {
        if (nsh) dnq_run<FSD == 0 ? F : FSD, CHSD, true, QW_DNQ_ROWS>(a, lut, V, g, t0, nt, 1, ready);
    }
    QW_DSTAMP(9);
    __syncthreads();
    for (uint32_t j = tid; j < nt * rw; j += blockDim.x) { // rank order, then the shared expert (qwk_cmb's arithmetic)
        const uint32_t t = j >> (4 + __builtin_ctz(tpw)), i = j & (rw - 1), r = g * rw + i;
        const float *w = L.wl + t * (K + 1), *p = L.part + t * (K + 1) * rw + i;
        float o = 0;
        for (uint32_t s = 0; s < K; s++) o = __builtin_fmaf(w[s], p[s * rw], o);
        float sh;
        if (nsh) sh = p[K * rw];
        else sh = a.Psh[(size_t)(t0 + t) * a.D + r]; // the caller's own shared product
        o = __builtin_fmaf(w[K], sh, o);
        a.out[(size_t)(t0 + t) * a.D + r] = qw_f2h(o);
    }
    QW_DSTAMP(14);
}
#define QW_DNQ(F, CH, FSD, CHSD, NAME)                                                              \
    extern "C" __global__ __launch_bounds__(QW_WG_DN) void NAME(qwk_dn_args a) {                    \
        __shared__ struct { u2 lut[QW_LUT_ENTRIES]; qw_dnq_lds d; } L;                               \
        dnq_body<F, CH, FSD, CHSD>(a, L.lut, L.d);                                                  \
    }
#if QW_IN_PART(4)
QW_DNQ(121, 2, 0, 1, qwk_dnq_f121_c2) QW_DNQ(121, 2, 121, 2, qwk_dnq_f121_c2_s121_c2) QW_DNQ(121, 2, 8, 4, qwk_dnq_f121_c2_s8_c4)
QW_DNQ(121, 1, 0, 1, qwk_dnq_f121_c1) QW_DNQ(121, 1, 121, 1, qwk_dnq_f121_c1_s121_c1) QW_DNQ(121, 1, 8, 4, qwk_dnq_f121_c1_s8_c4)
#endif

// ================================================================ routed gate/up, down and combine as one launch
// (kernels/moe_gg.metal:600-663 in one pass.) Three launches a layer each pay their own start: the launch itself, the
// table and the record into LDS, the first round trip to memory. Here the persistent workgroups of the gate/up launch go
// on into the down projection: the table and the selection stay in LDS, and every wave asks for its first down tiles
// before it waits for the others. What the two phases hand over is H, produced column by column all over the grid and
// consumed row by row: the SwiGLU values of a workgroup's tiles are kept in LDS while it streams (a store of device
// scope among the weight loads would hold up every wait for them) and leave in one burst of device-scope stores at the
// end; then one barrier over the grid; then every workgroup stages the H rows of its share of the tokens with loads
// of device scope and runs the down projection and the combine exactly as qwk_dnq_* does. Pg, Psh, H and the record
// are left in memory as the separate launches leave them.
struct qw_h_lds { // the gate/up phase's SwiGLU values in LDS: entry = one (tile, token), eight columns
    uint32_t *count, *off, *val; // val: hi | lo << 16
    uint16_t *H;
    uint32_t hplane, base;
    __device__ __forceinline__ void stamp(uint32_t k) const { QW_DSTAMP(k); }
    __device__ __forceinline__ void tile(uint32_t m) {
        uint32_t b = 0;
        if (qw_lane() == 0) b = atomicAdd(count, (uint32_t)__builtin_popcount(m));
        base = (uint32_t)__builtin_amdgcn_readfirstlane((int)b);
    }
    __device__ __forceinline__ void put(uint32_t m, uint32_t tok, size_t o, uint16_t hi, uint16_t lo) const {
        const uint32_t idx = base + (uint32_t)__builtin_popcount(m & ((1u << tok) - 1)), n = qw_lane() & 7;
        if (idx < QW_GUD_HCAP) {
            val[idx * 8 + n] = (uint32_t)hi | (uint32_t)lo << 16;
            if (n == 0) off[idx] = (uint32_t)o;
        } else { // (more results than the buffer holds: straight to memory)
            __hip_atomic_store(H + o, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(H + o + hplane, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
};
struct qw_gud_lds {
    u2 lut[QW_LUT_ENTRIES];
    union {
        u4 xf[QW_XF_MAXK * 2];                 // gate/up phase: the activations (and the selection's per-wave scratch behind them)
        u4 hrows[2 * 64 * QW_GUD_ROWS];        // down phase: the H rows of the share's tokens
    } big;
    qw_sel_cache sc;
    union {
        qw_sel_scratch ss;                                                    // while the selection is made
        struct { uint32_t off[QW_GUD_HCAP], val[QW_GUD_HCAP * 8]; } hb;       // gate/up phase
        float part[2 * 11 * 64];                                              // down phase: [local token][slot][row of the group]
    } u;
    float wl[QW_GUD_SHARE * 11];
    uint32_t ue[QW_DNQ_MAXU], slot4[QW_DNQ_MAXU];
    uint16_t mask[QW_DNQ_MAXU], vlist[32];
    uint32_t hcount, bail, dq[2];
};
static_assert(sizeof(qw_gud_lds) <= 160 * 1024, "LDS of the fused launch");
static_assert(QW_GUD_SHARE * 11 * 32 <= 2 * 11 * 64, "part holds three tokens by two tiles or two tokens by four");
#define QW_STAMP(k) QW_DSTAMP(k)
template <int FSD, int CHSD> __device__ __forceinline__ void gud_body(const qwk_gud_args &ga, qw_gud_lds &L) {
    constexpr int F = QW_F_PACKED, CH = 2; // tile-major IQ3_S, D a multiple of 512, I = 512
    const qwk_gu_args &a = ga.gu;
    const qwk_dn_args &d = ga.dn;
    const uint32_t K = d.topk, gnb = d.gnb, tid = threadIdx.x, lane = qw_lane(), nq = d.nq, tpw = d.tpw, rw = 16 * tpw;
    uint32_t gen0 = 0;
    QW_STAMP(0);
    if (tid == 0) gen0 = qw_ld_coh(ga.sync + QW_SYNC_GEN);
    // the down phase's place of this workgroup: tile group g, share q of the tokens (the shares of a group are eight
    // workgroups apart: one XCD); workgroups past the last group only take part in the gate/up phase
    const uint32_t hi8 = blockIdx.x >> 3, g = (hi8 / nq) * 8 + (blockIdx.x & 7), q = hi8 % nq;
    const bool active = g < d.D / 16 / tpw;
    const uint32_t base = d.nbr / nq, rem = d.nbr % nq, t0 = q * base + (q < rem ? q : rem);
    uint32_t nt = base + (q < rem ? 1 : 0);
    if (nt > QW_GUD_SHARE) nt = QW_GUD_SHARE; // (the host keeps the shares that small)
    uint32_t nv = 0;
    qw_h_lds hs = {&L.hcount, L.u.hb.off, L.u.hb.val, a.H, a.hplane, 0};
    gu_body<F, CH, 0, 1>(a, L.lut, L.big.xf, &L.sc, &L.u.ss, hs, true, [&] {
        // the down phase's lists, made while everything they come from is in LDS: gating weights of the share's tokens,
        // experts, masks, the share's slot bytes, and the unique experts its tokens picked in record order (every wave
        // makes the whole list: all write the same values)
        uint32_t GU = gnb * K;
        if (GU > QW_DNQ_MAXU) GU = QW_DNQ_MAXU;
        for (uint32_t i = tid; i < nt * (K + 1); i += blockDim.x) L.wl[i] = L.u.ss.w[t0 * (K + 1) + i];
        for (uint32_t i = tid; i < GU; i += blockDim.x) {
            uint32_t s4 = 0;
            for (uint32_t j = 0; j < nt; j++) s4 |= (uint32_t)L.sc.slot[i * gnb + t0 + j] << (8 * j);
            L.ue[i] = L.sc.ue[i], L.mask[i] = (uint16_t)L.sc.mask[i], L.slot4[i] = s4;
        }
        if (tid == 0) L.hcount = 0, L.bail = 0, L.dq[0] = blockDim.x >> 6, L.dq[1] = 0;
        uint32_t U = L.sc.U;
        if (U > GU) U = GU;
        const uint32_t want = (1u << nt) - 1;
        for (uint32_t u0 = 0; u0 < U; u0 += 64) {
            const uint32_t u = u0 + lane;
            const bool on = active && u < U && ((L.sc.mask[u] >> t0) & want);
            const unsigned long long bal = __ballot(on);
            const uint32_t at = nv + __builtin_amdgcn_mbcnt_hi((uint32_t)(bal >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)bal, 0));
            if (on && at < 32) L.vlist[at] = (uint16_t)u;
            nv += (uint32_t)__popcll(bal);
        }
        if (nv > 32) nv = 32; // (three tokens of ten experts: 30 at most)
        __syncthreads(); // the selection's scratch becomes the buffer of SwiGLU values
    });
    const uint32_t nsh = (FSD != 0 && d.Wsd) ? 1 : 0;
    bool met = false;
    // Once per wave, behind its first down loads (or straight away for a workgroup without a share): the hand-over.
    auto meet = [&] {
        if (met) return;
        met = true;
        QW_STAMP(3);
        __syncthreads(); // every wave of the workgroup has left the gate/up phase
        QW_STAMP(4);
        uint32_t cnt = L.hcount;
        if (cnt > QW_GUD_HCAP) cnt = QW_GUD_HCAP;
        for (uint32_t i = tid; i < cnt * 4; i += blockDim.x) { // two columns a thread, a dword a plane
            const uint32_t e = i >> 2, c = 2 * (i & 3), v0 = L.u.hb.val[e * 8 + c], v1 = L.u.hb.val[e * 8 + c + 1];
            uint32_t *p = (uint32_t *)(a.H + L.u.hb.off[e] + c);
            qw_st_coh(p, (v0 & 0xffffu) | (v1 << 16));
            qw_st_coh(p + a.hplane / 2, (v0 >> 16) | (v1 & 0xffff0000u));
        }
        __builtin_amdgcn_s_waitcnt(0); // this wave's stores (and its first down loads) have completed
        __syncthreads();
        QW_STAMP(5);
        if (tid == 0 && !qw_grid_barrier(ga.sync, gen0, 1, gridDim.x, ga.spin_limit)) L.bail = 1;
        __syncthreads();
        QW_STAMP(6);
        if (!active || L.bail) return;
        // every H row of the share's tokens into LDS in fragment order: a wave's load takes 8 rows x 128 bytes (whole
        // cache lines), lanes 0 .. 31 the first 64 bytes of a row, 32 .. 63 the rest
        const uint32_t upr = d.I / 8, cbs = upr / 8, used = nt * (K + 1), nrb = (used + 7) / 8, nunits = 2 * nrb * cbs, wv = qw_wave();
        constexpr uint32_t NW = QW_WG_GU / 64, PER = (2 * ((QW_GUD_ROWS + 7) / 8) * 8 + NW - 1) / NW; // 2 planes x 5 row blocks x 8 column blocks at most
        static_assert(PER == 7, "qw_ld_coh7 takes seven loads");
        u4 t[PER];
        const u4 *src[PER];
        uint32_t at[PER];
#pragma unroll
        for (uint32_t it = 0; it < PER; it++) {
            const uint32_t unit = wv + it * NW, cb = unit % cbs, rest = unit / cbs, rb = rest % nrb, pl = rest / nrb;
            const uint32_t r = 8 * rb + ((lane >> 2) & 7), c = 8 * cb + 4 * (lane >> 5) + (lane & 3);
            const bool on = unit < nunits && r < used;
            at[it] = on ? (pl * upr + c) * QW_GUD_ROWS + r : ~0u;
            src[it] = (const u4 *)(on ? d.H + pl * (size_t)d.hplane + ((size_t)t0 * (K + 1) + r) * d.I + 8 * c : d.H); // (off: a valid address, not kept)
        }
        qw_ld_coh7(t, src);
#pragma unroll
        for (uint32_t it = 0; it < PER; it++)
            if (at[it] != ~0u) L.big.hrows[at[it]] = t[it];
        __syncthreads();
        QW_STAMP(7);
    };
    if (!active) {
        meet();
        return;
    }
    const qw_dnq_view V = {L.big.hrows, L.u.part, L.ue, L.slot4, L.mask, L.vlist, L.dq};
    // the routed experts first; the shared expert's tiles go to the waves that the routed deal gave one tile fewer
    dnq_run<F, CH, false, QW_GUD_ROWS>(d, L.lut, V, g, t0, nt, nv, meet);
    if (FSD != 0) {
        if (nsh) dnq_run<FSD == 0 ? F : FSD, CHSD, true, QW_GUD_ROWS>(d, L.lut, V, g, t0, nt, 1, meet);
    }
    meet();
    QW_STAMP(8);
    __syncthreads();
    QW_STAMP(9);
    if (L.bail) return;
    for (uint32_t j = tid; j < nt * rw; j += blockDim.x) { // rank order, then the shared expert (qwk_cmb's arithmetic)
        const uint32_t t = j >> (4 + __builtin_ctz(tpw)), i = j & (rw - 1), r = g * rw + i;
        const float *w = L.wl + t * (K + 1), *p = L.u.part + t * (K + 1) * rw + i;
        float o = 0;
        for (uint32_t s = 0; s < K; s++) o = __builtin_fmaf(w[s], p[s * rw], o);
        float sh;
        if (nsh) sh = p[K * rw];
        else sh = d.Psh[(size_t)(t0 + t) * d.D + r]; // the caller's own shared product
        o = __builtin_fmaf(w[K], sh, o);
        d.out[(size_t)(t0 + t) * d.D + r] = qw_f2h(o);
    }
}
#define QW_GUD(FSD, CHSD, NAME)                                                                     \
    extern "C" __global__ __launch_bounds__(QW_WG_GU) void NAME(qwk_gud_args a) {                   \
        __shared__ qw_gud_lds L;                                                                    \
        gud_body<FSD, CHSD>(a, L);                                                                  \
    }
#if QW_IN_PART(4)
QW_GUD(0, 1, qwk_gud_f121_c2) QW_GUD(121, 2, qwk_gud_f121_c2_s121_c2) QW_GUD(8, 4, qwk_gud_f121_c2_s8_c4)
#endif

// Any I (multiple of the block size): one tile at a time, operand A straight from global memory.
template <int F> __device__ __forceinline__ void dn_any_tiles(const qwk_dn_args &a, const u2 *lut, const qw_sel_cache *sc, uint32_t w0, uint32_t nw) {
    typedef qw_chunk<F, 1> C;
    const uint32_t lane = qw_lane(), n = lane & 15, kg = lane >> 4, K = a.topk, gnb = a.gnb;
    const uint32_t tpe = a.D / 16, ntasks = sc->U * tpe, cpr = a.I / C::BLK_K;
    for (uint32_t task = w0; task < ntasks; task += nw) {
        const uint32_t u = task / tpe, r = 16 * (task % tpe) + n, m = sc->mask[u];
        qw_afrag_glb<true> af = {nullptr, nullptr};
        if (n < a.nbr && ((m >> n) & 1)) {
            af.rowhi = a.H + ((size_t)n * (K + 1) + sc->slot[u * gnb + n]) * a.I;
            af.rowlo = af.rowhi + a.hplane;
        }
        const uint8_t *row = a.Wd + ((size_t)sc->ue[u] * a.D + 16 * (task % tpe) + (lane >> 2)) * a.rowbytes; // quad order
        f4 acc = {0, 0, 0, 0};
        qw_pipeline<C>(cpr, [&](uint32_t i, C &c) { c.load(row + (size_t)i * C::BLK_B, lane & 3); },
                       [&](uint32_t i, const C &c) { c.mac(lut, af, i * C::BLK_K, kg, acc); });
#pragma unroll
        for (uint32_t j = 0; j < 4; j++) {
            const uint32_t tok = 4 * kg + j;
            if (tok < a.nbr && ((m >> tok) & 1)) a.P[((size_t)tok * K + sc->slot[u * gnb + tok]) * a.D + r] = acc[j];
        }
    }
}
template <int F, int FSD> __device__ __forceinline__ void dn_any_body(const qwk_dn_args &a, u2 *lut, qw_sel_cache *sc) {
    if (F == 21 || FSD == 21) qw_lut_copy(lut, (const u2 *)a.glut);
    if (F == 20 || FSD == 20) qw_kq_tab_build((uint32_t *)lut); // the byte table of the 4-bit codebook (IQ3_S never meets it here)
    qw_sel_load(*sc, a.sel, a.topk, a.gnb);
    __syncthreads();
    const uint32_t nw = gridDim.x * (blockDim.x >> 6), w0 = qw_wave() * gridDim.x + blockIdx.x /* wave-major: see gu_body */;
    if (FSD != 0) {
        if (a.Wsd) shared_down_tiles<FSD == 0 ? 8 : FSD, 1>(a, lut, w0, nw);
    }
    dn_any_tiles<F>(a, lut, sc, w0, nw);
}
// The same with both ggml types as arguments (qwk_dn_args.fd, fsd): every pair of types the reference's kernel takes
// (kernels/moe_gg.metal:336-395) that has no build of its own above. IQ3_S reads the big table, the 4-bit codebooks the
// byte table behind it.
__device__ __forceinline__ void dn_rt_body(const qwk_dn_args &a, u2 *lut, qw_sel_cache *sc) {
    const u2 *tab = lut + QW_LUT_ENTRIES;
    if (a.fd == 21 || a.fsd == 21) qw_lut_copy(lut, (const u2 *)a.glut);
    qw_kq_tab_build((uint32_t *)tab);
    qw_sel_load(*sc, a.sel, a.topk, a.gnb);
    __syncthreads();
    const uint32_t nw = gridDim.x * (blockDim.x >> 6), w0 = qw_wave() * gridDim.x + blockIdx.x;
    if (a.Wsd) switch (a.fsd) {
        case 8: shared_down_tiles<8, 1>(a, lut, w0, nw); break;
        case 21: shared_down_tiles<21, 1>(a, lut, w0, nw); break;
        case 20: shared_down_tiles<20, 1>(a, tab, w0, nw); break;
        case 12: shared_down_tiles<12, 1>(a, tab, w0, nw); break;
        case 13: shared_down_tiles<13, 1>(a, tab, w0, nw); break;
        case 14: shared_down_tiles<14, 1>(a, tab, w0, nw); break;
        case 23: shared_down_tiles<23, 1>(a, tab, w0, nw); break;
        default: break; // (the host launches this kernel for these seven only)
        }
    switch (a.fd) {
    case 8: dn_any_tiles<8>(a, lut, sc, w0, nw); break;
    case 21: dn_any_tiles<21>(a, lut, sc, w0, nw); break;
    case 20: dn_any_tiles<20>(a, tab, sc, w0, nw); break;
    case 12: dn_any_tiles<12>(a, tab, sc, w0, nw); break;
    case 13: dn_any_tiles<13>(a, tab, sc, w0, nw); break;
    case 14: dn_any_tiles<14>(a, tab, sc, w0, nw); break;
    case 23: dn_any_tiles<23>(a, tab, sc, w0, nw); break;
    default: break;
    }
}
#if QW_IN_PART(2)
extern "C" __global__ __launch_bounds__(QW_WG) void qwk_dn_rt(qwk_dn_args a) {
    __shared__ struct { u2 lut[QW_LUT_ENTRIES + QW_KQ_TAB / 2]; qw_sel_cache sc; } L;
    dn_rt_body(a, L.lut, &L.sc);
}
#endif
#define QW_DN_ANY(F, FSD, NAME)                                                       \
    extern "C" __global__ __launch_bounds__(QW_WG) void NAME(qwk_dn_args a) {         \
        __shared__ struct { u2 lut[(F == 21 || FSD == 21) ? QW_LUT_ENTRIES : (F == 20 || FSD == 20) ? QW_KQ_TAB / 2 : 1]; qw_sel_cache sc; } L; \
        dn_any_body<F, FSD>(a, L.lut, &L.sc);                                         \
    }
#if QW_IN_PART(2)
QW_DN_ANY(21, 0, qwk_dn_f21_any) QW_DN_ANY(21, 21, qwk_dn_f21_any_s21) QW_DN_ANY(21, 8, qwk_dn_f21_any_s8)
QW_DN_ANY(8, 0, qwk_dn_f8_any) QW_DN_ANY(8, 21, qwk_dn_f8_any_s21) QW_DN_ANY(8, 8, qwk_dn_f8_any_s8)
#endif
// IQ4_NL down rows (the routed and shared down projections of a layer with I = 640, bench/moe_bw.c:22-24 of the reference)
#if QW_IN_PART(2)
QW_DN_ANY(20, 0, qwk_dn_f20_any) QW_DN_ANY(20, 20, qwk_dn_f20_any_s20) QW_DN_ANY(20, 8, qwk_dn_f20_any_s8)
#endif

// ================================================================ ragged packing (kernels/moe_prefill.metal:15-119)
// P (token, expert) pairs -> per-expert counts -> exclusive prefix sums (first packed row of every expert, tile table)
// -> rows copied to packed order -> grouped product -> gathered, weighted sum. Integer work; bit-exact.
// The counters are cleared on the device, inside the recorded sequence (kernels/prefill.metal:601-603): a batch may hold
// the packing sequence several times, and all of it is recorded before any of it runs.
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(256) void qwk_zero(qwk_zero_args a) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < a.n) a.x[i] = 0;
}
extern "C" __global__ __launch_bounds__(256) void qwk_moe_count(qwk_count_args a) {
    const uint32_t p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p < a.P && a.ids[p] < a.E) atomicAdd(&a.counts[a.ids[p]], 1u);
}
#endif
// One workgroup of 1024 threads, thread e = expert e (E <= 1024): two exclusive scans (rows, tiles) by ballot-free
// wave scans (DPP row shifts through __shfl_up) and one pass over the sixteen wave totals.
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(1024) void qwk_moe_plan(qwk_plan_args a) {
    __shared__ uint32_t wr[16], wt[16];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t c = tid < a.E ? a.counts[tid] : 0, nt = (c + a.tm - 1) / a.tm;
    uint32_t pr = c, pt = nt; // inclusive scans inside the wave
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const uint32_t ur = __shfl_up(pr, o), ut = __shfl_up(pt, o);
        if (lane >= (uint32_t)o) pr += ur, pt += ut;
    }
    if (lane == 63) wr[wave] = pr, wt[wave] = pt;
    __syncthreads();
    uint32_t br = 0, bt = 0, total_t = 0;
    for (uint32_t w = 0; w < 16; w++) {
        if (w < wave) br += wr[w], bt += wt[w];
        total_t += wt[w];
    }
    const uint32_t row0 = br + pr - c, tile0 = bt + pt - nt;
    if (tid < a.E) {
        a.offs[tid] = row0;
        a.cursor[tid] = row0;
        for (uint32_t t = 0; t < nt; t++) {
            const uint32_t r = row0 + t * a.tm;
            if (tile0 + t < a.max_tiles) *(u4 *)(a.tiles + 4 * (tile0 + t)) = u4{tid, r, r + a.tm < row0 + c ? r + a.tm : row0 + c, 0};
        }
    }
    for (uint32_t t = total_t + tid; t < a.max_tiles; t += blockDim.x) *(u4 *)(a.tiles + 4 * t) = u4{0, 0, 0, 0}; // unused entries
}
#endif
// One workgroup per pair: take the next row of the pair's expert, remember it, copy the token's row there.
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(256) void qwk_moe_scatter(qwk_scatter_args a) {
    __shared__ uint32_t pos;
    const uint32_t p = blockIdx.x;
    if (threadIdx.x == 0) {
        const uint32_t e = a.ids[p];
        pos = e < a.E ? atomicAdd(&a.cursor[e], 1u) : 0xffffffffu;
        a.pos_of[p] = pos;
    }
    __syncthreads();
    if (pos >= a.P) return; // an expert id outside the table: the pair is dropped
    const u4 *src = (const u4 *)(a.X + (size_t)(p / a.topk) * a.KD);
    u4 *dst = (u4 *)(a.Xs + (size_t)pos * a.KD);
    for (uint32_t i = threadIdx.x; i < a.KD / 8; i += blockDim.x) dst[i] = src[i];
}
#endif
// The four launches above as one, for a step of a few thousand pairs at most: a workgroup per pair, and every workgroup
// counts all pairs itself (LDS atomics over the P ids), which gives it its own packed row without a hand-over: the rows
// of the experts below its own plus the earlier pairs of its own expert. The order inside an expert is therefore the
// order of the pairs (the cursor form leaves whatever order the atomics came in; both are permutations the grouped
// product and the combine do not care about). Workgroup 0 also leaves counts, offsets, cursors (where the scatter
// would have left them) and the tile table.
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(256) void qwk_moe_prep(qwk_prep_args a) {
    __shared__ uint32_t cnt[1024], red[4], wr[4], wt[4];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, p = blockIdx.x;
    const uint32_t ep = (uint32_t)__builtin_amdgcn_readfirstlane((int)a.ids[p]);
    for (uint32_t e = tid; e < a.E; e += 256) cnt[e] = 0;
    __syncthreads();
    uint32_t mine = 0; // earlier pairs of this pair's expert
    for (uint32_t q = tid; q < a.P; q += 256) {
        const uint32_t e = a.ids[q];
        if (e < a.E) atomicAdd(&cnt[e], 1u);
        mine += e == ep && q < p;
    }
    __syncthreads();
    if (ep < a.E)
        for (uint32_t e = tid; e < ep; e += 256) mine += cnt[e]; // rows of the experts below
#pragma unroll
    for (int o = 32; o; o >>= 1) mine += __shfl_xor(mine, o);
    if (lane == 0) red[wave] = mine;
    __syncthreads();
    const uint32_t pos = ep < a.E ? red[0] + red[1] + red[2] + red[3] : 0xffffffffu; // an expert id outside the table: the pair is dropped
    if (tid == 0) a.pos_of[p] = pos;
    if (pos < a.P) {
        const u4 *src = (const u4 *)(a.X + (size_t)(p / a.topk) * a.KD);
        u4 *dst = (u4 *)(a.Xs + (size_t)pos * a.KD);
        for (uint32_t i = tid; i < a.KD / 8; i += 256) dst[i] = src[i];
    }
    if (blockIdx.x != 0) return;
    // the tables (qwk_moe_plan's arithmetic): thread t has experts 4 t .. 4 t + 3
    uint32_t c[4], nt[4], sr = 0, st = 0;
#pragma unroll
    for (uint32_t i = 0; i < 4; i++) {
        const uint32_t e = 4 * tid + i;
        c[i] = e < a.E ? cnt[e] : 0, nt[i] = (c[i] + a.tm - 1) / a.tm;
        sr += c[i], st += nt[i];
    }
    uint32_t pr = sr, pt = st; // inclusive scans inside the wave
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const uint32_t ur = __shfl_up(pr, o), ut = __shfl_up(pt, o);
        if (lane >= (uint32_t)o) pr += ur, pt += ut;
    }
    if (lane == 63) wr[wave] = pr, wt[wave] = pt;
    __syncthreads();
    uint32_t row0 = pr - sr, tile0 = pt - st, total_t = 0;
    for (uint32_t w = 0; w < 4; w++) {
        if (w < wave) row0 += wr[w], tile0 += wt[w];
        total_t += wt[w];
    }
#pragma unroll
    for (uint32_t i = 0; i < 4; i++) {
        const uint32_t e = 4 * tid + i;
        if (e < a.E) {
            a.counts[e] = c[i], a.offs[e] = row0, a.cursor[e] = row0 + c[i];
            for (uint32_t t = 0; t < nt[i]; t++) {
                const uint32_t r = row0 + t * a.tm;
                if (tile0 + t < a.max_tiles) *(u4 *)(a.tiles + 4 * (tile0 + t)) = u4{e, r, r + a.tm < row0 + c[i] ? r + a.tm : row0 + c[i], 0};
            }
        }
        row0 += c[i], tile0 += nt[i];
    }
    for (uint32_t t = total_t + tid; t < a.max_tiles; t += 256) *(u4 *)(a.tiles + 4 * t) = u4{0, 0, 0, 0}; // unused entries
}
#endif
// H = SiLU(gate) * up, binary16 in and out, the product rounded once (kernels/moe_prefill.metal:95-103, kernels/prefill.metal:485-488)
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(256) void qwk_moe_act(qwk_act_args a) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= a.n) return;
    float g, u;
    if (a.U) g = qw_h2f(a.G[i]), u = qw_h2f(a.U[i]);
    else {
        const uint32_t r = i / a.I, j = i % a.I;
        g = qw_h2f(a.G[(size_t)r * 2 * a.I + j]), u = qw_h2f(a.G[(size_t)r * 2 * a.I + a.I + j]);
    }
    a.H[i] = qw_f2h(g / (1.0f + __expf(-g)) * u);
}
#endif
// y[t][c] = sum_s w[t][s] * D[pos_of[t][s]][c] in rank order; one thread per (token, 4 columns).
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(64) void qwk_moe_combine(qwk_combine_args a) {
    const uint32_t c4 = blockIdx.x * blockDim.x + threadIdx.x, t = blockIdx.y;
    if (c4 >= a.KD / 4 || t >= a.T) return;
    float acc[4] = {0, 0, 0, 0};
    for (uint32_t s = 0; s < a.topk; s++) {
        const uint32_t p = t * a.topk + s, pos = a.pos_of[p];
        if (pos >= a.P) continue;
        const u2 v = *(const u2 *)(a.Dm + (size_t)pos * a.KD + 4 * c4);
        const float w = a.w[p];
        acc[0] += w * qw_h2f((uint16_t)v.x), acc[1] += w * qw_h2f((uint16_t)(v.x >> 16));
        acc[2] += w * qw_h2f((uint16_t)v.y), acc[3] += w * qw_h2f((uint16_t)(v.y >> 16));
    }
    u2 o;
    o.x = (uint32_t)qw_f2h(acc[0]) | (uint32_t)qw_f2h(acc[1]) << 16;
    o.y = (uint32_t)qw_f2h(acc[2]) | (uint32_t)qw_f2h(acc[3]) << 16;
    *(u2 *)(a.Y + (size_t)t * a.KD + 4 * c4) = o;
}
#endif

// SwiGLU at the end of a tile of 8 gate + 8 up rows (a.H given): lane n < 8 has the gate value of a packed row and a
// column, lane n + 8 the up value of the same two; both as the binary16 the G and U buffers hold, the product rounded
// once, exactly as qwk_moe_act computes it from those buffers. Called by all lanes.
__device__ __forceinline__ void qw_pf_act(const qwk_pf_args &a, uint16_t y, uint32_t m, bool store, uint32_t col) {
    const float g = qw_h2f(y), u = qw_h2f((uint16_t)__shfl_xor((int)y, 8));
    if (store) a.H[(size_t)m * a.N + col] = qw_f2h(g / (1.0f + __expf(-g)) * u);
}
// Grouped product over the packed rows (kernels/moe_gg.metal:761-838): task = (tile entry, 16 weight rows); the
// weights of a task are decoded once and multiplied into up to four groups of 16 packed rows of the entry
// (tm <= 64). The non-empty entries are the first ones of the table; their number is counted here.
template <int F, int CH> __device__ __forceinline__ void pf_body(const qwk_pf_args &a, u2 *lut, u4 *tl /* max_tiles entries */, uint32_t *cnt) {
    typedef qw_chunk<F, CH> C;
    const uint32_t lane = qw_lane(), n = lane & 15, kg = lane >> 4;
    if (threadIdx.x == 0) *cnt = 0;
    if (qw_has_lut(F)) qw_lut_copy(lut, (const u2 *)a.glut);
    if (F == 20) qw_kq_tab_build((uint32_t *)lut); // the byte table of the 4-bit codebook
    __syncthreads();
    uint32_t mine = 0;
    for (uint32_t t = threadIdx.x; t < a.max_tiles; t += blockDim.x) {
        const u4 e = *(const u4 *)(a.tiles + 4 * t);
        tl[t] = e;
        mine += e.z > e.y;
    }
    if (mine) atomicAdd(cnt, mine);
    __syncthreads();
    const uint32_t used = *cnt, ntn = a.ntn, ntasks = used * ntn, cpr = a.K / (C::BLK_K * CH);
    const uint32_t nw = gridDim.x * (blockDim.x >> 6), w0 = qw_wave() * gridDim.x + blockIdx.x /* wave-major: see gu_body */;
    f4 acc[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
    qw_task_pipeline<C>(ntasks, w0, nw, cpr, CH * C::BLK_B, F == QW_F_PACKED ? lane : lane & 3,
        [&](uint32_t task) {
            const u4 e = tl[task / ntn];
            if constexpr (F == QW_F_PACKED) return a.W + ((size_t)e.x * ntn + task % ntn) * a.rowbytes; // the tile's slabs
            else return a.W + ((size_t)e.x * a.N + 16 * (task % ntn) + (lane >> 2)) * a.rowbytes;
        },
        [&](uint32_t task, uint32_t ci, const C &c) {
            const u4 e = tl[task / ntn];
            const uint32_t m0 = e.y, m1 = e.z, ng = (m1 - m0 + 15) / 16;
            const uint16_t *rows[4];
#pragma unroll
            for (uint32_t g = 0; g < 4; g++) {
                const uint32_t m = m0 + 16 * g + n;
                rows[g] = a.X + (size_t)(m < m1 ? m : m1 - 1) * a.K; // rows past the entry repeat its last row; never stored
            }
            const uint32_t k0 = ci * CH * C::BLK_K;
            if (ng <= 1) {
                const uint16_t *const r1[1] = {rows[0]};
                f4 a1[1] = {acc[0]};
                c.template mac_groups<1>(lut, r1, k0, kg, a1);
                acc[0] = a1[0];
            } else if (ng == 2) {
                const uint16_t *const r2[2] = {rows[0], rows[1]};
                f4 a2[2] = {acc[0], acc[1]};
                c.template mac_groups<2>(lut, r2, k0, kg, a2);
                acc[0] = a2[0], acc[1] = a2[1];
            } else {
                const uint16_t *const r4[4] = {rows[0], rows[1], rows[2], rows[3]};
                c.template mac_groups<4>(lut, r4, k0, kg, acc);
            }
            if (ci + 1 != cpr) return;
            // a tile of two matrices: rows 0..7 are matrix A's (-> Y), rows 8..15 matrix B's (-> Y1)
            const bool second = a.split == 8 && n >= 8;
            const uint32_t col = a.split == 8 ? 8 * (task % ntn) + (n & 7) : 16 * (task % ntn) + n;
            uint16_t *Y = second ? a.Y1 : a.Y;
#pragma unroll
            for (uint32_t g = 0; g < 4; g++) {
#pragma unroll
                for (uint32_t j = 0; j < 4; j++) {
                    const uint32_t m = m0 + 16 * g + 4 * kg + j;
                    const uint16_t y = qw_f2h(acc[g][j]);
                    if (m < m1) Y[(size_t)m * a.N + col] = y;
                    if (a.H) qw_pf_act(a, y, m, m < m1 && !second, col);
                }
                acc[g] = f4{0, 0, 0, 0};
            }
        });
}
#define QW_PF(F, CH, NAME)                                                                       \
    extern "C" __global__ __launch_bounds__(QW_WG) void NAME(qwk_pf_args a) {                    \
        __shared__ struct { u2 lut[qw_has_lut(F) ? QW_LUT_ENTRIES : F == 20 ? QW_KQ_TAB / 2 : 1]; u4 tl[2048]; uint32_t cnt; } L; \
        pf_body<F, CH>(a, L.lut, L.tl, &L.cnt);                                                  \
    }
#if QW_IN_PART(5)
QW_PF(21, 2, qwk_pf_f21_c2) QW_PF(21, 1, qwk_pf_f21_c1) QW_PF(8, 4, qwk_pf_f8_c4)
QW_PF(20, 4, qwk_pf_f20_c4) // IQ4_NL rows (the down projection of the reference model's layer: K = 640)
QW_PF(121, 2, qwk_pf_f121_c2) QW_PF(121, 1, qwk_pf_f121_c1) // tile-major IQ3_S: one matrix, or gate and up rows side by side
#endif

// The same product for entries of at most 16 packed rows over tile-major weights, the way the decode kernels work:
// a workgroup takes a contiguous range of (entry, weight tile) tasks - the tiles of one entry, or the end of one and
// the start of the next -, copies the entry's rows into LDS in fragment order once (after its first weight loads are
// issued) and its waves walk the tiles with the activations read from LDS.
template <int CH> __device__ __forceinline__ void pf_range_body(const qwk_pf_args &a, u2 *lut, u4 *xf, uint32_t *cnt) {
    typedef qw_chunk<QW_F_PACKED, CH> C;
    const uint32_t lane = qw_lane(), n = lane & 15, kg = lane >> 4, nwv = blockDim.x >> 6;
    if (threadIdx.x == 0) *cnt = 0;
    qw_lut_copy_issue(lut, (const u2 *)a.glut); // lands while the table of entries is read: one memory round trip for both
    __syncthreads();
    uint32_t mine = 0; // the non-empty entries are the first ones of the table
    for (uint32_t t = threadIdx.x; t < a.max_tiles; t += blockDim.x) {
        const u4 e = *(const u4 *)(a.tiles + 4 * t);
        mine += e.z > e.y;
    }
    if (mine) atomicAdd(cnt, mine);
    qw_lds_arrive();
    __syncthreads();
    const uint32_t used = *cnt, ntn = a.ntn, total = used * ntn, cpr = a.K / (C::BLK_K * CH);
    const uint32_t per = (total + gridDim.x - 1) / gridDim.x;
    const uint32_t end = (blockIdx.x + 1) * per < total ? (blockIdx.x + 1) * per : total;
    for (uint32_t pos = blockIdx.x * per; pos < end;) {
        const uint32_t entry = pos / ntn, t0 = pos % ntn, nt = ntn - t0 < end - pos ? ntn - t0 : end - pos;
        const u4 e = *(const u4 *)(a.tiles + 4 * entry);
        const uint32_t m0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)e.y), m1 = (uint32_t)__builtin_amdgcn_readfirstlane((int)e.z);
        const uint8_t *W = a.W + ((size_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)e.x) * ntn + t0) * a.rowbytes;
        bool staged = false;
        auto ready = [&] {
            if (staged) return;
            staged = true;
            __syncthreads(); // the waves are done with the rows of the segment before
            qw_stage_x(xf, a.X + (size_t)m0 * a.K, a.K, a.K, m1 - m0);
            __syncthreads();
        };
        const qw_afrag_lds af = {xf, n};
        f4 acc = {0, 0, 0, 0};
        qw_task_pipeline<C>(nt, qw_wave(), nwv, cpr, CH * C::BLK_B, lane, [&](uint32_t i) { return W + (size_t)i * a.rowbytes; },
            [&](uint32_t i, uint32_t ci, const C &c) {
                c.mac_lean(lut, af, ci * CH * C::BLK_K, kg, acc);
                if (ci + 1 != cpr) return;
                const bool second = a.split == 8 && n >= 8; // rows 8..15 of a two-matrix tile belong to the second output
                const uint32_t col = a.split == 8 ? 8 * (t0 + i) + (n & 7) : 16 * (t0 + i) + n;
                uint16_t *Y = second ? a.Y1 : a.Y;
#pragma unroll
                for (uint32_t j = 0; j < 4; j++) {
                    const uint32_t m = m0 + 4 * kg + j;
                    const uint16_t y = qw_f2h(acc[j]);
                    if (m < m1) Y[(size_t)m * a.N + col] = y;
                    if (a.H) qw_pf_act(a, y, m, m < m1 && !second, col);
                }
                acc = f4{0, 0, 0, 0};
            }, ready);
        pos += nt;
    }
}
#define QW_PFR(CH, NAME)                                                                          \
    extern "C" __global__ __launch_bounds__(QW_WG_GU) void NAME(qwk_pf_args a) {                 \
        __shared__ struct { u2 lut[QW_LUT_ENTRIES]; u4 xf[QW_XF_MAXK * 2]; uint32_t cnt; } L;     \
        pf_range_body<CH>(a, L.lut, L.xf, &L.cnt);                                                \
    }
#if QW_IN_PART(5)
QW_PFR(2, qwk_pfr_f121_c2) QW_PFR(1, qwk_pfr_f121_c1)
#endif

// ================================================================ combine (kernels/moe_gg.metal:655-663)
// Rank order, then the shared expert. One thread per (token, row).
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(256) void qwk_cmb(qwk_cmb_args a) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= a.nbr * a.D) return;
    const uint32_t t = i / a.D, row = i % a.D, K = a.topk;
    const float *w = (const float *)(a.sel + QW_SEL_OFF_W(a.gnb, K)) + t * (K + 1);
    float pg[16];
#pragma unroll
    for (uint32_t s = 0; s < 16; s++) pg[s] = s < K ? a.Pg[((size_t)t * K + s) * a.D + row] : 0.0f; // loads first
    float o = 0;
#pragma unroll
    for (uint32_t s = 0; s < 16; s++)
        if (s < K) o = __builtin_fmaf(w[s], pg[s], o);
    o = __builtin_fmaf(w[K], a.Psh[(size_t)t * a.D + row], o);
    a.out[(size_t)t * a.D + row] = qw_f2h(o);
}
#endif

// ================================================================ memory helpers
// Pure-read ceiling: every thread folds 16-byte loads into an XOR sink the compiler cannot drop
// (the method of the reference's kernels/ceiling_mem.metal:10-71). Grid-stride over n 16-byte units.
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(256) void qwk_bw_read(qwk_mem_args a) {
    const u4 *p = (const u4 *)a.src;
    u4 s = {0, 0, 0, 0};
    const uint64_t step = (uint64_t)gridDim.x * blockDim.x;
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i + 3 * step < a.n; i += 4 * step) {
        const u4 v0 = p[i], v1 = p[i + step], v2 = p[i + 2 * step], v3 = p[i + 3 * step];
        s ^= v0 ^ v1 ^ v2 ^ v3;
    }
    for (; i < a.n; i += step) s ^= p[i];
    if ((s.x ^ s.y ^ s.z ^ s.w) == 0x9e3779b9u && a.seed == 0x1234) ((u4 *)a.dst)[0] = s; // practically never taken
}
#endif
// ================================================================ hyper-connection, GGUF profile (kernels/hyper_gg.metal:94-233)
// Everything in binary32, as there. Two launches a hyper-connection whatever the token count: a launch boundary costs
// more here than recomputing nb x 320 activations per workgroup, which is what the reference's third kernel avoids.
__device__ __forceinline__ float qw_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
// 2 sigmoid(sum over the streams of their inject sums for stream s / HC) (kernels/hyper_gg.metal:47-51)
__device__ __forceinline__ float hc_coef(const float *injp, uint32_t s) {
    float t = 0;
#pragma unroll
    for (uint32_t q = 0; q < QW_HC; q++) t += injp[q * QW_HC + s];
    return 2.0f / (1.0f + expf(-t / QW_HC));
}
// Four sums at once over the lanes of a wave (W = 64) or of each half (W = 32): two exchange steps leave every lane with
// one of the four values summed over a quad of lanes, the remaining steps add the quads. Lane l ends with the whole sum
// of value number 2 (l & 1) + ((l >> 1) & 1). Seven (six) shuffles instead of four times six (five).
template <int W> __device__ __forceinline__ float qw_sum4(float d0, float d1, float d2, float d3, uint32_t lane) {
    const bool b0 = lane & 1, b1 = lane & 2;
    const float e0 = (b0 ? d2 : d0) + __shfl_xor(b0 ? d0 : d2, 1), e1 = (b0 ? d3 : d1) + __shfl_xor(b0 ? d1 : d3, 1);
    float f = (b1 ? e1 : e0) + __shfl_xor(b1 ? e0 : e1, 2);
#pragma unroll
    for (int o = 4; o < W; o <<= 1) f += __shfl_xor(f, o);
    return f;
}
// Down: residual, sums of squares and the un-normalised mix_down / inject sums (kernels/hyper_gg.metal:94-137).
// Workgroup (rb, s, tg): R weight rows (the last block = the four inject rows) against stream s of tokens
// 4 tg .. 4 tg + 3; thread c owns columns 8 c .. 8 c + 7 (16 bytes of a bfloat16 row). Everything a thread reads is
// asked for before anything is used, so the kernel is one memory round trip whatever the token count. Per token: the
// lane's eight h' w products, R dot products of eight and the squares, summed over the wave, then over the waves in
// order. R = 4 fills the machine at a few tokens; R = 16 re-reads h and out four times less often at many.
template <uint32_t R> __device__ __forceinline__ void hc_down_body(const qwk_hc_args &a, float (*part)[QW_HC_TG][17]) {
    const uint32_t rb = blockIdx.x, s = blockIdx.y, t0 = blockIdx.z * QW_HC_TG, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, nwv = blockDim.x >> 6;
    const uint32_t nt = a.nb - t0 < QW_HC_TG ? a.nb - t0 : QW_HC_TG;
    QW_HSTAMP(0);
    const bool is_inj = rb == QW_HC_LR / R;
    const uint32_t nrow = is_inj ? QW_HC : R; // rows of this block (uniform)
    const size_t HCD = (size_t)QW_HC * a.D, c0 = (size_t)s * a.D + 8 * tid;
    const uint16_t *W = is_inj ? a.Wi : a.Wd + (size_t)rb * R * HCD;
    u4 wu[R], ou[QW_HC_TG];
    f4 hv[QW_HC_TG][2];
#pragma unroll
    for (uint32_t r = 0; r < R; r++)
        if (r < nrow) wu[r] = *(const u4 *)(W + (size_t)r * HCD + c0);
    const f4 w0 = *(const f4 *)(a.w + c0), w1 = *(const f4 *)(a.w + c0 + 4);
#pragma unroll
    for (uint32_t tt = 0; tt < QW_HC_TG; tt++) {
        if (tt < nt) {
            hv[tt][0] = *(const f4 *)(a.h + (t0 + tt) * HCD + c0), hv[tt][1] = *(const f4 *)(a.h + (t0 + tt) * HCD + c0 + 4);
            if (a.apply) ou[tt] = *(const u4 *)(a.out + (size_t)(t0 + tt) * a.D + 8 * tid); // not read otherwise: it may never have been written
        }
    }
    QW_HSTAMP(1);
#pragma unroll
    for (uint32_t tt = 0; tt < QW_HC_TG; tt++) {
        if (tt >= nt) break;
        float v[8] = {hv[tt][0][0], hv[tt][0][1], hv[tt][0][2], hv[tt][0][3], hv[tt][1][0], hv[tt][1][1], hv[tt][1][2], hv[tt][1][3]};
        if (a.apply) {
            const float js = hc_coef(a.inj + (t0 + tt) * QW_HC * QW_HC, s);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                v[2 * k] = fmaf(qw_h2f((uint16_t)ou[tt][k]), js, v[2 * k]);
                v[2 * k + 1] = fmaf(qw_h2f((uint16_t)(ou[tt][k] >> 16)), js, v[2 * k + 1]);
            }
        }
        float ss = 0, x[8];
#pragma unroll
        for (int k = 0; k < 8; k++) ss = fmaf(v[k], v[k], ss), x[k] = v[k] * (k < 4 ? w0[k] : w1[k - 4]);
        ss = qw_wave_sum(ss);
        if (tt == 0) QW_HSTAMP(2);
        if (lane == 0) part[wave][tt][16] = ss;
#pragma unroll
        for (uint32_t r0 = 0; r0 < R; r0 += 4) {
            if (r0 >= nrow) break;
            float d[4];
#pragma unroll
            for (uint32_t r = 0; r < 4; r++) {
                d[r] = 0;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    d[r] = fmaf(__builtin_bit_cast(float, wu[r0 + r][k] << 16), x[2 * k], d[r]);
                    d[r] = fmaf(__builtin_bit_cast(float, wu[r0 + r][k] & 0xffff0000u), x[2 * k + 1], d[r]);
                }
            }
            const float f = qw_sum4<64>(d[0], d[1], d[2], d[3], lane);
            if (lane < 4) part[wave][tt][r0 + 2 * (lane & 1) + (lane >> 1)] = f;
        }
    }
    QW_HSTAMP(3);
    __syncthreads();
    QW_HSTAMP(4);
    for (uint32_t j = tid; j < nt * 17; j += blockDim.x) {
        const uint32_t tt = j / 17, r = j % 17;
        if (r < 16 && r >= nrow) continue;
        float sum = 0;
        for (uint32_t q = 0; q < nwv; q++) sum += part[q][tt][r];
        float *pd = a.pd + ((size_t)(t0 + tt) * QW_HC + s) * QW_HC_PDS;
        if (r < 16) pd[(is_inj ? QW_HC_LR : rb * R) + r] = sum;
        else if (rb == 0) pd[QW_HC_LR + QW_HC] = sum;
    }
    QW_HSTAMP(5);
}
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(512) void qwk_hc_down_r4(qwk_hc_args a) {
    __shared__ float part[8][QW_HC_TG][17]; // [wave][token][row | squares]
    hc_down_body<4>(a, part);
}
extern "C" __global__ __launch_bounds__(512) void qwk_hc_down_r8(qwk_hc_args a) {
    __shared__ float part[8][QW_HC_TG][17];
    hc_down_body<8>(a, part);
}
extern "C" __global__ __launch_bounds__(512) void qwk_hc_down_r16(qwk_hc_args a) {
    __shared__ float part[8][QW_HC_TG][17];
    hc_down_body<16>(a, part);
}
#endif
// What follows the down kernel for tokens t0 .. t0 + nt - 1, by the threads of one workgroup: the streams' 1 / rms,
// silu of the normalised mix_down sums, and (injo given) the inject sums in the caller's format
// (kernels/hyper_gg.metal:165-181, 312-340). rs [nt][HC] and sx [nt][LR] are in LDS; ends with a barrier.
__device__ __forceinline__ void hc_mid(const qwk_hc_args &a, uint32_t t0, uint32_t nt, float *rs, float *sx, float *injo) {
    const float *pd = a.pd + (size_t)t0 * QW_HC * QW_HC_PDS;
    for (uint32_t j = threadIdx.x; j < nt * QW_HC; j += blockDim.x) rs[j] = rsqrtf(pd[j * QW_HC_PDS + QW_HC_LR + QW_HC] / (float)a.D + 1e-6f);
    __syncthreads();
    for (uint32_t j0 = threadIdx.x; j0 < nt * QW_HC_LR; j0 += 4 * blockDim.x) { // four elements a round: their sixteen loads go out together
        float p[4][QW_HC];
#pragma unroll
        for (uint32_t e = 0; e < 4; e++) {
            const uint32_t j = j0 + e * blockDim.x, t = j / QW_HC_LR, r = j % QW_HC_LR;
#pragma unroll
            for (uint32_t q = 0; q < QW_HC; q++) p[e][q] = j < nt * QW_HC_LR ? pd[(t * QW_HC + q) * QW_HC_PDS + r] : 0.0f;
        }
#pragma unroll
        for (uint32_t e = 0; e < 4; e++) {
            const uint32_t j = j0 + e * blockDim.x, t = j / QW_HC_LR;
            if (j >= nt * QW_HC_LR) break;
            float d = 0;
#pragma unroll
            for (uint32_t q = 0; q < QW_HC; q++) d = fmaf(rs[t * QW_HC + q], p[e][q], d);
            d /= QW_HC;
            sx[j] = d / (1.0f + __expf(-d));
        }
    }
    if (injo)
        for (uint32_t j = threadIdx.x; j < nt * QW_HC * QW_HC; j += blockDim.x) // j = (t, s, q)
            injo[t0 * QW_HC * QW_HC + j] = rs[j / QW_HC] * pd[(j / QW_HC) * QW_HC_PDS + QW_HC_LR + j % QW_HC];
    __syncthreads();
}
// The middle kernel of the three-kernel form (kernels/hyper_gg.metal:312-340): a workgroup a token.
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(320) void qwk_hc_mid(qwk_hc_args a) {
    __shared__ float rs[QW_HC], sx[QW_HC_LR];
    const uint32_t t = blockIdx.x;
    hc_mid(a, t, 1, rs, sx, a.want_inj ? a.injo : nullptr);
    for (uint32_t r = threadIdx.x; r < QW_HC_LR; r += blockDim.x) a.sx[t * QW_HC_LR + r] = sx[r];
    if (threadIdx.x < QW_HC) a.rs[t * QW_HC + threadIdx.x] = rs[threadIdx.x];
}
#endif
// Up: mix_up, the gates and the mix over the streams, the write-back of h (kernels/hyper_gg.metal:141-233, 344-).
// A workgroup of 256 threads takes eight output columns i, one per group of 32 lanes, and QW_HC_TG tokens (grid y: the
// token groups; with all tokens in one workgroup a compute unit held four waves that walked sixteen tokens one after
// the other, and every workgroup repeated the middle step for all of them); a lane holds ten low-rank columns of the
// four mix_up rows s D + i (20 bytes each). GIVEN: sx and rs come from qwk_hc_mid instead of being made here.
template <bool GIVEN> __device__ __forceinline__ void hc_up_body(const qwk_hc_args &a) {
    __shared__ float sx[QW_HC_TG][QW_HC_LR], rs[QW_HC_TG][QW_HC], js[QW_HC_TG][QW_HC];
    const uint32_t tid = threadIdx.x, l32 = tid & 31, i = blockIdx.x * 8 + (tid >> 5), t0 = blockIdx.y * QW_HC_TG;
    const uint32_t nt = a.nb - t0 < QW_HC_TG ? a.nb - t0 : QW_HC_TG;
    const size_t HCD = (size_t)QW_HC * a.D;
    QW_HSTAMP(8);
    // Everything a thread will read is asked for here and without conditions (a lane without a token or a thread without
    // an element reads what element 0 would: valid memory, the value unused), so that the launch is one memory round
    // trip. Loads under conditions were a round trip each: the weights and h, out, the inject sums, the sums of squares,
    // the mix_down sums - five in a row.
    uint32_t u[QW_HC][5];
#pragma unroll
    for (uint32_t q = 0; q < QW_HC; q++) {
        const uint32_t *wr = (const uint32_t *)(a.Wu + ((size_t)q * a.D + i) * QW_HC_LR) + l32 * 5;
#pragma unroll
        for (int k = 0; k < 5; k++) u[q][k] = wr[k];
    }
    // lane l < 4 QW_HC_TG of a group owns token l / 4 of the workgroup's and the stream qw_sum4 leaves with it
    const uint32_t ts = l32 / QW_HC, sq = 2 * (l32 & 1) + ((l32 >> 1) & 1);
    const bool mine = ts < nt;
    const uint32_t tsc = mine ? ts : 0;
    const float wn = a.w[(size_t)sq * a.D + i];
    const float hv = a.h[(t0 + tsc) * HCD + (size_t)sq * a.D + i];
    // (out is not read unless it is applied: it may never have been written, nor the inject sums)
    const uint16_t ovr = *(a.apply ? a.out + (size_t)(t0 + tsc) * a.D + i : (const uint16_t *)a.h);
    const bool hasj = tid < nt * QW_HC; // this thread makes the values of (token jt / HC, stream jt % HC)
    const uint32_t jt = hasj ? tid : 0;
    const float *injp = a.apply ? a.inj + (t0 + jt / QW_HC) * QW_HC * QW_HC : a.pd;
    float iq[QW_HC];
#pragma unroll
    for (uint32_t q = 0; q < QW_HC; q++) iq[q] = injp[q * QW_HC + jt % QW_HC];
    // the middle step's inputs (hc_mid's arithmetic below, element tid + 256 e): sums of squares, mix_down sums, inject sums
    constexpr uint32_t EPT = (QW_HC_TG * QW_HC_LR + 255) / 256;
    const float *pd = a.pd + (size_t)t0 * QW_HC * QW_HC_PDS;
    float sq_raw = 0, ij_raw = 0, p[EPT][QW_HC];
    if (!GIVEN) {
        sq_raw = pd[jt * QW_HC_PDS + QW_HC_LR + QW_HC];
        const uint32_t ji = tid < nt * QW_HC * QW_HC ? tid : 0; // (t, s, q)
        ij_raw = pd[(ji / QW_HC) * QW_HC_PDS + QW_HC_LR + ji % QW_HC];
#pragma unroll
        for (uint32_t e = 0; e < EPT; e++) {
            const uint32_t j = tid + e * 256, jc = j < nt * QW_HC_LR ? j : 0, t = jc / QW_HC_LR, r = jc % QW_HC_LR;
#pragma unroll
            for (uint32_t q = 0; q < QW_HC; q++) p[e][q] = pd[(t * QW_HC + q) * QW_HC_PDS + r];
        }
    }
    QW_HSTAMP(9);
    if (hasj) {
        float t = 0;
#pragma unroll
        for (uint32_t q = 0; q < QW_HC; q++) t += iq[q];
        js[tid / QW_HC][tid % QW_HC] = a.apply ? 2.0f / (1.0f + expf(-t / QW_HC)) : 0.0f; // hc_coef
    }
    if (GIVEN) {
        for (uint32_t j0 = tid; j0 < nt * QW_HC_LR; j0 += 8 * blockDim.x) { // eight loads in flight a thread
            float v[8];
#pragma unroll
            for (uint32_t e = 0; e < 8; e++) v[e] = j0 + e * blockDim.x < nt * QW_HC_LR ? a.sx[t0 * QW_HC_LR + j0 + e * blockDim.x] : 0.0f;
#pragma unroll
            for (uint32_t e = 0; e < 8; e++)
                if (j0 + e * blockDim.x < nt * QW_HC_LR) (&sx[0][0])[j0 + e * blockDim.x] = v[e];
        }
        if (tid < nt * QW_HC) rs[tid / QW_HC][tid % QW_HC] = a.rs[t0 * QW_HC + tid];
    } else { // hc_mid for the workgroup's tokens, on the values read above
        if (hasj) (&rs[0][0])[tid] = rsqrtf(sq_raw / (float)a.D + 1e-6f);
        __syncthreads();
        QW_HSTAMP(10);
#pragma unroll
        for (uint32_t e = 0; e < EPT; e++) {
            const uint32_t j = tid + e * 256, t = j / QW_HC_LR;
            if (j < nt * QW_HC_LR) {
                float d = 0;
#pragma unroll
                for (uint32_t q = 0; q < QW_HC; q++) d = fmaf(rs[t][q], p[e][q], d);
                d /= QW_HC;
                (&sx[0][0])[j] = d / (1.0f + __expf(-d));
            }
        }
        if (blockIdx.x == 0 && a.want_inj && tid < nt * QW_HC * QW_HC) a.injo[t0 * QW_HC * QW_HC + tid] = (&rs[0][0])[tid / QW_HC] * ij_raw;
    }
    __syncthreads();
    QW_HSTAMP(11);
    const float ov = qw_h2f(ovr);
    float v[QW_HC][10];
#pragma unroll
    for (uint32_t q = 0; q < QW_HC; q++)
#pragma unroll
        for (int k = 0; k < 5; k++) v[q][2 * k] = __builtin_bit_cast(float, u[q][k] << 16), v[q][2 * k + 1] = __builtin_bit_cast(float, u[q][k] & 0xffff0000u);
    // mix_up: for every token four dot products of ten, summed over the group's 32 lanes; the lanes of the token's quad
    // keep the sums of their streams
    float uv = 0;
    for (uint32_t t = 0; t < nt; t++) {
        float xv[10];
#pragma unroll
        for (int k = 0; k < 10; k++) xv[k] = sx[t][l32 * 10 + k];
        float d[QW_HC];
#pragma unroll
        for (uint32_t q = 0; q < QW_HC; q++) {
            d[q] = 0;
#pragma unroll
            for (int k = 0; k < 10; k++) d[q] = fmaf(v[q][k], xv[k], d[q]);
        }
        const float f = qw_sum4<32>(d[0], d[1], d[2], d[3], l32); // this lane's stream, summed over the group
        uv = ts == t ? f : uv;
    }
    QW_HSTAMP(12);
    // the gates and the mix over the streams: the four streams of a token are neighbouring lanes
    float m = 0;
    if (mine) {
        float hq = hv;
        if (a.apply) {
            hq = fmaf(ov, js[ts][sq], hq);
            a.h[(t0 + ts) * HCD + (size_t)sq * a.D + i] = hq;
        }
        m = (hq * rs[ts][sq]) * wn / (1.0f + __expf(-uv));
    }
    m += __shfl_xor(m, 1);
    m += __shfl_xor(m, 2);
    if (mine && sq == 0) a.x[(size_t)(t0 + ts) * a.D + i] = qw_f2h(m / QW_HC);
    QW_HSTAMP(13);
}
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(256) void qwk_hc_up(qwk_hc_args a) { hc_up_body<false>(a); }
extern "C" __global__ __launch_bounds__(256) void qwk_hc_upv(qwk_hc_args a) { hc_up_body<true>(a); }
#endif

// Read pattern of a decode layer without the decoding (kernels/moe_bw.metal:7-26): workgroup (x, c) reads slice x
// (SL 16-byte units) of chunk c, every thread LD independent loads a round, folded into an XOR sink.
template <int LD> __device__ __forceinline__ void bw_chunks_body(const qwk_bwpat_args &a) {
    const uint32_t nt = blockDim.x, tid = threadIdx.x;
    const uint64_t start = a.chunks[2 * blockIdx.y];
    uint64_t len = a.chunks[2 * blockIdx.y + 1];
    if (start >= a.src_n) return;
    if (start + len > a.src_n) len = a.src_n - start; // a record that reaches past the arena reads what there is
    const uint64_t b = (uint64_t)blockIdx.x * a.sl;
    if (b >= len) return;
    const uint64_t e = b + a.sl < len ? b + a.sl : len;
    const u4 *p = (const u4 *)a.src + start;
    u4 acc[LD];
#pragma unroll
    for (int k = 0; k < LD; k++) acc[k] = u4{0, 0, 0, 0};
    uint64_t i = b + tid;
    for (; i + (uint64_t)(LD - 1) * nt < e; i += (uint64_t)LD * nt)
#pragma unroll
        for (int k = 0; k < LD; k++) acc[k] ^= p[i + (uint64_t)k * nt];
    for (; i < e; i += nt) acc[0] ^= p[i];
    u4 s = acc[0];
#pragma unroll
    for (int k = 1; k < LD; k++) s ^= acc[k];
    const uint32_t r = s.x ^ s.y ^ s.z ^ s.w;
    if (r == 0x9e3779b9u) a.out[tid] = r; // practically never taken
}
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(1024) void qwk_bw_chunks(qwk_bwpat_args a) {
    switch (a.ld) {
    case 1: bw_chunks_body<1>(a); break;
    case 2: bw_chunks_body<2>(a); break;
    case 4: bw_chunks_body<4>(a); break;
    default: bw_chunks_body<8>(a); break; // the host admits 1, 2, 4, 8
    }
}
#endif
// The row pattern (kernels/moe_bw.metal:30-41): a group of 32 lanes takes one row of RB bytes and reads it two bytes
// at a time, a unit of UB bytes per lane and step; workgroup (x, c) takes rows 8 x .. 8 x + 7 of chunk c. The
// reference's group is the 32-lane SIMD group of its hardware: here it is half of a wave, the same rows and loads.
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(256) void qwk_bw_rows(qwk_bwpat_args a) {
    const uint32_t sg = threadIdx.x >> 5, lane = threadIdx.x & 31;
    const uint64_t off = (uint64_t)a.chunks[2 * blockIdx.y] * 16 + ((uint64_t)blockIdx.x * 8 + sg) * a.rb;
    if (off + a.rb > a.src_n * 16) return; // a row past the arena is not read
    const uint8_t *row = (const uint8_t *)a.src + off;
    uint32_t acc = 0;
    for (uint32_t u = lane; u < a.rb / a.ub; u += 32)
        for (uint32_t j = 0; j < a.ub; j += 2) acc ^= *(const uint16_t *)(row + (size_t)u * a.ub + j);
    if (acc == 0x9e3779b9u) a.out[lane] = acc; // practically never taken
}
#endif
// Plain copy of n 16-byte units (the known-size kernel the hardware traffic counters are scaled against).
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(256) void qwk_copy(qwk_mem_args a) {
    const u4 *p = (const u4 *)a.src;
    u4 *q = (u4 *)a.dst;
    const uint64_t step = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.n; i += step) q[i] = p[i];
}
#endif
// Fill n 16-byte units with a counter-based hash of (seed, index): uniform random bytes.
__device__ __forceinline__ uint32_t qw_mix(uint64_t x) {
    x ^= x >> 33; x *= 0xff51afd7ed558ccdull; x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ull; x ^= x >> 33;
    return (uint32_t)x;
}
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(256) void qwk_fill_random(qwk_mem_args a) {
    u4 *q = (u4 *)a.dst;
    const uint64_t step = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.n; i += step) {
        const uint64_t c = a.seed + 4 * i;
        q[i] = u4{qw_mix(c), qw_mix(c + 1), qw_mix(c + 2), qw_mix(c + 3)};
    }
}
#endif

// Synthetic GGUF blocks, one thread per block: d = binary16(|N(0, sigma)|) by Box-Muller over two hashed uniforms,
// every other byte uniform (IQ3_S, IQ4_NL), or int8 uniform in [-127, 127] (Q8_0). Blocks are 2-byte aligned: 16-bit stores.
#if QW_IN_PART(5)
extern "C" __global__ __launch_bounds__(256) void qwk_fill_blocks(qwk_fill_args a) {
    const uint64_t step = (uint64_t)gridDim.x * blockDim.x;
    const uint32_t bb = a.type == 21 ? 110 : a.type == 20 ? 18 : 34; // IQ4_NL: d and sixteen uniform bytes
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.nblocks; i += step) {
        uint16_t *p = (uint16_t *)(a.dst + i * bb);
        const uint64_t c = a.seed + i * 64;
        const float u1 = ((float)(qw_mix(c) >> 8) + 1.0f) * (1.0f / 16777216.0f), u2 = (float)(qw_mix(c + 1) >> 8) * (1.0f / 16777216.0f);
        const float z = sqrtf(-2.0f * __logf(u1)) * __cosf(6.2831853f * u2);
        p[0] = qw_f2h(fabsf(z) * a.sigma);
        for (uint32_t w = 1; w < bb / 2; w++) {
            uint32_t r = qw_mix(c + 1 + w);
            if (a.type == 8) { // two int8 in [-127, 127]
                const uint32_t b0 = (r & 0xffff) % 255u, b1 = (r >> 16) % 255u;
                r = ((b0 - 127u) & 255u) | (((b1 - 127u) & 255u) << 8);
            }
            p[w] = (uint16_t)r;
        }
    }
}
#endif
