/* Kernel argument records shared by the HIP kernels (device side) and gpu_hip.c (host side, C23).
 * Every kernel takes exactly one of these by value. Plain C: fixed-width integers and pointers only. */
#pragma once
#include <stdint.h>

/* Selection record written by the select kernel and read by gate/up, down and combine. For gnb == 8 and
 * topk == 10 this is byte for byte the reference's struct gg_sel (kernels/moe_gg.metal:110-116), 1636 bytes;
 * gnb == 16 is the wide layout for up to 16 token columns (4548 bytes with topk == 10). GU = gnb * topk.
 *   uint32 U; uint32 ue[GU]; uint32 mask[GU]; uint8 slot[GU][gnb]; float w[gnb][topk + 1] */
#define QW_SEL_OFF_UE(gnb, topk) 4u
#define QW_SEL_OFF_MASK(gnb, topk) (4u + 4u * (gnb) * (topk))
#define QW_SEL_OFF_SLOT(gnb, topk) (4u + 8u * (gnb) * (topk))
#define QW_SEL_OFF_W(gnb, topk) (4u + 8u * (gnb) * (topk) + (gnb) * (topk) * (gnb))
#define QW_SEL_BYTES(gnb, topk) (QW_SEL_OFF_W(gnb, topk) + 4u * (gnb) * ((topk) + 1u))

/* Pre-signed IQ3_S table inside the lookup-table buffer the callers allocate (kernels/moe_gg.metal:89-95):
 * 8192 entries of four binary16 values at byte offset 49152; the whole buffer is 117760 bytes. */
#define QW_TAB_IQ3SS 49152u
#define QW_TAB_IQ4 114688u
#define QW_TAB_Q20 115712u
#define QW_TAB_BYTES 117760u

typedef struct { /* dq_test: rows x K values to float */
    const uint8_t *W;
    float *y;
    uint32_t K, rowbytes, rows, fmt; /* fmt: used by the kernel that serves the formats 1, 12, 13, 14, 20, 23, 30 */
} qwk_dq_args;

typedef struct { /* dense matvec, y[b][row] = W[row] . x[b] */
    const uint8_t *W;
    const uint16_t *x; /* binary16 [nb][xstride] */
    void *y;           /* binary16 or float [nb][ystride] */
    uint32_t N, K, rowbytes, xstride, ystride, nb, yfloat, ntiles;
    const void *glut; /* the backend's pre-signed IQ3_S table in global memory (64 KB) */
    uint32_t split, pad; /* waves a tile's chunks are cut over (1 .. 6; the chunk count of a row is a multiple of it) */
} qwk_qmv_args;

/* Dense matvec over up to four matrices that share the activations (kernels/qmv_ggm.metal:232-262; one matrix:
 * kernels/qmv_gg.metal:17-39) for the formats 1, 12, 13, 14, 20, 23, 30. 16-row tiles of all matrices form one list. */
#define QW_KQ_MAXK 4096u /* activations of up to 16 tokens staged in LDS: K * 32 bytes */
typedef struct {
    const uint8_t *W[4];
    void *y[4];        /* [nb][ystride[j]] binary16 or float */
    const uint16_t *x; /* binary16 [nb][xstride] */
    uint32_t N[4], fmt[4], rowbytes[4], ystride[4], ntiles[4];
    uint32_t K, xstride, nb, yfloat, nmat, sums; /* sums: some matrix is Q4_K / Q5_K (needs the 32-value sums of x) */
    uint32_t split, pad;                         /* waves a tile's K range is cut over (1 .. 6; > 1 needs K % (256 * split) == 0) */
    /* qwk_qmvm_swiglu (matrix 0 = gate rows, matrix 1 = up rows of a shared expert, N[0] = N[1] = I, split in
     * {2, 3, 5, 6}): nothing goes to y; H[t][topk][r] = silu(gate) * up as binary16 hi + lo planes, hplane halves apart */
    uint16_t *H;
    uint32_t topk, hplane;
} qwk_qmvm_args;

/* SwiGLU of the shared expert when its gate/up rows went through the multi-format matvec: g, u float [nb][I] ->
 * H[t][topk][j] as binary16 hi + lo planes */
typedef struct {
    const float *g, *u;
    uint16_t *H;
    uint32_t I, nb, topk, hplane;
} qwk_shact_args;

typedef struct { /* router: logits[t][r], r in [0, E] (row E = shared gate vector), row stride E + 1 */
    const uint16_t *Wr, *Wsg, *x;
    float *logits;
    uint32_t E, D, nb, pad;
} qwk_router_args;

typedef struct { /* selection + dedupe */
    const float *logits;
    uint8_t *sel;
    uint32_t nbr, E, topk, gnb;
} qwk_select_args;

typedef struct { /* build the lookup-table buffer */
    uint8_t *tab;
    uint32_t slot_order; /* 0: the reference's entry order; 1: the order this library's kernels read from LDS */
    uint32_t pad;
} qwk_tab_args;

/* gate/up + SwiGLU for a list of experts. routed: experts come from sel (U, ue, mask, slot). shared != 0: one
 * expert at Wg/Wu with every token in nbr selected, written to slot topk.
 * H is stored as two binary16 planes (value = hi + lo): Hhi = H, Hlo = H + nb_alloc * (topk + 1) * I halves. */
typedef struct {
    const uint8_t *Wg, *Wu; /* [E][I][rowbytes] */
    const uint16_t *x;      /* binary16 [nbr][D] */
    const uint8_t *sel;
    uint16_t *H;
    uint32_t D, I, rowbytes, nbr, topk, gnb, shared, hplane; /* hplane: halves between the hi and lo planes */
    const void *glut;
    /* the shared expert's gate/up, done by the same launch when Wsg != NULL: all tokens, slot topk */
    const uint8_t *Wsg, *Wsu;
    uint32_t sg_rowbytes, E;
    /* logits != NULL: the selection has not been made yet; every workgroup makes it from the logits [nbr][E + 1] for
     * itself and workgroup 0 also writes the record to sel (the later kernels of the layer read it from there) */
    const float *logits;
    /* qwk_gu_rt*: the routed rows' ggml type (12, 13, 14, 20 or 23), chosen when the kernel runs */
    uint32_t fgu, pad_fgu;
} qwk_gu_args;

/* down projection. routed: Pg[t][slot][row] for the tokens in mask[u]; shared != 0: Psh[t][row] from slot topk. */
typedef struct {
    const uint8_t *Wd; /* [E][D][rowbytes] */
    const uint16_t *H;
    const uint8_t *sel;
    float *P; /* Pg [nbr][topk][D] or Psh [nbr][D] */
    uint32_t D, I, rowbytes, nbr, topk, gnb, shared, hplane;
    const void *glut;
    /* the shared expert's down projection, done by the same launch when Wsd != NULL: Psh[t][row] from slot topk */
    const uint8_t *Wsd;
    float *Psh;
    uint32_t sd_rowbytes, snbr; /* snbr: token count of the shared part */
    /* down + combine in one launch (qwk_dnc_*, at most QW_DNC_MAXNB tokens): the layer's output [nbr][D] binary16;
     * Psh is then also read when the launch carries no shared expert */
    uint16_t *out;
    /* qwk_dnq_*: quarters of four tokens (nq of them) and weight tiles per workgroup (tpw: 1 or 2) */
    uint32_t nq, tpw;
    /* qwk_dn_rt: the ggml types of the routed and of the shared down rows (0: no shared expert in this launch),
     * chosen when the kernel runs */
    uint32_t fd, fsd;
} qwk_dn_args;
/* Down + combine with a quarter of the tokens per workgroup (qwk_dnq_*): limits of the staged H rows */
#define QW_DNQ_ROWS 44u /* 4 tokens x (topk + 1) rows, topk <= 10 */
#define QW_DNQ_MAXU 160u
#define QW_DNC_MAXNB 4

/* Synchronisation words of launches whose workgroups wait for one another (layout: QW_SYNC_* in qw_common.hip.h). */
#define QW_SYNC_BYTES 1536u
#define QW_SYNC_ALLOC 32768u /* what the backend allocates: the words above, the rest for working builds that leave time stamps */
#define QW_SYNC_ERR_WORD 352u
/* Routed gate/up, down and combine of a layer as one launch (qwk_gud_*: tile-major IQ3_S routed rows, D <= 2048 a
 * multiple of 512, I = 512, topk <= 10, 1 to 16 tokens): the argument records of the launches it stands for. The grid
 * is one workgroup per compute unit; all of them stream gate/up tiles, leave their SwiGLU values in H through stores
 * of device scope, meet at one barrier over the grid, and then run the down projection and the combine as qwk_dnq_*
 * does, with shares of at most QW_GUD_SHARE tokens: dn.nq shares, dn.tpw tiles of 16 output rows per workgroup,
 * D / 16 / dn.tpw * dn.nq <= grid workgroups take part in that phase. */
#define QW_GUD_SHARE 3u
#define QW_GUD_ROWS 33u /* staged H rows per workgroup: QW_GUD_SHARE tokens x (topk + 1) */
#define QW_GUD_HCAP 192u /* (tile, token) results of the gate/up phase a workgroup keeps in LDS; more go to memory directly */
typedef struct {
    qwk_gu_args gu;
    qwk_dn_args dn;
    uint32_t *sync;
    uint32_t spin_limit, pad; /* polls of the generation word after which a waiting workgroup gives up */
} qwk_gud_args;

/* front part of a layer: router rows on the first nrouter workgroups; when g.Wsg != NULL the shared expert's gate/up
 * on the workgroups after them (g: its arguments, shared = 1), one chunk of a tile per wave, summed through LDS. */
typedef struct {
    qwk_router_args r;
    uint32_t nrouter, pad;
    qwk_gu_args g;
} qwk_pre_args;
/* the front launch when the shared expert's gate/up rows are in the K-quant / IQ4 / plain family (qwk_pre_w1_kq):
 * m as for qwk_qmvm_swiglu, on the workgroups after the router's */
typedef struct {
    qwk_router_args r;
    uint32_t nrouter, pad;
    qwk_qmvm_args m;
} qwk_prekq_args;

typedef struct { /* out[t][row] = half(sum_s w[t][s] * Pg[t][s][row] + w[t][topk] * Psh[t][row]) */
    const float *Pg, *Psh;
    const uint8_t *sel;
    uint16_t *out;
    uint32_t D, nbr, topk, gnb;
} qwk_cmb_args;

typedef struct { /* pure-read ceiling and fill helpers */
    const void *src;
    void *dst;
    uint64_t n; /* 16-byte units */
    uint64_t seed;
} qwk_mem_args;

/* Hyper-connection of the GGUF profile (the reference's kernels/hyper_gg.metal): QW_HC streams of D values a token,
 * low rank QW_HC_LR. pd holds, per (token, stream), QW_HC_PDS floats: [0, LR) the stream's part of the mix_down sums
 * before normalisation, [LR, LR + HC) the same for the inject rows, [LR + HC] the stream's sum of squares. */
#define QW_HC 4u
#define QW_HC_LR 320u
#define QW_HC_PDS (QW_HC_LR + 2 * QW_HC)
#define QW_HC_TG 4u   /* tokens per workgroup of the down kernel */
typedef struct {
    float *h;                      /* [nb][HC][D]; the up kernels write it back when the residual is applied */
    const uint16_t *out;           /* binary16 [nb][D]: the sublayer output the residual adds */
    const float *inj;              /* [nb][HC][HC]: inject sums of the previous hyper-connection */
    const float *w;                /* [HC * D] norm weights */
    const uint16_t *Wd, *Wi, *Wu;  /* bfloat16: mix_down [LR][HC * D], inject [HC][HC * D], mix_up [HC * D][LR] */
    float *pd;                     /* [nb][HC][QW_HC_PDS] */
    float *sx, *rs;                /* three-kernel form: silu(mix_down) [nb][LR] and the streams' 1 / rms [nb][HC] */
    uint16_t *x;                   /* binary16 [nb][D] */
    float *injo;                   /* [nb][HC][HC] */
    uint32_t D, nb, apply, want_inj;
} qwk_hc_args;

typedef struct { /* read-pattern ceiling of a decode layer (the reference's kernels/moe_bw.metal:7-41) */
    const void *src;          /* the arena the chunks lie in */
    const uint32_t *chunks;   /* {start, length} per chunk, in 16-byte units; workgroup row y reads chunks[y] */
    uint32_t *out;            /* sink that is practically never written; holds at least one dword per thread */
    uint64_t src_n;           /* 16-byte units readable at src: chunk records that reach past it are clamped */
    uint32_t sl, ld, rb, ub;  /* SL: units per workgroup; LD: independent loads per thread and round; RB, UB: bytes per row and per unit */
} qwk_bwpat_args;

/* Tile-major copy of IQ3_S rows ("packed", format code QW_F_PACKED below): rows are taken 16 at a time (a tile) and
 * every (tile, block) slab of 16 x 110 bytes becomes QW_SLAB_BYTES contiguous bytes in the lane order of the matrix
 * instructions (lane l: row l & 15 of the tile, 64-value slice l >> 4 of the block):
 *     [0, 1024)     lane l: 16 bytes qs[16 kg .. 16 kg + 16)
 *     [1024, 1536)  lane l:  8 bytes signs[8 kg .. 8 kg + 8)
 *     [1536, 1792)  lane l:  4 bytes qh[2 kg], qh[2 kg + 1], scales[kg], one byte of d (low byte for even kg, high for odd)
 * so that a wave reads a slab with three fully coalesced loads. Slabs of a tile follow each other by block, tiles by
 * index. A tile's rows n < split come from matrix A (row tile * split + n), the others from matrix B
 * (row tile * (16 - split) + n - split): split 16 = one matrix, split 8 = gate rows and up rows side by side. */
#define QW_SLAB_BYTES 1792u
#define QW_F_PACKED 121
/* Measurement only (QW_HIP_ABLATE): the tile-major IQ3_S stream of QW_F_PACKED with the decoding and the matrix
 * instructions left out - the loaded registers are merely folded into the result, which is therefore meaningless. Times
 * what the gate/up launch costs without its arithmetic (same selection, table and activation staging, loads, stores). */
#define QW_F_ABLATE 122
/* Tile-major copy of IQ4_NL rows (format code QW_F_PACKED_NL; qwk_pack_args with split = QW_F_PACKED_NL, nblk = chunks
 * of ten blocks per row, so the row length is a multiple of 320): every (tile of 16 rows, chunk) becomes
 * QW_NL_CHUNK_BYTES = 16 x 180 contiguous bytes in the lane order of the matrix instruction (lane = row & 15 | k-group
 * << 4; a lane owns bytes 4 kg .. 4 kg + 3 of qs of every block of its row):
 *   [0, 1024)    blocks 0..3: 16 bytes per lane      [1024, 2048)  blocks 4..7: 16 bytes per lane
 *   [2048, 2560) blocks 8..9:  8 bytes per lane      [2560, 2880)  d of the ten blocks, 20 bytes per row
 * A wave reads a chunk with three fully coalesced loads plus 20 bytes of scales per lane. */
#define QW_F_PACKED_NL 120
/* Template argument of the kernels whose routed format is chosen when they run (qwk_gu_rt*: qwk_gu_args.fgu): not a format. */
#define QW_F_RT 99
#define QW_NL_CHUNK_BYTES 2880u
/* Tile-major copy of Q6_K rows (format code QW_F_PACKED_Q6; qwk_pack_args with split = QW_F_PACKED_Q6, nblk = blocks a
 * row): per (tile of 16 rows, block of 256 values) QW_Q6_SLAB_BYTES = 16 x 210 contiguous bytes in the lane order of the
 * matrix instruction (lane = row & 15 | k-group << 4): [0, 3072) three planes of 16 bytes a lane holding the twelve
 * dwords of ql and qh that the lane decodes (the r[0..11] of the Q6_K decoder), [3072, 3328) the sixteen int8 scales of
 * every row (16 bytes a row, read by the row's four lanes), [3328, 3360) d of every row. Exactly the matrix's bytes. */
#define QW_F_PACKED_Q6 114
#define QW_Q6_SLAB_BYTES 3360u
typedef struct {
    const uint8_t *A, *B;
    uint8_t *dst;
    uint64_t ntiles;
    uint32_t nblk, rowbytes, split, pad;
} qwk_pack_args;

/* Ragged packing of (token, expert) pairs and the grouped product over the packed rows (kernels/moe_prefill.metal,
 * kernels/moe_gg.metal:761-838). P pairs, flat index p = token * topk + rank. */
typedef struct { /* clear n dwords (kernels/prefill.metal:601-603) */
    uint32_t *x;
    uint32_t n, pad;
} qwk_zero_args;
typedef struct {
    const uint32_t *ids; /* [P] expert of pair p */
    uint32_t *counts;    /* [E] */
    uint32_t P, E;
} qwk_count_args;
typedef struct {
    const uint32_t *counts;
    uint32_t *offs, *cursor; /* [E] first packed row of each expert; cursor starts there */
    uint32_t *tiles;         /* [max_tiles][4] = {expert, first row, end row, 0}; unused entries are zero */
    uint32_t E, max_tiles, tm, pad;
} qwk_plan_args;
typedef struct {
    const uint16_t *X; /* [T][KD] binary16 */
    const uint32_t *ids;
    uint32_t *cursor;
    uint16_t *Xs;      /* [P][KD] rows in packed order */
    uint32_t *pos_of;  /* [P] packed row of pair p */
    uint32_t KD, topk, E, P;
} qwk_scatter_args;
typedef struct {
    const uint16_t *G, *U; /* U == NULL: G is [P][2 I] (gate then up in each row); else G, U are [n] each */
    uint16_t *H;
    uint32_t P, I, n, pad;
} qwk_act_args;
typedef struct {
    const uint16_t *Dm; /* [P][KD] binary16, packed order */
    const uint32_t *pos_of;
    const float *w;     /* [P] */
    uint16_t *Y;        /* [T][KD] */
    uint32_t KD, topk, T, P;
} qwk_combine_args;
typedef struct { /* Y[m][n] = X[m] . W[expert][n] for the rows m of every tile entry; binary16 in and out */
    const uint16_t *X;
    const uint8_t *W;     /* [E][N][rowbytes]; packed (QW_F_PACKED): [E][ntn][rowbytes] tiles, rowbytes = bytes of a tile */
    uint16_t *Y;          /* [M][N] */
    const uint32_t *tiles;
    uint32_t M, N, K, rowbytes, max_tiles, tm;
    uint32_t split, ntn;  /* packed: split 16 = one matrix of N rows; split 8 = a tile holds 8 rows of matrix A (-> Y) and 8 of
                           * matrix B (-> Y1), N rows each; ntn = tiles per expert (N / 16 or N / 8) */
    const void *glut;
    uint16_t *Y1;
    uint16_t *H;          /* split 8 only, may be null: [M][N] = SiLU(Y) * Y1 from the rounded values, as qwk_moe_act leaves it */
} qwk_pf_args;
/* count + prefix sums + tile table + rows to packed order in one launch of P workgroups (P <= QW_PREP_MAXP, E <= 1024) */
#define QW_PREP_MAXP 4096u
typedef struct {
    const uint32_t *ids;                  /* [P] */
    uint32_t *counts, *offs, *cursor;     /* [E]: as qwk_zero + qwk_moe_count, qwk_moe_plan and qwk_moe_scatter leave them */
    uint32_t *tiles, *pos_of;
    const uint16_t *X;
    uint16_t *Xs;
    uint32_t P, E, topk, KD, tm, max_tiles;
} qwk_prep_args;

typedef struct { /* synthetic weights: nblocks GGUF blocks of one type, scale d = binary16(|N(0, sigma)|), the rest uniform */
    uint8_t *dst;
    uint64_t nblocks, seed;
    uint32_t type; /* 8 or 21 */
    float sigma;
} qwk_fill_args;
