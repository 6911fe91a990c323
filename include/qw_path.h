/* Host side of the quantized decode path, above the GPU interface of gpu.h.
 *
 * These functions restate, against gpu.h only, what the reference's engine does for this path: build the kernel
 * name and the "#define" block, compile on a miss, bind by index, dispatch. They mirror
 *     qmv_gg()      src/engine.c:689-724      qw_path_qmv_gg()
 *     qmv_ggm()     src/engine.c:752-771      qw_path_qmv_ggm()
 *     gg_router()   src/engine.c:544-552      qw_path_gg_router()
 *     gg_kernel()   src/engine.c:460-517      (internal)
 *     gg_moe()      src/engine.c:568-647      qw_path_gg_moe()
 *     hyper_gg()    src/engine.c:1344-1412    qw_path_hyper_gg()
 * with the same binding indices, macro names and dispatch order, so that a parity test written against them
 * exercises exactly the call sequence engine.c would issue. The one extension is a token count above 8 (up to 16),
 * which the reference splits into two passes (src/engine.c:8783-8814).
 *
 * Failure: where the reference prints and calls exit(1) (src/engine.c:508-514), these return false after printing
 * the same kind of message to stderr; the batch must then be abandoned with qw_batch_end().
 */
#pragma once
#include "gpu.h"

#ifdef __cplusplus
extern "C" {
#endif

/* A quantized matrix in HBM: rows x cols values of one ggml type, rows contiguous (src/model.h:64-66). */
typedef struct {
    const qw_buf *buf;
    size_t offset;
    int type; /* ggml type. MoE weights: 8 = Q8_0, 21 = IQ3_S; router: 1 = F16, 30 = BF16; dense matvec: also
               * 12, 13, 14 = Q4_K, Q5_K, Q6_K, 20 = IQ4_NL, 23 = IQ4_XS, 1, 30 */
} qw_tensor;

/* One MoE layer's weights (the fields of the reference's qw_moe that this path reads, src/model.h). */
typedef struct {
    qw_tensor router;    /* [E][D], F16 or BF16 */
    qw_tensor sh_gate_w; /* [D] shared-expert gate vector, same type as router */
    qw_tensor gate, up;  /* routed, [E][I][D-row]; same type */
    qw_tensor down;      /* routed, [E][D][I-row] */
    qw_tensor sh_gate, sh_up, sh_down; /* shared expert */
} qw_moe_layer;

typedef struct qw_path qw_path;

/* Scratch buffers (lookup tables, H, Psh, Pg, counter) for layers of this shape and up to nbmax <= 16 tokens.
 * device_scratch: keep the intermediates in HBM only (no host shadow), as a serving loop would. */
qw_path *qw_path_open(qw_gpu *g, int D, int I, int E, int topk, int nbmax, bool device_scratch);
void qw_path_close(qw_path *p);
/* Bytes the caller must give the selection record and the logits for nb tokens. */
size_t qw_path_sel_bytes(const qw_path *p, int nb);
size_t qw_path_logits_bytes(const qw_path *p, int nb);
/* Token count a kernel is built for when nb tokens are asked (1, 2, 4, 8, 16; src/engine.c:447 stops at 8). */
int qw_path_nbv(int nb);

/* y[b][0..N) = W x[b], b < nb; x stride K, y stride N; fout selects float (else binary16) output. */
bool qw_path_qmv_gg(qw_path *p, qw_batch *b, const qw_tensor *W, int N, int K, const qw_buf *x, size_t xoff, const qw_buf *y,
                    size_t yoff, int nb, bool fout);
/* n <= 4 matrices W[i] (N[i] rows of K values, K a multiple of 256 up to 4096; types from 1, 12, 13, 14, 20, 23, 30,
 * mixed freely) times the same x [nb][K], one launch: y[i][b][0..N[i]) with row stride N[i]; nb <= 16. The weights'
 * first bytes must be 16-byte aligned. */
bool qw_path_qmv_ggm(qw_path *p, qw_batch *b, const qw_tensor *W, const int *N, int n, int K, const qw_buf *x, const qw_buf *const *y, int nb, bool fout);
/* logits[nb][E + 1] alone. */
bool qw_path_gg_router(qw_path *p, qw_batch *b, const qw_moe_layer *M, int nb, const qw_buf *x, const qw_buf *lg);
/* The whole layer: x [nb][D] binary16 -> out [nb][D] binary16; lg and sel receive the logits and the selection. */
bool qw_path_gg_moe(qw_path *p, qw_batch *b, const qw_moe_layer *M, int nb, const qw_buf *x, const qw_buf *lg, const qw_buf *sel,
                    const qw_buf *out);
/* The same with the router's logits given by the caller in lg (the reference's RBF = 0 build of moe_pre_gg plus a
 * moe_sel_gg dispatch): for forced routing. */
bool qw_path_gg_moe_lg(qw_path *p, qw_batch *b, const qw_moe_layer *M, int nb, const qw_buf *x, const qw_buf *lg, const qw_buf *sel,
                       const qw_buf *out);
/* nlayers layers in a row on the same input x (the FFN stack of the benchmark): layer l writes lg[l], sel[l] and,
 * each in turn, out. Equivalent to nlayers calls of qw_path_gg_moe. */
bool qw_path_gg_moe_stack(qw_path *p, qw_batch *b, const qw_moe_layer *M, int nlayers, int nb, const qw_buf *x, const qw_buf *lg,
                          const qw_buf *sel, const qw_buf *out);
/* After which layers of a stack the recorded part is submitted (qw_batch_flush) so that the GPU runs while the host
 * records the rest: bit l = after layer l, the reference's vb_flush (src/engine.c:142, :5997, where the default is 0).
 * Default here: 0x101 (after layers 0 and 8) — this backend launches at submit, so without it the GPU waits for the
 * whole step to be recorded; measured on the 48-layer step at one token: 1.73 ms a step unsplit, 1.72 with bit 0, 1.65
 * with bits 0 and 8, 1.72–1.97 with six flushes (each costs the host two events and a pass over the bound buffers).
 * A batch takes at most 8 flushes; a profiled batch is never split. */
void qw_path_set_flush(qw_path *p, uint64_t mask);
/* A ragged step of one layer, the way the reference's scheduler hands it over (qw_engine_par_vstep, src/engine.c:9138-9161,
 * and qw_engine_par_step, :8798-8814): slot i contributes n[i] >= 1 consecutive rows of x [R][D] (binary16), its first row
 * being r0[i] = n[0] + ... + n[i - 1]; R = sum n[i] <= QW_PAR_MAX. The rows are cut into groups of at most 16 by par's
 * measured table (qw_par_split), each group runs the layer in a batch of its own (the weights of the experts it picks are
 * read once per group) into the same rows of out [R][D], and the wall time of every group is fed back to par
 * (qw_par_observe; the first sample of a size is dropped, as src/engine.c:9037 does). A row's result does not depend on
 * the group it falls into (bit for bit). The path must have been opened for 16 tokens. info (may be NULL) receives the cut.
 * The packing path (qw_path_pf_moe) is the other form of such a step when the routing is known to the caller;
 * qw_par_choose() weighs the two. */
typedef struct {
    int rows, ngroups, groups[64], r0[64];
    double gpu_ms, wall_ms; /* summed over the groups */
} qw_vstep_info;
struct qw_par;
bool qw_path_par_vstep(qw_path *p, struct qw_par *par, const qw_moe_layer *M, const int *n, int B, const qw_buf *x, const qw_buf *out, qw_vstep_info *info);

/* Ragged batch through the packing path (the routed part of the reference's pf_moe(), src/engine.c:4203-4254, with
 * the kernels of kernels/moe_prefill.metal and moe_pf_gg): T rows of x, P = T * topk (token, expert) pairs given by
 * ids [P] (uint32) and weights w [P] (float); count -> plan -> scatter -> gate / up products -> SiLU -> down product
 * -> gathered weighted sum into out [T][D] binary16 (routed experts only). tm = rows per tile entry (16, 32 or 64).
 * qw_path_pf_reserve sizes the packing scratch for up to tmax rows; 0 .. 6 of qw_path_pf_scratch are counts, offsets,
 * tile table, pos_of, packed x, H, packed down output. */
bool qw_path_pf_reserve(qw_path *p, int tmax, int tm);
bool qw_path_pf_moe(qw_path *p, qw_batch *b, const qw_moe_layer *M, int T, const qw_buf *x, const qw_buf *ids, const qw_buf *w, const qw_buf *out);
const qw_buf *qw_path_pf_scratch(const qw_path *p, int which);
unsigned qw_path_pf_max_tiles(const qw_path *p);

/* The hyper-connection in front of a sublayer, GGUF profile (hyper_gg(), src/engine.c:1344-1412; kernels/hyper_gg.metal):
 * nb tokens with QW_PATH_HC residual streams of D values each. h [nb][HC][D] float (written back when apply),
 * out [nb][D] binary16 (the previous sublayer's output, read only when apply), inj [nb][HC][HC] float (inject sums of the
 * previous hyper-connection) -> x [nb][D] binary16 (the sublayer's input), inj_out [nb][HC][HC] (when H has inject rows).
 * Weights: hc_norm F32 [HC * D], mix_down BF16 [QW_PATH_HC_LR][HC * D], mix_up BF16 [HC * D][QW_PATH_HC_LR], inject
 * BF16 [HC][HC * D] (inject.buf NULL: none, as the reference's final mixer). pd is scratch of
 * qw_path_hyper_pd_bytes(nb) bytes. three: record the reference's three-kernel sequence (ghc_dsk, ghc_mid, ghc_upv;
 * its path for more than one token) instead of the two-kernel one; same results up to the float sums' order. D is the
 * path's; it must be a multiple of 512. All in binary32 on the device, as the reference. */
#define QW_PATH_HC 4
#define QW_PATH_HC_LR 320
typedef struct { qw_tensor hc_norm, mix_down, mix_up, inject; } qw_hyper_w;
size_t qw_path_hyper_pd_bytes(int nb);
bool qw_path_hyper_gg(qw_path *p, qw_batch *b, const qw_hyper_w *H, int nb, bool apply, bool three, const qw_buf *h, const qw_buf *out, const qw_buf *inj,
                      const qw_buf *inj_out, const qw_buf *pd, const qw_buf *x);

/* nlayers times: hyper-connection H[l] (h, and from the second layer on — or at once when pending — the residual of out)
 * -> x, then MoE layer M[l]: x -> out. The FFN half of the reference's layer loop (hyper_in then moe,
 * src/engine.c:1415-1423, :2169) with a real dependency from layer to layer. inj: two buffers of nb x HC x HC floats, the
 * first holding the inject sums to start from; they alternate as the reference swaps them. On return out holds the last
 * layer's output, still to be applied. lg and sel: one per layer, as for qw_path_gg_moe_stack. */
bool qw_path_hyper_moe_stack(qw_path *p, qw_batch *b, const qw_hyper_w *H, const qw_moe_layer *M, int nlayers, int nb, bool pending, const qw_buf *h,
                             const qw_buf *inj, const qw_buf *pd, const qw_buf *x, const qw_buf *lg, const qw_buf *sel, const qw_buf *out);

/* The layer for callers that cannot allocate. No counterpart in the reference: it exists for callers that must not call
 * hipMalloc or any allocating routine while they run the layer — a stream under HIP graph capture, a tight serving loop,
 * a harness that forbids allocation. It is qw_path_gg_moe() (same dispatches, same kernels, same results bit for bit)
 * with plain device pointers: the weights, x [nb][D] and out [nb][D] (binary16) are the caller's device memory; the
 * layer's intermediates (logits, selection record, H, Psh, Pg: what qw_path_open() allocates for qw_path_gg_moe()) live
 * in a per-device array of 4 MiB inside the library that the device holds until the process ends. Limits (larger shapes
 * are refused with a message): QW_NOALLOC_MAX_NB tokens, D <= QW_NOALLOC_MAX_D, I <= QW_NOALLOC_MAX_I, E <=
 * QW_NOALLOC_MAX_E, topk <= QW_NOALLOC_MAX_TOPK, and the formats qw_path_gg_moe() takes. The call records and launches on
 * `stream` (a hipStream_t; NULL = the stream qw_gpu_set_stream selected) and returns without waiting: no device or pinned
 * memory is allocated or freed, no event or stream is made, nothing is copied, and a tile-major copy of the weights is
 * used when an earlier allocating call made one, never made here (the GGUF rows are read directly otherwise; same
 * results). The first call for a shape registers that shape's kernel names with the device (a few small host
 * allocations and look-ups in the code object, nothing on the device): a caller that must not even do that makes one
 * call per shape beforehand. Every call on a device uses the same array, which keeps the last call's contents (nothing in it has to
 * start from zero): calls that overlap on one device, on any streams, race. */
#define QW_NOALLOC_MAX_NB 16
#define QW_NOALLOC_MAX_D 2560
#define QW_NOALLOC_MAX_I 640
#define QW_NOALLOC_MAX_E 1024
#define QW_NOALLOC_MAX_TOPK 16
typedef struct { /* device addresses and ggml types of one layer's weights (qw_moe_layer without the buffers) */
    const void *router, *sh_gate_w, *gate, *up, *down, *sh_gate, *sh_up, *sh_down;
    int router_type, gate_type, down_type, sh_gate_type, sh_up_type, sh_down_type;
} qw_moe_weights_dev;
bool qw_path_gg_moe_noalloc(qw_gpu *g, int D, int I, int E, int topk, const qw_moe_weights_dev *W, int nb, const void *x, void *out, void *stream);

/* The scratch buffers, for tests: 0 = lookup tables, 1 = H, 2 = Psh, 3 = Pg. */
const qw_buf *qw_path_scratch(const qw_path *p, int which);

#ifdef __cplusplus
}
#endif
