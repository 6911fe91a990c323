// Host side of the quantized decode path over gpu.h: the call sequences of the reference's engine for this path
// (src/engine.c:439-724), written against the interface only. See include/qw_path.h.
#include "qw_path.h"
#include "qw_hip_ext.h"
#include "qw_par.h"
#include "qw_internal.h"
#include "kernels/qw_kargs.h"
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

struct qw_path {
    qw_gpu *g;
    int D, I, E, topk, nbmax;
    qw_buf tab, H, psh, pd, cnt;
    bool tab_ready;
    // packing scratch (qw_path_pf_reserve)
    qw_buf pcnt, poffs, pcur, ptiles, ppos, pXs, pGg, pGu, pH, pDm;
    int pf_tmax, pf_tm;
    int rbf; // 1: moe_pre_gg computes the router (src/engine.c:577); 0: the logits are given
    bool device_scratch; // scratch without host shadows (qw_path_open)
    unsigned pf_max_tiles;
    uint64_t flush_mask; // bit l: submit what is recorded after layer l of a stack (src/engine.c:142, :5997 vb_flush)
    qw_buf vlg, vsel;    // logits and selection record of one group of a ragged step (qw_path_par_vstep), made at first use
};

static int blk_values(int type) { // src/gguf.c:15-25
    switch (type) {
    case 1: case 30: return 1;
    case 8: case 20: return 32;
    case 12: case 13: case 14: case 21: case 23: return 256;
    default: return 0;
    }
}
static int blk_bytes(int type) {
    switch (type) {
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
static int row_bytes(int type, int K) { return blk_values(type) ? K / blk_values(type) * blk_bytes(type) : 0; }

int qw_path_nbv(int nb) { return nb <= 1 ? 1 : nb <= 2 ? 2 : nb <= 4 ? 4 : nb <= 8 ? 8 : 16; }
static int gnb_of(int nb) { return qw_path_nbv(nb) <= 8 ? 8 : 16; }

size_t qw_path_sel_bytes(const qw_path *p, int nb) { return QW_SEL_BYTES((size_t)gnb_of(nb), (size_t)p->topk); }
size_t qw_path_logits_bytes(const qw_path *p, int nb) { return (size_t)nb * (size_t)(p->E + 1) * 4; }

qw_path *qw_path_open(qw_gpu *g, int D, int I, int E, int topk, int nbmax, bool device_scratch) {
    if (!g || nbmax < 1 || nbmax > 16) return NULL;
    qw_path *p = calloc(1, sizeof *p);
    if (!p) return NULL;
    *p = (qw_path){.g = g, .D = D, .I = I, .E = E, .topk = topk, .nbmax = nbmax, .flush_mask = 0x101, .device_scratch = device_scratch};
    const size_t nb = (size_t)qw_path_nbv(nbmax);
    bool (*mk)(qw_gpu *, size_t, qw_buf *) = device_scratch ? qw_hip_buf_new_device : qw_buf_new;
    // sizes as the engine allocates them: H [nb][topk + 1][I] float, Psh [nb][D] float, Pg [nb][topk][D] float (src/engine.c:157)
    if (!mk(g, QW_TAB_BYTES, &p->tab) || !mk(g, nb * (size_t)(topk + 1) * (size_t)I * 4, &p->H) || !mk(g, nb * (size_t)D * 4, &p->psh) ||
        !mk(g, nb * (size_t)topk * (size_t)D * 4, &p->pd) || !mk(g, 16, &p->cnt)) {
        qw_path_close(p);
        return NULL;
    }
    return p;
}

void qw_path_close(qw_path *p) {
    if (!p) return;
    qw_buf_free(&p->tab); qw_buf_free(&p->H); qw_buf_free(&p->psh); qw_buf_free(&p->pd); qw_buf_free(&p->cnt);
    qw_buf_free(&p->vlg); qw_buf_free(&p->vsel);
    qw_buf *pf[] = {&p->pcnt, &p->poffs, &p->pcur, &p->ptiles, &p->ppos, &p->pXs, &p->pGg, &p->pGu, &p->pH, &p->pDm};
    for (size_t i = 0; i < sizeof pf / sizeof *pf; i++) qw_buf_free(pf[i]);
    free(p);
}

const qw_buf *qw_path_scratch(const qw_path *p, int which) { return which == 0 ? &p->tab : which == 1 ? &p->H : which == 2 ? &p->psh : which == 3 ? &p->pd : NULL; }

static qw_kernel *compile_get(qw_path *p, const char *name, const char *defs) {
    char err[2048];
    qw_kernel *k = qw_kernel_get(p->g, name);
    if (k) return k;
    if (!qw_gpu_compile(p->g, defs, strlen(defs), err, sizeof err)) {
        fprintf(stderr, "compile %s failed: %s\n", name, err);
        return NULL;
    }
    k = qw_kernel_get(p->g, name);
    if (!k) fprintf(stderr, "kernel %s not found\n", name);
    return k;
}

// ---------------------------------------------------------------- dense matvec (src/engine.c:689-724)
bool qw_path_qmv_gg(qw_path *p, qw_batch *b, const qw_tensor *W, int N, int K, const qw_buf *x, size_t xoff, const qw_buf *y,
                    size_t yoff, int nb, bool fout) {
    char name[96], defs[512];
    const int f = W->type;
    snprintf(name, sizeof name, "qmv_gg_f%d_k%d_n%d%s", f, K, nb, fout ? "_f" : "");
    snprintf(defs, sizeof defs, "#define IQ_DQ_ONLY 1\n#define qmv_gg %s\n#define GF %d\n#define KD %d\n#define RB %d\n#define NB %d\n%s", name, f, K,
             row_bytes(f, K), nb, fout ? "#define YT float\n" : "");
    qw_kernel *k = compile_get(p, name, defs);
    if (!k) return false;
    struct { uint32_t N, xs, ys, pad; } a = {(uint32_t)N, (uint32_t)K, (uint32_t)N, 0};
    qw_batch_kernel(b, k);
    qw_batch_buf(b, 0, W->buf, W->offset);
    qw_batch_buf(b, 3, x, xoff);
    qw_batch_buf(b, 4, y, yoff);
    qw_batch_bytes(b, 5, &a, sizeof a);
    qw_batch_dispatch(b, ((unsigned)N + 7) / 8, 1, 1, 256, 1, 1);
    return true;
}

// ---------------------------------------------------------------- several matrices over one x (src/engine.c:730-771)
bool qw_path_qmv_ggm(qw_path *p, qw_batch *b, const qw_tensor *W, const int *N, int n, int K, const qw_buf *x, const qw_buf *const *y, int nb, bool fout) {
    if (n < 1 || n > 4 || nb < 1 || nb > 16 || K % 256) {
        fprintf(stderr, "qmv_ggm: %d matrices / %d tokens / K %d outside 1..4 / 1..16 / multiples of 256\n", n, nb, K);
        return false;
    }
    char base[128], name[140], defs[512];
    int f[4];
    for (int i = 0; i < 4; i++) f[i] = W[i < n ? i : 0].type;
    snprintf(base, sizeof base, "qmv_ggm_k%d_m%d_%d_%d_%d_%d%s", K, n, f[0], f[1], f[2], f[3], fout ? "_f" : "");
    snprintf(name, sizeof name, "%s_b%d", base, nb);
    snprintf(defs, sizeof defs, "#define IQ_DQ_ONLY 1\n#define qmv_ggm %s\n#define KD %d\n#define NB 0\n#define NMAT %d\n#define GF0 %d\n#define GF1 %d\n#define GF2 %d\n#define GF3 %d\n%s",
             base, K, n, f[0], f[1], f[2], f[3], fout ? "#define YT float\n" : "");
    qw_kernel *k = compile_get(p, name, defs);
    if (!k) return false;
    struct { uint32_t N[4], off[4], total, xstride; } a = {{0}, {0}, 0, (uint32_t)K};
    qw_batch_kernel(b, k);
    for (int i = 0; i < 4; i++) {
        const int j = i < n ? i : 0;
        qw_batch_buf(b, (unsigned)i, W[j].buf, W[j].offset);
        qw_batch_buf(b, 5u + (unsigned)i, y[j], 0);
        a.N[i] = i < n ? (uint32_t)N[i] : 0;
        a.off[i] = a.total;
        if (i < n) a.total += (uint32_t)N[i];
    }
    qw_batch_buf(b, 4, x, 0);
    qw_batch_bytes(b, 9, &a, sizeof a);
    qw_batch_dispatch(b, (a.total + 7) / 8, 1, 1, 256, 1, 1);
    return true;
}

// ---------------------------------------------------------------- MoE kernels by part (src/engine.c:460-517)
static qw_kernel *gg_kernel(qw_path *p, const char *base, const qw_moe_layer *M, int nb) {
    const int part = !strcmp(base, "moe_sel_gg") || !strcmp(base, "gg_tab_init") ? 0 : !strcmp(base, "moe_pre_gg") ? 1 : !strcmp(base, "moe_gu_gg") ? 2
                     : !strcmp(base, "moe_dn_gg") || !strcmp(base, "moe_cmb_gg") ? 3 : 4;
    const int nbv = part == 4 ? nb : qw_path_nbv(nb);
    const int rwf = M->router.type;
    char name[128], sfx[96], defs[2048];
    switch (part) {
    case 0: snprintf(sfx, sizeof sfx, "_n%d", nbv); break;
    case 1: snprintf(sfx, sizeof sfx, "_%d_%d_r%d_w%d_n%d", M->sh_gate.type, M->sh_up.type, p->rbf, rwf, nbv); break;
    case 2: snprintf(sfx, sizeof sfx, "_%d_%d_g%d_n%d", M->gate.type, M->sh_down.type, 1, nbv); break;
    case 3: snprintf(sfx, sizeof sfx, "_%d_s%d_n%d", M->down.type, 4, nbv); break;
    default: snprintf(sfx, sizeof sfx, "_w%d_n%d", rwf, nbv);
    }
    // one model per process in the reference, so its names carry no shape; a qw_gpu here may serve several shapes
    snprintf(sfx + strlen(sfx), sizeof sfx - strlen(sfx), "_e%dk%dd%di%d", p->E, p->topk, p->D, p->I);
    snprintf(name, sizeof name, "%s%s", base, sfx);
    qw_kernel *k = qw_kernel_get(p->g, name);
    if (k) return k;
    if (nb < 1 || nb > 16) {
        fprintf(stderr, "%s: unsupported token count %d\n", name, nb);
        return NULL;
    }
    int n = snprintf(defs, sizeof defs, "#define IQ_DQ_ONLY\n#define E %d\n#define TOPK %d\n#define D %d\n#define I %d\n#define NB %d\n#define RWF %d\n", p->E, p->topk,
                     p->D, p->I, nbv, rwf);
    switch (part) {
    case 0: snprintf(defs + n, sizeof defs - (size_t)n, "#define GG_PART 0\n#define moe_sel_gg moe_sel_gg%s\n#define gg_tab_init gg_tab_init%s\n", sfx, sfx); break;
    case 1:
        snprintf(defs + n, sizeof defs - (size_t)n, "#define GG_PART 1\n#define FSG %d\n#define FSU %d\n#define RBF %d\n#define moe_pre_gg moe_pre_gg%s\n", M->sh_gate.type,
                 M->sh_up.type, p->rbf, sfx);
        break;
    case 2:
        snprintf(defs + n, sizeof defs - (size_t)n, "#define GG_PART 2\n#define GSG %d\n#define RG %d\n#define FGU %d\n#define FSD %d\n#define moe_gu_gg moe_gu_gg%s\n", 8, 1,
                 M->gate.type, M->sh_down.type, sfx);
        break;
    case 3:
        snprintf(defs + n, sizeof defs - (size_t)n, "#define GG_PART 3\n#define FD %d\n#define DSGN %d\n#define moe_dn_gg moe_dn_gg%s\n#define moe_cmb_gg moe_cmb_gg%s\n",
                 M->down.type, 4, sfx, sfx);
        break;
    default:
        snprintf(defs + n, sizeof defs - (size_t)n, "#define GG_ROUTER\n#define moe_router_bf moe_router_bf%s\n#define p_router_bf p_router_bf%s\n"
                 "#define p_router_bf_refine p_router_bf_refine%s\n", sfx, sfx, sfx);
    }
    return compile_get(p, name, defs);
}

static void bind_t(qw_batch *b, unsigned index, const qw_tensor *t) { qw_batch_buf(b, index, t->buf, t->offset); }

// ---------------------------------------------------------------- hyper-connection (src/engine.c:1323-1412)
// The define block of gh_kernel (src/engine.c:1328-1333): the five kernel names carry the token count (and here the
// width, since one qw_gpu may serve several shapes); GH_R, GH_G, GU_SG, GV_SG, GV_RP and GK are the reference's
// defaults for its own kernels (src/engine.c:1295-1312) and mean nothing to this backend.
static qw_kernel *gh_kernel(qw_path *p, const char *base, int nb) {
    char name[64], defs[768];
    snprintf(name, sizeof name, "%s_n%d_d%d", base, nb, p->D);
    qw_kernel *k = qw_kernel_get(p->g, name);
    if (k) return k;
    snprintf(defs, sizeof defs,
             "#define ghc_down ghc_down_n%d_d%d\n#define ghc_up ghc_up_n%d_d%d\n#define ghc_dsk ghc_dsk_n%d_d%d\n#define ghc_mid ghc_mid_n%d_d%d\n"
             "#define ghc_upv ghc_upv_n%d_d%d\n#define D %d\n#define HC %d\n#define NB %d\n"
             "#define GH_R %d\n#define GH_G %d\n#define GU_SG %d\n#define GV_SG %d\n#define GV_RP %d\n#define GK %d\n",
             nb, p->D, nb, p->D, nb, p->D, nb, p->D, nb, p->D, p->D, QW_PATH_HC, nb, nb <= 4 ? 16 : 32, nb <= 2 ? 16 : 8, 8, 8, 10, 10);
    return compile_get(p, name, defs);
}
size_t qw_path_hyper_pd_bytes(int nb) { return (size_t)nb * (QW_PATH_HC * (QW_PATH_HC_LR + 2 * QW_PATH_HC) + QW_PATH_HC_LR + QW_PATH_HC) * 4; }

bool qw_path_hyper_gg(qw_path *p, qw_batch *b, const qw_hyper_w *H, int nb, bool apply, bool three, const qw_buf *h, const qw_buf *out, const qw_buf *inj,
                      const qw_buf *inj_out, const qw_buf *pd, const qw_buf *x) {
    if (nb < 1 || nb > 16) { fprintf(stderr, "hyper_gg: unsupported token count %d\n", nb); return false; }
    if (H->hc_norm.type != 0 || H->mix_down.type != 30 || H->mix_up.type != 30 || (H->inject.buf && H->inject.type != 30)) {
        fprintf(stderr, "hyper_gg: the norm weights must be F32 (0) and the matrices BF16 (30): got %d, %d, %d, %d\n", H->hc_norm.type, H->mix_down.type, H->mix_up.type, H->inject.type);
        return false;
    }
    const uint32_t fl[2] = {apply ? 1u : 0u, H->inject.buf ? 1u : 0u};
    const qw_tensor *inj_w = H->inject.buf ? &H->inject : &H->mix_down; // src/engine.c:1357-1358: something is bound at 5 either way
    qw_kernel *kd = gh_kernel(p, three ? "ghc_dsk" : "ghc_down", nb);
    if (!kd) return false;
    qw_batch_kernel(b, kd);
    qw_batch_buf(b, 0, h, 0);
    qw_batch_buf(b, 1, out, 0);
    qw_batch_buf(b, 2, inj, 0);
    bind_t(b, 3, &H->hc_norm);
    bind_t(b, 4, &H->mix_down);
    bind_t(b, 5, inj_w);
    qw_batch_buf(b, 6, pd, 0);
    qw_batch_bytes(b, 7, fl, sizeof fl);
    if (three) qw_batch_dispatch(b, 10, QW_PATH_HC, 10, 32 * 8, 1, 1);
    else qw_batch_dispatch(b, QW_PATH_HC_LR / (nb <= 4 ? 16 : 32) + 1, QW_PATH_HC, 1, (unsigned)p->D / 8, 1, 1);
    if (three) { // src/engine.c:1364-1386; sx and rs follow the partial sums in pd
        const size_t o_sx = (size_t)nb * QW_PATH_HC * (QW_PATH_HC_LR + 2 * QW_PATH_HC) * 4, o_rs = o_sx + (size_t)nb * QW_PATH_HC_LR * 4;
        qw_kernel *km = gh_kernel(p, "ghc_mid", nb), *kv = gh_kernel(p, "ghc_upv", nb);
        if (!km || !kv) return false;
        qw_batch_kernel(b, km);
        qw_batch_buf(b, 0, pd, 0);
        qw_batch_buf(b, 1, pd, o_sx);
        qw_batch_buf(b, 2, pd, o_rs);
        if (inj_out) qw_batch_buf(b, 3, inj_out, 0);
        qw_batch_bytes(b, 4, fl, sizeof fl);
        qw_batch_dispatch(b, (unsigned)nb, 1, 1, QW_PATH_HC_LR, 1, 1);
        qw_batch_kernel(b, kv);
        qw_batch_buf(b, 0, h, 0);
        qw_batch_buf(b, 1, out, 0);
        qw_batch_buf(b, 2, inj, 0);
        bind_t(b, 3, &H->hc_norm);
        bind_t(b, 4, &H->mix_up);
        qw_batch_buf(b, 5, pd, o_sx);
        qw_batch_buf(b, 6, pd, o_rs);
        qw_batch_buf(b, 7, x, 0);
        qw_batch_bytes(b, 8, fl, sizeof fl);
        qw_batch_dispatch(b, (unsigned)p->D / 8, 1, 1, 32 * 8, 1, 1);
        return true;
    }
    qw_kernel *ku = gh_kernel(p, "ghc_up", nb);
    if (!ku) return false;
    qw_batch_kernel(b, ku);
    qw_batch_buf(b, 0, h, 0);
    qw_batch_buf(b, 1, out, 0);
    qw_batch_buf(b, 2, inj, 0);
    bind_t(b, 3, &H->hc_norm);
    bind_t(b, 4, &H->mix_up);
    qw_batch_buf(b, 5, pd, 0);
    qw_batch_buf(b, 6, x, 0);
    if (inj_out) qw_batch_buf(b, 7, inj_out, 0);
    qw_batch_bytes(b, 8, fl, sizeof fl);
    qw_batch_dispatch(b, (unsigned)p->D / 8, 1, 1, 32 * 8, 1, 1);
    return true;
}

// src/engine.c:544-552
bool qw_path_gg_router(qw_path *p, qw_batch *b, const qw_moe_layer *M, int nb, const qw_buf *x, const qw_buf *lg) {
    qw_kernel *k = gg_kernel(p, "moe_router_bf", M, nb);
    if (!k) return false;
    qw_batch_kernel(b, k);
    bind_t(b, 0, &M->router);
    bind_t(b, 1, &M->sh_gate_w);
    qw_batch_buf(b, 2, x, 0);
    qw_batch_buf(b, 3, lg, 0);
    qw_batch_dispatch(b, ((unsigned)p->E + 1 + 7) / 8, 1, 1, 256, 1, 1);
    return true;
}

// src/engine.c:568-647: front part (router + shared gate/up + selection) -> routed gate/up + shared down -> routed down -> combine
static bool gg_moe_at(qw_path *p, qw_batch *b, const qw_moe_layer *M, int nb, const qw_buf *x, size_t xoff, const qw_buf *lg, const qw_buf *sel, const qw_buf *out, size_t outoff,
                      bool given);
static bool gg_moe(qw_path *p, qw_batch *b, const qw_moe_layer *M, int nb, const qw_buf *x, const qw_buf *lg, const qw_buf *sel, const qw_buf *out, bool given) {
    return gg_moe_at(p, b, M, nb, x, 0, lg, sel, out, 0, given);
}
bool qw_path_gg_moe(qw_path *p, qw_batch *b, const qw_moe_layer *M, int nb, const qw_buf *x, const qw_buf *lg, const qw_buf *sel,
                    const qw_buf *out) {
    return gg_moe(p, b, M, nb, x, lg, sel, out, false);
}
bool qw_path_gg_moe_lg(qw_path *p, qw_batch *b, const qw_moe_layer *M, int nb, const qw_buf *x, const qw_buf *lg, const qw_buf *sel,
                       const qw_buf *out) {
    return gg_moe(p, b, M, nb, x, lg, sel, out, true);
}
// x and out may be rows of larger buffers (byte offsets): the rows of one group of a step
static bool gg_moe_at(qw_path *p, qw_batch *b, const qw_moe_layer *M, int nb, const qw_buf *x, size_t xoff, const qw_buf *lg, const qw_buf *sel, const qw_buf *out, size_t outoff,
                      bool given) {
    p->rbf = given ? 0 : 1;
    if (nb < 1 || nb > p->nbmax) {
        fprintf(stderr, "gg_moe: %d tokens, scratch was sized for %d\n", nb, p->nbmax);
        return false;
    }
    qw_kernel *k;
    if (!p->tab_ready) { // first use: build the lookup tables in the same batch, before they are needed
        if (!(k = gg_kernel(p, "gg_tab_init", M, 1))) return false;
        qw_batch_kernel(b, k);
        qw_batch_buf(b, 0, &p->tab, 0);
        qw_batch_dispatch(b, 32, 1, 1, 256, 1, 1);
        p->tab_ready = true;
    }
    const uint32_t nbr = (uint32_t)nb;
    const unsigned E = (unsigned)p->E, I = (unsigned)p->I, D = (unsigned)p->D, K = (unsigned)p->topk;
    if (given) { // the selection from the caller's logits (src/engine.c:609-614)
        if (!(k = gg_kernel(p, "moe_sel_gg", M, nb))) return false;
        qw_batch_kernel(b, k);
        qw_batch_buf(b, 0, lg, 0);
        qw_batch_buf(b, 1, sel, 0);
        qw_batch_bytes(b, 2, &nbr, 4);
        qw_batch_dispatch(b, 1, 1, 1, 1024, 1, 1);
    }
    if (!(k = gg_kernel(p, "moe_pre_gg", M, nb))) return false;
    qw_batch_kernel(b, k);
    bind_t(b, 0, &M->router);
    bind_t(b, 1, &M->sh_gate_w);
    qw_batch_buf(b, 2, x, xoff);
    qw_batch_buf(b, 3, lg, 0);
    qw_batch_buf(b, 4, &p->cnt, 0);
    qw_batch_buf(b, 5, sel, 0);
    bind_t(b, 6, &M->sh_gate);
    bind_t(b, 7, &M->sh_up);
    qw_batch_buf(b, 8, &p->H, 0);
    for (unsigned i = 0; i < 2; i++) { // scale / bias slots of the MLX formats: bound to the weights as placeholders
        bind_t(b, 9 + 2 * i, i ? &M->sh_up : &M->sh_gate);
        bind_t(b, 10 + 2 * i, i ? &M->sh_up : &M->sh_gate);
    }
    qw_batch_buf(b, 13, &p->tab, 0);
    qw_batch_bytes(b, 14, &nbr, 4);
    qw_batch_dispatch(b, (E + 1 + 7) / 8 + I / 8, 1, 1, 256, 1, 1);

    if (!(k = gg_kernel(p, "moe_gu_gg", M, nb))) return false;
    qw_batch_kernel(b, k);
    bind_t(b, 0, &M->gate);
    bind_t(b, 1, &M->up);
    bind_t(b, 2, &M->sh_down);
    qw_batch_buf(b, 3, &p->psh, 0);
    qw_batch_buf(b, 4, x, xoff);
    qw_batch_buf(b, 5, sel, 0);
    qw_batch_buf(b, 6, &p->H, 0);
    bind_t(b, 7, &M->sh_down);
    bind_t(b, 8, &M->sh_down);
    qw_batch_buf(b, 11, &p->tab, 0);
    qw_batch_bytes(b, 12, &nbr, 4);
    {
        const unsigned a = I / 8, c = D / 32;
        qw_batch_dispatch(b, a > c ? a : c, nbr * K + 1, 1, 256, 1, 1);
    }

    if (!(k = gg_kernel(p, "moe_dn_gg", M, nb))) return false;
    qw_batch_kernel(b, k);
    bind_t(b, 0, &M->down);
    qw_batch_buf(b, 2, &p->H, 0);
    qw_batch_buf(b, 3, sel, 0);
    qw_batch_buf(b, 7, &p->tab, 0);
    qw_batch_buf(b, 9, &p->pd, 0);
    qw_batch_dispatch(b, D / 16, nbr * K, 1, 128, 1, 1);

    if (!(k = gg_kernel(p, "moe_cmb_gg", M, nb))) return false;
    qw_batch_kernel(b, k);
    qw_batch_buf(b, 1, &p->psh, 0);
    qw_batch_buf(b, 3, sel, 0);
    qw_batch_buf(b, 4, out, outoff);
    qw_batch_bytes(b, 8, &nbr, 4);
    qw_batch_buf(b, 9, &p->pd, 0);
    qw_batch_dispatch(b, D / 256, 1, 1, 256, 1, 1);
    return true;
}

bool qw_path_gg_moe_stack(qw_path *p, qw_batch *b, const qw_moe_layer *M, int nlayers, int nb, const qw_buf *x, const qw_buf *lg,
                          const qw_buf *sel, const qw_buf *out) {
    for (int l = 0; l < nlayers; l++) {
        if (!qw_path_gg_moe(p, b, &M[l], nb, x, &lg[l], &sel[l], out)) return false;
        // the recorded part goes to the GPU while the host records the rest (at most 8 times a batch, src/gpu.h:54-56)
        if (l < 64 && (p->flush_mask >> l & 1) && l + 1 < nlayers) qw_batch_flush(b);
    }
    return true;
}
void qw_path_set_flush(qw_path *p, uint64_t mask) { p->flush_mask = mask; }

// The FFN half of a decode step, layer after layer (the hyper_in -> moe pair of the reference's layer loop,
// src/engine.c:1415-1423 and :2169): hyper-connection l turns the streams h into the layer's input x, applying the
// residual of what the layer before left in out; the MoE layer turns x into out. The inject sums alternate between
// inj[0] and inj[1] as src/engine.c:1421 swaps them.
bool qw_path_hyper_moe_stack(qw_path *p, qw_batch *b, const qw_hyper_w *H, const qw_moe_layer *M, int nlayers, int nb, bool pending, const qw_buf *h,
                             const qw_buf *inj, const qw_buf *pd, const qw_buf *x, const qw_buf *lg, const qw_buf *sel, const qw_buf *out) {
    int cur = 0;
    for (int l = 0; l < nlayers; l++) {
        if (!qw_path_hyper_gg(p, b, &H[l], nb, pending, false, h, out, &inj[cur], &inj[cur ^ 1], pd, x)) return false;
        if (H[l].inject.buf) cur ^= 1;
        if (!qw_path_gg_moe(p, b, &M[l], nb, x, &lg[l], &sel[l], out)) return false;
        pending = true;
        if (l < 64 && (p->flush_mask >> l & 1) && l + 1 < nlayers) qw_batch_flush(b);
    }
    return true;
}

// ---------------------------------------------------------------- a ragged step (src/engine.c:8783-8814, :9138-9161, :9037)
// Slot i brings n[i] rows; its first row is r0[i] = n[0] + ... + n[i - 1] (src/engine.c:9150-9161). The R rows are cut
// into groups by the measured table (qw_par_split: the reference's par_split with groups of up to 16 rows), every
// group is one batch through the layer (the reference's par_step runs its groups one after the other, each reading
// the weights once, src/engine.c:8805-8812), and each group's wall time goes back into the table (src/engine.c:9037).
bool qw_path_par_vstep(qw_path *p, qw_par *par, const qw_moe_layer *M, const int *n, int B, const qw_buf *x, const qw_buf *out, qw_vstep_info *info) {
    if (!p || !par || !M || !n || !x || !out || B < 1 || B > QW_PAR_MAX) return false;
    int R = 0, r0[QW_PAR_MAX];
    for (int i = 0; i < B; i++) {
        if (n[i] < 1) return false; // src/engine.c:9141
        r0[i] = R;
        R += n[i];
    }
    if (R > QW_PAR_MAX || p->nbmax < QW_PAR_VBMAX) {
        fprintf(stderr, "qw_path_par_vstep: %d rows (at most %d), path opened for %d tokens (needs %d)\n", R, QW_PAR_MAX, p->nbmax, QW_PAR_VBMAX);
        return false;
    }
    if ((size_t)R * (size_t)p->D * 2 > x->size || (size_t)R * (size_t)p->D * 2 > out->size) return false;
    if (!p->vlg.handle && (!qw_hip_buf_new_device(p->g, qw_path_logits_bytes(p, QW_PAR_VBMAX), &p->vlg) || !qw_hip_buf_new_device(p->g, qw_path_sel_bytes(p, QW_PAR_VBMAX), &p->vsel)))
        return false;
    int grp[QW_PAR_MAX];
    const int ng = qw_par_split(par, R, grp);
    if (info) {
        *info = (qw_vstep_info){.rows = R, .ngroups = ng};
        memcpy(info->r0, r0, sizeof(int) * (size_t)B);
        memcpy(info->groups, grp, sizeof(int) * (size_t)ng);
    }
    double gpu = 0, wall = 0;
    for (int gi = 0, c = 0; gi < ng; c += grp[gi++]) {
        const double t0 = qw_now();
        qw_batch *b = qw_batch_begin(p->g, false);
        if (!b) return false;
        const bool rec = gg_moe_at(p, b, M, grp[gi], x, (size_t)c * (size_t)p->D * 2, &p->vlg, &p->vsel, out, (size_t)c * (size_t)p->D * 2, false);
        const double t = qw_batch_end(b);
        if (!rec || t < 0) return false;
        const double ms = (qw_now() - t0) * 1e3;
        qw_par_observe(par, grp[gi], ms);
        gpu += t * 1e3, wall += ms;
    }
    if (info) info->gpu_ms = gpu, info->wall_ms = wall;
    return true;
}

// ---------------------------------------------------------------- ragged batch through the packing path (src/engine.c:4133-4254)
bool qw_path_pf_reserve(qw_path *p, int tmax, int tm) {
    if (tmax < 1 || (tm != 16 && tm != 32 && tm != 64)) return false;
    if (p->pf_tmax >= tmax && p->pf_tm == tm) return true;
    qw_buf *pf[] = {&p->pcnt, &p->poffs, &p->pcur, &p->ptiles, &p->ppos, &p->pXs, &p->pGg, &p->pGu, &p->pH, &p->pDm};
    for (size_t i = 0; i < sizeof pf / sizeof *pf; i++) qw_buf_free(pf[i]);
    const size_t P = (size_t)tmax * (size_t)p->topk, E = (size_t)p->E;
    p->pf_max_tiles = (unsigned)((P + (size_t)tm - 1) / (size_t)tm + E); // src/engine.c:4135
    p->pf_tmax = 0;
    // with host shadows every one of these (several MB at full size) would be copied back at every wait
    bool (*mk)(qw_gpu *, size_t, qw_buf *) = p->device_scratch ? qw_hip_buf_new_device : qw_buf_new;
    if (!mk(p->g, E * 4, &p->pcnt) || !mk(p->g, E * 4, &p->poffs) || !mk(p->g, E * 4, &p->pcur) ||
        !mk(p->g, (size_t)p->pf_max_tiles * 16, &p->ptiles) || !mk(p->g, P * 4, &p->ppos) || !mk(p->g, P * (size_t)p->D * 2, &p->pXs) ||
        !mk(p->g, P * (size_t)p->I * 2, &p->pGg) || !mk(p->g, P * (size_t)p->I * 2, &p->pGu) || !mk(p->g, P * (size_t)p->I * 2, &p->pH) ||
        !mk(p->g, P * (size_t)p->D * 2, &p->pDm)) return false;
    p->pf_tmax = tmax;
    p->pf_tm = tm;
    return true;
}
unsigned qw_path_pf_max_tiles(const qw_path *p) { return p->pf_max_tiles; }
const qw_buf *qw_path_pf_scratch(const qw_path *p, int which) {
    const qw_buf *pf[] = {&p->pcnt, &p->poffs, &p->ptiles, &p->ppos, &p->pXs, &p->pH, &p->pDm};
    return which >= 0 && which < 7 ? pf[which] : NULL;
}

static qw_kernel *pk_kernel(qw_path *p, const char *base) { // bench/moe_prefill.c:84-88
    char name[96], defs[512];
    snprintf(name, sizeof name, "%s_e%dk%dd%di%dt%d", base, p->E, p->topk, p->D, p->I, p->pf_tm);
    qw_kernel *k = qw_kernel_get(p->g, name);
    if (k) return k;
    snprintf(defs, sizeof defs, "#define %s %s\n#define E %d\n#define TOPK %d\n#define KD %d\n#define I %d\n#define TM %d\n", base, name, p->E, p->topk, p->D, p->I, p->pf_tm);
    return compile_get(p, name, defs);
}
// src/engine.c:3231-3266: Y [P][N] = X [P][K] . W_e^T over the tile table
static bool pf_qmm_moe_iq(qw_path *p, qw_batch *b, const qw_tensor *W, int N, int K, const qw_buf *X, const qw_buf *Y, uint32_t P) {
    char name[96], defs[1024];
    snprintf(name, sizeof name, "moe_pf_gg_%d_k%d_tm%d_e%d", W->type, K, p->pf_tm, p->E);
    qw_kernel *k = qw_kernel_get(p->g, name);
    if (!k) {
        snprintf(defs, sizeof defs, "#define IQ_DQ_ONLY\n#define E %d\n#define TOPK %d\n#define D %d\n#define I %d\n#define NB 1\n#define GG_PART 5\n"
                 "#define PFF %d\n#define KD %d\n#define TM %d\n#define TN 64\n#define SG 4\n#define KC 64\n#define PFS 1\n#define PFT 1\n#define PFDBG 0\n#define moe_pf_gg %s\n",
                 p->E, p->topk, p->D, p->I, W->type, K, p->pf_tm, name);
        if (!(k = compile_get(p, name, defs))) return false;
    }
    const uint32_t a[2] = {P, (uint32_t)N};
    qw_batch_kernel(b, k);
    qw_batch_buf(b, 0, X, 0);
    qw_batch_buf(b, 1, W->buf, W->offset);
    qw_batch_buf(b, 4, Y, 0);
    qw_batch_bytes(b, 5, a, sizeof a);
    qw_batch_buf(b, 6, &p->ptiles, 0);
    qw_batch_buf(b, 7, &p->tab, 0);
    qw_batch_dispatch(b, (unsigned)N / 64, p->pf_max_tiles, 1, 128, 1, 1);
    return true;
}

bool qw_path_pf_moe(qw_path *p, qw_batch *b, const qw_moe_layer *M, int T, const qw_buf *x, const qw_buf *ids, const qw_buf *w, const qw_buf *out) {
    if (T < 1 || T > p->pf_tmax) {
        fprintf(stderr, "qw_path_pf_moe: %d rows, reserved %d\n", T, p->pf_tmax);
        return false;
    }
    const uint32_t P = (uint32_t)T * (uint32_t)p->topk, tm = (uint32_t)p->pf_tm, n = P * (uint32_t)p->I;
    qw_kernel *k;
    const uint32_t ne = (uint32_t)p->E; // the counters are cleared on the GPU, inside the batch (src/engine.c:4201-4206)
    if (!(k = pk_kernel(p, "p_zero"))) return false;
    qw_batch_kernel(b, k);
    qw_batch_buf(b, 0, &p->pcnt, 0);
    qw_batch_bytes(b, 1, &ne, 4);
    qw_batch_dispatch(b, (ne + 255) / 256, 1, 1, 256, 1, 1);
    if (!(k = pk_kernel(p, "moe_count"))) return false;
    qw_batch_kernel(b, k);
    qw_batch_buf(b, 0, ids, 0);
    qw_batch_buf(b, 1, &p->pcnt, 0);
    qw_batch_bytes(b, 2, &P, 4);
    qw_batch_dispatch(b, (P + 255) / 256, 1, 1, 256, 1, 1);
    if (!(k = pk_kernel(p, "moe_plan_t"))) return false; // src/engine.c:4137-4144
    qw_batch_kernel(b, k);
    qw_batch_buf(b, 0, &p->pcnt, 0);
    qw_batch_buf(b, 1, &p->poffs, 0);
    qw_batch_buf(b, 2, &p->pcur, 0);
    qw_batch_buf(b, 3, &p->ptiles, 0);
    qw_batch_bytes(b, 4, &p->pf_max_tiles, 4);
    qw_batch_bytes(b, 5, &tm, 4);
    qw_batch_dispatch(b, 1, 1, 1, (unsigned)p->E, 1, 1);
    if (!(k = pk_kernel(p, "moe_scatter"))) return false; // src/engine.c:4221-4227
    qw_batch_kernel(b, k);
    qw_batch_buf(b, 0, x, 0);
    qw_batch_buf(b, 1, ids, 0);
    qw_batch_buf(b, 2, &p->pcur, 0);
    qw_batch_buf(b, 3, &p->pXs, 0);
    qw_batch_buf(b, 4, &p->ppos, 0);
    qw_batch_dispatch(b, P, 1, 1, 256, 1, 1);
    if (!pf_qmm_moe_iq(p, b, &M->gate, p->I, p->D, &p->pXs, &p->pGg, P) || !pf_qmm_moe_iq(p, b, &M->up, p->I, p->D, &p->pXs, &p->pGu, P)) return false;
    if (!(k = pk_kernel(p, "p_act2"))) return false; // src/engine.c:4246-4251
    qw_batch_kernel(b, k);
    qw_batch_buf(b, 0, &p->pGg, 0);
    qw_batch_buf(b, 1, &p->pGu, 0);
    qw_batch_buf(b, 2, &p->pH, 0);
    qw_batch_bytes(b, 3, &n, 4);
    qw_batch_dispatch(b, (n + 255) / 256, 1, 1, 256, 1, 1);
    if (!pf_qmm_moe_iq(p, b, &M->down, p->D, p->I, &p->pH, &p->pDm, P)) return false;
    if (!(k = pk_kernel(p, "moe_combine"))) return false; // kernels/moe_prefill.metal:105-119
    qw_batch_kernel(b, k);
    qw_batch_buf(b, 0, &p->pDm, 0);
    qw_batch_buf(b, 1, &p->ppos, 0);
    qw_batch_buf(b, 2, w, 0);
    qw_batch_buf(b, 3, out, 0);
    qw_batch_dispatch(b, (unsigned)p->D / 4 / 64, (unsigned)T, 1, 64, 1, 1);
    return true;
}

// ---------------------------------------------------------------- the layer without any allocation (include/qw_path.h)
// qw_path_gg_moe over memory the caller owns and the device's scratch array: the same dispatches, translators and
// kernels, recorded into the device's fixed recorder and launched on the caller's stream.
bool qw_path_gg_moe_noalloc(qw_gpu *g, int D, int I, int E, int topk, const qw_moe_weights_dev *W, int nb, const void *x, void *out, void *stream) {
    if (!g || !W || !x || !out) return false;
    if (nb < 1 || nb > QW_NOALLOC_MAX_NB || D < 256 || D > QW_NOALLOC_MAX_D || I < 256 || I > QW_NOALLOC_MAX_I || E < 1 || E > QW_NOALLOC_MAX_E || topk < 1 ||
        topk > QW_NOALLOC_MAX_TOPK) {
        fprintf(stderr, "qw_path_gg_moe_noalloc: nb %d / D %d / I %d / E %d / top-%d beyond what the scratch array holds (%d tokens, D %d, I %d, E %d, top-%d)\n", nb, D, I, E,
                topk, QW_NOALLOC_MAX_NB, QW_NOALLOC_MAX_D, QW_NOALLOC_MAX_I, QW_NOALLOC_MAX_E, QW_NOALLOC_MAX_TOPK);
        return false;
    }
    void *base;
    size_t have;
    if (!qw_hip_noalloc_scratch(g, &base, &have)) {
        fprintf(stderr, "qw_path_gg_moe_noalloc: %s\n", qw_hip_last_error(g));
        return false;
    }
    // the array, cut at its largest shape (so that every shape finds its pieces at the same places), 256-byte aligned
    const size_t nbv = 16, gnb = 16, sz[7] = {QW_TAB_BYTES, nbv * (QW_NOALLOC_MAX_E + 1) * 4, QW_SEL_BYTES(gnb, (size_t)QW_NOALLOC_MAX_TOPK),
                                              nbv * (QW_NOALLOC_MAX_TOPK + 1) * (size_t)QW_NOALLOC_MAX_I * 4, nbv * (size_t)QW_NOALLOC_MAX_D * 4,
                                              nbv * QW_NOALLOC_MAX_TOPK * (size_t)QW_NOALLOC_MAX_D * 4, 16};
    size_t off[7], end = 0;
    for (int i = 0; i < 7; i++) off[i] = end, end = (end + sz[i] + 255) & ~(size_t)255;
    if (end > have) {
        fprintf(stderr, "qw_path_gg_moe_noalloc: the scratch array holds %zu bytes, the layer's intermediates need %zu\n", have, end);
        return false;
    }
    qw_hip_view v[7 + 10];
    qw_buf s[7], w[8], xb, ob;
    for (int i = 0; i < 7; i++) qw_hip_view_init(g, &v[i], (char *)base + off[i], sz[i], &s[i]);
    const int rt = W->router_type;
    if ((rt != 1 && rt != 30) || !blk_values(W->gate_type) || !blk_values(W->down_type) || !blk_values(W->sh_gate_type) || !blk_values(W->sh_up_type) || !blk_values(W->sh_down_type)) {
        fprintf(stderr, "qw_path_gg_moe_noalloc: unknown weight type\n");
        return false;
    }
    const size_t e = (size_t)E, ws[8] = {e * (size_t)D * 2, (size_t)D * 2, e * (size_t)I * (size_t)row_bytes(W->gate_type, D), e * (size_t)I * (size_t)row_bytes(W->gate_type, D),
                                         e * (size_t)D * (size_t)row_bytes(W->down_type, I), (size_t)I * (size_t)row_bytes(W->sh_gate_type, D), (size_t)I * (size_t)row_bytes(W->sh_up_type, D),
                                         (size_t)D * (size_t)row_bytes(W->sh_down_type, I)};
    const void *wp[8] = {W->router, W->sh_gate_w, W->gate, W->up, W->down, W->sh_gate, W->sh_up, W->sh_down};
    for (int i = 0; i < 8; i++) {
        if (!wp[i]) return false;
        qw_hip_view_init(g, &v[7 + i], (void *)(uintptr_t)wp[i], ws[i], &w[i]);
    }
    qw_hip_view_init(g, &v[15], (void *)(uintptr_t)x, (size_t)nb * (size_t)D * 2, &xb);
    qw_hip_view_init(g, &v[16], out, (size_t)nb * (size_t)D * 2, &ob);
    const qw_moe_layer M = {.router = {&w[0], 0, rt}, .sh_gate_w = {&w[1], 0, rt}, .gate = {&w[2], 0, W->gate_type}, .up = {&w[3], 0, W->gate_type}, .down = {&w[4], 0, W->down_type},
                            .sh_gate = {&w[5], 0, W->sh_gate_type}, .sh_up = {&w[6], 0, W->sh_up_type}, .sh_down = {&w[7], 0, W->sh_down_type}};
    // the kernels of this backend read its own table, never the caller's: no gg_tab_init dispatch here
    qw_path p = {.g = g, .D = D, .I = I, .E = E, .topk = topk, .nbmax = QW_NOALLOC_MAX_NB, .tab = s[0], .H = s[3], .psh = s[4], .pd = s[5], .cnt = s[6], .tab_ready = true};
    qw_batch *b = qw_hip_batch_begin_static(g, stream);
    if (!b) {
        fprintf(stderr, "qw_path_gg_moe_noalloc: the device's fixed recorder is missing or in use\n");
        return false;
    }
    const bool rec = gg_moe(&p, b, &M, nb, &xb, &s[1], &s[2], &ob, false);
    const bool ok = qw_hip_batch_launch_static(b, rec); // also releases the recorder; nothing is launched when the recording failed
    if (!ok) fprintf(stderr, "qw_path_gg_moe_noalloc: %s\n", qw_hip_last_error(g));
    return ok;
}
