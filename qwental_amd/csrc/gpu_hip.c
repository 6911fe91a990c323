// HIP implementation of the GPU interface in include/gpu.h (the reference's src/gpu.h, implemented there by
// src/gpu_metal.m). C23 over the HIP runtime's C API; the gfx950 code object built from kernels/qw_kernels.hip is
// embedded below and loaded with hipModuleLoadData. No kernel is compiled at run time.
//
// What a dispatch means here: callers record dispatches in Metal terms (kernel by name, sticky bindings by index,
// grid in threadgroups of 32-wide SIMD groups). Each kernel name was registered by qw_gpu_compile() from the
// caller's "#define" block, which names a kernel family and its parameters. At qw_batch_dispatch() the family's
// translator reads the bindings, checks every size, and records one or more HIP launches with this backend's own
// wave64 geometry. A translation that fails a check marks the batch failed; nothing of a failed batch is launched.
#define _GNU_SOURCE
#define __HIP_PLATFORM_AMD__ 1
#include "gpu.h"
#include "qw_hip_ext.h"
#include "qw_internal.h"
#include "kernels/qw_kargs.h"
#include <hip/hip_runtime_api.h>
#include <pthread.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#include <unistd.h>

static const unsigned char qw_code_object[] = {
#embed <qw_kernels_gfx950.hsaco>
};

#define QW_DNQ_MIN_DEFAULT 2u // token count from which down + combine run as one launch of token quarters (qwk_dnq_*)
enum { QW_MAX_ARGS = 256, QW_MAX_KERNELS = 4096, QW_MAX_BIND = 32, QW_MAX_BYTES = 256, QW_PROF_MAX = 8192, QW_MAX_FUNCS = 256 };

// ---------------------------------------------------------------- records
typedef enum {
    FAM_DQ_TEST, FAM_QMV_GG, FAM_QMV_GGM, FAM_ROUTER, FAM_TAB_INIT, FAM_SEL, FAM_PRE, FAM_GU, FAM_DN, FAM_CMB,
    FAM_BW_READ, FAM_COPY, FAM_FILL, FAM_FILL_BLOCKS,
    FAM_BW_CHUNKS, FAM_BW_ROWS, // read pattern of a decode layer (bench/moe_bw.c)
    FAM_HC_DOWN, FAM_HC_MID, FAM_HC_UP, FAM_HC_UPV, // hyper-connection of the GGUF profile (kernels/hyper_gg.metal)
    FAM_PK_COUNT, FAM_PK_PLAN, FAM_PK_PLAN_T, FAM_PK_SCATTER, FAM_PK_ACT, FAM_PK_ACT2, FAM_PK_COMBINE, FAM_PK_ZERO, FAM_PF, // ragged packing and the grouped product
} qw_family;

typedef struct { // parameters taken from the define block
    int F, K, RB, NB, yfloat;            // dq_test / qmv_gg
    int E, topk, D, I, gnb;              // MoE
    int fgu, fd, fsg, fsu, fsd, rbf, rwf; // formats; rbf: router inside moe_pre_gg; rwf: router weight type (1 / 30)
    int tm;                              // packing: rows per tile entry
    int valu;                            // qmv_gg: QW_VALU in the block asks for the VALU GEMV (measurement)
    int nmat, gf[4];                     // qmv_ggm: number of matrices and their formats
    int sl, ld, ub;                      // bw_chunks / bw_rows (with RB)
} qw_kparams;

struct qw_kernel {
    char name[128];
    qw_family fam;
    qw_kparams p;
};

typedef struct qw_hbuf {
    void *dptr;
    void *host;      // shadow (NULL for device-only)
    size_t size;
    bool own_host;   // shadow allocated here (hipHostMalloc or calloc)
    bool pinned;
    bool wrapped, device_only;
    bool dirty;      // host copy is newer than HBM (or HBM never received it)
    unsigned mark;   // scratch for de-duplication while a batch is submitted
    int pending_out; // submitted batches that bind it in an output role and have not been waited for: HBM is newer than the shadow
    uint64_t out_seq; // the last batch that counted itself in pending_out
    struct qw_gpu *g;
    int npack;       // packed copies made from this buffer (dropped when its contents change)
    bool released;   // the device bytes were freed (qw_hip_buf_release_source): dptr is only the key of its tile-major copies
} qw_hbuf;

// A tile-major copy of IQ3_S weight rows (layout: qwk_pack_args), made at the first use of a weight matrix.
typedef struct {
    const void *A, *B;
    qw_hbuf *ha, *hb;
    uint64_t ntiles;
    uint32_t nblk, split;
    void *dst;
    size_t bytes;
} qw_pack;

typedef struct {
    hipFunction_t f;
    const char *fname;
    unsigned gx, gy, gz, bx;
    unsigned char args[QW_MAX_ARGS];
    size_t argsz;
    const char *kname; // caller-visible kernel name (for profiling)
    bool last_of_dispatch;
    bool side; // independent of the launches before it in the batch: runs on the side stream, beside them
    bool join; // needs the side stream's results: the main stream waits for them first
} qw_launch;

typedef struct { qw_hbuf *b; bool out; } qw_use;

// measurement switches: read from the environment by qw_gpu_open (and again by qw_hip_reload_switches), never per batch
typedef struct { unsigned dnc_nb, dnq_min, spin_limit, hc_rows; int side, load_threads; bool dn_any, nl_c4, no_swiglu_matvec, shared_in_gu, split_select, pk_split, kq_own, no_fuse, ablate, verbose, quiet; } qw_switches;

struct qw_batch {
    qw_gpu *g;
    int stream;
    bool failed, submitted, prof;
    struct qw_kernel *k;
    struct { const qw_buf *buf; qw_hbuf *h; size_t off; } buf[QW_MAX_BIND];
    unsigned char bytes[QW_MAX_BIND][QW_MAX_BYTES];
    size_t blen[QW_MAX_BIND];
    qw_launch *l;
    int nl, capl, done_l; // done_l: launches already submitted by a flush
    qw_use *use;
    int nuse, capuse, done_use;
    bool noalloc;      // the device's static recorder (qw_hip_batch_begin_static): fixed storage, no tile-major copies made
    bool allow_released; // set by a translator while it binds weights that a tile-major copy may stand in for
    hipStream_t xstream; // noalloc: the caller's stream (NULL: the device's)
    uint64_t seq;      // this batch's number (qw_hbuf.out_seq)
    qw_hbuf **outs;    // buffers whose pending_out this batch raised
    int nouts, capouts;
    hipEvent_t ev[2 * 9]; // start/stop per submitted segment (end + at most 8 flushes)
    int nseg;
    hipEvent_t *pev;      // profiling: 2 events per launch
    int npev;
    // Work deferred from one dispatch of a layer to the next (the reference's front part also computes the shared
    // expert's gate/up, and its gate/up dispatch the shared down; here they ride in the next launch, where they cost
    // almost nothing): set by moe_pre_gg / moe_gu_gg, consumed by moe_gu_gg / moe_dn_gg of the same batch.
    struct { bool valid; int fmt; const uint8_t *Wsg, *Wsu; qw_hbuf *hg, *hu; uint32_t rowbytes, nbr; } pend_sg;
    struct { bool valid; int fmt; const uint8_t *Wsd; qw_hbuf *hd; float *Psh; uint32_t rowbytes, nbr; } pend_sd;
    struct { bool valid; qwk_select_args a; } pend_sel; // the selection moe_pre_gg owes: made inside the gate/up launch, or by a launch of its own
    // a grouped product over IQ3_S rows that waits for its twin (gate, then up over the same packed rows: one launch
    // over the tile-major copy that holds both); launched alone at the next other dispatch or at submit
    struct { bool valid; qwk_pf_args a; qw_hbuf *hw, *hx, *hy; int E; } pend_pf;
    // a gate / up pair of grouped products that runs as one launch, waiting for the p_act2 dispatch that may ride in it
    struct { bool valid; qwk_pf_args f, second; qw_hbuf *hw, *hwb; int E; const char *kname; } pend_tw;
    // p_zero, moe_count and moe_plan(_t) waiting for the moe_scatter dispatch with which they run as one launch (stage = how many wait)
    struct { int stage; qwk_zero_args z; qwk_count_args c; qwk_plan_args pl; const char *kn[3]; } pend_pk;
    // a down projection over a few tokens that waits for the combine of the same layer: both in one launch
    // (qwk_dnc_*); launched as it is at any other dispatch or at submit
    struct { bool valid; qwk_dn_args a; const char *fname, *fused, *kname; unsigned grid, fused_grid; bool quarters; } pend_dn;
    // a routed gate/up launch that waits for the down projection and the combine of the same layer: the three run as one
    // launch (qwk_gud_*) when the down dispatch qualifies for the form by token shares; launched as it is otherwise
    struct { bool valid; qwk_gu_args a; const char *fname, *kname; unsigned grid; } pend_gu;
    bool uses_sync;    // some launch of this batch has its workgroups wait for one another: the error word is read back at the end
    qw_switches sw; // the device's switches when the batch began (no_fuse also set for what must not wait for its workgroups)
};

#define QW_LD_MAX 16
struct qw_gpu {
    int dev;
    char name[256];
    size_t total_mem;
    int ncu;
    hipModule_t mod;
    void *tabs;   // this backend's own lookup tables in HBM (QW_TAB_BYTES); the pre-signed IQ3_S table sits at QW_TAB_IQ3SS
    hipStream_t stream[2];
    int cur_stream;
    struct qw_kernel *kernels;
    int nkernels;
    struct { char name[48]; hipFunction_t f; } funcs[QW_MAX_FUNCS];
    int nfuncs;
    char err[1024];
    bool prof;
    int nprof;
    const char *prof_name[QW_PROF_MAX];
    const char *prof_fname[QW_PROF_MAX];
    double prof_us[QW_PROF_MAX];
    unsigned mark;
    uint64_t batch_seq;
    qw_pack *packs;
    int npacks, cappacks;
    struct qw_ldlane { void *pin[2]; hipStream_t st; hipEvent_t ev[2]; } ld[QW_LD_MAX]; // staging of qw_hip_buf_write_fd, made at first use
    int nld;
    hipStream_t side[2]; // one beside each stream: launches of a batch that do not depend on the ones before them (made at first use)
    hipEvent_t sev[256];  // fork / join events between a stream and its side stream, used round robin (made at first use)
    unsigned nsev;
    // Launch sequences that come again unchanged (a decode step over resident weights) replayed as HIP graphs: hash of
    // the sequence, a copy of it for the exact comparison, the instantiated graph; seen = hashes of the last sequences
    // that were launched eagerly (a graph is built only when a sequence repeats). Off unless QW_HIP_GRAPH=1 / qw_hip_set_graphs.
    struct qw_graph { uint64_t hash; int nl; size_t bytes; unsigned char *key; hipGraphExec_t exec; } graphs[8];
    unsigned ngraph_next, ngraph_launches;
    uint64_t seen_hash[8];
    unsigned nseen;
    bool use_graphs;
    void *na_scratch;    // the scratch array of the no-allocation entry point on this device (csrc/qw_noalloc.hip); NULL: set-up failed
    size_t na_bytes;
    const char *na_err;
    struct qw_batch *na_batch; // its recorder, with fixed storage (made by qw_gpu_open)
    bool na_busy;
    qw_switches sw;
    uint32_t *sync;      // QW_SYNC_BYTES: synchronisation words of launches whose workgroups wait for one another (stream 0 only)
    uint32_t *sync_host; // pinned: the error word of those launches, copied back when a batch is waited for
    bool fuse_broken;    // such a launch gave up once: the layers stay separate launches from then on
    float *shgu;         // [2 streams][2][16][QW_SHGU_MAXI] gate and up results of a shared expert in the K-quant format family
    bool repack;         // make packed copies (QW_HIP_REPACK=0 in the environment or qw_hip_set_repack turn it off)
    size_t pack_bytes, released_bytes;
};

static void set_err(qw_gpu *g, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g->err, sizeof g->err, fmt, ap);
    va_end(ap);
    if (g->sw.verbose) fprintf(stderr, "[qw_hip] %s\n", g->err);
}
#define HIPOK(g, call) (hip_ok((g), (call), #call))
static bool hip_ok(qw_gpu *g, hipError_t e, const char *what) {
    if (e == hipSuccess) return true;
    set_err(g, "%s: %s", what, hipGetErrorString(e));
    return false;
}

double qw_now(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + (double)ts.tv_nsec * 1e-9;
}

static void read_switches(qw_gpu *g) {
    qw_switches *w = &g->sw;
    const char *e = getenv("QW_HIP_DNC_NB"); // token count up to which down + combine run as one launch (0: never)
    w->dnc_nb = e ? (unsigned)atoi(e) : 2;
    if (w->dnc_nb > QW_DNC_MAXNB) w->dnc_nb = QW_DNC_MAXNB;
    e = getenv("QW_HIP_DNQ_MIN"); // token count from which down + combine run as one launch of token shares (0: never)
    w->dnq_min = e ? (unsigned)atoi(e) : QW_DNQ_MIN_DEFAULT;
    e = getenv("QW_HIP_SIDE"); // the side stream for launches that depend on the step's input alone: 1 on
    w->side = e && e[0] == '1';
    w->dn_any = getenv("QW_HIP_DN_ANY") != NULL, w->nl_c4 = getenv("QW_HIP_NL_C4") != NULL;
    w->no_swiglu_matvec = getenv("QW_HIP_NO_SWIGLU_MATVEC") != NULL, w->shared_in_gu = getenv("QW_HIP_SHARED_IN_GU") != NULL;
    w->split_select = getenv("QW_HIP_SPLIT_SELECT") != NULL;
    w->pk_split = getenv("QW_HIP_PK_SPLIT") != NULL; // the packing sequence one launch per dispatch
    w->kq_own = getenv("QW_HIP_KQ_OWN_LAUNCH") != NULL; // a K-quant / IQ4 / plain shared expert's gate/up as a launch of its own
    e = getenv("QW_HIP_FUSE"); // 1: routed gate/up, down and combine of a layer as one launch (off unless asked for: measured as no gain)
    w->no_fuse = !(e && e[0] == '1');
    w->ablate = getenv("QW_HIP_ABLATE") != NULL; // measurement: the routed gate/up launch without its arithmetic (results are meaningless)
    e = getenv("QW_HIP_HC_ROWS"); // mix_down rows per workgroup of the hyper-connection's down launch: 4, 8 or 16 (0: by token count)
    w->hc_rows = e ? (unsigned)atoi(e) : 0;
    e = getenv("QW_HIP_SPIN_LIMIT"); // polls after which a workgroup of a fused launch stops waiting for the others
    w->spin_limit = e ? (unsigned)strtoul(e, NULL, 10) : 1u << 16;
    e = getenv("QW_HIP_LOAD_THREADS");
    w->load_threads = e && atoi(e) > 0 ? (atoi(e) > QW_LD_MAX ? QW_LD_MAX : atoi(e)) : 4;
    w->verbose = getenv("QW_HIP_VERBOSE") != NULL, w->quiet = getenv("QW_HIP_QUIET") != NULL;
}
bool qw_hip_sync_words(qw_gpu *g, uint32_t *dst, size_t nwords) {
    if (nwords * 4 > QW_SYNC_ALLOC) return false;
    return hipDeviceSynchronize() == hipSuccess && hipMemcpy(dst, g->sync, nwords * 4, hipMemcpyDeviceToHost) == hipSuccess;
}
void qw_hip_reload_switches(qw_gpu *g) {
    read_switches(g);
    g->fuse_broken = false; // fused launches are tried again
}

static hipFunction_t find_func(qw_gpu *g, const char *fname) {
    hipFunction_t f;
    if (hipModuleGetFunction(&f, g->mod, fname) == hipSuccess) return f;
    (void)hipGetLastError();
    return NULL;
}

// ---------------------------------------------------------------- device
qw_gpu *qw_gpu_open(void) {
    int n = 0;
    if (hipInit(0) != hipSuccess || hipGetDeviceCount(&n) != hipSuccess || n < 1) return NULL;
    qw_gpu *g = calloc(1, sizeof *g);
    if (!g) return NULL;
    hipDeviceProp_t pr;
    if (hipSetDevice(0) != hipSuccess || hipGetDeviceProperties(&pr, 0) != hipSuccess) { free(g); return NULL; }
    snprintf(g->name, sizeof g->name, "%s (%s, %d CUs)", pr.name[0] ? pr.name : "AMD Instinct", pr.gcnArchName, pr.multiProcessorCount);
    g->total_mem = pr.totalGlobalMem;
    g->ncu = pr.multiProcessorCount;
    if (strncmp(pr.gcnArchName, "gfx950", 6) != 0) {
        fprintf(stderr, "qw_gpu_open: device is %s; this library holds gfx950 code only\n", pr.gcnArchName);
        free(g);
        return NULL;
    }
    if (hipModuleLoadData(&g->mod, qw_code_object) != hipSuccess) {
        fprintf(stderr, "qw_gpu_open: the embedded gfx950 code object does not load\n");
        free(g);
        return NULL;
    }
    for (int i = 0; i < 2; i++)
        if (hipStreamCreateWithFlags(&g->stream[i], hipStreamNonBlocking) != hipSuccess) { free(g); return NULL; }
    g->kernels = calloc(QW_MAX_KERNELS, sizeof *g->kernels);
    read_switches(g);
    {
        const char *e = getenv("QW_HIP_REPACK"); // these two have setters of their own; the environment gives the start value
        g->repack = !(e && e[0] == '0');
        e = getenv("QW_HIP_GRAPH"); // off unless asked for: measured as no gain on this path (the steps are bound by the GPU)
        g->use_graphs = e && e[0] == '1';
    }
    { // build the pre-signed table once; every weight kernel copies it into LDS
        hipFunction_t f;
        qwk_tab_args ta;
        void *params[] = {&ta};
        if (hipMalloc(&g->tabs, QW_TAB_BYTES) != hipSuccess || hipMemset(g->tabs, 0, QW_TAB_BYTES) != hipSuccess ||
            hipMalloc((void **)&g->shgu, (size_t)2 * 2 * 16 * 4096 * 4) != hipSuccess ||
            hipMalloc((void **)&g->sync, QW_SYNC_ALLOC) != hipSuccess || hipMemset(g->sync, 0, QW_SYNC_ALLOC) != hipSuccess ||
            hipHostMalloc((void **)&g->sync_host, 64, hipHostMallocDefault) != hipSuccess ||
            !(f = find_func(g, "qwk_tab_init"))) { free(g->kernels); free(g); return NULL; }
        ta = (qwk_tab_args){.tab = g->tabs, .slot_order = 1};
        if (hipDeviceSynchronize() != hipSuccess || hipModuleLaunchKernel(f, 32, 1, 1, 256, 1, 1, 0, g->stream[0], params, NULL) != hipSuccess ||
            hipStreamSynchronize(g->stream[0]) != hipSuccess) {
            fprintf(stderr, "qw_gpu_open: the table kernel does not run\n");
            free(g->kernels);
            free(g);
            return NULL;
        }
    }
    // the entry point that allocates nothing: its scratch array's address on this device and its recorder, made now
    if (!qw_noalloc_scratch(g->dev, &g->na_scratch, &g->na_bytes, &g->na_err)) g->na_scratch = NULL;
#ifdef QW_STAMPS // working builds: the kernels' time stamps go behind the synchronisation words
    {
        hipDeviceptr_t p;
        size_t sz;
        if (hipModuleGetGlobal(&p, &sz, g->mod, "qw_stamp_ptr") == hipSuccess) (void)hipMemcpy((void *)p, &g->sync, sizeof g->sync, hipMemcpyHostToDevice);
        else (void)hipGetLastError();
    }
#endif
    g->na_batch = calloc(1, sizeof *g->na_batch);
    if (g->na_batch) {
        g->na_batch->capl = 64, g->na_batch->l = calloc(64, sizeof(qw_launch));
        g->na_batch->capuse = 1024, g->na_batch->use = calloc(1024, sizeof(qw_use));
    }
    return g;
}

void qw_gpu_close(qw_gpu *g) {
    if (!g) return;
    (void)hipDeviceSynchronize();
    for (int i = 0; i < 2; i++) (void)hipStreamDestroy(g->stream[i]);
    for (int i = 0; i < 2; i++)
        if (g->side[i]) (void)hipStreamDestroy(g->side[i]);
    for (int i = 0; i < 256; i++)
        if (g->sev[i]) (void)hipEventDestroy(g->sev[i]);
    for (int i = 0; i < g->nld; i++) {
        for (int k = 0; k < 2; k++) {
            if (g->ld[i].ev[k]) (void)hipEventDestroy(g->ld[i].ev[k]);
            if (g->ld[i].pin[k]) (void)hipHostFree(g->ld[i].pin[k]);
        }
        if (g->ld[i].st) (void)hipStreamDestroy(g->ld[i].st);
    }
    for (int i = 0; i < g->npacks; i++) {
        (void)hipFree(g->packs[i].dst);
        if (g->packs[i].ha) g->packs[i].ha->npack = 0;
        if (g->packs[i].hb) g->packs[i].hb->npack = 0;
    }
    free(g->packs);
    (void)hipFree(g->tabs);
    for (int i = 0; i < 8; i++) {
        if (g->graphs[i].exec) (void)hipGraphExecDestroy(g->graphs[i].exec);
        free(g->graphs[i].key);
    }
    (void)hipFree(g->shgu);
    (void)hipFree(g->sync);
    (void)hipHostFree(g->sync_host);
    if (g->na_batch) { free(g->na_batch->l); free(g->na_batch->use); free(g->na_batch); }
    (void)hipModuleUnload(g->mod);
    free(g->kernels);
    free(g);
}

const char *qw_gpu_name(const qw_gpu *g) { return g->name; }
size_t qw_gpu_max_working_set(const qw_gpu *g) { return g->total_mem; }
const char *qw_hip_last_error(const qw_gpu *g) { return g->err; }
int qw_hip_cu_count(const qw_gpu *g) { return g->ncu; }
const char *qw_hip_arch(void) { return "gfx950"; }

static hipFunction_t get_func(qw_gpu *g, const char *fname) {
    for (int i = 0; i < g->nfuncs; i++)
        if (!strcmp(g->funcs[i].name, fname)) return g->funcs[i].f;
    if (g->nfuncs >= QW_MAX_FUNCS) return NULL;
    hipFunction_t f = find_func(g, fname);
    if (!f) { set_err(g, "no entry point %s in the code objects", fname); return NULL; }
    snprintf(g->funcs[g->nfuncs].name, sizeof g->funcs[0].name, "%s", fname);
    g->funcs[g->nfuncs].f = f;
    return g->funcs[g->nfuncs++].f;
}

// ---------------------------------------------------------------- define block -> kernels
// The block is the run of "#define NAME VALUE" lines at the start of the source (src/engine.c:478-507, :709-710,
// tools/dqtest.c:27). Later definitions of a name win, as in the preprocessor.
typedef struct { char name[48], val[80]; } qw_def;

static int parse_defs(const char *src, size_t len, qw_def *d, int max) {
    int n = 0;
    size_t i = 0;
    while (i < len) {
        while (i < len && (src[i] == ' ' || src[i] == '\t' || src[i] == '\r' || src[i] == '\n')) i++;
        if (i + 7 >= len || strncmp(src + i, "#define", 7) != 0) break;
        i += 7;
        while (i < len && (src[i] == ' ' || src[i] == '\t')) i++;
        size_t a = i;
        while (i < len && src[i] != ' ' && src[i] != '\t' && src[i] != '\n' && src[i] != '\r') i++;
        size_t nl = i - a;
        while (i < len && (src[i] == ' ' || src[i] == '\t')) i++;
        size_t b = i;
        while (i < len && src[i] != '\n' && src[i] != '\r') i++;
        size_t vl = i - b;
        while (vl && (src[b + vl - 1] == ' ' || src[b + vl - 1] == '\t')) vl--;
        if (n < max && nl && nl < sizeof d->name && vl < sizeof d->val) {
            memcpy(d[n].name, src + a, nl); d[n].name[nl] = 0;
            memcpy(d[n].val, src + b, vl); d[n].val[vl] = 0;
            n++;
        }
    }
    return n;
}
static const char *def_get(const qw_def *d, int n, const char *name) {
    for (int i = n - 1; i >= 0; i--)
        if (!strcmp(d[i].name, name)) return d[i].val;
    return NULL;
}
static bool def_int(const qw_def *d, int n, const char *name, int *out) {
    const char *v = def_get(d, n, name);
    if (!v || !*v) return false;
    char *end;
    long x = strtol(v, &end, 0);
    if (*end) return false;
    *out = (int)x;
    return true;
}

static bool fmt_ok(int f) { return f == 8 || f == 21; } // formats of the MoE kernels
// formats of the multi-format dense matvec: binary16, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS, bfloat16 (src/gguf.c:15-25)
static bool kq_ok(int f) { return f == 1 || f == 12 || f == 13 || f == 14 || f == 20 || f == 23 || f == 30; }
// the other quantised types the reference's MoE kernels take (kernels/moe_gg.metal:336-395): served by the kernels whose
// type is an argument (qwk_gu_rt*, qwk_dn_rt)
static bool rt_ok(int f) { return f == 12 || f == 13 || f == 14 || f == 20 || f == 23; }
static int fmt_qb(int f) { return f == 1 || f == 30 || f == 8 || f == 20 ? 32 : 256; } // values per decoding unit (plain rows: 32 at a time)
static int fmt_bb(int f) {
    switch (f) {
    case 1: case 30: return 64;
    case 8: return 34;
    case 20: return 18;
    case 12: return 144;
    case 13: return 176;
    case 14: return 210;
    case 23: return 136;
    default: return 110;
    }
}
static size_t fmt_rb(int f, int K) { return (size_t)(K / fmt_qb(f)) * (size_t)fmt_bb(f); }

static bool reg_kernel(qw_gpu *g, const qw_def *d, int n, const char *base, qw_family fam, const qw_kparams *p, char *err, size_t errlen) {
    const char *nm = def_get(d, n, base); // "#define base newname" renames the kernel (src/engine.c:149)
    if (!nm || !*nm) nm = base;
    for (int i = 0; i < g->nkernels; i++)
        if (!strcmp(g->kernels[i].name, nm)) { g->kernels[i].fam = fam; g->kernels[i].p = *p; return true; }
    if (g->nkernels >= QW_MAX_KERNELS) { snprintf(err, errlen, "too many kernels"); return false; }
    struct qw_kernel *k = &g->kernels[g->nkernels++];
    snprintf(k->name, sizeof k->name, "%s", nm);
    k->fam = fam;
    k->p = *p;
    return true;
}

bool qw_gpu_compile(qw_gpu *g, const char *src, size_t len, char *err, size_t errlen) {
    char dummy[8];
    if (!err || !errlen) { err = dummy; errlen = sizeof dummy; }
    err[0] = 0;
    qw_def *d = calloc(128, sizeof *d);
    const int n = parse_defs(src, len, d, 128);
    qw_kparams p = {0};
    int v;
    bool ok = true;
#define FAIL(...) do { snprintf(err, errlen, __VA_ARGS__); ok = false; goto out; } while (0)
    if (def_int(d, n, "DQ_TEST", &v)) { // tools/dqtest.c:27
        if (!fmt_ok(v) && !kq_ok(v)) FAIL("dq_test: ggml type %d has no gfx950 build (have 1, 8, 12, 13, 14, 20, 21, 23, 30)", v);
        p.F = v;
        if (!reg_kernel(g, d, n, "dq_test", FAM_DQ_TEST, &p, err, errlen)) { ok = false; goto out; }
    }
    if (def_get(d, n, "GF") && def_get(d, n, "KD")) { // src/engine.c:709-710
        if (!def_int(d, n, "GF", &p.F) || !def_int(d, n, "KD", &p.K) || !def_int(d, n, "RB", &p.RB) || !def_int(d, n, "NB", &p.NB))
            FAIL("qmv_gg: GF, KD, RB and NB must be integer macros");
        if (!fmt_ok(p.F) && !kq_ok(p.F)) FAIL("qmv_gg: ggml type %d has no gfx950 build (have 1, 8, 12, 13, 14, 20, 21, 23, 30)", p.F);
        if (p.K <= 0 || p.K % fmt_qb(p.F) || (size_t)p.RB != fmt_rb(p.F, p.K)) FAIL("qmv_gg: K %d / row bytes %d do not fit type %d", p.K, p.RB, p.F);
        if (kq_ok(p.F) && p.K > (int)QW_KQ_MAXK) FAIL("qmv_gg: K %d beyond %u for type %d in this build", p.K, QW_KQ_MAXK, p.F);
        if (p.NB < 1 || p.NB > 16) FAIL("qmv_gg: NB %d outside 1..16", p.NB);
        const char *yt = def_get(d, n, "YT");
        p.yfloat = yt && !strcmp(yt, "float");
        p.valu = def_get(d, n, "QW_VALU") != NULL;
        if (yt && strcmp(yt, "float") && strcmp(yt, "half")) FAIL("qmv_gg: YT %s is neither half nor float", yt);
        if (!reg_kernel(g, d, n, "qmv_gg", FAM_QMV_GG, &p, err, errlen)) { ok = false; goto out; }
    }
    if (def_get(d, n, "NMAT") && def_get(d, n, "GF0")) { // src/engine.c:730-744: one launch for up to four matrices over the same activations
        p = (qw_kparams){0};
        if (!def_int(d, n, "KD", &p.K) || !def_int(d, n, "NB", &p.NB) || !def_int(d, n, "NMAT", &p.nmat) || !def_int(d, n, "GF0", &p.gf[0]))
            FAIL("qmv_ggm: KD, NB, NMAT and GF0 must be integer macros");
        if (p.nmat < 1 || p.nmat > 4) FAIL("qmv_ggm: NMAT %d outside 1..4", p.nmat);
        if (p.NB < 0 || p.NB > 16) FAIL("qmv_ggm: NB %d outside 0..16", p.NB);
        for (int j = 1; j < 4; j++) {
            char nm[8];
            snprintf(nm, sizeof nm, "GF%d", j);
            if (!def_int(d, n, nm, &p.gf[j])) p.gf[j] = p.gf[0]; // kernels/qmv_ggm.metal:20-28
        }
        for (int j = 0; j < p.nmat; j++)
            if (!kq_ok(p.gf[j])) FAIL("qmv_ggm: ggml type %d has no gfx950 build here (have 1, 12, 13, 14, 20, 23, 30)", p.gf[j]);
        if (p.K <= 0 || p.K % 256 || p.K > (int)QW_KQ_MAXK) FAIL("qmv_ggm: KD %d must be a multiple of 256 up to %u", p.K, QW_KQ_MAXK);
        const char *yt = def_get(d, n, "YT");
        if (yt && strcmp(yt, "float") && strcmp(yt, "half")) FAIL("qmv_ggm: YT %s is neither half nor float", yt);
        p.yfloat = yt && !strcmp(yt, "float");
        if (p.NB > 0) {
            if (!reg_kernel(g, d, n, "qmv_ggm", FAM_QMV_GGM, &p, err, errlen)) { ok = false; goto out; }
        } else { // NB 0: one kernel per token count, <name>_b1 ... (kernels/qmv_ggm.metal:251-262; here up to 16)
            const char *nm = def_get(d, n, "qmv_ggm");
            if (!nm || !*nm) nm = "qmv_ggm";
            for (int nb = 1; nb <= 16; nb++) {
                char full[128];
                snprintf(full, sizeof full, "%s_b%d", nm, nb);
                qw_def one = {"qmv_ggm", ""};
                snprintf(one.val, sizeof one.val, "%s", full);
                p.NB = nb;
                if (!reg_kernel(g, &one, 1, "qmv_ggm", FAM_QMV_GGM, &p, err, errlen)) { ok = false; goto out; }
            }
        }
    }
    const bool router = def_get(d, n, "GG_ROUTER") != NULL;
    int part = -1;
    if (router || def_int(d, n, "GG_PART", &part)) { // src/engine.c:478-507
        p = (qw_kparams){0};
        if (!def_int(d, n, "E", &p.E) || !def_int(d, n, "TOPK", &p.topk) || !def_int(d, n, "D", &p.D) || !def_int(d, n, "I", &p.I) || !def_int(d, n, "NB", &p.NB))
            FAIL("moe_gg: E, TOPK, D, I and NB must be integer macros");
        if (p.NB < 1 || p.NB > 16) FAIL("moe_gg: NB %d outside 1..16", p.NB);
        if (p.E < 1 || p.E > 1024 || p.topk < 1 || p.topk > 16 || p.topk > p.E) FAIL("moe_gg: E %d / TOPK %d outside this build (E <= 1024, TOPK <= 16)", p.E, p.topk);
        // the reference asks D % 512 == 0 and I % 128 == 0 (kernels/moe_gg.metal:419); its model has D = 2560, I = 640
        if (p.D % 256 || p.I % 128 || p.D > 2560 || p.D < 256 || p.I < 256) FAIL("moe_gg: D %d / I %d outside this build (D a multiple of 256 up to 2560, I a multiple of 128 from 256)", p.D, p.I);
        p.gnb = p.NB <= 8 ? 8 : 16; // 8 = the reference's gg_sel layout; 16 = the wide layout
        p.rwf = 30;
        if (def_int(d, n, "RWF", &v)) { if (v != 1 && v != 30) FAIL("moe_gg: RWF %d (router weight type) must be 1 or 30", v); p.rwf = v; }
        if (router) {
            if (!reg_kernel(g, d, n, "moe_router_bf", FAM_ROUTER, &p, err, errlen)) { ok = false; goto out; }
        } else if (part == 0) {
            if (!reg_kernel(g, d, n, "gg_tab_init", FAM_TAB_INIT, &p, err, errlen) || !reg_kernel(g, d, n, "moe_sel_gg", FAM_SEL, &p, err, errlen)) { ok = false; goto out; }
        } else if (part == 1) {
            if (!def_int(d, n, "FSG", &p.fsg) || !def_int(d, n, "FSU", &p.fsu) || !def_int(d, n, "RBF", &p.rbf)) FAIL("moe_pre_gg: FSG, FSU, RBF missing");
            if (!(fmt_ok(p.fsg) && p.fsu == p.fsg) && !(kq_ok(p.fsg) && kq_ok(p.fsu)))
                FAIL("moe_pre_gg: shared gate/up types %d/%d: this build needs equal types from {8, 21} or two of {1, 12, 13, 14, 20, 23, 30}", p.fsg, p.fsu);
            if (kq_ok(p.fsg) && (p.D > (int)QW_KQ_MAXK)) FAIL("moe_pre_gg: D %d too wide for shared gate/up types %d/%d", p.D, p.fsg, p.fsu);
            if (!reg_kernel(g, d, n, "moe_pre_gg", FAM_PRE, &p, err, errlen)) { ok = false; goto out; }
        } else if (part == 2) {
            if (!def_int(d, n, "FGU", &p.fgu) || !def_int(d, n, "FSD", &p.fsd)) FAIL("moe_gu_gg: FGU, FSD missing");
            if (!(fmt_ok(p.fgu) || rt_ok(p.fgu)) || !(fmt_ok(p.fsd) || rt_ok(p.fsd))) FAIL("moe_gu_gg: types %d/%d have no gfx950 build (have 8, 12, 13, 14, 20, 21, 23)", p.fgu, p.fsd);
            if (p.I % fmt_qb(p.fsd)) FAIL("moe_gu_gg: I %d does not fit shared down rows of type %d", p.I, p.fsd);
            if (!reg_kernel(g, d, n, "moe_gu_gg", FAM_GU, &p, err, errlen)) { ok = false; goto out; }
        } else if (part == 3) {
            if (!def_int(d, n, "FD", &p.fd)) FAIL("moe_dn_gg: FD missing");
            if (!fmt_ok(p.fd) && !rt_ok(p.fd)) FAIL("moe_dn_gg: type %d has no gfx950 build (have 8, 12, 13, 14, 20, 21, 23)", p.fd);
            if (p.I % fmt_qb(p.fd)) FAIL("moe_dn_gg: I %d does not fit rows of type %d", p.I, p.fd);
            if (!reg_kernel(g, d, n, "moe_dn_gg", FAM_DN, &p, err, errlen) || !reg_kernel(g, d, n, "moe_cmb_gg", FAM_CMB, &p, err, errlen)) { ok = false; goto out; }
        } else if (part != 5) FAIL("moe_gg: GG_PART %d has no gfx950 build (have 0..3, 5 and GG_ROUTER)", part);
    }
    if (part == 5) { // the grouped product over packed rows, src/engine.c:3244-3248
        p = (qw_kparams){0};
        if (!def_int(d, n, "PFF", &p.F) || !def_int(d, n, "KD", &p.K) || !def_int(d, n, "TM", &p.tm) || !def_int(d, n, "E", &p.E)) FAIL("moe_pf_gg: PFF, KD, TM and E must be integer macros");
        if (!fmt_ok(p.F) && p.F != 20) FAIL("moe_pf_gg: ggml type %d has no gfx950 build (have 8, 20, 21)", p.F);
        if (p.K <= 0 || p.K % fmt_qb(p.F) || ((p.F == 8 || p.F == 20) && p.K % 128)) FAIL("moe_pf_gg: KD %d does not fit type %d", p.K, p.F);
        if (p.tm < 1 || p.tm > 64) FAIL("moe_pf_gg: TM %d outside this build (1..64 rows per tile entry)", p.tm);
        if (p.E < 1 || p.E > 1024) FAIL("moe_pf_gg: E %d outside this build (E <= 1024)", p.E);
        if (!reg_kernel(g, d, n, "moe_pf_gg", FAM_PF, &p, err, errlen)) { ok = false; goto out; }
    } else if (part < 0 && !router && !def_get(d, n, "GF") && !def_get(d, n, "BITS") && def_get(d, n, "KD") && def_get(d, n, "TM") && def_get(d, n, "TOPK")) {
        // kernels/moe_prefill.metal: E, TOPK, KD, I, TM (bench/moe_prefill.c:86-87)
        p = (qw_kparams){0};
        if (!def_int(d, n, "E", &p.E) || !def_int(d, n, "TOPK", &p.topk) || !def_int(d, n, "KD", &p.K) || !def_int(d, n, "I", &p.I) || !def_int(d, n, "TM", &p.tm))
            FAIL("moe_prefill: E, TOPK, KD, I and TM must be integer macros");
        if (p.E < 1 || p.E > 1024 || p.topk < 1 || p.topk > 16) FAIL("moe_prefill: E %d / TOPK %d outside this build (E <= 1024, TOPK <= 16)", p.E, p.topk);
        if (p.K < 8 || p.K % 8 || p.I < 1 || p.tm < 1) FAIL("moe_prefill: KD %d / I %d / TM %d outside this build (KD a multiple of 8)", p.K, p.I, p.tm);
        if (!reg_kernel(g, d, n, "moe_count", FAM_PK_COUNT, &p, err, errlen) || !reg_kernel(g, d, n, "moe_plan", FAM_PK_PLAN, &p, err, errlen) ||
            !reg_kernel(g, d, n, "moe_plan_t", FAM_PK_PLAN_T, &p, err, errlen) || !reg_kernel(g, d, n, "moe_scatter", FAM_PK_SCATTER, &p, err, errlen) ||
            !reg_kernel(g, d, n, "moe_act", FAM_PK_ACT, &p, err, errlen) || !reg_kernel(g, d, n, "p_act2", FAM_PK_ACT2, &p, err, errlen) || !reg_kernel(g, d, n, "moe_combine", FAM_PK_COMBINE, &p, err, errlen) ||
            !reg_kernel(g, d, n, "p_zero", FAM_PK_ZERO, &p, err, errlen)) { ok = false; goto out; }
    }
    if (def_get(d, n, "HC") && (def_get(d, n, "ghc_down") || def_get(d, n, "ghc_up") || def_get(d, n, "ghc_dsk"))) { // src/engine.c:1323-1341
        memset(&p, 0, sizeof p);
        int hc;
        if (!def_int(d, n, "D", &p.D) || !def_int(d, n, "HC", &hc) || !def_int(d, n, "NB", &p.NB)) FAIL("hyper_gg: D, HC and NB must be integers");
        if (hc != (int)QW_HC) FAIL("hyper_gg: HC %d (this build has %u streams)", hc, QW_HC);
        if (p.D <= 0 || p.D % 512 || p.D > 4096) FAIL("hyper_gg: D %d must be a multiple of 512 up to 4096", p.D);
        if (p.NB < 1 || p.NB > 16) FAIL("hyper_gg: NB %d (1 to 16)", p.NB);
        // GH_R, GH_G, GU_SG, GV_SG, GV_RP and GK tune the reference's own kernels; the ones here have their own shape
        if (!reg_kernel(g, d, n, "ghc_down", FAM_HC_DOWN, &p, err, errlen) || !reg_kernel(g, d, n, "ghc_up", FAM_HC_UP, &p, err, errlen) ||
            !reg_kernel(g, d, n, "ghc_dsk", FAM_HC_DOWN, &p, err, errlen) || !reg_kernel(g, d, n, "ghc_mid", FAM_HC_MID, &p, err, errlen) ||
            !reg_kernel(g, d, n, "ghc_upv", FAM_HC_UPV, &p, err, errlen)) { ok = false; goto out; }
    }
    if (def_get(d, n, "SL") && def_get(d, n, "LD") && def_get(d, n, "UB")) { // bench/moe_bw.c:29-41: one source, one of its two kernels renamed
        memset(&p, 0, sizeof p);
        if (!def_int(d, n, "SL", &p.sl) || !def_int(d, n, "LD", &p.ld) || !def_int(d, n, "RB", &p.RB) || !def_int(d, n, "UB", &p.ub)) FAIL("bw_chunks / bw_rows: SL, LD, RB and UB must be integers");
        // Both kernels are in the source; the one the block renames is the one the caller asks for. Its parameters are
        // checked when it is dispatched (the other one's are placeholders).
        if (!reg_kernel(g, d, n, "bw_chunks", FAM_BW_CHUNKS, &p, err, errlen) || !reg_kernel(g, d, n, "bw_rows", FAM_BW_ROWS, &p, err, errlen)) { ok = false; goto out; }
    }
    if (def_get(d, n, "QW_HIP_MEM")) { // this backend's own measurement helpers
        p = (qw_kparams){0};
        if (!reg_kernel(g, d, n, "qw_bw_read", FAM_BW_READ, &p, err, errlen) || !reg_kernel(g, d, n, "qw_copy", FAM_COPY, &p, err, errlen) ||
            !reg_kernel(g, d, n, "qw_fill_random", FAM_FILL, &p, err, errlen) || !reg_kernel(g, d, n, "qw_fill_blocks", FAM_FILL_BLOCKS, &p, err, errlen)) { ok = false; goto out; }
    }
#undef FAIL
out:
    free(d);
    return ok;
}

bool qw_hip_compile_check(const char *src, size_t len, char *err, size_t errlen, char *names, size_t nameslen) {
    qw_gpu *g = calloc(1, sizeof *g); // no device behind it: only the kernel registry is touched
    if (!g) return false;
    g->kernels = calloc(QW_MAX_KERNELS, sizeof *g->kernels);
    const bool ok = g->kernels && qw_gpu_compile(g, src, len, err, errlen);
    if (ok && names && nameslen) {
        size_t n = 0;
        names[0] = 0;
        for (int i = 0; i < g->nkernels; i++) n += (size_t)snprintf(names + n, n < nameslen ? nameslen - n : 0, "%s%s", i ? "," : "", g->kernels[i].name);
    }
    free(g->kernels);
    free(g);
    return ok;
}

qw_kernel *qw_kernel_get(qw_gpu *g, const char *name) {
    for (int i = 0; i < g->nkernels; i++)
        if (!strcmp(g->kernels[i].name, name)) return &g->kernels[i];
    return NULL;
}
unsigned qw_kernel_max_threads(const qw_kernel *k) { (void)k; return 1024; }
unsigned qw_kernel_simd_width(const qw_kernel *k) { (void)k; return 64; }

// ---------------------------------------------------------------- buffers
static qw_hbuf *hbuf_new(qw_gpu *g, size_t size) {
    qw_hbuf *h = calloc(1, sizeof *h);
    if (!h) return NULL;
    // the memset runs on the null stream; the batches run on non-blocking streams, so wait for it here
    if (!HIPOK(g, hipMalloc(&h->dptr, size ? size : 1)) || !HIPOK(g, hipMemset(h->dptr, 0, size)) || !HIPOK(g, hipDeviceSynchronize())) { free(h); return NULL; }
    h->size = size;
    h->g = g;
    return h;
}

bool qw_buf_new(qw_gpu *g, size_t size, qw_buf *out) {
    qw_hbuf *h = hbuf_new(g, size);
    if (!h) return false;
    if (size <= ((size_t)64 << 20) && hipHostMalloc(&h->host, size ? size : 1, hipHostMallocDefault) == hipSuccess) {
        h->pinned = true;
        memset(h->host, 0, size);
    } else {
        h->host = calloc(size ? size : 1, 1);
        if (!h->host) { (void)hipFree(h->dptr); free(h); return false; }
    }
    h->own_host = true;
    h->dirty = true; // the caller may fill it through ptr at any time before its first use: the first bind copies it
    out->handle = h;
    out->ptr = h->host;
    out->size = size;
    return true;
}

bool qw_hip_buf_new_device(qw_gpu *g, size_t size, qw_buf *out) {
    qw_hbuf *h = hbuf_new(g, size);
    if (!h) return false;
    h->device_only = true;
    out->handle = h;
    out->ptr = NULL;
    out->size = size;
    return true;
}

bool qw_buf_wrap(qw_gpu *g, void *ptr, size_t len, qw_buf *out) {
    const size_t page = (size_t)sysconf(_SC_PAGESIZE);
    if ((uintptr_t)ptr % page) return false;
    qw_hbuf *h = hbuf_new(g, len);
    if (!h) return false;
    h->host = ptr;
    h->wrapped = true;
    h->dirty = true; // copied to HBM at the first submit that binds it
    out->handle = h;
    out->ptr = ptr;
    out->size = len;
    return true;
}

// The packed copies made from h are stale (its contents changed or it goes away): free them.
static void packs_drop(qw_hbuf *h) {
    if (!h || !h->npack) return;
    qw_gpu *g = h->g;
    (void)hipDeviceSynchronize(); // a batch in flight may still read them
    int n = 0;
    for (int i = 0; i < g->npacks; i++) {
        qw_pack *p = &g->packs[i];
        if (p->ha == h || p->hb == h) {
            qw_hbuf *other = p->ha == h ? p->hb : p->ha;
            if (other && other != h && other->released)
                fprintf(stderr, "qw_hip: a tile-major copy is dropped whose other source buffer was released: that buffer's matrix can no longer be dispatched\n");
            (void)hipFree(p->dst);
            g->pack_bytes -= p->bytes;
            if (p->ha && p->ha != h) p->ha->npack--;
            if (p->hb && p->hb != h && p->hb != p->ha) p->hb->npack--;
        } else g->packs[n++] = *p;
    }
    g->npacks = n;
    h->npack = 0;
}

void qw_buf_free(qw_buf *b) {
    if (!b || !b->handle) return;
    qw_hbuf *h = b->handle;
    packs_drop(h);
    if (!h->released) (void)hipFree(h->dptr);
    if (h->own_host) {
        if (h->pinned) (void)hipHostFree(h->host);
        else free(h->host);
    }
    free(h);
    b->handle = NULL;
    b->ptr = NULL;
    b->size = 0;
}

void *qw_pool_push(void) { return NULL; }
void qw_pool_pop(void *pool) { (void)pool; }

void qw_hip_buf_mark_dirty(qw_buf *b) {
    if (!b || !b->handle || ((qw_hbuf *)b->handle)->released) return; // a released buffer has nothing to refresh
    ((qw_hbuf *)b->handle)->dirty = true;
    packs_drop(b->handle);
}
void qw_hip_set_repack(qw_gpu *g, bool on) { g->repack = on; }
unsigned qw_hip_graph_launches(const qw_gpu *g) { return g->ngraph_launches; }
void qw_hip_set_graphs(qw_gpu *g, bool on) { g->use_graphs = on; }
size_t qw_hip_packed_bytes(const qw_gpu *g) { return g->pack_bytes; }
void *qw_hip_buf_devptr(const qw_buf *b) { return b && b->handle && !((qw_hbuf *)b->handle)->released ? ((qw_hbuf *)b->handle)->dptr : NULL; }
static bool range_ok(const qw_hbuf *h, size_t off, size_t len) { return !h->released && off <= h->size && len <= h->size - off; } // a released buffer has no bytes to copy
// Free the device bytes of a weight buffer and keep its tile-major copies (include/qw_hip_ext.h).
// Bytes of h that some tile-major copy was made from: the union of the copies' source ranges inside the buffer.
static size_t packed_source_bytes(const qw_hbuf *h) {
    const qw_gpu *g = h->g;
    enum { MAXIV = 256 };
    size_t lo[MAXIV], hi[MAXIV];
    int n = 0;
    for (int i = 0; i < g->npacks && n + 2 <= MAXIV; i++) {
        const qw_pack *p = &g->packs[i];
        const bool nl = p->split == QW_F_PACKED_NL, q6 = p->split == QW_F_PACKED_Q6;
        const size_t rowb = (size_t)p->nblk * (nl ? 180u : q6 ? 210u : 110u), rows_a = nl || q6 ? 16 : p->split, rows_b = nl || q6 ? 0 : 16 - p->split;
        if (p->ha == h && p->A) lo[n] = (size_t)((const char *)p->A - (const char *)h->dptr), hi[n] = lo[n] + (size_t)p->ntiles * rows_a * rowb, n++;
        if (p->hb == h && p->B && rows_b) lo[n] = (size_t)((const char *)p->B - (const char *)h->dptr), hi[n] = lo[n] + (size_t)p->ntiles * rows_b * rowb, n++;
    }
    for (int i = 1; i < n; i++) // by start (few intervals: insertion sort)
        for (int j = i; j > 0 && lo[j] < lo[j - 1]; j--) {
            const size_t a = lo[j], c = hi[j];
            lo[j] = lo[j - 1], hi[j] = hi[j - 1], lo[j - 1] = a, hi[j - 1] = c;
        }
    size_t total = 0, end = 0;
    for (int i = 0; i < n; i++) {
        const size_t from = lo[i] > end ? lo[i] : end;
        if (hi[i] > from) total += hi[i] - from, end = hi[i];
    }
    return total;
}
bool qw_hip_buf_release_source(qw_buf *b) {
    qw_hbuf *h = b ? b->handle : NULL;
    if (!h || h->released || !h->npack || h->pending_out) return false;
    // Every byte of the buffer must have a copy to stand in for it (up to the alignment gaps of an arena: 256 bytes a
    // copy): a matrix without one could never be dispatched again.
    const size_t covered = packed_source_bytes(h);
    if (covered + (size_t)256 * (size_t)h->npack * 2 < h->size) {
        set_err(h->g, "qw_hip_buf_release_source: tile-major copies stand in for %zu of the buffer's %zu bytes; run every matrix of it once first", covered, h->size);
        return false;
    }
    if (hipDeviceSynchronize() != hipSuccess) return false; // a batch in flight may still read the bytes
    if (hipFree(h->dptr) != hipSuccess) { (void)hipGetLastError(); return false; }
    h->released = true; // dptr stays as the key the copies were filed under; nothing dereferences it from here on
    h->dirty = false;
    h->g->released_bytes += h->size;
    return true;
}
size_t qw_hip_released_bytes(const qw_gpu *g) { return g->released_bytes; }
bool qw_hip_buf_upload(qw_buf *b, size_t off, size_t len) {
    qw_hbuf *h = b ? b->handle : NULL;
    if (h && h->released) return false;
    packs_drop(h);
    return h && h->host && range_ok(h, off, len) && hipMemcpy((char *)h->dptr + off, (char *)h->host + off, len, hipMemcpyHostToDevice) == hipSuccess;
}
bool qw_hip_buf_download(qw_buf *b, size_t off, size_t len) {
    qw_hbuf *h = b ? b->handle : NULL;
    return h && h->host && !h->wrapped && range_ok(h, off, len) && hipMemcpy((char *)h->host + off, (char *)h->dptr + off, len, hipMemcpyDeviceToHost) == hipSuccess;
}
bool qw_hip_buf_write(qw_buf *b, size_t off, const void *src, size_t len) {
    qw_hbuf *h = b ? b->handle : NULL;
    if (h && h->released) return false;
    if (!h || !range_ok(h, off, len)) return false;
    packs_drop(h);
    // A buffer with a host side keeps it in step: a later upload of the shadow (a new or marked buffer is sent whole at
    // its next bind, a small one at every submit) then carries these bytes instead of wiping them out.
    if (h->host && !h->wrapped) memcpy((char *)h->host + off, src, len);
    return hipMemcpy((char *)h->dptr + off, src, len, hipMemcpyHostToDevice) == hipSuccess;
}
// File -> HBM through pinned staging. Chunk c of the range belongs to lane c % nth; a lane is two pinned buffers, a
// stream (default priority) and two events, kept by the device handle from their first use: the pread() of a lane's
// next chunk runs while the DMA of its previous one is in flight. One thread per lane for the duration of a call.
#define QW_FD_CHUNK ((size_t)4 << 20)
typedef struct {
    qw_hbuf *h;
    struct qw_ldlane *lane;
    size_t off, len;
    int fd, tid, nth;
    uint64_t foff;
    bool ok;
} fd_job;
static void *fd_worker(void *arg) {
    fd_job *j = arg;
    struct qw_ldlane *L = j->lane;
    bool used[2] = {false, false}, ok = hipSetDevice(j->h->g->dev) == hipSuccess;
    int slot = 0;
    for (size_t c = (size_t)j->tid * QW_FD_CHUNK; ok && c < j->len; c += (size_t)j->nth * QW_FD_CHUNK, slot ^= 1) {
        const size_t n = j->len - c < QW_FD_CHUNK ? j->len - c : QW_FD_CHUNK;
        if (used[slot]) ok = hipEventSynchronize(L->ev[slot]) == hipSuccess; // the DMA that last read this staging buffer
        for (size_t got = 0; ok && got < n;) {
            const ssize_t r = pread(j->fd, (char *)L->pin[slot] + got, n - got, (off_t)(j->foff + c + got));
            if (r <= 0) ok = false; // an error, or the file ends inside the range
            else got += (size_t)r;
        }
        if (ok && j->h->host && !j->h->wrapped) memcpy((char *)j->h->host + j->off + c, L->pin[slot], n); // the host side keeps in step (qw_hip_buf_write)
        ok = ok && hipMemcpyAsync((char *)j->h->dptr + j->off + c, L->pin[slot], n, hipMemcpyHostToDevice, L->st) == hipSuccess;
        ok = ok && hipEventRecord(L->ev[slot], L->st) == hipSuccess;
        used[slot] = true;
    }
    ok = (hipStreamSynchronize(L->st) == hipSuccess) && ok; // also when a step failed: nothing of this call stays in flight
    j->ok = ok;
    return NULL;
}
// Lanes 0 .. n-1 of the device handle, made on the calling thread.
static bool ld_lanes(qw_gpu *g, int n) {
    for (; g->nld < n; g->nld++) {
        struct qw_ldlane *L = &g->ld[g->nld];
        memset(L, 0, sizeof *L);
        bool ok = HIPOK(g, hipHostMalloc(&L->pin[0], QW_FD_CHUNK, hipHostMallocDefault)) && HIPOK(g, hipHostMalloc(&L->pin[1], QW_FD_CHUNK, hipHostMallocDefault));
        ok = ok && HIPOK(g, hipStreamCreateWithFlags(&L->st, hipStreamNonBlocking));
        ok = ok && HIPOK(g, hipEventCreateWithFlags(&L->ev[0], hipEventDisableTiming)) && HIPOK(g, hipEventCreateWithFlags(&L->ev[1], hipEventDisableTiming));
        if (!ok) {
            for (int k = 0; k < 2; k++) {
                if (L->ev[k]) (void)hipEventDestroy(L->ev[k]);
                if (L->pin[k]) (void)hipHostFree(L->pin[k]);
            }
            if (L->st) (void)hipStreamDestroy(L->st);
            memset(L, 0, sizeof *L);
            return false;
        }
    }
    return true;
}
bool qw_hip_buf_write_fd(qw_buf *b, size_t off, int fd, uint64_t foff, size_t len) {
    qw_hbuf *h = b ? b->handle : NULL;
    if (!h || !range_ok(h, off, len) || fd < 0) return false;
    packs_drop(h);
    if (!len) return true;
    int nth = h->g->sw.load_threads;
    const size_t nchunk = (len + QW_FD_CHUNK - 1) / QW_FD_CHUNK;
    if ((size_t)nth > nchunk) nth = (int)nchunk;
    if (!ld_lanes(h->g, nth)) return false;
    fd_job job[QW_LD_MAX];
    pthread_t th[QW_LD_MAX];
    bool started[QW_LD_MAX] = {false};
    for (int i = 0; i < nth; i++) {
        job[i] = (fd_job){h, &h->g->ld[i], off, len, fd, i, nth, foff, false};
        if (i + 1 < nth) started[i] = pthread_create(&th[i], NULL, fd_worker, &job[i]) == 0;
    }
    bool ok = true;
    for (int i = nth - 1; i >= 0; i--) { // the calling thread takes the last lane, and any whose thread did not start
        if (started[i]) pthread_join(th[i], NULL);
        else fd_worker(&job[i]);
        ok = ok && job[i].ok;
    }
    if (!ok) set_err(h->g, "qw_hip_buf_write_fd: read or copy failed");
    return ok; // (a host side got the same bytes; whether it still holds others that HBM lacks stays as it was)
}
bool qw_hip_buf_read(const qw_buf *b, size_t off, void *dst, size_t len) {
    const qw_hbuf *h = b ? b->handle : NULL;
    return h && range_ok(h, off, len) && hipMemcpy(dst, (const char *)h->dptr + off, len, hipMemcpyDeviceToHost) == hipSuccess;
}

// ---------------------------------------------------------------- batches: recording
qw_batch *qw_batch_begin(qw_gpu *g, bool concurrent) {
    (void)concurrent; // an in-order stream already gives the serial order; "concurrent" batches are serial too
    qw_batch *b = calloc(1, sizeof *b);
    if (!b) return NULL;
    b->g = g;
    b->seq = ++g->batch_seq;
    b->stream = g->cur_stream;
    b->prof = g->prof;
    g->err[0] = 0;
    b->sw = g->sw;
    b->sw.no_fuse = g->sw.no_fuse || g->fuse_broken || b->stream != 0; // launches that wait for all their workgroups: one stream only
    return b;
}

void qw_batch_kernel(qw_batch *b, qw_kernel *k) {
    b->k = k;
    if (!k) { b->failed = true; set_err(b->g, "qw_batch_kernel: NULL kernel"); }
}

void qw_batch_buf(qw_batch *b, unsigned index, const qw_buf *buf, size_t offset) {
    if (index >= QW_MAX_BIND) { b->failed = true; set_err(b->g, "binding index %u out of range", index); return; }
    b->buf[index].buf = buf;
    b->buf[index].h = buf ? buf->handle : NULL;
    b->buf[index].off = offset;
    b->blen[index] = 0;
}

void qw_batch_bytes(qw_batch *b, unsigned index, const void *data, size_t len) {
    if (index >= QW_MAX_BIND || len > QW_MAX_BYTES) { b->failed = true; set_err(b->g, "inline bytes: index %u / length %zu out of range", index, len); return; }
    memcpy(b->bytes[index], data, len);
    b->blen[index] = len;
    b->buf[index].h = NULL;
}

void qw_batch_threadgroup_mem(qw_batch *b, unsigned index, size_t len) { (void)b; (void)index; (void)len; } // LDS sizes are fixed per kernel here
void qw_batch_barrier(qw_batch *b) { (void)b; }

static bool fail(qw_batch *b, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(b->g->err, sizeof b->g->err, fmt, ap);
    va_end(ap);
    if (b->g->sw.verbose) fprintf(stderr, "[qw_hip] %s\n", b->g->err);
    b->failed = true;
    return false;
}

// Binding `index` as a device pointer with at least `need` bytes after its offset; records the use.
static bool bind_ptr(qw_batch *b, unsigned index, size_t need, bool out, const char *what, void **p) {
    qw_hbuf *h = b->buf[index].h;
    if (!h) return fail(b, "%s: nothing bound at index %u (%s)", b->k->name, index, what);
    const size_t off = b->buf[index].off;
    if (off > h->size || need > h->size - off) return fail(b, "%s: %s at index %u needs %zu bytes after offset %zu, buffer has %zu", b->k->name, what, index, need, off, h->size);
    if (out && h->wrapped) return fail(b, "%s: %s at index %u is a wrapped (read-only) buffer", b->k->name, what, index);
    if (h->released && (out || !b->allow_released))
        return fail(b, "%s: %s at index %u: the buffer's GGUF-order bytes were released (qw_hip_buf_release_source); only dispatches that a tile-major copy serves may bind it", b->k->name, what, index);
    if (out) packs_drop(h); // a kernel is about to write it
    *p = (char *)h->dptr + off;
    if (b->nuse == b->capuse) {
        if (b->noalloc) return fail(b, "%s: more than %d bindings in the fixed recorder", b->k->name, b->capuse);
        b->capuse = b->capuse ? 2 * b->capuse : 64;
        b->use = realloc(b->use, sizeof *b->use * (size_t)b->capuse);
    }
    b->use[b->nuse++] = (qw_use){h, out};
    return true;
}
static bool bind_bytes(qw_batch *b, unsigned index, void *dst, size_t len, const char *what) {
    if (b->blen[index] < len) return fail(b, "%s: %s at index %u needs %zu inline bytes, has %zu", b->k->name, what, index, len, b->blen[index]);
    memcpy(dst, b->bytes[index], len);
    return true;
}

_Static_assert(sizeof(qwk_prekq_args) <= QW_MAX_ARGS, "argument record");
_Static_assert(sizeof(qwk_pre_args) <= QW_MAX_ARGS && sizeof(qwk_gu_args) <= QW_MAX_ARGS && sizeof(qwk_dn_args) <= QW_MAX_ARGS && sizeof(qwk_qmv_args) <= QW_MAX_ARGS,
               "a kernel argument record is larger than the launch record's copy of it");

static bool add_launch(qw_batch *b, const char *fname, unsigned gx, unsigned bx, const void *args, size_t argsz) {
    if (argsz > QW_MAX_ARGS) return fail(b, "%s: argument record of %zu bytes", fname, argsz);
    hipFunction_t f = get_func(b->g, fname);
    if (!f) return fail(b, "%s: entry point %s missing from the code object", b->k->name, fname);
    if (gx == 0) return true; // nothing to do
    if (b->nl == b->capl) {
        if (b->noalloc) return fail(b, "%s: more than %d launches in the fixed recorder", b->k->name, b->capl);
        b->capl = b->capl ? 2 * b->capl : 64;
        b->l = realloc(b->l, sizeof *b->l * (size_t)b->capl);
    }
    qw_launch *l = &b->l[b->nl++];
    memset(l, 0, sizeof *l);
    l->f = f;
    l->fname = fname;
    l->gx = gx; l->gy = 1; l->gz = 1; l->bx = bx;
    memcpy(l->args, args, argsz);
    l->argsz = argsz;
    l->kname = b->k->name;
    l->join = !strncmp(fname, "qwk_dn", 6); // the down launches read H of the shared expert, which a side launch may write
    return true;
}

static unsigned umin(unsigned a, unsigned b) { return a < b ? a : b; }
static unsigned cdiv(unsigned a, unsigned b) { return (a + b - 1) / b; }
// Persistent grids: one 512-thread workgroup per compute unit (the LDS tables leave room for one), fewer if the
// work is smaller. tasks are per-wave units; 8 waves per workgroup.
static unsigned persistent_grid(const qw_gpu *g, unsigned wave_tasks, unsigned waves) { return umin((unsigned)g->ncu, cdiv(wave_tasks, waves)); }
// waves per workgroup: gate/up + matvec kernels, front / any-shape down kernels, down range kernels
enum { QW_WAVES_GU = 12, QW_WAVES_DN = 8, QW_WAVES_DNR = 12 }; // (the routed gate/up launch with 8 or 10 waves a workgroup: 2 % slower at 16 tokens)

static const char *fname_fmt(char *buf, size_t n, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, n, fmt, ap);
    va_end(ap);
    return buf;
}
// entry-point names live as long as the process: intern them
static const char *intern(const char *s) {
    static char *tab[256];
    static int n;
    for (int i = 0; i < n; i++)
        if (!strcmp(tab[i], s)) return tab[i];
    if (n == 256) return "?";
    return tab[n++] = strdup(s);
}


// ---------------------------------------------------------------- family translators
static bool tr_dq_test(qw_batch *b, unsigned gx) { // tools/dqtest.c:39-45: 0 W, 1 y, 2 {K, row bytes}; grid = rows
    const qw_kparams *p = &b->k->p;
    uint32_t a2[2];
    if (!bind_bytes(b, 2, a2, sizeof a2, "{K, rowbytes}")) return false;
    if (a2[0] == 0 || a2[0] % (unsigned)fmt_qb(p->F) || a2[1] < fmt_rb(p->F, (int)a2[0])) return fail(b, "dq_test: K %u / row bytes %u do not fit type %d", a2[0], a2[1], p->F);
    qwk_dq_args a = {.K = a2[0], .rowbytes = a2[1], .rows = gx, .fmt = (uint32_t)p->F};
    if (!bind_ptr(b, 0, (size_t)gx * a2[1], false, "W", (void **)&a.W) || !bind_ptr(b, 1, (size_t)gx * a2[0] * 4, true, "y", (void **)&a.y)) return false;
    if (kq_ok(p->F)) {
        if ((b->buf[0].h && b->buf[0].off % 16) || a2[1] % (p->F == 14 || p->F == 20 ? 2 : p->F == 23 ? 8 : 16)) return fail(b, "dq_test: rows of type %d must keep the alignment of its blocks (offset %zu, row bytes %u)", p->F, b->buf[0].off, a2[1]);
        return add_launch(b, "qwk_dq_test_kq", gx, 64, &a, sizeof a);
    }
    return add_launch(b, p->F == 21 ? "qwk_dq_test_f21" : "qwk_dq_test_f8", gx, 64, &a, sizeof a);
}

static const void *glut(const qw_gpu *g) { return (const char *)g->tabs + QW_TAB_IQ3SS; }

// Blocks per prefetch chunk for a row of K values (the kernels are instantiated for these; 1 = any K).
static int chunk_of(int F, int K) { return K % 512 == 0 ? (F == 21 ? 2 : 16) : 1; }

static const uint8_t *get_pack(qw_batch *b, qw_hbuf *ha, const void *A, qw_hbuf *hb, const void *B, uint64_t ntiles, uint32_t nblk, uint32_t rowbytes, uint32_t split);
// One launch of the multi-format matvec over nmat matrices; W / y already bound into a.
// Few tiles: the parts a tile's K range is cut into, one wave each — the largest divisor of the chunk count up to 6
// that the wave slots of the device hold (a workgroup's waves beyond a whole number of tiles stay idle).
static unsigned pick_split(unsigned chunks, unsigned tiles, unsigned slots) {
    for (unsigned s = 6; s > 1; s--)
        if (chunks % s == 0 && tiles * s <= slots) return s;
    return 1;
}
// hw: the buffers the matrices lie in (NULL: no tile-major copies are looked for)
#define QW_Q6_PACK_MIN_ROWS 16384u
static bool launch_qmvm(qw_batch *b, qwk_qmvm_args *a, qw_hbuf *const *hw) {
    unsigned tiles = 0;
    a->sums = 0;
    for (uint32_t j = 0; j < a->nmat; j++) {
        // A large Q6_K matrix (the vocabulary projection, src/engine.c:658-704) is read from a tile-major copy made at
        // its first use: five coalesced loads a block instead of seventeen 4-byte ones and seventeen cross-lane moves.
        if (hw && a->fmt[j] == 14 && a->K % 256 == 0 && a->N[j] % 16 == 0 && a->N[j] >= QW_Q6_PACK_MIN_ROWS) {
            const uint32_t nblk = a->K / 256;
            const uint8_t *pk = get_pack(b, hw[j], a->W[j], NULL, NULL, a->N[j] / 16, nblk, a->rowbytes[j], QW_F_PACKED_Q6);
            if (pk) a->W[j] = pk, a->fmt[j] = QW_F_PACKED_Q6, a->rowbytes[j] = nblk * QW_Q6_SLAB_BYTES;
        }
        a->ntiles[j] = cdiv(a->N[j], 16);
        tiles += a->ntiles[j];
        if (a->fmt[j] == 12 || a->fmt[j] == 13) a->sums = 1;
    }
    if (!tiles) return true;
    // few tiles: cut every tile's K range over several waves, as far as the wave slots of the device and K allow
    const unsigned waves = QW_WAVES_GU, slots = (unsigned)b->g->ncu * waves;
    a->split = a->K % 256 == 0 ? pick_split(a->K / 256, tiles, slots) : 1;
    if (a->split > 1) {
        unsigned groups = 0;
        for (uint32_t j = 0; j < a->nmat; j++) groups += cdiv(a->ntiles[j], waves / a->split);
        return add_launch(b, "qwk_qmvm", umin((unsigned)b->g->ncu, groups), 64 * waves, a, sizeof *a);
    }
    return add_launch(b, "qwk_qmvm", persistent_grid(b->g, tiles, waves), 64 * waves, a, sizeof *a);
}

static bool tr_qmvm(qw_batch *b) { // src/engine.c:752-771: 0..3 W, 4 x, 5..8 y, 9 {N[4], off[4], total, xstride}; y stride = N
    const qw_kparams *p = &b->k->p;
    struct { uint32_t N[4], off[4], total, xstride; } in;
    if (!bind_bytes(b, 9, &in, sizeof in, "{N[4], off[4], total, xstride}")) return false;
    qwk_qmvm_args a = {.K = (uint32_t)p->K, .xstride = in.xstride, .nb = (uint32_t)p->NB, .yfloat = (uint32_t)p->yfloat, .nmat = (uint32_t)p->nmat};
    if (a.xstride < a.K || a.xstride % 8) return fail(b, "qmv_ggm: xstride %u (needs >= K, multiple of 8)", a.xstride);
    if (b->buf[4].h && b->buf[4].off % 16) return fail(b, "qmv_ggm: x offset %zu is not 16-byte aligned", b->buf[4].off);
    if (!bind_ptr(b, 4, ((size_t)(a.nb - 1) * a.xstride + a.K) * 2, false, "x", (void **)&a.x)) return false;
    uint32_t total = 0;
    for (int j = 0; j < p->nmat; j++) {
        a.N[j] = in.N[j], a.fmt[j] = (uint32_t)p->gf[j], a.rowbytes[j] = (uint32_t)fmt_rb(p->gf[j], p->K), a.ystride[j] = in.N[j];
        if (in.off[j] != total) return fail(b, "qmv_ggm: off[%d] = %u, expected %u (rows of the matrices before it)", j, in.off[j], total);
        total += in.N[j];
        if (!in.N[j]) return fail(b, "qmv_ggm: matrix %d has no rows", j);
        if (b->buf[j].h && b->buf[j].off % 16) return fail(b, "qmv_ggm: offset %zu of matrix %d is not 16-byte aligned", b->buf[j].off, j);
        if (!bind_ptr(b, (unsigned)j, (size_t)a.N[j] * a.rowbytes[j], false, "W", (void **)&a.W[j]) ||
            !bind_ptr(b, 5u + (unsigned)j, (size_t)a.nb * a.N[j] * (a.yfloat ? 4 : 2), true, "y", &a.y[j])) return false;
    }
    if (in.total != total) return fail(b, "qmv_ggm: total %u, the matrices have %u rows", in.total, total);
    qw_hbuf *hm[4] = {b->buf[0].h, b->buf[1].h, b->buf[2].h, b->buf[3].h};
    return launch_qmvm(b, &a, hm);
}

static bool tr_qmv(qw_batch *b) { // src/engine.c:717-723: 0 W, 3 x, 4 y, 5 {N, xstride, ystride, pad}
    const qw_kparams *p = &b->k->p;
    uint32_t a4[4];
    if (!bind_bytes(b, 5, a4, sizeof a4, "{N, xstride, ystride, pad}")) return false;
    if (kq_ok(p->F)) { // the multi-format kernel with one matrix
        qwk_qmvm_args m = {.K = (uint32_t)p->K, .xstride = a4[1], .nb = (uint32_t)p->NB, .yfloat = (uint32_t)p->yfloat, .nmat = 1,
                           .N = {a4[0]}, .fmt = {(uint32_t)p->F}, .rowbytes = {(uint32_t)p->RB}, .ystride = {a4[2]}};
        if (!m.N[0]) return true;
        if (m.xstride < m.K || m.xstride % 8 || m.ystride[0] < m.N[0]) return fail(b, "qmv_gg: xstride %u (needs >= K, multiple of 8) / ystride %u (needs >= N)", m.xstride, m.ystride[0]);
        if ((b->buf[3].h && b->buf[3].off % 16) || (b->buf[0].h && b->buf[0].off % 16)) return fail(b, "qmv_gg: x / W offsets must be 16-byte aligned");
        if (!bind_ptr(b, 0, (size_t)m.N[0] * m.rowbytes[0], false, "W", (void **)&m.W[0]) ||
            !bind_ptr(b, 3, ((size_t)(m.nb - 1) * m.xstride + m.K) * 2, false, "x", (void **)&m.x) ||
            !bind_ptr(b, 4, ((size_t)(m.nb - 1) * m.ystride[0] + m.N[0]) * (m.yfloat ? 4 : 2), true, "y", &m.y[0])) return false;
        qw_hbuf *hm[4] = {b->buf[0].h};
        return launch_qmvm(b, &m, hm);
    }
    qwk_qmv_args a = {.N = a4[0], .K = (uint32_t)p->K, .rowbytes = (uint32_t)p->RB, .xstride = a4[1], .ystride = a4[2], .nb = (uint32_t)p->NB, .yfloat = (uint32_t)p->yfloat,
                      .glut = glut(b->g)};
    if (a.N == 0) return true;
    if (a.xstride < a.K || a.xstride % 8 || a.ystride < a.N) return fail(b, "qmv_gg: xstride %u (needs >= K, multiple of 8) / ystride %u (needs >= N)", a.xstride, a.ystride);
    if (b->buf[3].h && b->buf[3].off % 16) return fail(b, "qmv_gg: x offset %zu is not 16-byte aligned", b->buf[3].off);
    a.ntiles = cdiv(a.N, 16);
    b->allow_released = true; // W may be a buffer of which only the tile-major copy is left
    const bool bound = bind_ptr(b, 0, (size_t)a.N * a.rowbytes, false, "W", (void **)&a.W);
    b->allow_released = false;
    if (!bound || !bind_ptr(b, 3, ((size_t)(a.nb - 1) * a.xstride + a.K) * 2, false, "x", (void **)&a.x) ||
        !bind_ptr(b, 4, ((size_t)(a.nb - 1) * a.ystride + a.N) * (a.yfloat ? 4 : 2), true, "y", &a.y)) return false;
    char fn[48];
    int F = p->F;
    if (F == 21 && p->K <= 2560 && a.N % 16 == 0) { // tile-major copy of the rows, made at first use
        const uint32_t nblk = (uint32_t)p->K / 256;
        const uint8_t *pk = get_pack(b, b->buf[0].h, a.W, NULL, NULL, a.N / 16, nblk, a.rowbytes, 16);
        if (pk) F = QW_F_PACKED, a.W = pk, a.rowbytes = nblk * QW_SLAB_BYTES;
    }
    if (b->buf[0].h->released && F != QW_F_PACKED) return fail(b, "%s: the GGUF-order bytes of the weights were released and no tile-major copy serves this dispatch", b->k->name);
    if (p->valu) { // the VALU GEMV, for measurement against the matrix-core form
        if (F != QW_F_PACKED || p->K % 512 || p->NB > 4) return fail(b, "qmv_gg: the VALU form needs packed IQ3_S weights, K a multiple of 512 and NB <= 4");
        fname_fmt(fn, sizeof fn, "qwk_qmv_valu_n%d", p->NB <= 1 ? 1 : p->NB <= 2 ? 2 : 4);
    } else {
        const int base = 21 == F || F == QW_F_PACKED ? 21 : F, ch = p->K > 2560 ? 1 : chunk_of(base, p->K);
        if (p->K > 2560) fname_fmt(fn, sizeof fn, "qwk_qmv_f%d_c1g", F);
        else fname_fmt(fn, sizeof fn, "qwk_qmv_f%d_c%d", F, ch);
        // few tiles: cut every tile's chunks over several waves, as far as the wave slots of the device allow
        const unsigned cpr = (unsigned)p->K / ((unsigned)fmt_qb(base) * (unsigned)ch), slots = (unsigned)b->g->ncu * QW_WAVES_GU;
        a.split = pick_split(cpr, a.ntiles, slots);
        if (a.split > 1) return add_launch(b, intern(fn), umin((unsigned)b->g->ncu, cdiv(a.ntiles, QW_WAVES_GU / a.split)), 64 * QW_WAVES_GU, &a, sizeof a);
    }
    a.split = 1;
    return add_launch(b, intern(fn), persistent_grid(b->g, a.ntiles, QW_WAVES_GU), 64 * QW_WAVES_GU, &a, sizeof a);
}

static bool fill_router(qw_batch *b, qwk_router_args *a, unsigned iWr, unsigned iWsg, unsigned ix, unsigned ilg, uint32_t nbr) {
    const qw_kparams *p = &b->k->p;
    *a = (qwk_router_args){.E = (uint32_t)p->E, .D = (uint32_t)p->D, .nb = nbr};
    return bind_ptr(b, iWr, (size_t)p->E * p->D * 2, false, "router weights", (void **)&a->Wr) && bind_ptr(b, iWsg, (size_t)p->D * 2, false, "shared gate vector", (void **)&a->Wsg) &&
           bind_ptr(b, ix, (size_t)nbr * p->D * 2, false, "x", (void **)&a->x) && bind_ptr(b, ilg, (size_t)nbr * (p->E + 1) * 4, true, "logits", (void **)&a->logits);
}

static bool fill_select(qw_batch *b, qwk_select_args *a, unsigned ilg, unsigned isel, uint32_t nbr) {
    const qw_kparams *p = &b->k->p;
    *a = (qwk_select_args){.nbr = nbr, .E = (uint32_t)p->E, .topk = (uint32_t)p->topk, .gnb = (uint32_t)p->gnb};
    return bind_ptr(b, ilg, (size_t)nbr * (p->E + 1) * 4, false, "logits", (void **)&a->logits) && bind_ptr(b, isel, QW_SEL_BYTES((size_t)p->gnb, (size_t)p->topk), true, "selection", (void **)&a->sel);
}
static bool launch_select(qw_batch *b, unsigned ilg, unsigned isel, uint32_t nbr) {
    qwk_select_args a;
    return fill_select(b, &a, ilg, isel, nbr) && add_launch(b, "qwk_select", 1, 1024, &a, sizeof a);
}
// The selection that a moe_pre_gg dispatch left pending and no gate/up dispatch took over: a launch of its own.
static bool flush_select(qw_batch *b) {
    if (!b->pend_sel.valid) return true;
    b->pend_sel.valid = false;
    return add_launch(b, "qwk_select", 1, 1024, &b->pend_sel.a, sizeof b->pend_sel.a);
}

static bool nbr_ok(qw_batch *b, uint32_t nbr) {
    if (nbr < 1 || nbr > (uint32_t)b->k->p.NB) return fail(b, "%s: %u tokens, kernel was built for at most NB = %d", b->k->name, nbr, b->k->p.NB);
    return true;
}

// gate/up arguments. shared: one expert at (iWg, iWu), all tokens, slot topk.
// The packed copy of IQ3_S rows: tiles of `split` rows of A and 16 - split rows of B (B = NULL, split 16: one matrix);
// split = QW_F_PACKED_NL: the packed copy of one matrix of IQ4_NL rows, nblk chunks of ten blocks a row.
// Made at the first request, on the batch's stream, and complete when this returns; NULL when packing is off, the
// source may change without notice (a small buffer with a host shadow is copied at every submit) or memory is short:
// the caller then reads the GGUF rows directly.
static const uint8_t *get_pack(qw_batch *b, qw_hbuf *ha, const void *A, qw_hbuf *hb, const void *B, uint64_t ntiles, uint32_t nblk, uint32_t rowbytes, uint32_t split) {
    qw_gpu *g = b->g;
    if (!g->repack) return NULL;
    for (int i = 0; i < g->npacks; i++) {
        const qw_pack *p = &g->packs[i];
        if (p->A != A || p->B != B || p->ntiles != ntiles || p->nblk != nblk || p->split != split) continue;
        // The addresses are the key (a view of the same memory under another handle finds the copy too) — unless the
        // source was released: its address may since have been given to another allocation, so only its own handle matches.
        const bool gone = (p->ha && p->ha->released) || (p->hb && p->hb->released);
        if (!gone || (p->ha == ha && p->hb == hb)) return p->dst;
    }
    if (b->noalloc) return NULL; // a copy that exists was found above; none is made here
    if ((ha && ha->released) || (hb && hb->released)) return NULL; // nothing left to copy from
    qw_hbuf *hs[2] = {ha, hb};
    for (int i = 0; i < 2; i++) {
        qw_hbuf *h = hs[i];
        if (!h) continue;
        if (!h->device_only && !h->wrapped && h->size <= QW_HIP_SMALL_BYTES) return NULL;
        // A dispatch recorded earlier in this batch writes the source and has not been launched yet (launches wait for
        // the submit): a copy made now would hold the old bytes.
        for (int u = b->done_use; u < b->nuse; u++)
            if (b->use[u].b == h && b->use[u].out) return NULL;
        if (h->dirty && h->host) { // what the next submit would do for this buffer
            if (hipMemcpyAsync(h->dptr, h->host, h->size, hipMemcpyHostToDevice, g->stream[b->stream]) != hipSuccess) return NULL;
            h->dirty = false;
        }
    }
    const bool nl = split == QW_F_PACKED_NL, q6 = split == QW_F_PACKED_Q6; // IQ4_NL rows: nblk counts chunks of ten blocks; Q6_K rows: blocks
    hipFunction_t f = get_func(g, nl ? "qwk_pack_nl" : q6 ? "qwk_pack_q6" : "qwk_pack_iq3");
    if (!f) return NULL;
    const size_t bytes = (size_t)ntiles * nblk * (nl ? QW_NL_CHUNK_BYTES : q6 ? QW_Q6_SLAB_BYTES : QW_SLAB_BYTES);
    void *dst;
    if (hipMalloc(&dst, bytes) != hipSuccess) {
        (void)hipGetLastError();
        return NULL;
    }
    qwk_pack_args pa = {.A = A, .B = B, .dst = dst, .ntiles = ntiles, .nblk = nblk, .rowbytes = rowbytes, .split = split};
    void *params[] = {&pa};
    const uint64_t nslab = ntiles * nblk;
    const unsigned gx = (unsigned)(nslab / 4 < 65536 ? (nslab + 3) / 4 : 65536);
    if (hipModuleLaunchKernel(f, gx, 1, 1, 256, 1, 1, 0, g->stream[b->stream], params, NULL) != hipSuccess || hipStreamSynchronize(g->stream[b->stream]) != hipSuccess) {
        (void)hipFree(dst);
        return NULL;
    }
    if (g->npacks == g->cappacks) {
        g->cappacks = g->cappacks ? 2 * g->cappacks : 64;
        g->packs = realloc(g->packs, sizeof *g->packs * (size_t)g->cappacks);
    }
    g->packs[g->npacks++] = (qw_pack){.A = A, .B = B, .ha = ha, .hb = hb, .ntiles = ntiles, .nblk = nblk, .split = split, .dst = dst, .bytes = bytes};
    g->pack_bytes += bytes;
    if (ha) ha->npack++;
    if (hb && hb != ha) hb->npack++;
    return dst;
}

static bool fill_gu(qw_batch *b, qwk_gu_args *a, int F, unsigned iWg, unsigned iWu, unsigned ix, unsigned iH, uint32_t nbr, bool shared) {
    const qw_kparams *p = &b->k->p;
    const size_t rb = fmt_rb(F, p->D), ne = shared ? 1 : (size_t)p->E;
    *a = (qwk_gu_args){.D = (uint32_t)p->D, .I = (uint32_t)p->I, .rowbytes = (uint32_t)rb, .nbr = nbr, .topk = (uint32_t)p->topk, .gnb = (uint32_t)p->gnb, .shared = shared,
                       .hplane = (uint32_t)p->NB * (uint32_t)(p->topk + 1) * (uint32_t)p->I, .glut = glut(b->g)};
    b->allow_released = !shared; // the routed matrices may be buffers of which only the tile-major copy is left (the caller checks that one serves)
    const bool bound = bind_ptr(b, iWg, ne * p->I * rb, false, "gate weights", (void **)&a->Wg) && bind_ptr(b, iWu, ne * p->I * rb, false, "up weights", (void **)&a->Wu);
    b->allow_released = false;
    if (!bound || !bind_ptr(b, ix, (size_t)nbr * p->D * 2, false, "x", (void **)&a->x) || !bind_ptr(b, iH, (size_t)a->hplane * 4, true, "H", (void **)&a->H)) return false;
    if (b->buf[ix].off % 16) return fail(b, "%s: x offset %zu is not 16-byte aligned", b->k->name, b->buf[ix].off);
    return true;
}

static bool tr_router(qw_batch *b) { // src/engine.c:546-551; NB = token count
    qwk_router_args a;
    if (!fill_router(b, &a, 0, 1, 2, 3, (uint32_t)b->k->p.NB)) return false;
    return add_launch(b, b->k->p.rwf == 30 ? "qwk_router_w30" : "qwk_router_w1", cdiv((unsigned)b->k->p.E + 1, 4), 256, &a, sizeof a);
}

static bool tr_tab_init(qw_batch *b) { // src/engine.c:572-574
    qwk_tab_args a = {0}; // the caller's buffer gets the reference's entry order
    if (!bind_ptr(b, 0, QW_TAB_BYTES, true, "lookup tables", (void **)&a.tab)) return false;
    return add_launch(b, "qwk_tab_init", 32, 256, &a, sizeof a);
}

static bool tr_sel(qw_batch *b) { // src/engine.c:609-614: 0 logits, 1 sel, 2 nbr
    uint32_t nbr;
    return bind_bytes(b, 2, &nbr, 4, "nbr") && nbr_ok(b, nbr) && launch_select(b, 0, 1, nbr);
}

// A shared expert whose gate and up rows are in the other format family (Q4_K gate and IQ4_XS up in the reference's
// model, bench/moe_bw.c:19-20): the multi-format matvec over the two matrices, then SwiGLU into H.
#define QW_SHGU_MAXI 4096
// front: the router's arguments when the caller is the front launch, which then takes this work onto the workgroups
// after the router's (one launch, qwk_pre_w1_kq) when it can; *rode tells whether it did.
static bool shared_gu_kq(qw_batch *b, uint32_t nbr, const uint16_t *x, uint16_t *h, const qwk_pre_args *front, bool *rode) {
    const qw_kparams *p = &b->k->p;
    if (rode) *rode = false;
    if (p->I > QW_SHGU_MAXI) return fail(b, "moe_pre_gg: I %d too wide for shared gate/up types %d/%d", p->I, p->fsg, p->fsu);
    if (b->buf[2].off % 16 || b->buf[6].off % 16 || b->buf[7].off % 16) return fail(b, "moe_pre_gg: x and shared gate/up offsets must be 16-byte aligned for types %d/%d", p->fsg, p->fsu);
    float *gy = b->g->shgu + (size_t)b->stream * 2 * 16 * QW_SHGU_MAXI, *uy = gy + (size_t)16 * p->I;
    qwk_qmvm_args m = {.K = (uint32_t)p->D, .xstride = (uint32_t)p->D, .nb = nbr, .yfloat = 1, .nmat = 2, .x = x,
                       .W = {b->pend_sg.Wsg, b->pend_sg.Wsu}, .y = {gy, uy}, .N = {(uint32_t)p->I, (uint32_t)p->I}, .fmt = {(uint32_t)p->fsg, (uint32_t)p->fsu},
                       .rowbytes = {(uint32_t)fmt_rb(p->fsg, p->D), (uint32_t)fmt_rb(p->fsu, p->D)}, .ystride = {(uint32_t)p->I, (uint32_t)p->I}};
    qwk_shact_args sa = {.g = gy, .u = uy, .H = h, .I = (uint32_t)p->I, .nb = nbr, .topk = (uint32_t)p->topk, .hplane = (uint32_t)p->NB * (uint32_t)(p->topk + 1) * (uint32_t)p->I};
    b->pend_sg.valid = false; // done here
    // This work depends on x alone, so it may run beside the router and the routed gate/up on the side stream
    // (QW_HIP_SIDE=1). Off by default: with the matvec and SwiGLU as two launches it paid with one or two tokens (48
    // layers of the reference model's shape: 2.89 -> 2.70 ms a token) and cost with more (6.81 -> 6.93 ms at 16); as
    // the one launch it is now, the fork and join cost as much as the overlap gives at every token count.
    const int first = b->nl;
    // one launch when the K range splits so that a workgroup holds whole (gate tile, up tile) pairs; else matvec, then SwiGLU
    unsigned sw = 0;
    for (unsigned s = 6; s > 1 && !sw; s--)
        if (s != 4 && (unsigned)(p->D / 256) % s == 0 && !b->sw.no_swiglu_matvec) sw = s;
    if (sw) {
        m.split = sw, m.sums = 0, m.H = h, m.topk = (uint32_t)p->topk, m.hplane = sa.hplane;
        for (int j = 0; j < 2; j++) {
            m.ntiles[j] = cdiv((unsigned)p->I, 16);
            if (m.fmt[j] == 12 || m.fmt[j] == 13) m.sums = 1;
        }
        const unsigned wgs = umin((unsigned)b->g->ncu, cdiv(m.ntiles[0], QW_WAVES_GU / sw / 2));
        if (front && p->rwf == 1 && b->sw.side != 1 && !b->sw.kq_own) { // binary16 router: its workgroups first, then these
            qwk_prekq_args f = {.r = front->r, .nrouter = front->nrouter, .m = m};
            if (!add_launch(b, "qwk_pre_w1_kq", f.nrouter + wgs, 64 * QW_WAVES_GU, &f, sizeof f)) return false;
            *rode = true;
            return true;
        }
        if (!add_launch(b, "qwk_qmvm_swiglu", wgs, 64 * QW_WAVES_GU, &m, sizeof m)) return false;
    } else if (!launch_qmvm(b, &m, NULL) || !add_launch(b, "qwk_sh_act", cdiv(nbr * (unsigned)p->I, 256), 256, &sa, sizeof sa)) return false;
    if (b->sw.side == 1)
        for (int i = first; i < b->nl; i++) b->l[i].side = true;
    return true;
}

// src/engine.c:588-607: 0 Wr, 1 shared gate vector, 2 x, 3 logits, 4 counter, 5 sel, 6/7 shared gate/up, 8 H, 13 tables, 14 nbr.
// Two launches: router rows, then the selection. The shared expert's gate/up is checked and remembered here and
// runs inside the gate/up launch that follows.
static bool tr_pre(qw_batch *b) {
    const qw_kparams *p = &b->k->p;
    uint32_t nbr;
    if (!bind_bytes(b, 14, &nbr, 4, "nbr") || !nbr_ok(b, nbr) || !flush_select(b)) return false;
    const size_t rb = fmt_rb(p->fsg, p->D);
    uint16_t *h;
    b->pend_sg.valid = false;
    if (!bind_ptr(b, 6, (size_t)p->I * rb, false, "shared gate weights", (void **)&b->pend_sg.Wsg) || !bind_ptr(b, 7, (size_t)p->I * fmt_rb(p->fsu, p->D), false, "shared up weights", (void **)&b->pend_sg.Wsu) ||
        !bind_ptr(b, 8, (size_t)p->NB * (p->topk + 1) * p->I * 4, true, "H", (void **)&h)) return false;
    b->pend_sg.valid = true;
    b->pend_sg.hg = b->buf[6].h;
    b->pend_sg.hu = b->buf[7].h;
    b->pend_sg.fmt = p->fsg;
    b->pend_sg.rowbytes = (uint32_t)rb;
    b->pend_sg.nbr = nbr;
    if (!p->rbf) { // router and selection come as dispatches of their own
        const uint16_t *x;
        return !kq_ok(p->fsg) || (bind_ptr(b, 2, (size_t)nbr * p->D * 2, false, "x", (void **)&x) && shared_gu_kq(b, nbr, x, h, NULL, NULL));
    }
    // router rows per workgroup: 16 on the matrix cores (binary16 router), 8 on the vector units (bf16 router)
    qwk_pre_args a = {.nrouter = cdiv((unsigned)p->E + 1, p->rwf == 1 ? 16 : 8)};
    if (!fill_router(b, &a.r, 0, 1, 2, 3, nbr)) return false;
    if (b->buf[2].off % 16) return fail(b, "moe_pre_gg: x offset %zu is not 16-byte aligned", b->buf[2].off);
    if (p->rwf == 1 && (b->buf[0].off % 16 || b->buf[1].off % 16)) return fail(b, "moe_pre_gg: router weight offsets must be 16-byte aligned");
    // The shared expert's gate/up runs on the workgroups after the router's when a tile row splits into at most 8
    // chunks (D a multiple of 512, at most 4096) and the weights are Q8_0 or packed IQ3_S; otherwise it is left for
    // the gate/up launch (pend_sg).
    char fn[48];
    fname_fmt(fn, sizeof fn, "qwk_pre_w%d", p->rwf == 30 ? 30 : 1);
    unsigned grid = a.nrouter;
    const unsigned cpr = (unsigned)p->D / 512;
    if (p->D % 512 == 0 && cpr <= 8 && !b->sw.shared_in_gu) {
        const uint32_t nblk = (uint32_t)p->D / 256;
        const uint8_t *ps = p->fsg == 21 ? get_pack(b, b->pend_sg.hg, b->pend_sg.Wsg, b->pend_sg.hu, b->pend_sg.Wsu, (uint64_t)(p->I / 8), nblk, (uint32_t)rb, 8) : NULL;
        if (p->fsg == 8 || ps) {
            a.g = (qwk_gu_args){.Wg = ps ? ps : b->pend_sg.Wsg, .Wu = ps ? NULL : b->pend_sg.Wsu, .x = a.r.x, .H = h, .D = (uint32_t)p->D, .I = (uint32_t)p->I,
                                .rowbytes = ps ? nblk * QW_SLAB_BYTES : (uint32_t)rb, .nbr = nbr, .topk = (uint32_t)p->topk, .gnb = (uint32_t)p->gnb, .shared = 1,
                                .hplane = (uint32_t)p->NB * (uint32_t)(p->topk + 1) * (uint32_t)p->I, .glut = glut(b->g)};
            fname_fmt(fn, sizeof fn, "qwk_pre_w%d_s%d_c%d", p->rwf == 30 ? 30 : 1, ps ? QW_F_PACKED : 8, ps ? 2 : 16);
            grid += cdiv((unsigned)p->I / 8, 8 / cpr);
            b->pend_sg.valid = false; // done here
        }
    }
    // the counter buffer of the reference's hand-over (index 4) is not used
    bool rode = false;
    if (kq_ok(p->fsg) && !shared_gu_kq(b, nbr, a.r.x, h, &a, &rode)) return false; // first: side launches fork where they stand in the batch
    if (!rode && !add_launch(b, intern(fn), grid, 512, &a, sizeof a)) return false;
    if (!fill_select(b, &b->pend_sel.a, 3, 5, nbr)) return false;
    b->pend_sel.valid = true; // made by the gate/up launch if one follows for the same record, else by its own launch
    return true;
}

// src/engine.c:616-629: 0 Wg, 1 Wu, 2 shared down, 3 Psh, 4 x, 5 sel, 6 H, 11 tables, 12 nbr.
// One launch: the shared expert's gate/up tiles (remembered from moe_pre_gg) and the routed gate/up tiles of the
// selected experts. The shared down is checked and remembered for the down launch.
static bool tr_gu(qw_batch *b) {
    const qw_kparams *p = &b->k->p;
    uint32_t nbr;
    if (!bind_bytes(b, 12, &nbr, 4, "nbr") || !nbr_ok(b, nbr)) return false;
    qwk_gu_args a;
    if (!fill_gu(b, &a, p->fgu, 0, 1, 4, 6, nbr, false)) return false;
    if (!bind_ptr(b, 5, QW_SEL_BYTES((size_t)p->gnb, (size_t)p->topk), false, "selection", (void **)&a.sel)) return false;
    b->pend_sd.valid = false;
    b->pend_sd.rowbytes = (uint32_t)fmt_rb(p->fsd, p->I);
    if (!bind_ptr(b, 2, (size_t)p->D * b->pend_sd.rowbytes, false, "shared down weights", (void **)&b->pend_sd.Wsd) || !bind_ptr(b, 3, (size_t)nbr * p->D * 4, true, "Psh", (void **)&b->pend_sd.Psh)) return false;
    b->pend_sd.valid = true;
    b->pend_sd.hd = b->buf[2].h;
    b->pend_sd.fmt = p->fsd;
    b->pend_sd.nbr = nbr;
    int cg = chunk_of(p->fgu, p->D), fs = 0, cs = 1;
    qw_hbuf *hsg = NULL, *hsu = NULL;
    if (b->pend_sg.valid) {
        hsg = b->pend_sg.hg, hsu = b->pend_sg.hu;
        if (b->pend_sg.nbr != nbr) return fail(b, "moe_gu_gg: %u tokens after a front part of %u", nbr, b->pend_sg.nbr);
        fs = b->pend_sg.fmt;
        cs = chunk_of(fs, p->D);
        a.Wsg = b->pend_sg.Wsg;
        a.Wsu = b->pend_sg.Wsu;
        a.sg_rowbytes = b->pend_sg.rowbytes;
        b->pend_sg.valid = false;
        if (cg == 1 || cs == 1) cg = cs = 1; // any-shape builds come in pairs
    }
    if (b->pend_sel.valid && b->pend_sel.a.sel == a.sel && b->pend_sel.a.nbr == nbr && b->pend_sel.a.E == (uint32_t)p->E && b->pend_sel.a.topk == (uint32_t)p->topk &&
        b->pend_sel.a.gnb == (uint32_t)p->gnb && !b->sw.split_select) {
        a.logits = b->pend_sel.a.logits;
        a.E = (uint32_t)p->E;
        b->pend_sel.valid = false;
    } else if (!flush_select(b)) return false;
    int fgu = p->fgu;
    const bool rt = rt_ok(fgu); // a type the kernel takes as an argument: one block a chunk, the shared expert's rows in GGUF order
    if (rt) {
        if (fs && fs != 8 && fs != 21) return fail(b, "moe_gu_gg: gate/up types %d (routed) / %d (shared) have no common gfx950 kernel", fgu, fs);
        a.fgu = (uint32_t)fgu;
        cg = cs = 1;
    }
    if (fgu == 21) { // tile-major copies of the IQ3_S rows, made at first use
        const uint32_t nblk = (uint32_t)p->D / 256, tileb = nblk * QW_SLAB_BYTES;
        const uint8_t *pk = get_pack(b, b->buf[0].h, a.Wg, b->buf[1].h, a.Wu, (uint64_t)p->E * (uint64_t)(p->I / 8), nblk, a.rowbytes, 8);
        const uint8_t *ps = pk && fs == 21 ? get_pack(b, hsg, a.Wsg, hsu, a.Wsu, (uint64_t)(p->I / 8), nblk, a.sg_rowbytes, 8) : NULL;
        if (pk && (fs != 21 || ps)) {
            fgu = QW_F_PACKED;
            a.Wg = pk, a.Wu = NULL, a.rowbytes = tileb;
            if (fs == 21) fs = QW_F_PACKED, a.Wsg = ps, a.Wsu = NULL, a.sg_rowbytes = tileb;
        }
    }
    if ((b->buf[0].h->released || b->buf[1].h->released) && fgu != QW_F_PACKED) return fail(b, "%s: the GGUF-order bytes of the weights were released and no tile-major copy serves this dispatch", b->k->name);
    char fn[64];
    if (rt) {
        if (fs) fname_fmt(fn, sizeof fn, "qwk_gu_rt_s%d_c1", fs);
        else fname_fmt(fn, sizeof fn, "qwk_gu_rt");
    } else if (fs) fname_fmt(fn, sizeof fn, "qwk_gu_f%d_c%d_s%d_c%d", fgu, cg, fs, cs);
    else fname_fmt(fn, sizeof fn, "qwk_gu_f%d_c%d", fgu, cg);
    const unsigned tasks = umin((unsigned)p->E, nbr * (unsigned)p->topk) * (unsigned)(p->I / 8) + (fs ? (unsigned)p->I / 8 : 0);
    // With few tiles (one or two tokens: 640 to 1280 of them) every compute unit still gets a workgroup: the waves are
    // numbered wave-major, so the tiles spread over all compute units instead of filling the waves of the first
    // workgroups (48-layer step at one token: gate/up launch 18.3 -> 13.4 us, 615 -> 715 tokens/s).
    if (b->sw.ablate && fgu == QW_F_PACKED && cg == 2 && !fs) fname_fmt(fn, sizeof fn, "qwk_gu_f%d_c2", QW_F_ABLATE);
    const unsigned grid = umin((unsigned)b->g->ncu, tasks);
    // Tile-major IQ3_S rows of the shape the fused launch is built for: wait for the down dispatch (qwk_gud_*)
    if (!b->sw.no_fuse && !b->sw.ablate && b->sw.side != 1 && fgu == QW_F_PACKED && cg == 2 && !fs && p->D <= 2048 && p->I == 512 && p->topk <= 10 && p->gnb * p->topk <= (int)QW_DNQ_MAXU &&
        b->buf[6].off % 4 == 0) {
        b->pend_gu.valid = true;
        b->pend_gu.a = a;
        b->pend_gu.fname = intern(fn), b->pend_gu.kname = b->k->name, b->pend_gu.grid = grid;
        return true;
    }
    return add_launch(b, intern(fn), grid, 64 * QW_WAVES_GU, &a, sizeof a);
}

// The gate/up launch that waited for a down dispatch to join it, on its own after all.
static bool flush_gu(qw_batch *b) {
    if (!b->pend_gu.valid) return true;
    b->pend_gu.valid = false;
    const int first = b->nl;
    if (!add_launch(b, b->pend_gu.fname, b->pend_gu.grid, 64 * QW_WAVES_GU, &b->pend_gu.a, sizeof b->pend_gu.a)) return false;
    if (b->nl > first) b->l[b->nl - 1].kname = b->pend_gu.kname, b->l[b->nl - 1].last_of_dispatch = true;
    return true;
}
// Shares of the tokens and tiles per workgroup of the fused launch's down phase: at most QW_GUD_SHARE tokens a share.
static void gud_shape(unsigned nbr, unsigned *nq, unsigned *tpw) {
    unsigned q = 1;
    while (q < 8 && (nbr == 1 ? q < 1 : cdiv(nbr, q) > QW_GUD_SHARE || q < 2)) q *= 2;
    *nq = q;
    *tpw = q > 2 ? q / 2 : 1;
}

static bool flush_dn(qw_batch *b) {
    if (!b->pend_dn.valid) return true;
    b->pend_dn.valid = false;
    const int first = b->nl;
    if (!add_launch(b, b->pend_dn.fname, b->pend_dn.grid, 64 * QW_WAVES_DNR, &b->pend_dn.a, sizeof b->pend_dn.a)) return false;
    if (b->nl > first) b->l[b->nl - 1].kname = b->pend_dn.kname, b->l[b->nl - 1].last_of_dispatch = true;
    return true;
}

// The fused down + combine launch (qwk_dnq_*) shares the tokens over two quarters up to 8 tokens and over four up to 16:
// every quarter has four tokens at most, and with one tile of rows per workgroup for two quarters and two tiles for four
// the launch has D / 8 workgroups either way.
static unsigned dnq_quarters(unsigned nbr) { return nbr <= 8 ? 2 : 4; }

// src/engine.c:633-639: 0 Wd, 2 H, 3 sel, 7 tables, 9 Pg. The token count is not bound: the masks carry it.
// The shared down tiles (remembered from moe_gu_gg) run in the same launch.
static bool tr_dn_inner(qw_batch *b);
static bool tr_dn(qw_batch *b) {
    const int first = b->nl;
    if (!tr_dn_inner(b)) return false;
    if (!b->pend_gu.valid) return true;
    // a gate/up launch waits: it stays only if this dispatch became a down + combine by token shares over its H and record
    const qwk_gu_args *gu = &b->pend_gu.a;
    const qwk_dn_args *d = &b->pend_dn.a;
    if (b->pend_dn.valid && b->pend_dn.quarters && b->nl == first && d->H == gu->H && d->sel == gu->sel && d->D == gu->D && d->I == gu->I && d->topk == gu->topk && d->gnb == gu->gnb &&
        d->hplane == gu->hplane) return true;
    // otherwise it goes in front of what this dispatch launched
    const int n = b->nl - first;
    if (!flush_gu(b)) return false;
    if (n > 0 && b->nl == first + n + 1) {
        const qw_launch gl = b->l[b->nl - 1];
        memmove(&b->l[first + 1], &b->l[first], sizeof(qw_launch) * (size_t)n);
        b->l[first] = gl;
        b->l[first].last_of_dispatch = true;
    }
    return true;
}
static bool tr_dn_inner(qw_batch *b) {
    const qw_kparams *p = &b->k->p;
    const uint32_t nbr = (uint32_t)p->NB;
    const size_t rb = fmt_rb(p->fd, p->I);
    qwk_dn_args a = {.D = (uint32_t)p->D, .I = (uint32_t)p->I, .rowbytes = (uint32_t)rb, .nbr = nbr, .topk = (uint32_t)p->topk, .gnb = (uint32_t)p->gnb, .shared = 0,
                     .hplane = (uint32_t)p->NB * (uint32_t)(p->topk + 1) * (uint32_t)p->I, .glut = glut(b->g)};
    b->allow_released = true; // Wd may be a buffer of which only the tile-major copy is left
    const bool bound = bind_ptr(b, 0, (size_t)p->E * p->D * rb, false, "down weights", (void **)&a.Wd);
    b->allow_released = false;
    const bool rel = bound && b->buf[0].h->released;
    if (!bound || !bind_ptr(b, 2, (size_t)a.hplane * 4, false, "H", (void **)&a.H) ||
        !bind_ptr(b, 9, (size_t)nbr * p->topk * p->D * 4, true, "Pg", (void **)&a.P) ||
        !bind_ptr(b, 3, QW_SEL_BYTES((size_t)p->gnb, (size_t)p->topk), false, "selection", (void **)&a.sel)) return false;
    int fs = 0;
    qw_hbuf *hsd = NULL;
    if (b->pend_sd.valid) {
        hsd = b->pend_sd.hd;
        fs = b->pend_sd.fmt;
        a.Wsd = b->pend_sd.Wsd;
        a.Psh = b->pend_sd.Psh;
        a.sd_rowbytes = b->pend_sd.rowbytes;
        a.snbr = b->pend_sd.nbr;
        b->pend_sd.valid = false;
    }
    const unsigned umax = umin((unsigned)p->E, nbr * (unsigned)p->topk);
    int fd = p->fd;
    // A pair of types without a build of its own (Q4_K, Q5_K, Q6_K or IQ4_XS on either side; IQ4_NL beside IQ3_S): the
    // kernel that takes both types as arguments, rows in GGUF order.
    const bool kq_d = rt_ok(fd) && fd != 20, kq_s = rt_ok(fs) && fs != 20;
    if (kq_d || kq_s || ((fd == 20 || fs == 20) && (fd != 20 || (fs != 0 && fs != 20 && fs != 8)))) {
        if (rel) return fail(b, "%s: the GGUF-order bytes of the weights were released and no tile-major copy serves this dispatch", b->k->name);
        a.fd = (uint32_t)fd, a.fsd = (uint32_t)fs;
        return add_launch(b, "qwk_dn_rt", persistent_grid(b->g, umax * (unsigned)(p->D / 16) + (unsigned)p->D / 16, QW_WAVES_DN), 64 * QW_WAVES_DN, &a, sizeof a);
    }
    if (fd == 21 && p->I <= 512) {
        const uint32_t nblk = (uint32_t)p->I / 256, tileb = nblk * QW_SLAB_BYTES;
        const uint8_t *pk = get_pack(b, b->buf[0].h, a.Wd, NULL, NULL, (uint64_t)p->E * (uint64_t)(p->D / 16), nblk, a.rowbytes, 16);
        const uint8_t *ps = pk && fs == 21 ? get_pack(b, hsd, a.Wsd, NULL, NULL, (uint64_t)(p->D / 16), nblk, a.sd_rowbytes, 16) : NULL;
        if (pk && (fs != 21 || ps)) {
            fd = QW_F_PACKED;
            a.Wd = pk, a.rowbytes = tileb;
            if (fs == 21) fs = QW_F_PACKED, a.Wsd = ps, a.sd_rowbytes = tileb;
        }
    }
    if (rel && fd != QW_F_PACKED && fd != 20) return fail(b, "%s: the GGUF-order bytes of the weights were released and no tile-major copy serves this dispatch", b->k->name);
    char fn[48], sfx[16] = "";
    if (fs) fname_fmt(sfx, sizeof sfx, "_s%d", fs);
    // (IQ4_NL routed rows from here on have no shared expert beside them, or one in IQ4_NL or Q8_0)
    if (fd == 20 && p->I <= 640 && !b->sw.dn_any) { // the range kernel with rows of up to 640 staged
        if (p->I % 320 == 0) { // tile-major copies, as for IQ3_S rows (the shared expert's only together with the routed ones)
            const uint32_t nch = (uint32_t)p->I / 320, tileb = nch * QW_NL_CHUNK_BYTES;
            const uint8_t *pk = get_pack(b, b->buf[0].h, a.Wd, NULL, NULL, (uint64_t)p->E * (uint64_t)(p->D / 16), nch, a.rowbytes, QW_F_PACKED_NL);
            const uint8_t *ps = pk && fs == 20 ? get_pack(b, hsd, a.Wsd, NULL, NULL, (uint64_t)(p->D / 16), nch, a.sd_rowbytes, QW_F_PACKED_NL) : NULL;
            if (pk && (fs != 20 || ps)) {
                a.Wd = pk, a.rowbytes = tileb;
                if (fs == 20) a.Wsd = ps, a.sd_rowbytes = tileb;
                char tail[24] = "";
                if (fs) fname_fmt(tail, sizeof tail, "_s%d_c%d", fs == 20 ? QW_F_PACKED_NL : fs, fs == 20 ? 10 : 4);
                fname_fmt(fn, sizeof fn, "qwk_dnr_f120_c10%s", tail);
                const unsigned grid = persistent_grid(b->g, umax * (unsigned)(p->D / 16) + (unsigned)p->D / 16, QW_WAVES_DNR);
                if (nbr <= b->sw.dnc_nb) { // a few tokens: wait for the combine, the two run as one launch
                    char fu[48];
                    fname_fmt(fu, sizeof fu, "qwk_dnc_f120_c10%s", tail);
                    b->pend_dn.valid = true;
                    b->pend_dn.a = a;
                    b->pend_dn.fname = intern(fn), b->pend_dn.fused = intern(fu), b->pend_dn.kname = b->k->name, b->pend_dn.grid = grid, b->pend_dn.fused_grid = (unsigned)p->D / 16, b->pend_dn.quarters = false;
                    return true;
                }
                return add_launch(b, intern(fn), grid, 64 * QW_WAVES_DNR, &a, sizeof a);
            }
        }
        if (rel) return fail(b, "%s: the GGUF-order bytes of the weights were released and no tile-major copy serves this dispatch", b->k->name);
        const int ch = p->I % 320 == 0 && !b->sw.nl_c4 ? 10 : 4; // blocks per chunk
        if (fs) fname_fmt(fn, sizeof fn, "qwk_dnr_f20_c%d_s%d_c%d", ch, fs, fs == 20 ? ch : 4);
        else fname_fmt(fn, sizeof fn, "qwk_dnr_f20_c%d", ch);
        return add_launch(b, intern(fn), persistent_grid(b->g, umax * (unsigned)(p->D / 16) + (unsigned)p->D / 16, QW_WAVES_DNR), 64 * QW_WAVES_DNR, &a, sizeof a);
    }
    if (fd != 20 && p->I <= 512 && p->I % 256 == 0) { // contiguous task ranges per workgroup, operand A staged in LDS
        const int ch = fd == 8 ? 4 : p->I / 256;
        if (fs) fname_fmt(fn, sizeof fn, "qwk_dnr_f%d_c%d_s%d_c%d", fd, ch, fs, fs == 8 ? 4 : p->I / 256);
        else fname_fmt(fn, sizeof fn, "qwk_dnr_f%d_c%d", fd, ch);
        const unsigned grid = persistent_grid(b->g, umax * (unsigned)(p->D / 16) + (unsigned)p->D / 16, QW_WAVES_DNR);
        // Down + combine as one launch in which a workgroup owns one or two tiles of output rows and a share of the
        // tokens (qwk_dnq_*): for tile-major IQ3_S rows when a share's H rows fit in LDS beside the table.
        const unsigned tpe = (unsigned)p->D / 16, nq = dnq_quarters(nbr), tpw = nq > 2 ? 2 : 1;
        // (a gate/up launch that waits to be joined asks for this form at any token count)
        const bool by_shares = (b->pend_gu.valid || (b->sw.dnq_min && nbr >= b->sw.dnq_min)) && nbr <= 16 && fd == QW_F_PACKED && (fs == 0 || fs == 8 || fs == QW_F_PACKED) && p->topk <= 10 &&
                               p->gnb * p->topk <= (int)QW_DNQ_MAXU && tpe % 16 == 0;
        // a few tokens: wait for the combine, the two run as one launch (tile-major IQ3_S or Q8_0 routed rows; a shared
        // expert in either of these)
        if (!by_shares && nbr <= b->sw.dnc_nb && (fd == QW_F_PACKED || fd == 8) && (fs == 0 || fs == 8 || (fs == QW_F_PACKED && fd == QW_F_PACKED))) {
            char fu[48];
            if (fs) fname_fmt(fu, sizeof fu, "qwk_dnc_f%d_c%d_s%d_c%d", fd, ch, fs, fs == 8 ? 4 : p->I / 256);
            else fname_fmt(fu, sizeof fu, "qwk_dnc_f%d_c%d", fd, ch);
            b->pend_dn.valid = true;
            b->pend_dn.a = a;
            b->pend_dn.fname = intern(fn), b->pend_dn.fused = intern(fu), b->pend_dn.kname = b->k->name, b->pend_dn.grid = grid, b->pend_dn.fused_grid = (unsigned)p->D / 16, b->pend_dn.quarters = false;
            return true;
        }
        if (by_shares) { // waits for the combine too
            char fu[48];
            if (fs) fname_fmt(fu, sizeof fu, "qwk_dnq_f%d_c%d_s%d_c%d", fd, ch, fs, fs == 8 ? 4 : p->I / 256);
            else fname_fmt(fu, sizeof fu, "qwk_dnq_f%d_c%d", fd, ch);
            a.nq = nq, a.tpw = tpw;
            b->pend_dn.valid = true;
            b->pend_dn.a = a;
            b->pend_dn.fname = intern(fn), b->pend_dn.fused = intern(fu), b->pend_dn.kname = b->k->name, b->pend_dn.grid = grid, b->pend_dn.fused_grid = tpe / tpw * nq, b->pend_dn.quarters = true;
            return true;
        }
        return add_launch(b, intern(fn), grid, 64 * QW_WAVES_DNR, &a, sizeof a);
    }
    // wider rows: one tile at a time, operand A from global memory
    fname_fmt(fn, sizeof fn, "qwk_dn_f%d_any%s", p->fd, sfx);
    if (rel && fd != QW_F_PACKED) return fail(b, "%s: the GGUF-order bytes of the weights were released and no tile-major copy serves this dispatch", b->k->name);
    return add_launch(b, intern(fn), persistent_grid(b->g, umax * (unsigned)(p->D / 16) + (unsigned)p->D / 16, QW_WAVES_DN), 64 * QW_WAVES_DN, &a, sizeof a);
}

// src/engine.c:640-646: 1 Psh, 3 sel, 4 out, 8 nbr, 9 Pg
static bool tr_cmb(qw_batch *b) {
    const qw_kparams *p = &b->k->p;
    uint32_t nbr;
    if (!bind_bytes(b, 8, &nbr, 4, "nbr") || !nbr_ok(b, nbr)) return false;
    qwk_cmb_args a = {.D = (uint32_t)p->D, .nbr = nbr, .topk = (uint32_t)p->topk, .gnb = (uint32_t)p->gnb};
    if (!bind_ptr(b, 9, (size_t)nbr * p->topk * p->D * 4, false, "Pg", (void **)&a.Pg) || !bind_ptr(b, 1, (size_t)nbr * p->D * 4, false, "Psh", (void **)&a.Psh) ||
        !bind_ptr(b, 3, QW_SEL_BYTES((size_t)p->gnb, (size_t)p->topk), false, "selection", (void **)&a.sel) || !bind_ptr(b, 4, (size_t)nbr * p->D * 2, true, "out", (void **)&a.out)) return false;
    if (b->pend_dn.valid) {
        qwk_dn_args *d = &b->pend_dn.a;
        // the down dispatch counts tokens by its compiled NB, the combine by the bound count: the masks carry the rest
        const bool same = d->P == a.Pg && d->sel == a.sel && d->nbr >= nbr && d->D == a.D && d->topk == a.topk && d->gnb == a.gnb && (!d->Wsd || (d->Psh == a.Psh && d->snbr >= nbr));
        if (same) {
            b->pend_dn.valid = false;
            d->nbr = nbr;
            d->out = a.out;
            d->Psh = (float *)a.Psh;
            if (b->pend_gu.valid && b->pend_dn.quarters && b->pend_gu.a.nbr == nbr && (!d->Wsd || d->snbr == nbr)) { // gate/up, down and combine as one launch
                unsigned nq, tpw;
                gud_shape(nbr, &nq, &tpw);
                const unsigned grid = (unsigned)b->g->ncu, tpe = a.D / 16;
                if (tpe % (8 * tpw) == 0 && tpe / tpw * nq <= grid && grid % 8 == 0) {
                    b->pend_gu.valid = false;
                    qwk_gud_args f = {.gu = b->pend_gu.a, .dn = *d, .sync = b->g->sync, .spin_limit = b->sw.spin_limit};
                    f.dn.nq = nq, f.dn.tpw = tpw;
                    char fu[48];
                    fname_fmt(fu, sizeof fu, "qwk_gud%s", b->pend_dn.fused + 7); // the same formats as the qwk_dnq_* launch
                    b->uses_sync = true;
                    return add_launch(b, intern(fu), grid, 64 * QW_WAVES_GU, &f, sizeof f);
                }
            }
            if (!flush_gu(b)) return false;
            if (b->pend_dn.quarters) { // the quarters and the tiles per workgroup follow the bound token count, not the compiled one
                d->nq = dnq_quarters(nbr), d->tpw = d->nq > 2 ? 2 : 1;
                b->pend_dn.fused_grid = a.D / 16 / d->tpw * d->nq;
            }
            return add_launch(b, b->pend_dn.fused, b->pend_dn.fused_grid, 64 * QW_WAVES_DNR, d, sizeof *d);
        }
        if (!flush_gu(b) || !flush_dn(b)) return false;
    }
    if (!flush_gu(b)) return false;
    return add_launch(b, "qwk_cmb", cdiv(nbr * (unsigned)p->D, 256), 256, &a, sizeof a);
}

// ---------------------------------------------------------------- ragged packing (kernels/moe_prefill.metal; src/engine.c:4133-4224)
// The sequence p_zero (the counters), moe_count, moe_plan(_t), moe_scatter of a step with at most QW_PREP_MAXP pairs runs as
// one launch (qwk_moe_prep): each of the first three dispatches waits for the next one as long as it continues the
// sequence on the same buffers; anything else launches what waits, one kernel per dispatch (QW_HIP_PK_SPLIT: always).
static bool add_named(qw_batch *b, const char *kname, const char *fname, unsigned gx, unsigned bx, const void *args, size_t argsz) {
    const int first = b->nl;
    if (!add_launch(b, fname, gx, bx, args, argsz)) return false;
    if (b->nl > first) b->l[b->nl - 1].kname = kname, b->l[b->nl - 1].last_of_dispatch = true;
    return true;
}
static bool flush_pk(qw_batch *b) {
    const int st = b->pend_pk.stage;
    b->pend_pk.stage = 0;
    if (st >= 1 && !add_named(b, b->pend_pk.kn[0], "qwk_zero", cdiv(b->pend_pk.z.n, 256), 256, &b->pend_pk.z, sizeof b->pend_pk.z)) return false;
    if (st >= 2 && !add_named(b, b->pend_pk.kn[1], "qwk_moe_count", cdiv(b->pend_pk.c.P, 256), 256, &b->pend_pk.c, sizeof b->pend_pk.c)) return false;
    if (st >= 3 && !add_named(b, b->pend_pk.kn[2], "qwk_moe_plan", 1, 1024, &b->pend_pk.pl, sizeof b->pend_pk.pl)) return false;
    return true;
}
static bool tr_pk_count(qw_batch *b) { // 0 ids, 1 counts, 2 P
    qwk_count_args a = {.E = (uint32_t)b->k->p.E};
    if (!bind_bytes(b, 2, &a.P, 4, "P") || !bind_ptr(b, 0, (size_t)a.P * 4, false, "ids", (void **)&a.ids) || !bind_ptr(b, 1, (size_t)a.E * 4, true, "counts", (void **)&a.counts)) return false;
    if (b->pend_pk.stage == 1 && b->pend_pk.z.x == a.counts && b->pend_pk.z.n == a.E && a.E <= 1024 && a.P <= QW_PREP_MAXP) {
        b->pend_pk.stage = 2, b->pend_pk.c = a, b->pend_pk.kn[1] = b->k->name;
        return true;
    }
    if (!flush_pk(b)) return false;
    return add_launch(b, "qwk_moe_count", cdiv(a.P, 256), 256, &a, sizeof a);
}
static bool tr_pk_zero(qw_batch *b) { // kernels/prefill.metal:601-603: 0 x, 1 n (dwords to clear)
    qwk_zero_args a = {0};
    if (!bind_bytes(b, 1, &a.n, 4, "n") || !bind_ptr(b, 0, (size_t)a.n * 4, true, "x", (void **)&a.x)) return false;
    if (!flush_pk(b)) return false;
    if (!b->sw.pk_split) {
        b->pend_pk.stage = 1, b->pend_pk.z = a, b->pend_pk.kn[0] = b->k->name;
        return true;
    }
    return add_launch(b, "qwk_zero", cdiv(a.n, 256), 256, &a, sizeof a);
}
static bool tr_pk_plan(qw_batch *b, bool tm_bound) { // 0 counts, 1 offs, 2 cursor, 3 tiles, 4 max_tiles (, 5 tm)
    const qw_kparams *p = &b->k->p;
    qwk_plan_args a = {.E = (uint32_t)p->E, .tm = (uint32_t)p->tm};
    if (!bind_bytes(b, 4, &a.max_tiles, 4, "max_tiles") || (tm_bound && !bind_bytes(b, 5, &a.tm, 4, "tm"))) return false;
    if (a.tm < 1) return fail(b, "%s: tm 0", b->k->name);
    if (!bind_ptr(b, 0, (size_t)a.E * 4, false, "counts", (void **)&a.counts) || !bind_ptr(b, 1, (size_t)a.E * 4, true, "offs", (void **)&a.offs) ||
        !bind_ptr(b, 2, (size_t)a.E * 4, true, "cursor", (void **)&a.cursor) || !bind_ptr(b, 3, (size_t)a.max_tiles * 16, true, "tiles", (void **)&a.tiles)) return false;
    if (b->buf[3].off % 16) return fail(b, "%s: tile table offset %zu is not 16-byte aligned", b->k->name, b->buf[3].off);
    if (b->pend_pk.stage == 2 && b->pend_pk.c.counts == a.counts && b->pend_pk.c.E == a.E) {
        b->pend_pk.stage = 3, b->pend_pk.pl = a, b->pend_pk.kn[2] = b->k->name;
        return true;
    }
    if (!flush_pk(b)) return false;
    return add_launch(b, "qwk_moe_plan", 1, 1024, &a, sizeof a);
}
static bool tr_pk_scatter(qw_batch *b, unsigned gx) { // 0 X, 1 ids, 2 cursor, 3 Xs, 4 pos_of; grid x = P
    const qw_kparams *p = &b->k->p;
    qwk_scatter_args a = {.KD = (uint32_t)p->K, .topk = (uint32_t)p->topk, .E = (uint32_t)p->E, .P = gx};
    if (gx % (unsigned)p->topk) return fail(b, "moe_scatter: %u pairs is not a multiple of TOPK %d", gx, p->topk);
    if (!bind_ptr(b, 0, (size_t)(gx / p->topk) * p->K * 2, false, "X", (void **)&a.X) || !bind_ptr(b, 1, (size_t)gx * 4, false, "ids", (void **)&a.ids) ||
        !bind_ptr(b, 2, (size_t)p->E * 4, true, "cursor", (void **)&a.cursor) || !bind_ptr(b, 3, (size_t)gx * p->K * 2, true, "Xs", (void **)&a.Xs) ||
        !bind_ptr(b, 4, (size_t)gx * 4, true, "pos_of", (void **)&a.pos_of)) return false;
    if (b->buf[0].off % 16 || b->buf[3].off % 16) return fail(b, "moe_scatter: row buffers must be 16-byte aligned");
    if (b->pend_pk.stage == 3 && b->pend_pk.pl.cursor == a.cursor && b->pend_pk.c.ids == a.ids && b->pend_pk.c.P == a.P && b->pend_pk.c.E == a.E && a.KD % 8 == 0) {
        const qwk_plan_args *pl = &b->pend_pk.pl;
        const qwk_prep_args f = {.ids = a.ids, .counts = b->pend_pk.c.counts, .offs = pl->offs, .cursor = pl->cursor, .tiles = pl->tiles, .pos_of = a.pos_of, .X = a.X, .Xs = a.Xs,
                                 .P = a.P, .E = a.E, .topk = a.topk, .KD = a.KD, .tm = pl->tm, .max_tiles = pl->max_tiles};
        b->pend_pk.stage = 0;
        return add_launch(b, "qwk_moe_prep", a.P, 256, &f, sizeof f);
    }
    if (!flush_pk(b)) return false;
    return add_launch(b, "qwk_moe_scatter", gx, 256, &a, sizeof a);
}
static bool tr_pk_act(qw_batch *b) { // 0 G [P][2 I], 1 H [P][I], 2 P
    const qw_kparams *p = &b->k->p;
    qwk_act_args a = {.I = (uint32_t)p->I};
    if (!bind_bytes(b, 2, &a.P, 4, "P")) return false;
    a.n = a.P * a.I;
    if (!bind_ptr(b, 0, (size_t)a.n * 4, false, "G", (void **)&a.G) || !bind_ptr(b, 1, (size_t)a.n * 2, true, "H", (void **)&a.H)) return false;
    return add_launch(b, "qwk_moe_act", cdiv(a.n, 256), 256, &a, sizeof a);
}
static bool flush_tw(qw_batch *b, uint16_t *H, bool *acted);
static bool tr_pk_act2(qw_batch *b) { // kernels/prefill.metal:485-488: 0 G, 1 U, 2 H, 3 n
    qwk_act_args a = {0};
    if (!bind_bytes(b, 3, &a.n, 4, "n")) return false;
    if (!bind_ptr(b, 0, (size_t)a.n * 2, false, "G", (void **)&a.G) || !bind_ptr(b, 1, (size_t)a.n * 2, false, "U", (void **)&a.U) || !bind_ptr(b, 2, (size_t)a.n * 2, true, "H", (void **)&a.H)) return false;
    if (b->pend_tw.valid) { // SwiGLU of exactly what the waiting gate / up launch writes: it rides at that launch's end
        const qwk_pf_args *f = &b->pend_tw.f;
        const bool rides = !b->sw.pk_split && f->Y == a.G && f->Y1 == a.U && (uint64_t)f->M * f->N == a.n && a.H != f->Y && a.H != f->Y1 && (const uint16_t *)a.H != f->X;
        bool acted = false;
        if (!flush_tw(b, rides ? a.H : NULL, &acted)) return false;
        if (acted) return true;
    }
    return add_launch(b, "qwk_moe_act", cdiv(a.n, 256), 256, &a, sizeof a);
}
static bool tr_pk_combine(qw_batch *b, unsigned gy) { // 0 D, 1 pos_of, 2 w, 3 Y; grid = (KD / 4 / 64, T)
    const qw_kparams *p = &b->k->p;
    qwk_combine_args a = {.KD = (uint32_t)p->K, .topk = (uint32_t)p->topk, .T = gy, .P = gy * (uint32_t)p->topk};
    if (!bind_ptr(b, 0, (size_t)a.P * p->K * 2, false, "D", (void **)&a.Dm) || !bind_ptr(b, 1, (size_t)a.P * 4, false, "pos_of", (void **)&a.pos_of) ||
        !bind_ptr(b, 2, (size_t)a.P * 4, false, "w", (void **)&a.w) || !bind_ptr(b, 3, (size_t)gy * p->K * 2, true, "Y", (void **)&a.Y)) return false;
    if (!add_launch(b, "qwk_moe_combine", cdiv((unsigned)p->K / 4, 64), 64, &a, sizeof a)) return false;
    if (gy) b->l[b->nl - 1].gy = gy;
    return true;
}
// src/engine.c:3257-3264: 0 X, 1 W, 4 Y, 5 {M, N}, 6 tiles, 7 tables; grid y = entries of the tile table
// One grouped-product launch. IQ3_S weights go through the tile-major copy when there is one: wb != NULL = the second
// matrix of a gate / up pair (tiles of 8 + 8 rows, outputs a->Y and a->Y1), else a single matrix (tiles of 16 rows).
static bool launch_pf(qw_batch *b, qwk_pf_args *a, int F, int E, qw_hbuf *hw, qw_hbuf *hwb, const uint8_t *wb) {
    a->split = 16, a->ntn = a->N / 16;
    if (!wb) a->H = NULL, a->Y1 = NULL; // SwiGLU rides only in a launch that holds both matrices
    char fn[32];
    if (F == 21 && a->K % 256 == 0) {
        const uint32_t nblk = a->K / 256, split = wb ? 8 : 16;
        const uint64_t ntiles = (uint64_t)E * (a->N / split);
        const uint8_t *pk = get_pack(b, hw, a->W, wb ? hwb : NULL, wb, ntiles, nblk, a->rowbytes, split);
        if (pk) {
            a->W = pk, a->rowbytes = nblk * QW_SLAB_BYTES, a->split = split, a->ntn = a->N / split;
            if (a->tm <= 16 && a->K <= 2560) { // entries of one group of rows: the rows are staged in LDS per workgroup range
                fname_fmt(fn, sizeof fn, "qwk_pfr_f121_c%d", a->K % 512 == 0 ? 2 : 1);
                return add_launch(b, intern(fn), umin((unsigned)b->g->ncu, a->max_tiles * a->ntn), 64 * QW_WAVES_GU, a, sizeof *a);
            }
            fname_fmt(fn, sizeof fn, "qwk_pf_f121_c%d", a->K % 512 == 0 ? 2 : 1);
            return add_launch(b, intern(fn), persistent_grid(b->g, a->max_tiles * a->ntn, 8), 512, a, sizeof *a);
        }
        if (wb) return false; // the caller launches the two matrices one by one
    }
    if (hw && hw->released) return fail(b, "%s: the GGUF-order bytes of the weights were released and no tile-major copy serves this dispatch", b->k->name);
    if (F == 21) fname_fmt(fn, sizeof fn, "qwk_pf_f21_c%d", a->K % 512 == 0 ? 2 : 1);
    else fname_fmt(fn, sizeof fn, "qwk_pf_f%d_c4", F == 20 ? 20 : 8);
    // every entry can hold a tile: the grid covers the whole table, the kernel counts the entries in use
    return add_launch(b, intern(fn), persistent_grid(b->g, a->max_tiles * a->ntn, 8), 512, a, sizeof *a);
}

static bool flush_pf(qw_batch *b) {
    if (!b->pend_pf.valid) return true;
    b->pend_pf.valid = false;
    return launch_pf(b, &b->pend_pf.a, 21, b->pend_pf.E, b->pend_pf.hw, NULL, NULL);
}
// The waiting gate / up pair: one launch over the tile-major copy of both (H: SwiGLU of the two results at its end, *acted
// tells whether it was done), or the two matrices one by one when there is no such copy (small buffers, copies switched off).
static bool flush_tw(qw_batch *b, uint16_t *H, bool *acted) {
    if (acted) *acted = false;
    if (!b->pend_tw.valid) return true;
    b->pend_tw.valid = false;
    const int first = b->nl;
    qwk_pf_args f = b->pend_tw.f;
    f.H = H;
    bool ok = launch_pf(b, &f, 21, b->pend_tw.E, b->pend_tw.hw, b->pend_tw.hwb, b->pend_tw.second.W);
    if (ok) {
        if (acted) *acted = H != NULL;
    } else {
        if (b->failed) return false;
        qwk_pf_args one = b->pend_tw.f, two = b->pend_tw.second;
        ok = launch_pf(b, &one, 21, b->pend_tw.E, b->pend_tw.hw, NULL, NULL) && launch_pf(b, &two, 21, b->pend_tw.E, b->pend_tw.hwb, NULL, NULL);
    }
    for (int i = first; ok && i < b->nl; i++) b->l[i].kname = b->pend_tw.kname;
    return ok;
}

static bool tr_pf(qw_batch *b, unsigned gy) {
    const qw_kparams *p = &b->k->p;
    uint32_t mn[2];
    if (!bind_bytes(b, 5, mn, sizeof mn, "{M, N}")) return false;
    if (mn[1] == 0 || mn[1] % 16) return fail(b, "moe_pf_gg: N %u is not a multiple of 16", mn[1]);
    if (gy > 2048) return fail(b, "moe_pf_gg: %u tile entries, this build takes at most 2048", gy);
    const size_t rb = fmt_rb(p->F, p->K);
    qwk_pf_args a = {.M = mn[0], .N = mn[1], .K = (uint32_t)p->K, .rowbytes = (uint32_t)rb, .max_tiles = gy, .tm = (uint32_t)p->tm, .glut = glut(b->g)};
    b->allow_released = true; // the weights may be a buffer of which only the tile-major copy is left (launch_pf checks that one serves)
    const bool bound = bind_ptr(b, 1, (size_t)p->E * a.N * rb, false, "weights", (void **)&a.W);
    b->allow_released = false;
    if (!bound || !bind_ptr(b, 0, (size_t)a.M * p->K * 2, false, "X", (void **)&a.X) ||
        !bind_ptr(b, 4, (size_t)a.M * a.N * 2, true, "Y", (void **)&a.Y) || !bind_ptr(b, 6, (size_t)gy * 16, false, "tiles", (void **)&a.tiles)) return false;
    if (b->buf[0].off % 16 || b->buf[6].off % 16) return fail(b, "moe_pf_gg: X and the tile table must be 16-byte aligned");
    qw_hbuf *hw = b->buf[1].h, *hx = b->buf[0].h, *hy = b->buf[4].h;
    if (b->pend_pf.valid) {
        // the twin of the waiting product: same packed rows, table and shape, other weights and output
        const qwk_pf_args *q = &b->pend_pf.a;
        const bool twin = p->F == 21 && q->X == a.X && q->tiles == a.tiles && q->M == a.M && q->N == a.N && q->K == a.K && q->max_tiles == a.max_tiles &&
                          q->W != a.W && q->Y != a.Y && b->pend_pf.E == p->E && hy != b->pend_pf.hx && b->pend_pf.hy != hx && b->pend_pf.hy != hy;
        if (twin) { // launched at the next dispatch (flush_tw): a p_act2 over the two results rides in the same launch
            b->pend_pf.valid = false;
            b->pend_tw.valid = true;
            b->pend_tw.f = *q, b->pend_tw.f.Y1 = a.Y, b->pend_tw.second = a;
            b->pend_tw.hw = b->pend_pf.hw, b->pend_tw.hwb = hw, b->pend_tw.E = p->E, b->pend_tw.kname = b->k->name;
            return true;
        }
        if (!flush_pf(b)) return false;
    }
    if (p->F == 21 && p->K % 256 == 0 && b->g->repack) { // may be the first of a pair: wait for the next dispatch
        b->pend_pf.valid = true;
        b->pend_pf.a = a;
        b->pend_pf.hw = hw, b->pend_pf.hx = hx, b->pend_pf.hy = hy, b->pend_pf.E = p->E;
        return true;
    }
    return launch_pf(b, &a, p->F, p->E, hw, NULL, NULL);
}

// helpers: 0 src, 1 dst, 2 {n16 (uint64), seed (uint64)}; grid x = workgroups of 256 threads
static bool tr_mem(qw_batch *b, unsigned gx) {
    uint64_t a2[2];
    if (!bind_bytes(b, 2, a2, sizeof a2, "{n, seed}")) return false;
    qwk_mem_args a = {.n = a2[0], .seed = a2[1]};
    const qw_family f = b->k->fam;
    if (f != FAM_FILL && !bind_ptr(b, 0, a.n * 16, false, "src", (void **)&a.src)) return false;
    if (!bind_ptr(b, 1, f == FAM_BW_READ ? 16 : a.n * 16, true, "dst", &a.dst)) return false;
    return add_launch(b, f == FAM_BW_READ ? "qwk_bw_read" : f == FAM_COPY ? "qwk_copy" : "qwk_fill_random", gx, 256, &a, sizeof a);
}

// Hyper-connection (src/engine.c:1344-1412). Bindings of ghc_down / ghc_dsk: 0 h, 1 out, 2 inj, 3 norm weights, 4 mix_down,
// 5 inject, 6 partial sums, 7 {apply, want inject}; ghc_up: 0 h, 1 out, 2 inj, 3 norm weights, 4 mix_up, 5 partial sums, 6 x,
// 7 new inject sums, 8 flags; ghc_mid: 0 partial sums, 1 sx, 2 rs, 3 new inject sums, 4 flags; ghc_upv: as ghc_up with 5 sx, 6 rs,
// 7 x, 8 flags. The caller's grids are the reference kernels' own; these launches have theirs.
static bool hc_aligned(qw_batch *b, const unsigned *idx, int n) {
    for (int i = 0; i < n; i++)
        if (b->buf[idx[i]].off % 16) return fail(b, "%s: the offset of binding %u must be a multiple of 16", b->k->name, idx[i]);
    return true;
}
static bool tr_hc(qw_batch *b) {
    const qw_kparams *p = &b->k->p;
    const qw_family f = b->k->fam;
    const size_t D = (size_t)p->D, nb = (size_t)p->NB, HCD = QW_HC * D;
    uint32_t fl[2];
    qwk_hc_args a = {.D = (uint32_t)p->D, .nb = (uint32_t)p->NB};
    if (!bind_bytes(b, f == FAM_HC_DOWN ? 7 : f == FAM_HC_MID ? 4 : 8, fl, sizeof fl, "{apply, want inject}")) return false;
    a.apply = fl[0] != 0, a.want_inj = fl[1] != 0;
    if (f == FAM_HC_MID) {
        static const unsigned al[] = {0, 1, 2, 3};
        if (!hc_aligned(b, al, 4)) return false;
        if (!bind_ptr(b, 0, nb * QW_HC * QW_HC_PDS * 4, false, "partial sums", (void **)&a.pd) || !bind_ptr(b, 1, nb * QW_HC_LR * 4, true, "sx", (void **)&a.sx) ||
            !bind_ptr(b, 2, nb * QW_HC * 4, true, "rs", (void **)&a.rs)) return false;
        if (a.want_inj && !bind_ptr(b, 3, nb * QW_HC * QW_HC * 4, true, "new inject sums", (void **)&a.injo)) return false;
        return add_launch(b, "qwk_hc_mid", (unsigned)nb, QW_HC_LR, &a, sizeof a);
    }
    static const unsigned al[] = {0, 1, 2, 3, 4, 5, 6, 7};
    if (!hc_aligned(b, al, f == FAM_HC_DOWN ? 7 : 8)) return false;
    // h is written back by the up kernels when the residual is applied; out is only read then (it may not exist yet otherwise)
    if (!bind_ptr(b, 0, nb * HCD * 4, a.apply && f != FAM_HC_DOWN, "h", (void **)&a.h) || !bind_ptr(b, 3, HCD * 4, false, "norm weights", (void **)&a.w)) return false;
    if (a.apply && (!bind_ptr(b, 1, nb * D * 2, false, "out", (void **)&a.out) || !bind_ptr(b, 2, nb * QW_HC * QW_HC * 4, false, "inject sums", (void **)&a.inj))) return false;
    if (f == FAM_HC_DOWN) {
        if (!bind_ptr(b, 4, QW_HC_LR * HCD * 2, false, "mix_down", (void **)&a.Wd) || !bind_ptr(b, 6, nb * QW_HC * QW_HC_PDS * 4, true, "partial sums", (void **)&a.pd)) return false;
        if (a.want_inj && !bind_ptr(b, 5, QW_HC * HCD * 2, false, "inject", (void **)&a.Wi)) return false;
        // rows per workgroup. Measured per launch at D = 2048 (4 / 8 / 16 rows): 6.2 / 6.5 / 7.9 us at one token, 10.0 / 11.7 /
        // 13.6 at eight, 12.5 / 12.3 / 14.1 at sixteen: many small workgroups beat fewer re-reads of h up to about a dozen tokens
        unsigned R = nb <= 12 ? 4 : 8;
        if (b->sw.hc_rows == 4 || b->sw.hc_rows == 8 || b->sw.hc_rows == 16) R = b->sw.hc_rows;
        if (!add_launch(b, R == 4 ? "qwk_hc_down_r4" : R == 8 ? "qwk_hc_down_r8" : "qwk_hc_down_r16", QW_HC_LR / R + (a.want_inj ? 1 : 0), (unsigned)(D / 8), &a, sizeof a)) return false;
        b->l[b->nl - 1].gy = QW_HC;
        b->l[b->nl - 1].gz = (unsigned)(nb + QW_HC_TG - 1) / QW_HC_TG; // tokens four at a time
        return true;
    }
    if (!bind_ptr(b, 4, HCD * QW_HC_LR * 2, false, "mix_up", (void **)&a.Wu)) return false;
    if (f == FAM_HC_UP) {
        if (!bind_ptr(b, 5, nb * QW_HC * QW_HC_PDS * 4, false, "partial sums", (void **)&a.pd) || !bind_ptr(b, 6, nb * D * 2, true, "x", (void **)&a.x)) return false;
        if (a.want_inj && !bind_ptr(b, 7, nb * QW_HC * QW_HC * 4, true, "new inject sums", (void **)&a.injo)) return false;
    } else if (!bind_ptr(b, 5, nb * QW_HC_LR * 4, false, "sx", (void **)&a.sx) || !bind_ptr(b, 6, nb * QW_HC * 4, false, "rs", (void **)&a.rs) ||
               !bind_ptr(b, 7, nb * D * 2, true, "x", (void **)&a.x)) return false;
    if (!add_launch(b, f == FAM_HC_UP ? "qwk_hc_up" : "qwk_hc_upv", (unsigned)(D / 8), 256, &a, sizeof a)) return false;
    b->l[b->nl - 1].gy = (unsigned)(nb + QW_HC_TG - 1) / QW_HC_TG; // tokens four at a time
    return true;
}

// bench/moe_bw.c:82-91, 106-112: 0 arena, 1 chunk records at the dispatch's first chunk, 2 sink; grid (slices or row groups, chunks)
static bool tr_bwpat(qw_batch *b, unsigned gx, unsigned gy, unsigned tx) {
    const qw_kparams *p = &b->k->p;
    const bool rows = b->k->fam == FAM_BW_ROWS;
    qwk_bwpat_args a = {.sl = (uint32_t)p->sl, .ld = (uint32_t)p->ld, .rb = (uint32_t)p->RB, .ub = (uint32_t)p->ub};
    if (rows) {
        if (p->RB <= 0 || p->ub < 2 || p->ub % 2 || tx != 256) return fail(b, "bw_rows: RB %d, UB %d (even, at least 2), %u threads (256)", p->RB, p->ub, tx);
    } else if (p->sl <= 0 || (p->ld != 1 && p->ld != 2 && p->ld != 4 && p->ld != 8) || tx == 0 || tx > 1024 || tx % 64)
        return fail(b, "bw_chunks: SL %d, LD %d (1, 2, 4 or 8), %u threads (a multiple of 64 up to 1024)", p->sl, p->ld, tx);
    if (gy == 0 || gy > 65535) return fail(b, "%s: %u chunks in one dispatch", b->k->name, gy);
    if (!b->buf[0].h) return fail(b, "%s: no arena bound at 0", b->k->name);
    if (b->buf[0].off > b->buf[0].h->size) return fail(b, "%s: arena offset past its end", b->k->name);
    const size_t avail = b->buf[0].h->size - b->buf[0].off;
    if (b->buf[0].off % 16 || !bind_ptr(b, 0, avail, false, "arena", (void **)&a.src)) return fail(b, "%s: arena binding", b->k->name);
    a.src_n = avail / 16;
    if (b->buf[1].off % 8 || !bind_ptr(b, 1, (size_t)gy * 8, false, "chunk records", (void **)&a.chunks)) return false;
    if (!bind_ptr(b, 2, 1024 * 4, true, "sink", (void **)&a.out)) return false;
    if (!add_launch(b, rows ? "qwk_bw_rows" : "qwk_bw_chunks", gx, tx, &a, sizeof a)) return false;
    if (gx) b->l[b->nl - 1].gy = gy;
    return true;
}

// synthetic weights: 1 dst (+ offset), 2 {nblocks (uint64), seed (uint64), type (uint32), sigma (float)}
static bool tr_fill_blocks(qw_batch *b) {
    struct { uint64_t nblocks, seed; uint32_t type; float sigma; } in;
    if (!bind_bytes(b, 2, &in, sizeof in, "{nblocks, seed, type, sigma}")) return false;
    if (!fmt_ok((int)in.type) && in.type != 20) return fail(b, "qw_fill_blocks: type %u", in.type);
    qwk_fill_args a = {.nblocks = in.nblocks, .seed = in.seed, .type = in.type, .sigma = in.sigma};
    if (!bind_ptr(b, 1, (size_t)in.nblocks * (size_t)fmt_bb((int)in.type), true, "dst", (void **)&a.dst)) return false;
    if (b->buf[1].off % 2) return fail(b, "qw_fill_blocks: odd offset");
    const uint64_t wg = (in.nblocks + 255) / 256;
    return add_launch(b, "qwk_fill_blocks", (unsigned)(wg < 65536 ? wg : 65536), 256, &a, sizeof a);
}

void qw_batch_dispatch(qw_batch *b, unsigned gx, unsigned gy, unsigned gz, unsigned tx, unsigned ty, unsigned tz) {
    (void)gz; (void)tx; (void)ty; (void)tz;
    if (b->failed) return;
    if (!b->k) { fail(b, "qw_batch_dispatch without a kernel"); return; }
    b->allow_released = false;
    const int first = b->nl;
    bool ok;
    if (b->k->fam != FAM_GU && b->k->fam != FAM_PRE && !flush_select(b)) return;
    if (b->k->fam != FAM_PK_ACT2 && !flush_tw(b, NULL, NULL)) return;
    if (b->k->fam != FAM_PF && !flush_pf(b)) return;
    // a gate/up launch waits for the down dispatch of its layer, a down launch for the combine; anything else sends them off
    if (b->k->fam != FAM_CMB && (b->k->fam != FAM_DN || b->pend_dn.valid) && (!flush_gu(b) || !flush_dn(b))) return;
    if (b->k->fam != FAM_PK_ZERO && b->k->fam != FAM_PK_COUNT && b->k->fam != FAM_PK_PLAN && b->k->fam != FAM_PK_PLAN_T && b->k->fam != FAM_PK_SCATTER && !flush_pk(b)) return;
    switch (b->k->fam) {
    case FAM_DQ_TEST: ok = tr_dq_test(b, gx); break;
    case FAM_QMV_GGM: ok = tr_qmvm(b); break;
    case FAM_QMV_GG: ok = tr_qmv(b); break;
    case FAM_ROUTER: ok = tr_router(b); break;
    case FAM_TAB_INIT: ok = tr_tab_init(b); break;
    case FAM_SEL: ok = tr_sel(b); break;
    case FAM_PRE: ok = tr_pre(b); break;
    case FAM_GU: ok = tr_gu(b); break;
    case FAM_DN: ok = tr_dn(b); break;
    case FAM_CMB: ok = tr_cmb(b); break;
    case FAM_FILL_BLOCKS: ok = tr_fill_blocks(b); break;
    case FAM_BW_CHUNKS: case FAM_BW_ROWS: ok = tr_bwpat(b, gx, gy, tx); break;
    case FAM_HC_DOWN: case FAM_HC_MID: case FAM_HC_UP: case FAM_HC_UPV: ok = tr_hc(b); break;
    case FAM_PK_ZERO: ok = tr_pk_zero(b); break;
    case FAM_PK_COUNT: ok = tr_pk_count(b); break;
    case FAM_PK_PLAN: ok = tr_pk_plan(b, false); break;
    case FAM_PK_PLAN_T: ok = tr_pk_plan(b, true); break;
    case FAM_PK_SCATTER: ok = tr_pk_scatter(b, gx); break;
    case FAM_PK_ACT: ok = tr_pk_act(b); break;
    case FAM_PK_ACT2: ok = tr_pk_act2(b); break;
    case FAM_PK_COMBINE: ok = tr_pk_combine(b, gy); break;
    case FAM_PF: ok = tr_pf(b, gy); break;
    default: ok = tr_mem(b, gx);
    }
    if (ok && b->nl > first) b->l[b->nl - 1].last_of_dispatch = true;
}

// ---------------------------------------------------------------- batches: submission
// The side stream of a stream (default priority, made at first use), and an ordering edge "to goes on after what from
// holds now" through an event of the pool.
static hipStream_t side_of(qw_gpu *g, int stream) {
    if (!g->side[stream] && hipStreamCreateWithFlags(&g->side[stream], hipStreamNonBlocking) != hipSuccess) g->side[stream] = NULL;
    return g->side[stream];
}
static bool side_link(qw_gpu *g, hipStream_t from, hipStream_t to) {
    if (!from || !to) { set_err(g, "no side stream"); return false; }
    hipEvent_t *e = &g->sev[g->nsev++ % 256];
    if (!*e && !HIPOK(g, hipEventCreateWithFlags(e, hipEventDisableTiming))) return false;
    return HIPOK(g, hipEventRecord(*e, from)) && HIPOK(g, hipStreamWaitEvent(to, *e, 0));
}

// A batch's launches as a HIP graph. The key of a sequence is every launch's function, grid and argument record;
// it is replayed only after an exact comparison. Returns 1 when the sequence ran as a graph, 0 when the caller should
// launch it eagerly, -1 on an error. Graphs hold kernel nodes only (no copies, no memsets).
static size_t graph_key(const qw_batch *b, unsigned char *out) {
    size_t n = 0;
    for (int i = 0; i < b->nl; i++) {
        const qw_launch *l = &b->l[i];
        const unsigned hdr[4] = {l->gx, l->bx, (unsigned)l->argsz, 0};
        if (out) { memcpy(out + n, &l->f, sizeof l->f); memcpy(out + n + sizeof l->f, hdr, sizeof hdr); memcpy(out + n + sizeof l->f + sizeof hdr, l->args, l->argsz); }
        n += sizeof l->f + sizeof hdr + l->argsz;
    }
    return n;
}
static int graph_run(qw_batch *b, hipStream_t st) {
    qw_gpu *g = b->g;
    if (!g->use_graphs || b->prof || b->done_l != 0 || b->nl < 8) return 0;
    for (int i = 0; i < b->nl; i++)
        if (b->l[i].side) return 0;
    const size_t bytes = graph_key(b, NULL);
    unsigned char *key = malloc(bytes);
    if (!key) return 0;
    graph_key(b, key);
    uint64_t h = 1469598103934665603ull; // FNV-1a
    for (size_t i = 0; i < bytes; i++) h = (h ^ key[i]) * 1099511628211ull;
    for (int i = 0; i < 8; i++) {
        struct qw_graph *c = &g->graphs[i];
        if (c->exec && c->hash == h && c->nl == b->nl && c->bytes == bytes && !memcmp(c->key, key, bytes)) {
            free(key);
            g->ngraph_launches++;
            return HIPOK(g, hipGraphLaunch(c->exec, st)) ? 1 : -1;
        }
    }
    bool seen = false;
    for (int i = 0; i < 8; i++) seen = seen || g->seen_hash[i] == h;
    if (!seen) { // first time: eagerly, and remembered
        g->seen_hash[g->nseen++ % 8] = h;
        free(key);
        return 0;
    }
    hipGraph_t graph = NULL;
    hipGraphExec_t exec = NULL;
    if (hipStreamBeginCapture(st, hipStreamCaptureModeRelaxed) != hipSuccess) { (void)hipGetLastError(); free(key); return 0; }
    bool ok = true;
    for (int i = 0; i < b->nl && ok; i++) {
        qw_launch *l = &b->l[i];
        void *params[] = {l->args};
        ok = hipModuleLaunchKernel(l->f, l->gx, l->gy, l->gz, l->bx, 1, 1, 0, st, params, NULL) == hipSuccess;
    }
    if (hipStreamEndCapture(st, &graph) != hipSuccess || !ok || !graph || hipGraphInstantiate(&exec, graph, NULL, NULL, 0) != hipSuccess) {
        (void)hipGetLastError();
        if (graph) (void)hipGraphDestroy(graph);
        free(key);
        g->use_graphs = false; // this runtime does not capture these launches: stay eager
        return 0;
    }
    (void)hipGraphDestroy(graph);
    struct qw_graph *c = &g->graphs[g->ngraph_next++ % 8];
    if (c->exec) (void)hipGraphExecDestroy(c->exec);
    free(c->key);
    *c = (struct qw_graph){.hash = h, .nl = b->nl, .bytes = bytes, .key = key, .exec = exec};
    g->ngraph_launches++;
    return HIPOK(g, hipGraphLaunch(exec, st)) ? 1 : -1;
}

static bool submit_segment(qw_batch *b) {
    qw_gpu *g = b->g;
    hipStream_t st = g->stream[b->stream];
    if (b->failed || !flush_select(b) || !flush_tw(b, NULL, NULL) || !flush_pf(b) || !flush_gu(b) || !flush_dn(b) || !flush_pk(b)) return false;
    if (b->nseg >= 9) return fail(b, "too many flushes in one batch");
    // host -> device for what this segment binds
    const unsigned mark = ++g->mark;
    for (int i = b->done_use; i < b->nuse; i++) {
        qw_hbuf *h = b->use[i].b;
        if (h->mark == mark) continue;
        h->mark = mark;
        if (h->device_only || !h->host) continue;
        // A kernel of a batch that was submitted (or of an earlier segment of this one) and not yet waited for wrote
        // this buffer: HBM holds the newer contents, and the shadow must not overwrite them.
        if (h->released) continue; // no device bytes: its tile-major copies are what the kernels read
        if (h->pending_out > 0 && !h->dirty) continue;
        if (h->dirty || (!h->wrapped && h->size <= QW_HIP_SMALL_BYTES)) {
            if (!HIPOK(g, hipMemcpyAsync(h->dptr, h->host, h->size, hipMemcpyHostToDevice, st))) { b->failed = true; return false; }
            h->dirty = false;
        }
    }
    for (int i = b->done_use; i < b->nuse; i++) { // outputs of this segment: the device side is the newer one until the batch is waited for
        qw_hbuf *h = b->use[i].b;
        if (!b->use[i].out || h->device_only || !h->host || h->wrapped || h->out_seq == b->seq) continue;
        if (b->nouts == b->capouts) {
            b->capouts = b->capouts ? 2 * b->capouts : 16;
            b->outs = realloc(b->outs, sizeof *b->outs * (size_t)b->capouts);
        }
        h->out_seq = b->seq;
        h->pending_out++;
        b->outs[b->nouts++] = h;
    }
    hipEvent_t *ev = &b->ev[2 * b->nseg];
    if (!HIPOK(g, hipEventCreate(&ev[0])) || !HIPOK(g, hipEventCreate(&ev[1]))) { b->failed = true; return false; }
    b->nseg++;
    if (!HIPOK(g, hipEventRecord(ev[0], st))) { b->failed = true; return false; }
    const int as_graph = graph_run(b, st);
    if (as_graph < 0) { b->failed = true; return false; }
    bool side_open = false;
    for (int i = as_graph ? b->nl : b->done_l; i < b->nl; i++) {
        qw_launch *l = &b->l[i];
        if (l->side && !b->prof) { // fork: the side stream starts from where the main stream stands now
            if (!side_open && !(side_open = side_link(g, st, side_of(g, b->stream)))) { b->failed = true; return false; }
            void *sparams[] = {l->args};
            if (!HIPOK(g, hipModuleLaunchKernel(l->f, l->gx, l->gy, l->gz, l->bx, 1, 1, 0, g->side[b->stream], sparams, NULL))) { b->failed = true; return false; }
            continue;
        }
        if (l->join && side_open) { // join: the main stream goes on once the side stream has finished
            side_open = false;
            if (!side_link(g, g->side[b->stream], st)) { b->failed = true; return false; }
        }
        if (b->prof) { // an event pair brackets every launch
            b->pev = realloc(b->pev, sizeof *b->pev * (size_t)(b->npev + 2));
            if (!HIPOK(g, hipEventCreate(&b->pev[b->npev])) || !HIPOK(g, hipEventCreate(&b->pev[b->npev + 1])) || !HIPOK(g, hipEventRecord(b->pev[b->npev], st))) { b->failed = true; return false; }
        }
        void *params[] = {l->args}; // every kernel takes one record by value
        if (!HIPOK(g, hipModuleLaunchKernel(l->f, l->gx, l->gy, l->gz, l->bx, 1, 1, 0, st, params, NULL))) { b->failed = true; return false; }
        if (b->prof) {
            if (!HIPOK(g, hipEventRecord(b->pev[b->npev + 1], st))) { b->failed = true; return false; }
            b->npev += 2;
        }
    }
    if (side_open && !side_link(g, g->side[b->stream], st)) { b->failed = true; return false; }
    if (!HIPOK(g, hipEventRecord(ev[1], st))) { b->failed = true; return false; }
    b->done_l = b->nl;
    b->done_use = b->nuse;
    return true;
}

void qw_batch_flush(qw_batch *b) {
    if (b->prof) return; // as in the reference: a profiled batch is not split
    if (b->nseg >= 8) return;
    submit_segment(b);
}

void qw_batch_submit(qw_batch *b) {
    if (b->submitted) return;
    b->submitted = true;
    submit_segment(b);
}

bool qw_batch_poll(qw_batch *b) {
    if (b->failed || !b->submitted) return true;
    return hipEventQuery(b->ev[2 * b->nseg - 1]) != hipErrorNotReady;
}

static void batch_free(qw_batch *b) {
    for (int i = 0; i < b->nouts; i++) b->outs[i]->pending_out--;
    free(b->outs);
    for (int i = 0; i < 2 * b->nseg; i++) (void)hipEventDestroy(b->ev[i]);
    for (int i = 0; i < b->npev; i++) (void)hipEventDestroy(b->pev[i]);
    free(b->pev);
    free(b->l);
    free(b->use);
    free(b);
}

double qw_batch_wait(qw_batch *b) {
    qw_gpu *g = b->g;
    hipStream_t st = g->stream[b->stream];
    if (!b->submitted) qw_batch_submit(b);
    double secs = -1;
    if (b->failed) {
        (void)hipStreamSynchronize(st);
        if (!g->err[0]) set_err(g, "batch failed");
        if (!g->sw.quiet) fprintf(stderr, "qw_batch: %s\n", g->err);
        batch_free(b);
        return -1;
    }
    // device -> host for everything bound in an output role
    const unsigned mark = ++g->mark;
    bool ok = true;
    for (int i = 0; i < b->nuse && ok; i++) {
        qw_hbuf *h = b->use[i].b;
        if (!b->use[i].out || h->mark == mark) continue;
        h->mark = mark;
        if (h->device_only || !h->host || h->wrapped || h->size > QW_HIP_BIG_OUT_BYTES) continue;
        ok = HIPOK(g, hipMemcpyAsync(h->host, h->dptr, h->size, hipMemcpyDeviceToHost, st));
    }
    if (ok && b->uses_sync) ok = HIPOK(g, hipMemcpyAsync(g->sync_host, g->sync + QW_SYNC_ERR_WORD, 4, hipMemcpyDeviceToHost, st));
    ok = ok && HIPOK(g, hipStreamSynchronize(st));
    if (ok && b->uses_sync && g->sync_host[0]) { // a launch whose workgroups wait for one another gave up: its results are not valid
        (void)hipMemset(g->sync, 0, QW_SYNC_BYTES);
        g->fuse_broken = true;
        set_err(g, "a fused layer launch timed out waiting for its workgroups (are other kernels running on this device?); layers run as separate launches from now on");
        ok = false;
    }
    if (ok) {
        secs = 0;
        for (int s = 0; s < b->nseg; s++) {
            float ms = 0;
            if (!HIPOK(g, hipEventElapsedTime(&ms, b->ev[2 * s], b->ev[2 * s + 1]))) { ok = false; break; }
            secs += (double)ms * 1e-3;
        }
    }
    if (ok && b->prof) {
        g->nprof = 0;
        for (int i = 0; i < b->nl && g->nprof < QW_PROF_MAX && 2 * i + 1 < b->npev; i++) {
            float ms = 0;
            (void)hipEventElapsedTime(&ms, b->pev[2 * i], b->pev[2 * i + 1]);
            g->prof_name[g->nprof] = b->l[i].kname;
            g->prof_fname[g->nprof] = b->l[i].fname;
            g->prof_us[g->nprof++] = (double)ms * 1e3;
        }
    }
    if (!ok) {
        if (!g->sw.quiet) fprintf(stderr, "qw_batch: %s\n", g->err);
        secs = -1;
    }
    batch_free(b);
    return secs;
}

double qw_batch_end(qw_batch *b) {
    qw_batch_submit(b);
    return qw_batch_wait(b);
}

void qw_gpu_set_stream(qw_gpu *g, int s) { g->cur_stream = s == 1 ? 1 : 0; }

// ---------------------------------------------------------------- the recorder with fixed storage (qw_internal.h)
_Static_assert(sizeof(qw_hbuf) <= sizeof(qw_hip_view), "qw_hip_view is too small for a buffer handle");
void qw_hip_view_init(qw_gpu *g, qw_hip_view *v, void *devptr, size_t size, qw_buf *out) {
    qw_hbuf *h = (qw_hbuf *)v;
    memset(h, 0, sizeof *h);
    h->dptr = devptr;
    h->size = size;
    h->device_only = true;
    h->g = g;
    *out = (qw_buf){.handle = h, .ptr = NULL, .size = size};
}
bool qw_hip_noalloc_scratch(qw_gpu *g, void **ptr, size_t *bytes) {
    if (!g->na_scratch) { set_err(g, "no scratch array on this device: %s", g->na_err ? g->na_err : "not set up"); return false; }
    *ptr = g->na_scratch;
    *bytes = g->na_bytes;
    return true;
}
qw_batch *qw_hip_batch_begin_static(qw_gpu *g, void *stream) {
    qw_batch *b = g->na_batch;
    if (!b || !b->l || !b->use || g->na_busy) return NULL;
    qw_launch *l = b->l;
    qw_use *use = b->use;
    memset(b, 0, sizeof *b);
    *b = (qw_batch){.g = g, .seq = ++g->batch_seq, .stream = g->cur_stream, .noalloc = true, .xstream = (hipStream_t)stream, .l = l, .capl = 64, .use = use, .capuse = 1024};
    b->sw.dnq_min = QW_DNQ_MIN_DEFAULT;
    b->sw.dnc_nb = 2; // the defaults; the measurement switches of the environment do not apply here
    b->sw.no_fuse = true; // the caller's stream may run beside other work of this device: no launch that waits for all of its workgroups
    g->na_busy = true;
    g->err[0] = 0;
    return b;
}
bool qw_hip_batch_launch_static(qw_batch *b, bool recorded) {
    qw_gpu *g = b->g;
    hipStream_t st = b->xstream ? b->xstream : g->stream[b->stream];
    bool ok = recorded && !b->failed && flush_select(b) && flush_tw(b, NULL, NULL) && flush_pf(b) && flush_gu(b) && flush_dn(b) && flush_pk(b) && !b->failed;
    for (int i = 0; ok && i < b->nl; i++) {
        qw_launch *l = &b->l[i];
        void *params[] = {l->args};
        ok = HIPOK(g, hipModuleLaunchKernel(l->f, l->gx, l->gy, l->gz, l->bx, 1, 1, 0, st, params, NULL));
    }
    g->na_busy = false;
    return ok;
}

// ---------------------------------------------------------------- profiling and bench utilities
void qw_profile_enable(qw_gpu *g, bool on) { g->prof = on; }
int qw_profile_count(const qw_gpu *g) { return g->nprof; }
const char *qw_profile_get(const qw_gpu *g, int i, double *us) {
    if (i < 0 || i >= g->nprof) return NULL;
    if (us) *us = g->prof_us[i];
    return g->prof_name[i];
}
const char *qw_hip_profile_entry(const qw_gpu *g, int i, double *us) {
    if (i < 0 || i >= g->nprof) return NULL;
    if (us) *us = g->prof_us[i];
    return g->prof_fname[i];
}
double qw_hip_profile_mean(const qw_gpu *g, const char *prefix, int *count) {
    double s = 0;
    int n = 0;
    for (int i = 0; i < g->nprof; i++)
        if (!strncmp(g->prof_fname[i], prefix, strlen(prefix)) || !strncmp(g->prof_name[i], prefix, strlen(prefix))) { s += g->prof_us[i]; n++; }
    if (count) *count = n;
    return n ? s / n * 1e-6 : 0;
}

double qw_gpu_empty_commit_latency(qw_gpu *g, qw_kernel *k, int n) {
    (void)k;
    if (n < 1) return 0;
    hipStream_t st = g->stream[g->cur_stream];
    hipEvent_t ev;
    if (hipEventCreate(&ev) != hipSuccess) return -1;
    const double t0 = qw_now();
    for (int i = 0; i < n; i++) {
        (void)hipEventRecord(ev, st);
        (void)hipEventSynchronize(ev);
    }
    const double t = (qw_now() - t0) / n;
    (void)hipEventDestroy(ev);
    return t;
}

void qw_power_desc(char *out, size_t len) { snprintf(out, len, "power: mains (accelerator card); thermal state not reported"); }
bool qw_on_battery(void) { return false; }
