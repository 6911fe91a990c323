// GGUF reader and weight residency (include/qw_gguf.h). Host code above gpu.h and qw_hip_ext.h only.
#define _GNU_SOURCE
#include "qw_gguf.h"
#include "qw_hip_ext.h"
#include <dirent.h>
#include <fcntl.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

enum { T_F32 = 0, T_F16 = 1, T_BF16 = 30 };
#define ARENA_ALIGN 256u
#define MAX_SHARDS 16 // src/gguf.c:299

typedef struct {
    char *path;
    int fd;
    uint64_t fsize, data0;
    uint32_t version, align;
    void *map;
} shard;

struct qw_gguf {
    shard *sh;
    int nsh;
    qw_gguf_tensor *t;
    int nt;
    int *by_name, *by_model; // tensor indices sorted by name / by model-side name (mapped tensors only)
    int nmodel;
    // residency
    qw_gpu *g;
    qw_buf arena;
    bool only_experts; // the arena holds routed expert matrices and nothing else (qw_gguf_release_source)
    bool loaded;
    uint64_t *dev_off; // per tensor; valid when res_type >= 0
    size_t resident;
    double load_s;
};

static bool fail(char *err, size_t errlen, const char *fmt, ...) {
    if (err && errlen) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(err, errlen, fmt, ap);
        va_end(ap);
    }
    return false;
}

// ---------------------------------------------------------------- type table (src/gguf.c:15-37)
static const struct { int t, qb, bb; const char *name; } TYPES[] = {
    {0, 1, 4, "F32"},        {1, 1, 2, "F16"},        {30, 1, 2, "BF16"},      {2, 32, 18, "Q4_0"},     {3, 32, 20, "Q4_1"},
    {6, 32, 22, "Q5_0"},     {7, 32, 24, "Q5_1"},     {8, 32, 34, "Q8_0"},     {10, 256, 84, "Q2_K"},   {11, 256, 110, "Q3_K"},
    {12, 256, 144, "Q4_K"},  {13, 256, 176, "Q5_K"},  {14, 256, 210, "Q6_K"},  {16, 256, 66, "IQ2_XXS"}, {17, 256, 74, "IQ2_XS"},
    {18, 256, 98, "IQ3_XXS"}, {19, 256, 50, "IQ1_S"}, {20, 32, 18, "IQ4_NL"},  {21, 256, 110, "IQ3_S"}, {22, 256, 82, "IQ2_S"},
    {23, 256, 136, "IQ4_XS"}, {29, 256, 56, "IQ1_M"}, {42, 64, 18, "Q2_0(42)"},
};
bool qw_ggml_block(int type, int *qb, int *bb) {
    for (size_t i = 0; i < sizeof TYPES / sizeof *TYPES; i++)
        if (TYPES[i].t == type) {
            *qb = TYPES[i].qb;
            *bb = TYPES[i].bb;
            return true;
        }
    return false;
}
const char *qw_ggml_name(int type) {
    for (size_t i = 0; i < sizeof TYPES / sizeof *TYPES; i++)
        if (TYPES[i].t == type) return TYPES[i].name;
    return "?";
}

// One word of a QW_GGUF_PARTS list (src/gguf.c:38-52 gives the words and what they select).
static unsigned part_of_word(const char *w, size_t n) {
    static const char *const words[] = {"moe", "shared", "router", "attn", "lin", "hyper", "lm", "embed", "ple"};
    static const unsigned bits[] = {QW_GG_MOE, QW_GG_SHARED, QW_GG_ROUTER, QW_GG_ATTN, QW_GG_LIN, QW_GG_HYPER, QW_GG_LM, QW_GG_EMBED, QW_GG_PLE};
    for (size_t i = 0; i < sizeof bits / sizeof *bits; i++)
        if (strlen(words[i]) == n && !memcmp(w, words[i], n)) return bits[i];
    return 0; // a word that names nothing selects nothing
}
unsigned qw_gguf_parse_parts(const char *s) {
    if (!s || !*s || !strcmp(s, "all")) return QW_GG_ALL;
    unsigned parts = 0;
    while (*s) { // comma-separated, read in place
        const size_t n = strcspn(s, ",");
        parts |= part_of_word(s, n);
        s += n;
        if (*s == ',') s++;
    }
    return parts;
}

// ---------------------------------------------------------------- names (src/gguf.c:181-273)
// Per-layer tensors "blk.<l>.<suffix>" -> "language_model.model.layers.<l>.<model suffix>"
static const struct { const char *g; unsigned part; const char *m; int kind; } LAYER_NAMES[] = {
    {"ffn_gate_exps.weight", QW_GG_MOE, "mlp.switch_mlp.gate_proj.iq", QW_GK_EXP},
    {"ffn_up_exps.weight", QW_GG_MOE, "mlp.switch_mlp.up_proj.iq", QW_GK_EXP},
    {"ffn_down_exps.weight", QW_GG_MOE, "mlp.switch_mlp.down_proj.iq", QW_GK_EXP},
    {"ffn_gate_shexp.weight", QW_GG_SHARED, "mlp.shared_expert.gate_proj.weight", QW_GK_LIN},
    {"ffn_up_shexp.weight", QW_GG_SHARED, "mlp.shared_expert.up_proj.weight", QW_GK_LIN},
    {"ffn_down_shexp.weight", QW_GG_SHARED, "mlp.shared_expert.down_proj.weight", QW_GK_LIN},
    {"ffn_gate_inp.weight", QW_GG_ROUTER, "mlp.gate.weight", QW_GK_LIN},
    {"ffn_gate_inp_shexp.weight", QW_GG_ROUTER, "mlp.shared_expert_gate.weight", QW_GK_SMALL},
    {"attn_q.weight", QW_GG_ATTN, "self_attn.q_proj.weight", QW_GK_LIN},
    {"attn_k.weight", QW_GG_ATTN, "self_attn.k_proj.weight", QW_GK_LIN},
    {"attn_v.weight", QW_GG_ATTN, "self_attn.v_proj.weight", QW_GK_LIN},
    {"attn_output.weight", QW_GG_ATTN, "self_attn.o_proj.weight", QW_GK_LIN},
    {"attn_q_norm.weight", QW_GG_ATTN, "self_attn.q_norm.weight", QW_GK_F32},
    {"attn_k_norm.weight", QW_GG_ATTN, "self_attn.k_norm.weight", QW_GK_F32},
    {"attn_qkv.weight", QW_GG_LIN, "linear_attn.in_proj_qkv.weight", QW_GK_LIN},
    {"attn_gate.weight", QW_GG_LIN, "linear_attn.in_proj_z.weight", QW_GK_LIN},
    {"ssm_alpha.weight", QW_GG_LIN, "linear_attn.in_proj_a.weight", QW_GK_LIN},
    {"ssm_beta.weight", QW_GG_LIN, "linear_attn.in_proj_b.weight", QW_GK_LIN},
    {"ssm_out.weight", QW_GG_LIN, "linear_attn.out_proj.weight", QW_GK_LIN},
    {"ssm_a", QW_GG_LIN, "linear_attn.A_neg", QW_GK_F32},
    {"ssm_dt.bias", QW_GG_LIN, "linear_attn.dt_bias", QW_GK_SMALL},
    {"ssm_conv1d.weight", QW_GG_LIN, "linear_attn.conv1d.weight", QW_GK_SMALL},
    {"ssm_norm.weight", QW_GG_LIN, "linear_attn.norm.weight", QW_GK_SMALL},
    // the two hyper-connections of a layer (src/gguf.c:222-229): BF16 matrices as they are, inject as a small tensor, norm F32
    {"hc_attn_down.weight", QW_GG_HYPER, "attn_hyper_connection.input_mix_weight_down.weight", QW_GK_LIN},
    {"hc_attn_up.weight", QW_GG_HYPER, "attn_hyper_connection.input_mix_weight_up.weight", QW_GK_LIN},
    {"hc_attn_inject.weight", QW_GG_HYPER, "attn_hyper_connection.block_inject_weight.weight", QW_GK_SMALL},
    {"hc_attn_norm.weight", QW_GG_HYPER, "attn_hyper_connection.hc_norm.weight", QW_GK_F32},
    {"hc_ffn_down.weight", QW_GG_HYPER, "mlp_hyper_connection.input_mix_weight_down.weight", QW_GK_LIN},
    {"hc_ffn_up.weight", QW_GG_HYPER, "mlp_hyper_connection.input_mix_weight_up.weight", QW_GK_LIN},
    {"hc_ffn_inject.weight", QW_GG_HYPER, "mlp_hyper_connection.block_inject_weight.weight", QW_GK_SMALL},
    {"hc_ffn_norm.weight", QW_GG_HYPER, "mlp_hyper_connection.hc_norm.weight", QW_GK_F32},
};
static const struct { const char *g; unsigned part; const char *m; int kind; } TOP_NAMES[] = {
    {"output.weight", QW_GG_LM, "language_model.lm_head.weight", QW_GK_LIN},
    {"token_embd.weight", QW_GG_EMBED, "language_model.model.embed_tokens.weight", QW_GK_LIN},
    // the mixer after the last layer (src/gguf.c:250-252): no inject rows
    {"output_hc_down.weight", QW_GG_HYPER, "language_model.model.hyper_connection_mixer.input_mix_weight_down.weight", QW_GK_LIN},
    {"output_hc_up.weight", QW_GG_HYPER, "language_model.model.hyper_connection_mixer.input_mix_weight_up.weight", QW_GK_LIN},
    {"output_hc_norm.weight", QW_GG_HYPER, "language_model.model.hyper_connection_mixer.hc_norm.weight", QW_GK_F32},
};

static char *map_name(const char *g, unsigned *part, int *kind) {
    int l = -1, n = 0;
    char out[256];
    *part = 0;
    *kind = QW_GK_LIN;
    if (sscanf(g, "blk.%d.%n", &l, &n) == 1 && n > 0 && l >= 0) {
        for (size_t i = 0; i < sizeof LAYER_NAMES / sizeof *LAYER_NAMES; i++)
            if (!strcmp(g + n, LAYER_NAMES[i].g)) {
                *part = LAYER_NAMES[i].part;
                *kind = LAYER_NAMES[i].kind;
                snprintf(out, sizeof out, "language_model.model.layers.%d.%s", l, LAYER_NAMES[i].m);
                return strdup(out);
            }
        return strdup("");
    }
    for (size_t i = 0; i < sizeof TOP_NAMES / sizeof *TOP_NAMES; i++)
        if (!strcmp(g, TOP_NAMES[i].g)) {
            *part = TOP_NAMES[i].part;
            *kind = TOP_NAMES[i].kind;
            return strdup(TOP_NAMES[i].m);
        }
    return strdup("");
}

// ---------------------------------------------------------------- parsing
// What the header of a file holds and which files are refused follows the reference's parser (src/gguf.c:73-173): GGUF
// version 2 or later, strings of at most 16 MiB, tensors of at most four dimensions, no arrays of arrays, of the metadata
// only general.alignment kept (default 32), the data start rounded up to the alignment. Here the file is mapped first
// and the header is walked in the mapping by a cursor that can never leave it: a read past the end yields zero and
// marks the cursor, and the caller looks at the mark when a section is done.
typedef struct {
    const uint8_t *base;
    uint64_t size, at;
    bool overrun;
} cursor;
// n bytes at the cursor, or NULL (and the mark) when fewer are left
static const uint8_t *cur_take(cursor *c, uint64_t n) {
    if (c->overrun || n > c->size - c->at) {
        c->overrun = true;
        return NULL;
    }
    const uint8_t *p = c->base + c->at;
    c->at += n;
    return p;
}
// a little-endian unsigned integer of 1 to 8 bytes
static uint64_t cur_uint(cursor *c, unsigned width) {
    const uint8_t *p = cur_take(c, width);
    uint64_t v = 0;
    for (unsigned i = 0; p && i < width; i++) v |= (uint64_t)p[i] << (8 * i);
    return v;
}
// a string (u64 length, then the bytes): pointer into the mapping and its length; longer than 16 MiB counts as damage
static const char *cur_text(cursor *c, uint64_t *len) {
    *len = cur_uint(c, 8);
    if (*len > ((uint64_t)1 << 24)) c->overrun = true;
    return (const char *)cur_take(c, *len);
}
enum { GV_STRING = 8, GV_ARRAY = 9, GV_TYPES = 13 };
// bytes of a scalar of each GGUF value type: u8 i8 u16 i16 u32 i32 f32 bool | string array | u64 i64 f64
static const uint8_t GV_WIDTH[GV_TYPES] = {1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8};
// Step over one metadata value of type vt. A scalar's integer value goes to *scalar when the caller wants it.
static void cur_skip_value(cursor *c, uint32_t vt, uint64_t *scalar) {
    uint64_t n;
    if (vt == GV_STRING) {
        (void)cur_text(c, &n);
    } else if (vt == GV_ARRAY) {
        const uint32_t et = (uint32_t)cur_uint(c, 4);
        n = cur_uint(c, 8);
        if (et == GV_ARRAY || et >= GV_TYPES) c->overrun = true; // (arrays of arrays are not accepted)
        else if (et == GV_STRING)
            for (uint64_t i = 0; i < n && !c->overrun; i++) {
                uint64_t l;
                (void)cur_text(c, &l);
            }
        else if (n > (c->size - c->at) / GV_WIDTH[et]) c->overrun = true;
        else (void)cur_take(c, n * GV_WIDTH[et]);
    } else if (vt < GV_TYPES) {
        const uint64_t v = cur_uint(c, GV_WIDTH[vt]);
        if (scalar) *scalar = v;
    } else c->overrun = true;
}
static char *text_dup(const char *p, uint64_t len) {
    char *s = malloc(len + 1);
    if (s) {
        memcpy(s, p, len);
        s[len] = 0;
    }
    return s;
}

// rows, rowbytes and nbytes of a tensor (nbytes 0 for a type that is not in the table); false when a product of its
// dimensions does not fit 64 bits.
static bool tensor_bytes(qw_gguf_tensor *t) {
    int qb, bb;
    t->rows = 1;
    t->rowbytes = t->nbytes = 0;
    uint64_t values;
    for (uint32_t d = 1; d < t->nd; d++)
        if (__builtin_mul_overflow(t->rows, t->dims[d], &t->rows)) return false;
    if (__builtin_mul_overflow(t->rows, t->nd ? t->dims[0] : 1, &values) || values > UINT64_MAX / 4) return false;
    if (!qw_ggml_block((int)t->type, &qb, &bb)) return true;
    t->rowbytes = t->dims[0] / (uint64_t)qb * (uint64_t)bb;
    return !__builtin_mul_overflow(t->rows, t->rowbytes, &t->nbytes);
}

static bool parse_shard(qw_gguf *G, int si, const char *path, char *err, size_t errlen) {
    shard *s = &G->sh[si];
    s->path = strdup(path);
    s->fd = open(path, O_RDONLY);
    if (s->fd < 0) return fail(err, errlen, "GGUF: cannot open %s", path);
    struct stat sb;
    if (fstat(s->fd, &sb)) return fail(err, errlen, "GGUF: cannot stat %s", path);
    s->fsize = (uint64_t)sb.st_size;
    if (s->fsize) {
        s->map = mmap(NULL, s->fsize, PROT_READ, MAP_SHARED, s->fd, 0);
        if (s->map == MAP_FAILED) {
            s->map = NULL;
            return fail(err, errlen, "GGUF: mmap of %s failed", path);
        }
    }
    cursor c = {.base = s->map, .size = s->fsize};
    const uint8_t *magic = cur_take(&c, 4);
    const uint32_t ver = (uint32_t)cur_uint(&c, 4);
    const uint64_t ntensors = cur_uint(&c, 8), nmeta = cur_uint(&c, 8);
    if (c.overrun || memcmp(magic, "GGUF", 4) || ver < 2) return fail(err, errlen, "GGUF: %s is not GGUF v2+", path);
    // every metadata entry takes at least 12 bytes and every tensor entry at least 24: a count beyond that is damage
    if (nmeta > s->fsize / 12 || ntensors > s->fsize / 24) return fail(err, errlen, "GGUF: %s: metadata is damaged", path);
    uint64_t align = 32;
    static const char ALIGN_KEY[] = "general.alignment";
    for (uint64_t i = 0; i < nmeta && !c.overrun; i++) {
        uint64_t klen;
        const char *key = cur_text(&c, &klen);
        const uint32_t vt = (uint32_t)cur_uint(&c, 4);
        const bool is_align = key && klen == sizeof ALIGN_KEY - 1 && !memcmp(key, ALIGN_KEY, klen);
        cur_skip_value(&c, vt, is_align ? &align : NULL);
    }
    align &= 0xffffffffu;
    if (c.overrun || align == 0) return fail(err, errlen, "GGUF: %s: metadata is damaged", path);
    qw_gguf_tensor *grown = realloc(G->t, sizeof *G->t * (size_t)(G->nt + (int)ntensors + 1));
    if (!grown) return fail(err, errlen, "GGUF: out of memory");
    G->t = grown;
    const int first = G->nt;
    for (uint64_t i = 0; i < ntensors; i++) {
        qw_gguf_tensor *t = &G->t[G->nt];
        memset(t, 0, sizeof *t);
        uint64_t nlen;
        const char *name = cur_text(&c, &nlen);
        t->nd = (uint32_t)cur_uint(&c, 4);
        if (t->nd > 4) c.overrun = true;
        for (uint32_t d = 0; d < t->nd && !c.overrun; d++) t->dims[d] = cur_uint(&c, 8);
        t->type = (uint32_t)cur_uint(&c, 4);
        t->offset = cur_uint(&c, 8); // relative to the data start until the loop below
        if (c.overrun || !(t->name = text_dup(name, nlen))) return fail(err, errlen, "GGUF: %s: tensor table is damaged", path);
        t->shard = si;
        t->res_type = -1;
        t->model = map_name(t->name, &t->part, &t->kind);
        G->nt++;
    }
    s->version = ver;
    s->align = (uint32_t)align;
    s->data0 = (c.at + align - 1) / align * align;
    for (int i = first; i < G->nt; i++) {
        qw_gguf_tensor *t = &G->t[i];
        if (!tensor_bytes(t) || __builtin_add_overflow(t->offset, s->data0, &t->offset)) return fail(err, errlen, "GGUF: %s: tensor table is damaged", path);
        if (t->offset > s->fsize || t->nbytes > s->fsize - t->offset) return fail(err, errlen, "GGUF: %s: tensor %s lies beyond the end of the file", path, t->name);
    }
    return true;
}

static int cmp_str(const void *a, const void *b) { return strcmp(*(char *const *)a, *(char *const *)b); }
static int cmp_by_name(const void *a, const void *b, void *G) { return strcmp(((const qw_gguf *)G)->t[*(const int *)a].name, ((const qw_gguf *)G)->t[*(const int *)b].name); }
static int cmp_by_model(const void *a, const void *b, void *G) { return strcmp(((const qw_gguf *)G)->t[*(const int *)a].model, ((const qw_gguf *)G)->t[*(const int *)b].model); }

qw_gguf *qw_gguf_open(const char *dir, char *err, size_t errlen) {
    if (err && errlen) err[0] = 0;
    DIR *d = opendir(dir);
    if (!d) {
        fail(err, errlen, "GGUF: cannot open directory %s", dir);
        return NULL;
    }
    char *names[MAX_SHARDS];
    int nn = 0;
    for (struct dirent *de; (de = readdir(d)) && nn < MAX_SHARDS;) {
        const size_t l = strlen(de->d_name);
        if (l > 5 && !strcmp(de->d_name + l - 5, ".gguf")) {
            char p[4096];
            snprintf(p, sizeof p, "%s/%s", dir, de->d_name);
            names[nn++] = strdup(p);
        }
    }
    closedir(d);
    if (!nn) {
        fail(err, errlen, "GGUF: no .gguf in %s", dir);
        return NULL;
    }
    qsort(names, (size_t)nn, sizeof *names, cmp_str);
    qw_gguf *G = calloc(1, sizeof *G);
    G->sh = calloc((size_t)nn, sizeof *G->sh);
    G->nsh = nn;
    bool ok = true;
    for (int i = 0; i < nn; i++) {
        G->sh[i].fd = -1;
        if (ok) ok = parse_shard(G, i, names[i], err, errlen);
        free(names[i]);
    }
    if (!ok) {
        qw_gguf_close(G);
        return NULL;
    }
    G->by_name = malloc(sizeof(int) * (size_t)(G->nt + 1));
    G->by_model = malloc(sizeof(int) * (size_t)(G->nt + 1));
    G->dev_off = calloc((size_t)G->nt + 1, sizeof *G->dev_off);
    for (int i = 0; i < G->nt; i++) {
        G->by_name[i] = i;
        if (G->t[i].part) G->by_model[G->nmodel++] = i;
    }
    qsort_r(G->by_name, (size_t)G->nt, sizeof(int), cmp_by_name, G);
    qsort_r(G->by_model, (size_t)G->nmodel, sizeof(int), cmp_by_model, G);
    return G;
}

void qw_gguf_close(qw_gguf *G) {
    if (!G) return;
    if (G->loaded) qw_buf_free(&G->arena);
    for (int i = 0; i < G->nt; i++) {
        free((char *)G->t[i].name);
        free((char *)G->t[i].model);
    }
    for (int i = 0; i < G->nsh; i++) {
        if (G->sh[i].map) munmap(G->sh[i].map, G->sh[i].fsize);
        if (G->sh[i].fd >= 0) close(G->sh[i].fd);
        free(G->sh[i].path);
    }
    free(G->t);
    free(G->sh);
    free(G->by_name);
    free(G->by_model);
    free(G->dev_off);
    free(G);
}

int qw_gguf_shards(const qw_gguf *G) { return G->nsh; }
const char *qw_gguf_shard_path(const qw_gguf *G, int i) { return i >= 0 && i < G->nsh ? G->sh[i].path : NULL; }
uint32_t qw_gguf_shard_alignment(const qw_gguf *G, int i) { return i >= 0 && i < G->nsh ? G->sh[i].align : 0; }
uint64_t qw_gguf_shard_data_start(const qw_gguf *G, int i) { return i >= 0 && i < G->nsh ? G->sh[i].data0 : 0; }
int qw_gguf_count(const qw_gguf *G) { return G->nt; }
const qw_gguf_tensor *qw_gguf_get(const qw_gguf *G, int i) { return i >= 0 && i < G->nt ? &G->t[i] : NULL; }

// Binary search over idx (sorted by the key that field selects); among equal names the first in file order wins.
static const qw_gguf_tensor *find_in(const qw_gguf *G, const int *idx, int n, const char *name, bool model) {
    int lo = 0, hi = n;
    while (lo < hi) {
        const int mid = (lo + hi) / 2;
        const qw_gguf_tensor *t = &G->t[idx[mid]];
        if (strcmp(model ? t->model : t->name, name) < 0) lo = mid + 1;
        else hi = mid;
    }
    const qw_gguf_tensor *best = NULL;
    for (; lo < n; lo++) {
        const qw_gguf_tensor *t = &G->t[idx[lo]];
        if (strcmp(model ? t->model : t->name, name)) break;
        if (!best || t < best) best = t;
    }
    return best;
}
const qw_gguf_tensor *qw_gguf_find(const qw_gguf *G, const char *name) {
    if (!name || !*name) return NULL;
    const qw_gguf_tensor *t = find_in(G, G->by_name, G->nt, name, false);
    return t ? t : find_in(G, G->by_model, G->nmodel, name, true);
}
const void *qw_gguf_host(const qw_gguf *G, const qw_gguf_tensor *t) {
    if (!t || t < G->t || t >= G->t + G->nt || !G->sh[t->shard].map) return NULL;
    return (const uint8_t *)G->sh[t->shard].map + t->offset;
}

// ---------------------------------------------------------------- residency
static float h2f(uint16_t h) {
    _Float16 x;
    memcpy(&x, &h, 2);
    return (float)x;
}

// Small float tensor -> float values; *exact = every value has a BF16 representation (src/gguf.c:275-280, 449-455).
static float *small_values(const qw_gguf *G, const qw_gguf_tensor *t, bool *exact) {
    const uint64_t n = t->rows * t->dims[0];
    const void *src = qw_gguf_host(G, t);
    float *v = malloc(sizeof(float) * (n ? n : 1));
    if (!v || !src) {
        free(v);
        return NULL;
    }
    *exact = true;
    for (uint64_t i = 0; i < n; i++) {
        if (t->type == T_F32) memcpy(&v[i], (const uint8_t *)src + 4 * i, 4);
        else if (t->type == T_F16) {
            uint16_t h;
            memcpy(&h, (const uint8_t *)src + 2 * i, 2);
            v[i] = h2f(h);
        } else {
            uint16_t h;
            memcpy(&h, (const uint8_t *)src + 2 * i, 2);
            const uint32_t u = (uint32_t)h << 16;
            memcpy(&v[i], &u, 4);
        }
        uint32_t u;
        memcpy(&u, &v[i], 4);
        if (u & 0xffff) *exact = false;
    }
    return v;
}

bool qw_gguf_load(qw_gguf *G, qw_gpu *g, unsigned parts, char *err, size_t errlen) {
    if (err && errlen) err[0] = 0;
    if (G->loaded) return fail(err, errlen, "GGUF: already loaded");
    // first pass: checks, and the place of every selected tensor in the arena
    uint64_t total = 0;
    int nsel = 0;
    for (int i = 0; i < G->nt; i++) {
        qw_gguf_tensor *t = &G->t[i];
        if (!t->part || !(t->part & parts)) continue;
        if (!t->rowbytes) return fail(err, errlen, "GGUF: format %u of %s is not supported", t->type, t->name);
        const bool is_float = t->type == T_F32 || t->type == T_F16 || t->type == T_BF16;
        uint64_t bytes;
        if (t->kind == QW_GK_LIN || t->kind == QW_GK_EXP) {
            if (is_float && t->type != T_BF16) return fail(err, errlen, "GGUF: %s is a %s matrix, which is not supported", t->name, qw_ggml_name((int)t->type));
            bytes = t->nbytes;
        } else {
            if (!is_float) return fail(err, errlen, "GGUF: %s should be floating point but is %s", t->name, qw_ggml_name((int)t->type));
            bytes = t->rows * t->dims[0] * 4; // at most F32
        }
        G->dev_off[i] = total;
        total += (bytes + ARENA_ALIGN - 1) / ARENA_ALIGN * ARENA_ALIGN;
        nsel++;
    }
    if (!nsel) return fail(err, errlen, "GGUF: no tensor of parts 0x%x", parts);
    G->only_experts = true;
    for (int i = 0; i < G->nt; i++)
        if (G->t[i].part && (G->t[i].part & parts) && G->t[i].kind != QW_GK_EXP) G->only_experts = false;
    if (!qw_hip_buf_new_device(g, (size_t)total, &G->arena)) return fail(err, errlen, "GGUF: cannot allocate %llu bytes of device memory: %s", (unsigned long long)total, qw_hip_last_error(g));
    G->g = g;
    G->loaded = true;
    const double t0 = qw_now();
    for (int i = 0; i < G->nt; i++) {
        qw_gguf_tensor *t = &G->t[i];
        if (!t->part || !(t->part & parts)) continue;
        const shard *s = &G->sh[t->shard];
        bool ok;
        if (t->kind == QW_GK_LIN || t->kind == QW_GK_EXP) {
            ok = qw_hip_buf_write_fd(&G->arena, (size_t)G->dev_off[i], s->fd, t->offset, (size_t)t->nbytes);
            t->res_type = (int)t->type;
            G->resident += t->nbytes;
        } else {
            bool exact;
            float *v = small_values(G, t, &exact);
            if (!v) return fail(err, errlen, "GGUF: cannot read %s", t->name);
            const uint64_t n = t->rows * t->dims[0];
            if (exact && t->kind == QW_GK_SMALL) {
                uint16_t *h = (uint16_t *)v; // in place: entry i of the halves lies below entry i of the floats
                for (uint64_t k = 0; k < n; k++) {
                    uint32_t u;
                    memcpy(&u, &v[k], 4);
                    h[k] = (uint16_t)(u >> 16);
                }
                ok = qw_hip_buf_write(&G->arena, (size_t)G->dev_off[i], h, (size_t)n * 2);
                t->res_type = T_BF16;
                G->resident += n * 2;
            } else {
                ok = qw_hip_buf_write(&G->arena, (size_t)G->dev_off[i], v, (size_t)n * 4);
                t->res_type = T_F32;
                G->resident += n * 4;
            }
            free(v);
        }
        if (!ok) {
            t->res_type = -1;
            return fail(err, errlen, "GGUF: copy of %s to the device failed: %s", t->name, qw_hip_last_error(g));
        }
    }
    G->load_s = qw_now() - t0;
    return true;
}

size_t qw_gguf_resident_bytes(const qw_gguf *G) { return G->resident; }
double qw_gguf_load_seconds(const qw_gguf *G) { return G->load_s; }

bool qw_gguf_tensor_at(const qw_gguf *G, const qw_gguf_tensor *t, qw_tensor *out) {
    if (!G->loaded || !t || t < G->t || t >= G->t + G->nt || t->res_type < 0) return false;
    out->buf = &G->arena;
    out->offset = (size_t)G->dev_off[t - G->t];
    out->type = t->res_type;
    return true;
}

bool qw_gguf_moe_layer(const qw_gguf *G, int layer, qw_moe_layer *M, int *D, int *I, int *E, char *err, size_t errlen) {
    if (err && errlen) err[0] = 0;
    static const char *const suffix[8] = {"ffn_gate_inp.weight",  "ffn_gate_inp_shexp.weight", "ffn_gate_exps.weight",  "ffn_up_exps.weight",
                                          "ffn_down_exps.weight", "ffn_gate_shexp.weight",     "ffn_up_shexp.weight",    "ffn_down_shexp.weight"};
    qw_tensor *const dst[8] = {&M->router, &M->sh_gate_w, &M->gate, &M->up, &M->down, &M->sh_gate, &M->sh_up, &M->sh_down};
    const qw_gguf_tensor *t[8];
    for (int i = 0; i < 8; i++) {
        char name[128];
        snprintf(name, sizeof name, "blk.%d.%s", layer, suffix[i]);
        t[i] = qw_gguf_find(G, name);
        if (!t[i]) return fail(err, errlen, "GGUF: %s is missing", name);
        if (!qw_gguf_tensor_at(G, t[i], dst[i])) return fail(err, errlen, "GGUF: %s is not resident", name);
    }
    const qw_gguf_tensor *r = t[0], *gw = t[1], *ga = t[2], *up = t[3], *dn = t[4], *sg = t[5], *su = t[6], *sd = t[7];
    if (ga->nd != 3 || up->nd != 3 || dn->nd != 3 || r->nd != 2 || sg->nd != 2 || su->nd != 2 || sd->nd != 2) return fail(err, errlen, "GGUF: layer %d: unexpected number of dimensions", layer);
    const uint64_t d = ga->dims[0], in = ga->dims[1], e = ga->dims[2];
    bool ok = up->dims[0] == d && up->dims[1] == in && up->dims[2] == e && dn->dims[0] == in && dn->dims[1] == d && dn->dims[2] == e;
    ok = ok && r->dims[0] == d && r->dims[1] == e && gw->rows * gw->dims[0] == d;
    ok = ok && sg->dims[0] == d && sg->dims[1] == in && su->dims[0] == d && su->dims[1] == in && sd->dims[0] == in && sd->dims[1] == d;
    if (!ok) return fail(err, errlen, "GGUF: layer %d: the shapes of the MoE tensors do not agree", layer);
    if (ga->type != up->type) return fail(err, errlen, "GGUF: layer %d: gate is %s but up is %s", layer, qw_ggml_name((int)ga->type), qw_ggml_name((int)up->type));
    // The shared expert's gate and up may differ inside the K-quant / IQ4 / plain family (Q4_K gate and IQ4_XS up in the
    // reference's model, bench/moe_bw.c:19-20); Q8_0 and IQ3_S rows run in kernels that take one type for both.
    if (sg->type != su->type && (sg->type == 8 || sg->type == 21 || su->type == 8 || su->type == 21))
        return fail(err, errlen, "GGUF: layer %d: shared gate is %s but shared up is %s", layer, qw_ggml_name((int)sg->type), qw_ggml_name((int)su->type));
    if (M->sh_gate_w.type != M->router.type)
        return fail(err, errlen, "GGUF: layer %d: the shared-expert gate vector is %s but the router is %s", layer, qw_ggml_name(M->sh_gate_w.type), qw_ggml_name(M->router.type));
    *D = (int)d;
    *I = (int)in;
    *E = (int)e;
    return true;
}

// The weights of one hyper-connection: which = 0 the one in front of a layer's attention / linear attention
// (blk.<layer>.hc_attn_*), 1 the one in front of its MoE (hc_ffn_*), 2 the mixer after the last layer (output_hc_*, layer
// ignored, no inject rows). Shapes (src/model.h:41-45): norm [HC D], mix_down [LR][HC D], mix_up [HC D][LR], inject [HC][HC D].
bool qw_gguf_hyper(const qw_gguf *G, int layer, int which, qw_hyper_w *H, int *D, char *err, size_t errlen) {
    if (err && errlen) err[0] = 0;
    if (which < 0 || which > 2) return fail(err, errlen, "GGUF: hyper-connection %d (0 attention, 1 MoE, 2 output mixer)", which);
    static const char *const part[4] = {"norm", "down", "up", "inject"};
    qw_tensor *const dst[4] = {&H->hc_norm, &H->mix_down, &H->mix_up, &H->inject};
    const qw_gguf_tensor *t[4] = {0};
    memset(H, 0, sizeof *H);
    for (int i = 0; i < (which == 2 ? 3 : 4); i++) {
        char name[128];
        if (which == 2) snprintf(name, sizeof name, "output_hc_%s.weight", part[i]);
        else snprintf(name, sizeof name, "blk.%d.hc_%s_%s.weight", layer, which ? "ffn" : "attn", part[i]);
        t[i] = qw_gguf_find(G, name);
        if (!t[i]) return fail(err, errlen, "GGUF: %s is missing", name);
        if (!qw_gguf_tensor_at(G, t[i], dst[i])) return fail(err, errlen, "GGUF: %s is not resident", name);
    }
    const uint64_t hcd = t[0]->dims[0] * t[0]->rows;
    if (hcd % QW_PATH_HC) return fail(err, errlen, "GGUF: hyper-connection norm of %llu values is not %d streams", (unsigned long long)hcd, QW_PATH_HC);
    bool ok = t[1]->nd == 2 && t[1]->dims[0] == hcd && t[1]->dims[1] == QW_PATH_HC_LR && t[2]->nd == 2 && t[2]->dims[0] == QW_PATH_HC_LR && t[2]->dims[1] == hcd;
    if (t[3]) ok = ok && t[3]->dims[0] == hcd && t[3]->rows == QW_PATH_HC;
    if (!ok) return fail(err, errlen, "GGUF: the shapes of the hyper-connection tensors do not agree");
    if (H->hc_norm.type != 0 || H->mix_down.type != 30 || H->mix_up.type != 30 || (t[3] && H->inject.type != 30))
        return fail(err, errlen, "GGUF: hyper-connection tensors must be resident as F32 norm and BF16 matrices (got %s, %s, %s, %s)", qw_ggml_name(H->hc_norm.type),
                    qw_ggml_name(H->mix_down.type), qw_ggml_name(H->mix_up.type), t[3] ? qw_ggml_name(H->inject.type) : "-");
    *D = (int)(hcd / QW_PATH_HC);
    return true;
}

// Keep only the tile-major copies of the routed experts of this handle (qw_hip_buf_release_source on its arena).
bool qw_gguf_release_source(qw_gguf *G, char *err, size_t errlen) {
    if (err && errlen) err[0] = 0;
    if (!G->loaded) return fail(err, errlen, "GGUF: nothing is resident");
    if (!G->only_experts) return fail(err, errlen, "GGUF: this handle's arena also holds tensors that are read as they are; load the routed experts (part moe) through a handle of their own");
    if (!qw_hip_buf_release_source(&G->arena)) return fail(err, errlen, "GGUF: no tile-major copy has been made from the arena yet (run every layer once), or a batch that writes it is in flight");
    return true;
}
