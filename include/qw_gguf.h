/* GGUF reader and weight residency for the quantized decode path.
 *
 * What the reference does in src/gguf.c, restated for a machine whose weights live in HBM instead of unified memory:
 *     gparse()          src/gguf.c:129-173   header, metadata (only general.alignment is kept), tensor table, data start
 *     qw_ggml_block()   src/gguf.c:15-25     values and bytes per block of a ggml type          (same name here)
 *     qw_ggml_name()    src/gguf.c:27-37     type name                                          (same name here)
 *     qw_gguf_parse_parts()  src/gguf.c:39-54   "all" or "moe,attn,..." -> QW_GG_* bits        (same name here)
 *     tbytes()          src/gguf.c:168-175   bytes of a tensor
 *     map_name()        src/gguf.c:181-273   GGUF tensor name -> part, model-side name, kind
 *     qw_gguf_attach()  src/gguf.c:296-547   every *.gguf of a directory in name order; matrices stay where they are in
 *                                            the file (shape [rows][row bytes], experts [E][rows][row bytes]); small
 *                                            float tensors are converted (BF16 when that is exact, else F32)
 * The reference maps whole files and hands the pages to the GPU with qw_buf_wrap() (src/gpu.h:40): zero copy on
 * unified memory. Here the selected tensors are read from the files straight into one HBM arena
 * (qw_hip_buf_write_fd: pread into pinned staging, DMA behind it); the mapping of the file stays as the host view.
 *
 * Not restated (their consumers are not part of this path): the hyper-connection, PLE and indexer tensors, whose names
 * map to part 0 here and are never loaded, and the st_model name index that the reference's model.c reads.
 * Failure: false / NULL and a message in err, like the reference; no function exits the process.
 */
#pragma once
#include "gpu.h"
#include "qw_path.h"
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Parts of the model that can be taken from the GGUF (src/model.h:111-120). */
enum {
    QW_GG_MOE = 1u << 0,    /* routed experts */
    QW_GG_SHARED = 1u << 1, /* shared expert */
    QW_GG_ROUTER = 1u << 2, /* router + shared-expert gate vector */
    QW_GG_ATTN = 1u << 3,   /* attention projections and norms */
    QW_GG_LIN = 1u << 4,    /* linear-attention projections and their small tensors */
    QW_GG_HYPER = 1u << 5,  /* hyper-connections of the layers and the output mixer */
    QW_GG_LM = 1u << 6,     /* lm_head */
    QW_GG_EMBED = 1u << 7,  /* token embedding */
    QW_GG_PLE = 1u << 8,    /* per-layer embedding (not loaded here) */
    QW_GG_ALL = (1u << 9) - 1,
};
/* What happens to a tensor when it is attached (src/gguf.c:178). */
enum {
    QW_GK_LIN = 0,   /* matrix, bytes as in the file: [rows][row bytes] */
    QW_GK_EXP = 1,   /* expert matrices, bytes as in the file: [E][rows][row bytes] */
    QW_GK_SMALL = 2, /* small float tensor: BF16 when every value is exact in BF16, else F32 */
    QW_GK_F32 = 3,   /* small float tensor kept as F32 (norm weights, A_neg) */
};

typedef struct {
    const char *name;  /* name in the file */
    const char *model; /* name the reference's model code looks it up by ("" when the tensor is not mapped) */
    unsigned part;     /* one QW_GG_* bit, 0 when the tensor is not mapped */
    int kind;          /* QW_GK_* */
    uint32_t type, nd; /* ggml type; number of dimensions (<= 4) */
    uint64_t dims[4];  /* dims[0] = values per row (innermost), as stored in the file */
    uint64_t rows, rowbytes, nbytes; /* rows = product of dims[1..]; nbytes = rows * rowbytes (0: type not known) */
    int shard;         /* index of the file that holds it */
    uint64_t offset;   /* of its first byte from the start of that file */
    int res_type;      /* after qw_gguf_load: type of the resident copy (type, or 30 / 0 for converted small tensors); -1 = not resident */
} qw_gguf_tensor;

typedef struct qw_gguf qw_gguf;

unsigned qw_gguf_parse_parts(const char *s);
bool qw_ggml_block(int type, int *qb, int *bb);
const char *qw_ggml_name(int type);

/* Parse every *.gguf of dir (sorted by file name) and map the files read-only. */
qw_gguf *qw_gguf_open(const char *dir, char *err, size_t errlen);
void qw_gguf_close(qw_gguf *f);
int qw_gguf_shards(const qw_gguf *f);
const char *qw_gguf_shard_path(const qw_gguf *f, int shard);
uint32_t qw_gguf_shard_alignment(const qw_gguf *f, int shard);
uint64_t qw_gguf_shard_data_start(const qw_gguf *f, int shard);
int qw_gguf_count(const qw_gguf *f);
const qw_gguf_tensor *qw_gguf_get(const qw_gguf *f, int i);
/* By the name in the file or by the model-side name. */
const qw_gguf_tensor *qw_gguf_find(const qw_gguf *f, const char *name);
/* The tensor's bytes in the mapping of its file. */
const void *qw_gguf_host(const qw_gguf *f, const qw_gguf_tensor *t);

/* Residency: every mapped tensor whose part is in parts goes to HBM (one device arena, 256-byte aligned tensors).
 * Matrices (QW_GK_LIN / QW_GK_EXP) must be quantized or BF16, small tensors float (src/gguf.c:417-421, 444), as in
 * the reference. May be called once per qw_gguf. */
bool qw_gguf_load(qw_gguf *f, qw_gpu *g, unsigned parts, char *err, size_t errlen);
size_t qw_gguf_resident_bytes(const qw_gguf *f);
double qw_gguf_load_seconds(const qw_gguf *f);
/* Where a resident tensor lies: buffer, offset, type (false when it is not resident). */
bool qw_gguf_tensor_at(const qw_gguf *f, const qw_gguf_tensor *t, qw_tensor *out);
/* The MoE weights of one layer (blk.<layer>.ffn_*), checked against each other; D, I, E receive the layer's sizes. */
bool qw_gguf_moe_layer(const qw_gguf *f, int layer, qw_moe_layer *M, int *D, int *I, int *E, char *err, size_t errlen);

/* Keep only the tile-major copies of the routed experts: frees the GGUF-order bytes of this handle's arena
 * (qw_hip_buf_release_source, include/qw_hip_ext.h) once every layer's experts have been dispatched at least once. Only
 * for a handle that loaded the routed expert matrices alone (parts = QW_GG_MOE): the other tensors are read as they are,
 * so they belong to a second handle on the same directory. */
bool qw_gguf_release_source(qw_gguf *f, char *err, size_t errlen);

/* The weights of one hyper-connection (src/gguf.c:222-229, :250-252): which = 0 blk.<layer>.hc_attn_*, 1 blk.<layer>.hc_ffn_*,
 * 2 the output mixer (no inject rows; H->inject.buf stays NULL); D receives the width of a stream. The inject rows must be
 * exact in BF16 (they are converted as a small tensor), as the reference's kernel reads them as BF16. */
bool qw_gguf_hyper(const qw_gguf *f, int layer, int which, qw_hyper_w *H, int *D, char *err, size_t errlen);

#ifdef __cplusplus
}
#endif
