/* Additions of the HIP backend that the reference's src/gpu.h has no counterpart for. None of them is needed by
 * the reference's callers; they exist because HBM is not host memory, and for measurement.
 *
 * Host shadow rules (qw_buf.ptr is host memory, the kernels read HBM):
 *   - host -> device, when a batch is submitted, for every buffer a dispatch of the batch binds:
 *       a buffer of at most QW_HIP_SMALL_BYTES is copied every time;
 *       a larger one is copied the first time it is bound and again only after qw_hip_buf_mark_dirty();
 *       qw_buf_wrap() buffers are copied once; device-only buffers never;
 *       none of this for a buffer that a submitted batch (or an earlier, flushed part of this one) binds in an
 *       output role and that has not been waited for yet: HBM then holds the newer contents (a layer's output that the
 *       next layer reads), and they stay until the wait copies them back.
 *   - device -> host, when the batch completes, for every buffer bound in an output role:
 *       always, unless the buffer is device-only or larger than QW_HIP_BIG_OUT_BYTES (then: qw_hip_buf_download()).
 */
#pragma once
#include "gpu.h"
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QW_HIP_SMALL_BYTES ((size_t)4 << 20)
#define QW_HIP_BIG_OUT_BYTES ((size_t)256 << 20)

/* Device memory without a host shadow (out->ptr = NULL). Zero-filled. For resident weights and scratch that the
 * host never looks at. */
bool qw_hip_buf_new_device(qw_gpu *g, size_t size, qw_buf *out);
/* The host changed a large buffer after its first use: copy it again at the next submit. */
void qw_hip_buf_mark_dirty(qw_buf *b);
/* Explicit copies (synchronous). upload/download move [offset, offset + len) between the shadow and HBM;
 * write/read move between caller memory and HBM (the only way to fill or inspect a device-only buffer). write and
 * write_fd also store the bytes in the host side of a buffer that has one (not a wrapped one: that memory is the
 * caller's), so that the upload at the buffer's next bind carries them. */
bool qw_hip_buf_upload(qw_buf *b, size_t offset, size_t len);
bool qw_hip_buf_download(qw_buf *b, size_t offset, size_t len);
bool qw_hip_buf_write(qw_buf *b, size_t offset, const void *src, size_t len);
bool qw_hip_buf_read(const qw_buf *b, size_t offset, void *dst, size_t len);
/* len bytes of the open file fd, from file offset file_off, into HBM at [offset, offset + len) of b: worker threads
 * pread() into pinned staging buffers and the DMA of one chunk runs while the next is read (no page of the file is
 * mapped). QW_HIP_LOAD_THREADS sets the number of threads (default 4, at most 16). Synchronous. */
bool qw_hip_buf_write_fd(qw_buf *b, size_t offset, int fd, uint64_t file_off, size_t len);
/* Device address of a buffer (for tools that pass it to their own code). */
void *qw_hip_buf_devptr(const qw_buf *b);

/* IQ3_S weight matrices of the MoE kernels are copied once, at their first use, into a tile-major layout that a wave
 * reads with fully coalesced loads (the copy costs 1792 / 1760 of the matrix's bytes of HBM; the GGUF bytes stay where
 * they are); IQ4_NL down matrices with rows of 640 values likewise (a copy of exactly their size). The copy is dropped when the source buffer is freed, marked dirty, uploaded, written, or bound as a
 * kernel's output. Buffers of at most QW_HIP_SMALL_BYTES with a host shadow are never copied. QW_HIP_REPACK=0 in the
 * environment, or qw_hip_set_repack(g, false), turns the copies off (kernels then read the GGUF rows directly). */
void qw_hip_set_repack(qw_gpu *g, bool on);
size_t qw_hip_packed_bytes(const qw_gpu *g);
/* Keep only the tile-major copies of a weight buffer: frees the buffer's device bytes (the GGUF-order rows) once the
 * copies that the kernels read have been made, i.e. after every matrix in it has been through a dispatch that makes one
 * (moe_gu_gg, moe_dn_gg, moe_pf_gg and qmv_gg over IQ3_S rows; moe_dn_gg over IQ4_NL rows of 320 or 640). Residency of
 * such a matrix drops from 2.018 to 1.018 times its bytes. Afterwards the buffer may only be bound as those weights:
 * a dispatch that no existing copy serves (another shape or split, a matrix that was never dispatched, dq_test, any output
 * role) fails the batch with a message, the explicit copy calls return false, qw_hip_buf_devptr gives NULL, and the
 * buffer is otherwise freed as usual. Returns false (and frees nothing, with a text in qw_hip_last_error) while copies
 * stand in for only a part of the buffer's bytes (a matrix in it has not been dispatched yet), or when the buffer is
 * written by a batch still in flight. Keep shared-expert and router tensors in buffers of their own: they are read in GGUF order. */
bool qw_hip_buf_release_source(qw_buf *b);
size_t qw_hip_released_bytes(const qw_gpu *g);

/* Optional: a batch whose launches (functions, grids, argument records) equal those of one of the last few batches —
 * a decode step over the same resident buffers — is instantiated as a HIP graph of kernel nodes and replayed from
 * then on for as long as the sequence stays the same (eight sequences are kept). Uploads of host-shadowed buffers and
 * the timing events stay outside the graph. Profiled batches and batches with launches on the side stream run
 * eagerly. Off by default: on the 48-layer decode step it measured 3.85 ms against 3.82 ms eager per step at 16
 * tokens and 1.72 against 1.73 ms at one (the step is bound by the GPU, not by the launches). QW_HIP_GRAPH=1 in the
 * environment at qw_gpu_open, or qw_hip_set_graphs(g, true), turns it on. Number of batches run as graphs so far: */
void qw_hip_set_graphs(qw_gpu *g, bool on);
unsigned qw_hip_graph_launches(const qw_gpu *g);

/* Measurement switches, read from the environment ONCE, by qw_gpu_open(); a batch takes the device's switches as they
 * are when it begins, and nothing reads the environment afterwards. A program that changes a variable while it holds
 * a device (the tests and the benchmark do, to time two forms on one shape) calls qw_hip_reload_switches() to have
 * them read again. Each switch routes a layer through kernels that other shapes or formats reach by themselves;
 * results do not change (tests/test_gpu_path.py runs a layer with each of them set).
 *   QW_HIP_FUSE=1             routed gate/up, down and combine of a layer run as one launch whose workgroups meet at a barrier
 *                             (qwk_gud_*: tile-major IQ3_S rows with D <= 2048, I = 512, top-k <= 10, on stream 0). Off by
 *                             default: the hand-over inside the launch costs what the two launch boundaries cost
 *   QW_HIP_ABLATE             MEASUREMENT ONLY, results are meaningless: the routed gate/up launch over tile-major IQ3_S rows runs
 *                             without decoding and matrix instructions (qwk_gu_f122_c2: same selection, staging, loads and
 *                             stores), so that bench.py can state what the launch costs without its arithmetic
 *   QW_HIP_HC_ROWS=4|8|16     mix_down rows per workgroup of the hyper-connection's down launch (default: 4 up to twelve tokens, else 8)
 *   QW_HIP_SPIN_LIMIT=n       polls of the barrier word after which a workgroup of that launch stops waiting for the others
 *                             (default 65536, some tenths of a second). A launch that gives up fails its batch with a message
 *                             (negative time from qw_batch_end); the device then keeps its layers as separate launches until
 *                             qw_hip_reload_switches() is called. All workgroups of such a launch must be resident at once:
 *                             it is used on stream 0 only and never by qw_path_gg_moe_noalloc (the caller's stream).
 *   QW_HIP_DNC_NB=n           token count up to which moe_dn_gg + moe_cmb_gg run as one launch (default 2, at most 4; 0: never)
 *   QW_HIP_DNQ_MIN=n          token count from which (up to 16) they run as the one launch by token shares, for tile-major IQ3_S
 *                             down rows (default 2; 0: never)
 *   QW_HIP_PK_SPLIT           the packing sequence (p_zero, moe_count, moe_plan_t, moe_scatter, moe_pf_gg x 2, p_act2) one launch per
 *                             dispatch instead of one launch for the first four and SwiGLU inside the gate / up launch
 *   QW_HIP_SIDE=1             a shared expert's gate/up in the K-quant / IQ4 / plain formats runs on a side stream beside the router
 *   QW_HIP_DN_ANY             IQ4_NL down rows take the any-shape kernel instead of the range kernel
 *   QW_HIP_NL_C4              IQ4_NL down rows from GGUF order in chunks of four blocks instead of ten
 *   QW_HIP_NO_SWIGLU_MATVEC   such a shared expert's gate/up as two launches (matvec, then SwiGLU) instead of one
 *   QW_HIP_KQ_OWN_LAUNCH      such a shared expert's gate/up as a launch of its own instead of on the workgroups behind the router's
 *   QW_HIP_SHARED_IN_GU       an IQ3_S / Q8_0 shared expert's gate/up inside the gate/up launch instead of the front launch
 *   QW_HIP_SPLIT_SELECT       the selection as a launch of its own instead of inside the gate/up launch
 * Read at the same two places: QW_HIP_LOAD_THREADS (threads of qw_hip_buf_write_fd), QW_HIP_VERBOSE (every error text
 * goes to stderr as it is set) and QW_HIP_QUIET (qw_batch_wait prints none). QW_HIP_REPACK=0 and QW_HIP_GRAPH=1 are
 * read by qw_gpu_open() only (see above); afterwards qw_hip_set_repack / qw_hip_set_graphs change them. */
void qw_hip_reload_switches(qw_gpu *g);
/* The device's synchronisation words (the first 384 are the barrier's: all zero between launches except word 0, the
 * generation; word 352 is the error word), copied to dst after a device synchronisation. For tests. */
bool qw_hip_sync_words(qw_gpu *g, uint32_t *dst, size_t nwords);

/* The define-block front end of qw_gpu_compile() without a device: parses src as qw_gpu_compile would, and on
 * success writes the names of the kernels it would register to names (comma separated). For host-side tests. */
bool qw_hip_compile_check(const char *src, size_t len, char *err, size_t errlen, char *names, size_t nameslen);

/* Last error text of this device (empty string if none); cleared by qw_batch_begin. */
const char *qw_hip_last_error(const qw_gpu *g);
/* Number of compute units and the name of the code-object architecture the library was built for. */
int qw_hip_cu_count(const qw_gpu *g);
const char *qw_hip_arch(void);

/* Average duration in seconds of the kernel whose entry-point name starts with `prefix`, over the dispatches of
 * the last completed batch that ran with profiling enabled; count receives how many matched. */
double qw_hip_profile_mean(const qw_gpu *g, const char *prefix, int *count);
/* Entry i of the last profiled batch by the code object's entry-point name (qw_profile_get gives the caller's
 * kernel name); one entry per launch, in launch order. */
const char *qw_hip_profile_entry(const qw_gpu *g, int i, double *us);

#ifdef __cplusplus
}
#endif
