/* GPU interface of the quantized decode path — the drop-in boundary.
 *
 * This header declares, symbol for symbol, the C interface the reference declares in src/gpu.h (its lines are
 * cited per declaration below) so that the reference's callers of this path — gg_moe(), qmv_gg(), gg_router()
 * in src/engine.c:439-724 and the small drivers tools/dqtest.c, tools/ggmtest.c, bench/moe_bw.c — compile and
 * link against libqwgpu_hip.so instead of gpu_metal.o without a source change. The implementation is
 * qwental_amd/csrc/gpu_hip.c (C23 over the HIP runtime); the kernels are HIP code for gfx950.
 *
 * Differences a caller can observe, all forced by a discrete GPU with its own HBM:
 *   - qw_buf.ptr is a host shadow of a device allocation, not shared memory. The backend copies host -> device
 *     when a batch that reads the buffer is submitted, and device -> host when a batch that wrote it completes
 *     (rules in qw_hip_ext.h: small buffers every time, large buffers once unless marked). After
 *     qw_batch_end / qw_batch_wait the shadow of every output buffer is current, as the callers expect.
 *   - qw_gpu_compile() receives the reference's kernel source with the caller's "#define" block in front. The
 *     block is the operator interface: its parameter macros and its "#define <kernel> <new name>" renames select
 *     and name a prebuilt gfx950 kernel. The Metal text after the block is ignored.
 *   - Launch geometry: callers pass grids sized for 32-wide SIMD groups. The backend knows each kernel family and
 *     launches its own wave64 geometry derived from the bound arguments; the caller's numbers are validated only.
 */
#pragma once
#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct qw_gpu qw_gpu;       /* src/gpu.h:7 */
typedef struct qw_kernel qw_kernel; /* src/gpu.h:8 */
typedef struct qw_batch qw_batch;   /* src/gpu.h:9 */

/* src/gpu.h:11-15. handle: backend object (device allocation record); ptr: host-addressable bytes; size in bytes. */
typedef struct {
    void *handle;
    void *ptr;
    size_t size;
} qw_buf;

/* ---- device (src/gpu.h:18-21). open returns NULL when no HIP device is usable. */
qw_gpu *qw_gpu_open(void);
void qw_gpu_close(qw_gpu *g);
const char *qw_gpu_name(const qw_gpu *g);
size_t qw_gpu_max_working_set(const qw_gpu *g); /* total HBM in bytes */

/* ---- kernels (src/gpu.h:25-30).
 * compile: true on success with err[0] = 0; false with a message in err when the define block asks for a kernel
 * family, format or shape that has no gfx950 build. A block that renames nothing known succeeds and registers
 * nothing (qw_kernel_get then returns NULL, which the reference's callers turn into exit(1), src/engine.c:513-514).
 * qw_kernel_get: exact-name lookup; the pointer stays valid until qw_gpu_close.
 * max_threads: 1024. simd_width: 64. */
bool qw_gpu_compile(qw_gpu *g, const char *src, size_t len, char *err, size_t errlen);
qw_kernel *qw_kernel_get(qw_gpu *g, const char *name);
unsigned qw_kernel_max_threads(const qw_kernel *k);
unsigned qw_kernel_simd_width(const qw_kernel *k);

/* ---- buffers (src/gpu.h:33-40). new: zero-filled device memory + zero-filled host shadow. free clears the struct.
 * pool push/pop exist for the reference's autorelease pools and do nothing here.
 * wrap: ptr must be page aligned (false otherwise, as in the reference); the bytes are copied to HBM once, at the
 * first batch that binds the buffer, and out->ptr stays the caller's pointer. */
bool qw_buf_new(qw_gpu *g, size_t size, qw_buf *out);
void qw_buf_free(qw_buf *b);
void *qw_pool_push(void);
void qw_pool_pop(void *pool);
bool qw_buf_wrap(qw_gpu *g, void *ptr, size_t len, qw_buf *out);

/* ---- batches (src/gpu.h:45-63). A batch is an ordered list of dispatches on one in-order HIP stream.
 * Bindings are sticky across dispatches, indices 0..31; inline bytes are limited to 256 per index.
 * dispatch takes the grid in threadgroups, as the reference does. barrier is a no-op on an in-order stream.
 * flush submits what is recorded so far and keeps recording. end = submit + wait. wait returns the GPU execution
 * time in seconds (HIP events around the batch's kernels; host<->device copies are outside it), negative on any
 * failure (unknown kernel, missing or undersized binding, HIP error), and frees the batch. */
qw_batch *qw_batch_begin(qw_gpu *g, bool concurrent);
void qw_batch_kernel(qw_batch *b, qw_kernel *k);
void qw_batch_buf(qw_batch *b, unsigned index, const qw_buf *buf, size_t offset);
void qw_batch_bytes(qw_batch *b, unsigned index, const void *data, size_t len);
void qw_batch_threadgroup_mem(qw_batch *b, unsigned index, size_t len);
void qw_batch_dispatch(qw_batch *b, unsigned gx, unsigned gy, unsigned gz, unsigned tx, unsigned ty, unsigned tz);
void qw_batch_barrier(qw_batch *b);
void qw_batch_flush(qw_batch *b);
double qw_batch_end(qw_batch *b);
void qw_batch_submit(qw_batch *b);
double qw_batch_wait(qw_batch *b);
bool qw_batch_poll(qw_batch *b);
/* src/gpu.h:66. Two independent in-order streams, 0 (default) and 1; both at the default priority. */
void qw_gpu_set_stream(qw_gpu *g, int s);

/* ---- profiling (src/gpu.h:70-72): per-dispatch microseconds and kernel name of the last completed batch. */
void qw_profile_enable(qw_gpu *g, bool on);
int qw_profile_count(const qw_gpu *g);
const char *qw_profile_get(const qw_gpu *g, int i, double *us);

/* ---- bench utilities (src/gpu.h:75-83). empty_commit_latency: mean wall seconds of n empty submissions.
 * power_desc / on_battery describe a laptop in the reference; here: a fixed description and false. */
double qw_gpu_empty_commit_latency(qw_gpu *g, qw_kernel *k, int n);
void qw_power_desc(char *out, size_t len);
bool qw_on_battery(void);
double qw_now(void); /* monotonic seconds */

#ifdef __cplusplus
}
#endif
