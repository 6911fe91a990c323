/* Declarations shared by the library's own translation units and not exported (hidden visibility). */
#pragma once
#include "gpu.h"
#include <stdbool.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QW_INTERNAL __attribute__((visibility("hidden")))

/* Size of the per-device scratch array of the entry point that allocates nothing (csrc/qw_noalloc.hip): the layer's
 * intermediates at the largest shape that entry point takes (16 tokens, D 2560, I 640, E 1024, top-16), 4 MiB. */
#define QW_NOALLOC_SCRATCH_BYTES ((size_t)4 << 20)

/* The device address of that array on device dev (looked up once per device) and its size; false + a text on failure. */
QW_INTERNAL bool qw_noalloc_scratch(int dev, void **ptr, size_t *bytes, const char **err);

/* gpu_hip.c: what the no-allocation entry point needs from the backend. */
typedef struct { _Alignas(16) unsigned char s[160]; } qw_hip_view; /* storage of one buffer handle, owned by the caller */
/* out becomes a qw_buf over [devptr, devptr + size) of device memory that someone else owns: device-only, never copied, never freed. */
QW_INTERNAL void qw_hip_view_init(qw_gpu *g, qw_hip_view *v, void *devptr, size_t size, qw_buf *out);
/* The device's scratch array (set up by qw_gpu_open); false + qw_hip_last_error when the set-up failed. */
QW_INTERNAL bool qw_hip_noalloc_scratch(qw_gpu *g, void **ptr, size_t *bytes);
/* The device's one recorder with fixed storage (64 launches): tile-major copies are only looked up, never made. NULL while
 * it is in use. stream: a hipStream_t, or NULL for the stream qw_gpu_set_stream selected. */
QW_INTERNAL qw_batch *qw_hip_batch_begin_static(qw_gpu *g, void *stream);
/* Launches what was recorded, in order, on the recorder's stream and releases the recorder; no copies, no events, no
 * synchronisation. recorded: whether the caller's recording went through; when it did not, or when a dispatch was
 * refused, nothing is launched. false + qw_hip_last_error in those cases and when a launch failed. */
QW_INTERNAL bool qw_hip_batch_launch_static(qw_batch *b, bool recorded);

#ifdef __cplusplus
}
#endif
