// Scratch memory for the entry point that allocates nothing (qw_path_gg_moe_noalloc, include/qw_path.h).
//
// The intermediates of a MoE decode layer (lookup tables, logits, selection record, H, Psh, Pg) live in a file-scope
// device array instead of buffers from hipMalloc, so that callers which must not allocate (a stream under graph
// capture, a serving loop with a fixed memory budget) can run the layer. Every device the library runs on holds its own
// copy of the array, at its own address, until the process ends. In host code the array's name is only a handle for
// hipGetSymbolAddress: the address a kernel may use is the one that call returns, asked for once per device with that
// device current, and kept here. Everything else in the library takes that address as an ordinary pointer.
#include <hip/hip_runtime.h>
#include <stddef.h>
#include "qw_internal.h"

static __device__ __align__(256) unsigned char scratch[QW_NOALLOC_SCRATCH_BYTES];

enum { QW_NOALLOC_MAX_DEVICES = 16 };
static void *scratch_ptr[QW_NOALLOC_MAX_DEVICES]; // per device; NULL until asked for

extern "C" __attribute__((visibility("hidden"))) bool qw_noalloc_scratch(int dev, void **ptr, size_t *bytes, const char **err) {
    static const char *const e_dev = "device index outside the table of scratch addresses", *const e_cur = "hipSetDevice failed",
                             *const e_sym = "hipGetSymbolAddress(scratch) failed";
    *ptr = NULL;
    *bytes = 0;
    if (dev < 0 || dev >= QW_NOALLOC_MAX_DEVICES) { *err = e_dev; return false; }
    if (!scratch_ptr[dev]) {
        int cur = -1;
        if (hipGetDevice(&cur) != hipSuccess || (cur != dev && hipSetDevice(dev) != hipSuccess)) { *err = e_cur; return false; }
        void *p = NULL;
        const hipError_t rc = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (cur != dev && cur >= 0) (void)hipSetDevice(cur);
        if (rc != hipSuccess || !p) { (void)hipGetLastError(); *err = e_sym; return false; }
        scratch_ptr[dev] = p;
    }
    *ptr = scratch_ptr[dev];
    *bytes = QW_NOALLOC_SCRATCH_BYTES;
    return true;
}
