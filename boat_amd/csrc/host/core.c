/* core.c - errors, memory seam and reference-counted tensors with a host mirror and a device copy.
 *
 * Mirrors the behaviour of src/core/tensor.c:65-300 (zero-filled creation, ref/unref, views that
 * share their parent's payload), src/core/memory.c:46-247 (header-tracked allocation with
 * statistics; here the `device` argument selects real HBM) and src/core/error.c:1-79.
 */
#include "boat_internal.h"

#include <stdarg.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ errors */

static _Thread_local boat_error_t g_last_error = BOAT_SUCCESS;
static _Thread_local char g_last_message[256] = "";   /* the size of the reference's buffer (error.c:18): longer messages are cut at 255 bytes */

void boat_fail(boat_error_t code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_message, sizeof(g_last_message), fmt, ap);
    va_end(ap);
    g_last_error = code;
    /* the reference reports failures on stderr and returns NULL/false (dense.c:203-217) */
    fprintf(stderr, "Error: %s\n", g_last_message);
}

bool boat_hip_ok(int rc, const char* what) {
    if (rc == BH_OK) return true;
    boat_fail(rc == BH_ENOMEM ? BOAT_ERROR_OUT_OF_MEMORY : rc == BH_EINVAL ? BOAT_ERROR_INVALID_ARGUMENT : BOAT_ERROR_DEVICE,
              "%s: %s", what, bh_last_error());
    return false;
}

void boat_init(void) {
    if (bh_init() != BH_OK) boat_fail(BOAT_ERROR_DEVICE, "boat_init: %s", bh_last_error());
}
void boat_cleanup(void) { bh_shutdown(); }

const char* boat_error_string(boat_error_t error) {
    switch (error) {
        case BOAT_SUCCESS: return "Success";
        case BOAT_ERROR_INVALID_ARGUMENT: return "Invalid argument";
        case BOAT_ERROR_OUT_OF_MEMORY: return "Out of memory";
        case BOAT_ERROR_INVALID_OPERATION: return "Invalid operation";
        case BOAT_ERROR_DEVICE: return "Device error";
        case BOAT_ERROR_FILE_IO: return "File I/O error";
        case BOAT_ERROR_FORMAT: return "Format error";
        case BOAT_ERROR_NOT_IMPLEMENTED: return "Not implemented";
        case BOAT_ERROR_UNKNOWN: return "Unknown error";
        default: return "Invalid error code";
    }
}
boat_error_t boat_get_last_error(void) { return g_last_error; }
const char* boat_get_last_error_message(void) { return g_last_message; }
void boat_set_error(boat_error_t error, const char* message) {
    g_last_error = error;
    snprintf(g_last_message, sizeof(g_last_message), "%s", message ? message : "");
}
/* src/core/error.c:64-80 */
void boat_set_errorf(boat_error_t error, const char* format, ...) {
    va_list ap;
    va_start(ap, format);
    g_last_error = error;
    vsnprintf(g_last_message, sizeof(g_last_message), format ? format : "", ap);
    va_end(ap);
}
void boat_reset_error(void) { boat_clear_error(); }
void boat_clear_error(void) {
    g_last_error = BOAT_SUCCESS;
    g_last_message[0] = 0;
}
bool boat_has_error(void) { return g_last_error != BOAT_SUCCESS; }
void boat_hip_synchronize(void) { boat_hip_ok(bh_synchronize(), "boat_hip_synchronize"); }

/* ------------------------------------------------------------------ memory */

#define BOAT_MEM_MAGIC 0xB0A7A11Cu
typedef struct {
    uint32_t magic;
    uint32_t device;
    size_t size;
} mem_header_t;

static boat_memory_stats_t g_stats;

/* memory.c:28-43: allocated_bytes is what is live now, the block counts only grow */
static void stats_alloc(size_t size) {
    g_stats.allocated_bytes += size;
    g_stats.allocated_blocks++;
    if (g_stats.allocated_bytes > g_stats.peak_allocated_bytes) g_stats.peak_allocated_bytes = g_stats.allocated_bytes;
}
static void stats_free(size_t size) {
    g_stats.allocated_bytes -= size < g_stats.allocated_bytes ? size : g_stats.allocated_bytes;   /* a reset may lie between */
    g_stats.freed_bytes += size;
    g_stats.freed_blocks++;
}

/* device blocks handed out through the memory seam, so boat_memory_free can tell them apart */
static struct { void* ptr; size_t size; }* g_dev_blocks = NULL;
static size_t g_dev_count = 0, g_dev_cap = 0;

static void* device_block_alloc(size_t size) {
    void* p = bh_malloc(size);
    if (!p) {
        boat_fail(BOAT_ERROR_OUT_OF_MEMORY, "device allocation of %zu bytes failed: %s", size, bh_last_error());
        return NULL;
    }
    if (g_dev_count == g_dev_cap) {
        size_t cap = g_dev_cap ? g_dev_cap * 2 : 16;
        void* grown = realloc(g_dev_blocks, cap * sizeof(*g_dev_blocks));
        if (!grown) {
            bh_free(p);
            return NULL;
        }
        g_dev_blocks = grown;
        g_dev_cap = cap;
    }
    g_dev_blocks[g_dev_count].ptr = p;
    g_dev_blocks[g_dev_count].size = size;
    g_dev_count++;
    stats_alloc(size);
    return p;
}
static bool device_block_free(void* ptr) {
    for (size_t i = 0; i < g_dev_count; i++) {
        if (g_dev_blocks[i].ptr == ptr) {
            stats_free(g_dev_blocks[i].size);
            bh_free(ptr);
            g_dev_blocks[i] = g_dev_blocks[--g_dev_count];
            return true;
        }
    }
    return false;
}

void* boat_memory_allocate(size_t size, boat_device_t device, const char* file, int line) {
    (void)file;
    (void)line;
    if (size == 0) return NULL;   /* memory.c:48-50 */
    if (device == BOAT_DEVICE_HIP) return device_block_alloc(size);
    mem_header_t* h = (mem_header_t*)malloc(sizeof(mem_header_t) + size);
    if (!h) return NULL;
    h->magic = BOAT_MEM_MAGIC;
    h->device = (uint32_t)device;
    h->size = size;
    stats_alloc(size);
    return h + 1;
}
void* boat_memory_allocate_zero(size_t size, boat_device_t device, const char* file, int line) {
    void* p = boat_memory_allocate(size, device, file, line);
    if (p) boat_memory_set(p, 0, size, device);
    return p;
}
void boat_memory_free(void* ptr) {
    if (!ptr) return;
    if (device_block_free(ptr)) return;
    mem_header_t* h = (mem_header_t*)ptr - 1;
    if (h->magic != BOAT_MEM_MAGIC) {
        boat_fail(BOAT_ERROR_INVALID_ARGUMENT, "boat_memory_free: pointer %p was not allocated by boat_memory_allocate", ptr);
        return;
    }
    h->magic = 0;
    stats_free(h->size);
    free(h);
}
void boat_memory_free_safe(void** ptr_ptr) {   /* memory.c:137-142 */
    if (ptr_ptr && *ptr_ptr) {
        boat_memory_free(*ptr_ptr);
        *ptr_ptr = NULL;
    }
}
/* memory.c:189-227: a host block over-allocated by alignment + one word, the original pointer kept in the word before the
 * aligned address.  Device blocks come from hipMalloc, which aligns to 256 bytes and more: they are handed out as they are
 * when that satisfies the request (a header cannot be written into device memory from here). */
void* boat_memory_allocate_aligned(size_t size, size_t alignment, boat_device_t device, const char* file, int line) {
    if (alignment < sizeof(void*)) alignment = sizeof(void*);
    if (alignment & (alignment - 1)) {
        boat_fail(BOAT_ERROR_INVALID_ARGUMENT, "boat_memory_allocate_aligned: alignment %zu is not a power of two", alignment);
        return NULL;
    }
    if (device == BOAT_DEVICE_HIP) {
        void* p = boat_memory_allocate(size, device, file, line);
        if (p && ((uintptr_t)p & (alignment - 1))) {
            boat_memory_free(p);
            boat_fail(BOAT_ERROR_INVALID_ARGUMENT, "boat_memory_allocate_aligned: device blocks are aligned to 256 bytes, %zu was asked", alignment);
            return NULL;
        }
        return p;
    }
    const size_t total = size + alignment + sizeof(size_t);
    void* ptr = boat_memory_allocate(total, device, file, line);
    if (!ptr) return NULL;
    const uintptr_t aligned = ((uintptr_t)ptr + alignment + sizeof(size_t)) & ~(uintptr_t)(alignment - 1);
    *(void**)(aligned - sizeof(size_t)) = ptr;
    return (void*)aligned;
}
void boat_memory_free_aligned(const void* aligned_ptr) {
    if (!aligned_ptr) return;
    if (device_block_free((void*)aligned_ptr)) return;
    boat_memory_free(*(void**)((uintptr_t)aligned_ptr - sizeof(size_t)));
}
void* boat_memory_reallocate(void* ptr, size_t new_size, boat_device_t device, const char* file, int line) {
    /* memory.c:85-120: NULL allocates, size 0 frees, otherwise the block keeps its contents up to the smaller size */
    if (!ptr) return boat_memory_allocate(new_size, device, file, line);
    if (new_size == 0) {
        boat_memory_free(ptr);
        return NULL;
    }
    mem_header_t* h = (mem_header_t*)ptr - 1;
    if (device == BOAT_DEVICE_HIP || h->magic != BOAT_MEM_MAGIC) {
        boat_fail(BOAT_ERROR_INVALID_ARGUMENT, "boat_memory_reallocate: only host blocks of boat_memory_allocate can be resized");
        return NULL;
    }
    const size_t old_size = h->size;
    mem_header_t* grown = (mem_header_t*)realloc(h, sizeof(mem_header_t) + new_size);
    if (!grown) {
        fprintf(stderr, "Memory reallocation failed: %zu bytes at %s:%d\n", new_size, file ? file : "?", line);
        return NULL;
    }
    grown->size = new_size;
    stats_free(old_size);
    stats_alloc(new_size);
    return grown + 1;
}
void* boat_memory_allocate_device(size_t size, boat_device_t device, const char* file, int line) {
    return boat_memory_allocate(size, device, file, line);
}
void boat_memory_free_device(void* ptr, boat_device_t device) {
    (void)device;
    boat_memory_free(ptr);
}
void boat_memory_copy(void* dest, const void* src, size_t size, boat_device_t dest_device, boat_device_t src_device) {
    if (!dest || !src || size == 0) return;
    const bool dd = dest_device == BOAT_DEVICE_HIP, sd = src_device == BOAT_DEVICE_HIP;
    if (!dd && !sd) memcpy(dest, src, size);
    else if (dd && !sd) boat_hip_ok(bh_memcpy_h2d(dest, src, size), "boat_memory_copy");
    else if (!dd && sd) boat_hip_ok(bh_memcpy_d2h(dest, src, size), "boat_memory_copy");
    else boat_hip_ok(bh_memcpy_d2d(dest, src, size), "boat_memory_copy");
}
void boat_memory_set(void* dest, int value, size_t size, boat_device_t device) {
    if (!dest || size == 0) return;
    if (device != BOAT_DEVICE_HIP) {
        memset(dest, value, size);
        return;
    }
    if (value == 0) {
        boat_hip_ok(bh_memset_zero(dest, size), "boat_memory_set");
    } else {
        void* tmp = malloc(size);
        if (!tmp) return;
        memset(tmp, value, size);
        boat_hip_ok(bh_memcpy_h2d(dest, tmp, size), "boat_memory_set");
        free(tmp);
    }
}
boat_memory_stats_t boat_memory_get_stats(void) { return g_stats; }
void boat_memory_reset_stats(void) { memset(&g_stats, 0, sizeof(g_stats)); }
void boat_memory_print_stats(FILE* stream) {
    if (!stream) stream = stdout;
    fprintf(stream, "Memory: live %zu B, %zu blocks allocated so far, freed %zu B in %zu blocks, peak %zu B; device in use %zu B, cached %zu B\n",
            g_stats.allocated_bytes, g_stats.allocated_blocks, g_stats.freed_bytes, g_stats.freed_blocks,
            g_stats.peak_allocated_bytes, bh_bytes_in_use(), bh_bytes_cached());
}

/* ------------------------------------------------------------------ tensor */

size_t boat_dtype_size(boat_dtype_t dtype) {
    switch (dtype) {
        case BOAT_DTYPE_FLOAT64: return 8;
        case BOAT_DTYPE_FLOAT32: return 4;
        case BOAT_DTYPE_FLOAT16: return 2;
        case BOAT_DTYPE_FLOAT8: return 1;
        case BOAT_DTYPE_FLOAT4: return 1;
        case BOAT_DTYPE_INT64: return 8;
        case BOAT_DTYPE_INT32: return 4;
        case BOAT_DTYPE_UINT8: return 1;
        case BOAT_DTYPE_BITS2: return 1;
        case BOAT_DTYPE_BITS1: return 1;
        case BOAT_DTYPE_BOOL: return sizeof(bool);
        default: return 0;
    }
}
const char* boat_dtype_name(boat_dtype_t dtype) {
    static const char* names[] = {"float64", "float32", "float16", "float8", "float4", "int64",
                                  "int32", "uint8", "bits2", "bits1", "bool"};
    return (int)dtype >= 0 && dtype < BOAT_DTYPE_COUNT ? names[dtype] : "unknown";
}

static boat_tensor_t* tensor_alloc(const int64_t* shape, size_t ndim, boat_dtype_t dtype, boat_device_t device,
                                   boat_storage_t* share) {
    if (ndim > BOAT_MAX_DIMS || (ndim > 0 && !shape)) return NULL;
    if ((int)dtype < 0 || dtype >= BOAT_DTYPE_COUNT) return NULL;
    size_t n = 1;
    for (size_t i = 0; i < ndim; i++) {
        if (shape[i] < 0) return NULL;
        n *= (size_t)shape[i];
    }
    boat_tensor_t* t = (boat_tensor_t*)calloc(1, sizeof(*t));
    if (!t) return NULL;
    t->shape = (int64_t*)malloc(sizeof(int64_t) * (ndim ? ndim : 1));
    if (!t->shape) {
        free(t);
        return NULL;
    }
    if (ndim) memcpy(t->shape, shape, sizeof(int64_t) * ndim);
    t->ndim = ndim;
    t->dtype = dtype;
    t->device = device;
    t->nelements = n;
    t->nbytes = n * boat_dtype_size(dtype);
    /* packed types, tensor.c:105-115 */
    if (dtype == BOAT_DTYPE_FLOAT4) t->nbytes = (n + 1) / 2;
    else if (dtype == BOAT_DTYPE_BITS2) t->nbytes = (n + 3) / 4;
    else if (dtype == BOAT_DTYPE_BITS1) t->nbytes = (n + 7) / 8;
    t->is_contiguous = true;
    t->ref_count = 1;
    if (share) {
        t->st = share;
        share->refs++;
        t->is_view = true;
    } else {
        boat_storage_t* st = (boat_storage_t*)calloc(1, sizeof(*st));
        if (!st) {
            free(t->shape);
            free(t);
            return NULL;
        }
        st->nbytes = t->nbytes;
        st->refs = 1;
        t->st = st;   /* neither copy valid yet == logically all zeros (tensor.c:132 zero-fills) */
        stats_alloc(t->nbytes);
    }
    return t;
}

static void shadow_release(boat_storage_t* st);
static void storage_unref(boat_storage_t* st) {
    if (--st->refs > 0) return;
    shadow_release(st);
    free(st->host);
    if (st->dev) bh_buffer_unref(st->dev);
    stats_free(st->nbytes);
    free(st);
}

boat_tensor_t* boat_tensor_create(const int64_t* shape, size_t ndim, boat_dtype_t dtype, boat_device_t device) {
    if ((int)device < 0 || device >= BOAT_DEVICE_COUNT) return NULL;
    return tensor_alloc(shape, ndim, dtype, device, NULL);
}
boat_tensor_t* boat_tensor_create_like(const boat_tensor_t* other) {
    if (!other) return NULL;
    return boat_tensor_create(other->shape, other->ndim, other->dtype, other->device);
}
boat_tensor_t* bt_new_uninit(const int64_t* shape, size_t ndim, boat_device_t device) {
    return boat_tensor_create(shape, ndim, BOAT_DTYPE_FLOAT32, device);
}
boat_tensor_t* bt_new_like_uninit(const boat_tensor_t* like) {
    return like ? boat_tensor_create(like->shape, like->ndim, BOAT_DTYPE_FLOAT32, like->device) : NULL;
}

/* ---- coherent-pointer mode ----
 * Boat's callers keep the float* that boat_tensor_data() gave them: they write through it before a later call
 * (tests/unit/test_attention_gradient_check.c:22-41) and read results through it after one
 * (tests/unit/test_optimizer_adam.c:96-108).  The reference's pointer IS the tensor's storage, so this mode is the
 * default: a tensor whose pointer was handed out is "exposed": its host mirror is uploaded before every device read
 * (the caller may have written), and device writes to it are copied back before the public call returns (the caller
 * may read).  Correct for any caller, at the price of PCIe transfers for exposed tensors.  Switched off
 * (boat_hip_set_coherent_pointers(0) or BOAT_HIP_COHERENT_POINTERS=0), a pointer is only promised until the next call
 * that takes the tensor, and parameters stay resident on the device whatever the caller looked at. */
static int g_coherent = -1;
static int g_reference_exact = -1;

/* Reference-exact mode: every place where this library deliberately computes something else than the reference does
 * follows the reference instead (see boat_hip_set_reference_exact in boat_api.h). */
bool bt_reference_exact(void) {
    if (g_reference_exact < 0) {
        const char* e = getenv("BOAT_HIP_REFERENCE_EXACT");
        g_reference_exact = e && *e && *e != '0';
    }
    return g_reference_exact != 0;
}
void boat_hip_set_reference_exact(int enable) { g_reference_exact = enable != 0; }
static boat_storage_t** g_pending = NULL;
static size_t g_pending_n = 0, g_pending_cap = 0;

static bool coherent_mode(void) {
    if (g_coherent < 0) {
        const char* e = getenv("BOAT_HIP_COHERENT_POINTERS");   /* on unless the environment says 0 */
        g_coherent = !(e && *e == '0');
    }
    return g_coherent != 0;
}
void boat_hip_set_coherent_pointers(int enable) {
    bt_flush_exposed();
    g_coherent = enable != 0;
}

/* ---- the shadow of an exposed storage ----
 * Without it every device read of an exposed tensor has to upload the host mirror (the caller may have written) and wait,
 * and every write-back waits per tensor.  With it a read costs one memcmp of the mirror against the shadow (equal: the
 * device copy is current), an upload is a memcpy into the shadow plus a queued copy that nobody waits for, and the
 * write-backs of one call share one wait.  Page-locked memory is finite: storages above kShadowLimit keep the plain path. */
static const size_t kShadowLimit = (size_t)256 << 20;
static uint64_t g_ticket = 0, g_synced_ticket = 0;   /* queued uploads issued / known to have completed */

static void stream_synced(void) { g_synced_ticket = g_ticket; }
static bool shadow_ensure(boat_storage_t* st) {
    if (st->shadow) return true;
    if (!st->exposed || st->nbytes == 0 || st->nbytes > kShadowLimit) return false;
    st->shadow = bh_host_alloc(st->nbytes);
    st->shadow_valid = false;
    return st->shadow != NULL;
}
/* the shadow is about to be written (or freed): a queued upload out of it must have run */
static void shadow_settle(boat_storage_t* st) {
    if (st->shadow && st->upload_ticket > g_synced_ticket && bh_synchronize() == BH_OK) stream_synced();
}
static void shadow_release(boat_storage_t* st) {
    if (!st->shadow) return;
    shadow_settle(st);
    bh_host_free(st->shadow);
    st->shadow = NULL;
    st->shadow_valid = false;
}

static void mark_device_write(boat_storage_t* st) {
    st->shadow_valid = false;
    if (!st->exposed || st->pending) return;
    if (g_pending_n == g_pending_cap) {
        const size_t cap = g_pending_cap ? 2 * g_pending_cap : 64;
        boat_storage_t** grown = (boat_storage_t**)realloc(g_pending, cap * sizeof(*grown));
        if (!grown) return;   /* the tensor stays readable through boat_tensor_data(), which downloads */
        g_pending = grown;
        g_pending_cap = cap;
    }
    st->pending = true;
    st->refs++;               /* alive until written back */
    g_pending[g_pending_n++] = st;
}

/* One event per queued write-back when a call writes back several large tensors: the copy shadow -> mirror of one tensor
 * then runs while the next tensors are still crossing PCIe, instead of after a wait for all of them. */
static const size_t kPipelinedFlushMin = (size_t)8 << 20;
static bh_event_t** g_flush_events = NULL;
static size_t g_flush_events_n = 0;
static bool flush_events_ensure(size_t n) {
    if (n <= g_flush_events_n) return true;
    bh_event_t** grown = (bh_event_t**)realloc(g_flush_events, n * sizeof(*grown));
    if (!grown) return false;
    g_flush_events = grown;
    while (g_flush_events_n < n) {
        bh_event_t* e = bh_event_create();
        if (!e) return false;
        g_flush_events[g_flush_events_n++] = e;
    }
    return true;
}

void bt_flush_exposed(void) {
    if (g_pending_n == 0) return;
    /* storages with a shadow: all copies queued, then shadow -> mirror as they land; the others one waiting copy each */
    size_t queued = 0, queued_bytes = 0, shadowed = 0;
    for (size_t i = 0; i < g_pending_n; i++) {
        boat_storage_t* st = g_pending[i];
        if (st->refs > 1 && st->host && st->dev && st->dev_valid && !st->host_valid && st->exposed && st->nbytes && st->nbytes <= kShadowLimit) {
            shadowed++;
            queued_bytes += st->nbytes;
        }
    }
    const bool pipelined = shadowed > 1 && queued_bytes >= kPipelinedFlushMin && flush_events_ensure(shadowed);
    for (size_t i = 0; i < g_pending_n; i++) {
        boat_storage_t* st = g_pending[i];
        st->pending = false;
        if (!(st->refs > 1 && st->host && st->dev && st->dev_valid && !st->host_valid)) continue;
        if (shadow_ensure(st)) {
            shadow_settle(st);
            if (boat_hip_ok(bh_memcpy_d2h_async(st->shadow, bh_buffer_ptr(st->dev), st->nbytes), "write-back of an exposed tensor") &&
                (!pipelined || queued >= g_flush_events_n || boat_hip_ok(bh_event_record(g_flush_events[queued]), "write-back of an exposed tensor"))) {
                st->pending = true;   /* marks: copy queued (the queued-th of this call) */
                queued++;
                continue;
            }
        }
        if (boat_hip_ok(bh_memcpy_d2h(st->host, bh_buffer_ptr(st->dev), st->nbytes), "write-back of an exposed tensor")) {
            st->host_valid = true;
            stream_synced();
        }
    }
    const bool per_copy = pipelined && queued <= g_flush_events_n;
    bool landed = queued > 0 && !per_copy && boat_hip_ok(bh_synchronize(), "write-back of exposed tensors");
    if (landed) stream_synced();
    size_t nth = 0;
    for (size_t i = 0; i < g_pending_n; i++) {
        boat_storage_t* st = g_pending[i];
        if (st->pending) {
            st->pending = false;
            if (per_copy) landed = boat_hip_ok(bh_event_wait(g_flush_events[nth]), "write-back of exposed tensors");
            nth++;
            if (landed) {
                bt_bytes_copy(st->host, st->shadow, st->nbytes);
                st->host_valid = true;
                st->shadow_valid = true;
            }
        }
    }
    if (per_copy && landed && nth > 0) stream_synced();   /* the last event is behind everything queued before it */
    /* (a storage freed by the unref below may wait for the stream itself: only after every copy of this call was handled) */
    const size_t n = g_pending_n;
    g_pending_n = 0;
    for (size_t i = 0; i < n; i++) storage_unref(g_pending[i]);
}

static bool storage_host_ready(boat_storage_t* st) {
    if (!st->host) {
        st->host = calloc(1, st->nbytes ? st->nbytes : 1);
        if (!st->host) return false;
        if (!st->dev_valid) st->host_valid = true;   /* zero state */
    }
    if (!st->host_valid) {
        if (st->dev_valid) {
            if (!boat_hip_ok(bh_memcpy_d2h(st->host, bh_buffer_ptr(st->dev), st->nbytes), "tensor download")) return false;
            stream_synced();
            if (st->shadow) {          /* mirror and device agree again: so does the shadow */
                bt_bytes_copy(st->shadow, st->host, st->nbytes);
                st->shadow_valid = true;
            }
        } else {
            memset(st->host, 0, st->nbytes);
        }
        st->host_valid = true;
    }
    return true;
}

static bool storage_dev_ready(boat_storage_t* st, bool need_contents) {
    if (!st->dev) {
        const bool zero = need_contents && !st->host_valid;
        st->dev = bh_buffer_create(st->nbytes ? st->nbytes : 4, zero);
        if (!st->dev) {
            boat_fail(BOAT_ERROR_OUT_OF_MEMORY, "device allocation of %zu bytes failed: %s", st->nbytes, bh_last_error());
            return false;
        }
        if (zero) st->dev_valid = true;
    }
    /* an exposed tensor may have been written through the caller's pointer since the last upload: it was not if the
     * mirror still equals the shadow, the copy of what was uploaded or written back last */
    if (need_contents && st->exposed && !st->pending && st->host_valid &&
        !(st->dev_valid && st->shadow && st->shadow_valid && bt_bytes_equal(st->host, st->shadow, st->nbytes)))
        st->dev_valid = false;
    if (need_contents && !st->dev_valid) {
        if (st->host_valid && shadow_ensure(st)) {
            /* staged: the caller may overwrite the mirror as soon as this call returns, the queued copy reads the shadow */
            shadow_settle(st);
            bt_bytes_copy(st->shadow, st->host, st->nbytes);
            if (!boat_hip_ok(bh_memcpy_h2d_async(bh_buffer_ptr(st->dev), st->shadow, st->nbytes), "tensor upload")) return false;
            st->upload_ticket = ++g_ticket;
            st->shadow_valid = true;
        } else if (st->host_valid) {
            if (!boat_hip_ok(bh_memcpy_h2d(bh_buffer_ptr(st->dev), st->host, st->nbytes), "tensor upload")) return false;
            stream_synced();
        } else {
            if (!boat_hip_ok(bh_memset_zero(bh_buffer_ptr(st->dev), st->nbytes), "tensor zero fill")) return false;
        }
        st->dev_valid = true;
    }
    return true;
}

const float* bt_dev_read(const boat_tensor_t* t) {
    if (!t || !storage_dev_ready(t->st, true)) return NULL;
    return (const float*)((const char*)bh_buffer_ptr(t->st->dev) + t->offset);
}
float* bt_dev_write(boat_tensor_t* t) {
    if (!t) return NULL;
    /* a reshaped view covers its whole parent payload, so a full overwrite is still full; a slice covers a part of
     * it and the rest has to stay what it is */
    if (t->nbytes != t->st->nbytes) return bt_dev_rw(t);
    if (!storage_dev_ready(t->st, false)) return NULL;
    t->st->dev_valid = true;
    t->st->host_valid = false;
    mark_device_write(t->st);
    return (float*)bh_buffer_ptr(t->st->dev);
}
float* bt_dev_rw(boat_tensor_t* t) {
    if (!t || !storage_dev_ready(t->st, true)) return NULL;
    t->st->host_valid = false;
    mark_device_write(t->st);
    return (float*)((char*)bh_buffer_ptr(t->st->dev) + t->offset);
}

bool bt_is_zero(const boat_tensor_t* t) {
    return t && t->st && !t->st->host_valid && !t->st->dev_valid && !t->st->exposed && t->nbytes == t->st->nbytes;
}
bool bt_set_zero(boat_tensor_t* t) {
    if (!t || !t->st) return false;
    boat_storage_t* st = t->st;
    if (t->nbytes != st->nbytes || st->exposed || st->pending) return false;
    st->host_valid = false;
    st->dev_valid = false;
    st->shadow_valid = false;
    return true;
}
float* bt_dev_accumulate(boat_tensor_t* t, int* accumulate) {
    if (bt_is_zero(t)) {
        *accumulate = 0;
        return bt_dev_write(t);
    }
    *accumulate = 1;
    return bt_dev_rw(t);
}

boat_tensor_t* boat_tensor_from_data(const int64_t* shape, size_t ndim, boat_dtype_t dtype, const void* data) {
    boat_tensor_t* t = boat_tensor_create(shape, ndim, dtype, BOAT_DEVICE_CPU);
    if (!t) return NULL;
    if (data) {
        void* dst = bt_host_rw(t);
        if (!dst) {
            boat_tensor_free(t);
            return NULL;
        }
        memcpy(dst, data, t->nbytes);
    }
    return t;
}

void boat_tensor_free(boat_tensor_t* tensor) {
    if (!tensor) return;
    if (--tensor->ref_count == 0) {
        storage_unref(tensor->st);
        free(tensor->shape);
        free(tensor);
    }
}
void boat_tensor_ref(boat_tensor_t* tensor) {
    if (tensor) tensor->ref_count++;
}
void boat_tensor_unref(boat_tensor_t* tensor) { boat_tensor_free(tensor); }

const int64_t* boat_tensor_shape(const boat_tensor_t* t) { return t ? t->shape : NULL; }
size_t boat_tensor_ndim(const boat_tensor_t* t) { return t ? t->ndim : 0; }
boat_dtype_t boat_tensor_dtype(const boat_tensor_t* t) { return t ? t->dtype : BOAT_DTYPE_FLOAT32; }
boat_device_t boat_tensor_device(const boat_tensor_t* t) { return t ? t->device : BOAT_DEVICE_CPU; }
size_t boat_tensor_nbytes(const boat_tensor_t* t) { return t ? t->nbytes : 0; }
size_t boat_tensor_nelements(const boat_tensor_t* t) { return t ? t->nelements : 0; }
bool boat_tensor_is_contiguous(const boat_tensor_t* t) { return t ? t->is_contiguous : false; }

void* bt_host_rw(boat_tensor_t* tensor) {
    if (!tensor) return NULL;
    boat_storage_t* st = tensor->st;
    if (tensor->device == BOAT_DEVICE_HIP) return bt_dev_rw(tensor);
    if (!storage_host_ready(st)) return NULL;
    /* written through the pointer -- unless a shadow will tell whether it really was */
    if (!(st->exposed && st->shadow && st->shadow_valid)) st->dev_valid = false;
    return (char*)st->host + tensor->offset;
}
void* boat_tensor_data(const boat_tensor_t* tensor) {
    void* p = bt_host_rw((boat_tensor_t*)tensor);
    if (p && tensor->device != BOAT_DEVICE_HIP && coherent_mode()) tensor->st->exposed = true;   /* the caller keeps it */
    return p;
}
const void* boat_tensor_const_data(const boat_tensor_t* tensor) {
    if (!tensor) return NULL;
    if (tensor->device == BOAT_DEVICE_HIP) return bt_dev_read(tensor);
    if (!storage_host_ready(tensor->st)) return NULL;
    if (coherent_mode()) tensor->st->exposed = true;
    return (const char*)tensor->st->host + tensor->offset;
}

boat_tensor_t* boat_tensor_reshape(const boat_tensor_t* tensor, const int64_t* new_shape, size_t new_ndim) {
    if (!tensor || !new_shape) return NULL;
    size_t n = 1;
    for (size_t i = 0; i < new_ndim; i++) n *= (size_t)new_shape[i];
    if (n != tensor->nelements) {
        fprintf(stderr, "Error: Reshape element count mismatch: %zu != %zu\n", n, tensor->nelements);
        return NULL;
    }
    boat_tensor_t* v = tensor_alloc(new_shape, new_ndim, tensor->dtype, tensor->device, tensor->st);
    if (v) {
        v->is_contiguous = false;   /* the reference marks reshaped views so (tensor.c:289) */
        v->offset = tensor->offset;
    }
    return v;
}

/* tensor.c:302-456: a view that starts at element `start` (row-major) of a contiguous tensor and is read as a dense
 * tensor of the new extents, i.e. exact for ranges of the leading dimension (a batch of samples), which is how the
 * callers use it (examples/mnist/mnist_autodiff.c:2387-2392).  Steps other than 1 are refused, as there. */
boat_tensor_t* boat_tensor_slice(const boat_tensor_t* tensor, const size_t* start, const size_t* end, const size_t* step) {
    if (!tensor || !start || !end) return NULL;
    const size_t ndim = tensor->ndim;
    if (ndim == 0) {
        fprintf(stderr, "Error: Cannot slice scalar tensor\n");
        return NULL;
    }
    int64_t shape[BOAT_MAX_DIMS];
    for (size_t i = 0; i < ndim; i++) {
        if (step && step[i] == 0) {
            fprintf(stderr, "Error: Step cannot be zero\n");
            return NULL;
        }
    }
    for (size_t i = 0; i < ndim; i++) {
        const size_t dim = (size_t)tensor->shape[i], st = step ? step[i] : 1;
        if (start[i] >= dim || end[i] > dim || start[i] > end[i]) {
            fprintf(stderr, "Error: Invalid slice range for dimension %zu: [%zu, %zu) (dim size: %zu)\n", i, start[i], end[i], dim);
            return NULL;
        }
        shape[i] = (int64_t)((end[i] - start[i] + st - 1) / st);
        if (shape[i] == 0) {
            fprintf(stderr, "Error: Slice results in zero-size dimension %zu\n", i);
            return NULL;
        }
    }
    if (!tensor->is_contiguous) {
        fprintf(stderr, "Error: Slicing non-contiguous tensors not supported\n");
        return NULL;
    }
    size_t first = 0, stride = 1;
    for (size_t i = ndim; i-- > 0;) {
        first += start[i] * stride;
        stride *= (size_t)tensor->shape[i];
    }
    for (size_t i = 0; i < ndim; i++) {
        if (step && step[i] != 1) {
            fprintf(stderr, "Error: Non-unit step slicing not yet implemented\n");
            return NULL;
        }
    }
    boat_tensor_t* v = tensor_alloc(shape, ndim, tensor->dtype, tensor->device, tensor->st);
    if (!v) return NULL;
    v->offset = tensor->offset + first * boat_dtype_size(tensor->dtype);
    v->is_contiguous = false;   /* tensor.c:436 */
    if (v->offset + v->nbytes > tensor->st->nbytes) {   /* a range that is not made of whole leading rows can run past the payload */
        fprintf(stderr, "Error: slice does not fit the tensor's payload\n");
        boat_tensor_free(v);
        return NULL;
    }
    return v;
}

boat_tensor_t* boat_tensor_clone(const boat_tensor_t* tensor) {
    if (!tensor) return NULL;
    boat_tensor_t* c = boat_tensor_create_like(tensor);
    if (!c) return NULL;
    boat_storage_t* st = tensor->st;
    if (st->dev_valid) {
        float* dst = bt_dev_write(c);
        if (!dst || !boat_hip_ok(bh_memcpy_d2d(dst, (const char*)bh_buffer_ptr(st->dev) + tensor->offset, tensor->nbytes), "boat_tensor_clone")) {
            boat_tensor_free(c);
            return NULL;
        }
    } else if (st->host_valid) {
        void* dst = bt_host_rw(c);
        if (!dst) {
            boat_tensor_free(c);
            return NULL;
        }
        memcpy(dst, (const char*)st->host + tensor->offset, tensor->nbytes);
    }
    return c;
}

boat_tensor_t* boat_tensor_to_device(const boat_tensor_t* tensor, boat_device_t dev) {
    if (!tensor || (int)dev < 0 || dev >= BOAT_DEVICE_COUNT) return NULL;
    boat_tensor_t* out = boat_tensor_create(tensor->shape, tensor->ndim, tensor->dtype, dev);
    if (!out) return NULL;
    boat_storage_t* src = tensor->st;
    if (!src->dev_valid && !src->host_valid) return out;   /* zeros */
    if (dev == BOAT_DEVICE_HIP) {
        float* dst = bt_dev_write(out);
        bool ok = dst != NULL;
        if (ok && src->dev_valid) ok = boat_hip_ok(bh_memcpy_d2d(dst, (const char*)bh_buffer_ptr(src->dev) + tensor->offset, tensor->nbytes), "boat_tensor_to_device");
        else if (ok) ok = boat_hip_ok(bh_memcpy_h2d(dst, (const char*)src->host + tensor->offset, tensor->nbytes), "boat_tensor_to_device");
        if (!ok) {
            boat_tensor_free(out);
            return NULL;
        }
    } else {
        void* dst = bt_host_rw(out);
        bool ok = dst != NULL;
        if (ok && src->host_valid) memcpy(dst, (const char*)src->host + tensor->offset, tensor->nbytes);
        else if (ok) ok = boat_hip_ok(bh_memcpy_d2h(dst, (const char*)bh_buffer_ptr(src->dev) + tensor->offset, tensor->nbytes), "boat_tensor_to_device");
        if (!ok) {
            boat_tensor_free(out);
            return NULL;
        }
    }
    return out;
}

bool bt_same_shape(const boat_tensor_t* a, const boat_tensor_t* b) {
    if (!a || !b || a->ndim != b->ndim) return false;
    for (size_t i = 0; i < a->ndim; i++)
        if (a->shape[i] != b->shape[i]) return false;
    return true;
}
bool bt_is_f32(const boat_tensor_t* t) { return t && t->dtype == BOAT_DTYPE_FLOAT32; }
