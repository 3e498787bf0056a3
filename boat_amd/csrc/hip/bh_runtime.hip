// bh_runtime.hip - device, stream, cached device memory, reference-counted buffers, events.
//
// Replaces the device seam the reference leaves unimplemented: boat_memory_allocate's
// `device` argument is recorded and ignored (src/core/memory.c:46-74), the device
// allocators are stubs (:174-186) and cross-device copies print "not implemented"
// (:230-247).  Here device memory is real HBM, handed out from a size-keyed cache so
// that the many short-lived temporaries of a backward pass cost no hipMalloc/hipFree.
// Reuse is safe without events because every kernel and copy of this library runs on
// the one stream: a block freed by the host is only re-issued to work enqueued later.
#include "bh_common.h"

#include <stdarg.h>
#include <string.h>

#include <map>
#include <vector>
#include <mutex>
#include <unordered_map>

namespace bh {

static hipStream_t g_stream = nullptr;
static bool g_ready = false;
static char g_err[512] = "";
static char g_name[256] = "";
static int g_cus = 0;
static std::mutex g_mu;

// cache: free blocks keyed by capacity; live blocks remember their capacity
static std::multimap<size_t, void*> g_free;
static std::unordered_map<void*, size_t> g_live;
static size_t g_in_use = 0, g_cached = 0;

hipStream_t stream() { return g_stream; }
bool ready() { return g_ready; }

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return BH_OK;
    return set_error(BH_EDEVICE, "%s: %s", what, hipGetErrorString(e));
}

// ---- profiling: one start/stop event pair per instrumented call, taken from a pool created when profiling is
// switched on (nothing is created inside a timed region); of nested scopes (bh_dense_backward calling bh_gemm) only
// the outermost is recorded.  A benchmark hook for ONE host thread: this state is not guarded by the library's
// mutex, so while profiling is on no second thread may call into the library.
struct ProfRec {
    int cls;
    double work;
    hipEvent_t a, b;
};
static bool g_prof_on = false;
static std::vector<ProfRec> g_prof;
static std::vector<hipEvent_t> g_prof_pool;
static int g_prof_depth = 0;

void prof_open(int cls, double work, int* slot) {
    *slot = -1;
    if (!g_prof_on) return;
    *slot = -2;
    if (g_prof_depth++ > 0) return;          // called from an instrumented entry point: the outer call is the record
    if (g_prof_pool.size() < 2) return;
    ProfRec r{cls, work, g_prof_pool.back(), nullptr};
    g_prof_pool.pop_back();
    r.b = g_prof_pool.back();
    g_prof_pool.pop_back();
    if (hipEventRecord(r.a, g_stream) != hipSuccess) {   // not recorded: the pair goes back to the pool
        g_prof_pool.push_back(r.b);
        g_prof_pool.push_back(r.a);
        return;
    }
    g_prof.push_back(r);
    *slot = (int)g_prof.size() - 1;
}
void prof_close(int slot) {
    if (g_prof_depth > 0) g_prof_depth--;
    if (slot >= 0 && slot < (int)g_prof.size()) (void)hipEventRecord(g_prof[slot].b, g_stream);
}

static size_t round_capacity(size_t n) {
    if (n == 0) n = 1;
    if (n <= (1u << 20)) return (n + 511) & ~size_t(511);          // 512 B granules below 1 MiB
    return (n + ((1u << 20) - 1)) & ~size_t((1u << 20) - 1);        // 1 MiB granules above
}

}  // namespace bh

using namespace bh;

extern "C" {

int bh_init(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_ready) return BH_OK;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n < 1)
        return set_error(BH_EDEVICE, "bh_init: no HIP device visible (%s)", hipGetErrorString(e));
    int rc = check_hip(hipSetDevice(0), "hipSetDevice");
    if (rc) return rc;
    hipDeviceProp_t prop;
    rc = check_hip(hipGetDeviceProperties(&prop, 0), "hipGetDeviceProperties");
    if (rc) return rc;
    snprintf(g_name, sizeof(g_name), "%s (%s)", prop.name, prop.gcnArchName);
    g_cus = prop.multiProcessorCount;
    rc = check_hip(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking), "hipStreamCreate");
    if (rc) return rc;
    rc = ln_scratch_setup();
    if (rc) return rc;
    g_ready = true;
    return BH_OK;
}

int bh_shutdown(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_ready) return BH_OK;
    (void)hipStreamSynchronize(g_stream);
    for (auto& kv : g_free) (void)hipFree(kv.second);
    g_free.clear();
    g_cached = 0;
    (void)hipStreamDestroy(g_stream);
    g_stream = nullptr;
    g_ready = false;
    return BH_OK;
}

int bh_synchronize(void) {
    BH_REQUIRE_INIT();
    return check_hip(hipStreamSynchronize(g_stream), "hipStreamSynchronize");
}

const char* bh_last_error(void) { return g_err; }
const char* bh_device_name(void) { return bh_init() == BH_OK ? g_name : ""; }
int bh_device_cu_count(void) { return bh_init() == BH_OK ? g_cus : 0; }
void* bh_stream(void) { return bh_init() == BH_OK ? (void*)g_stream : nullptr; }

void* bh_malloc(size_t nbytes) {
    if (!ready() && bh_init() != BH_OK) return nullptr;
    size_t cap = round_capacity(nbytes);
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_free.lower_bound(cap);
    // accept a cached block up to 12.5 % larger than asked
    if (it != g_free.end() && it->first <= cap + cap / 8) {
        void* p = it->second;
        size_t c = it->first;
        g_free.erase(it);
        g_cached -= c;
        g_live[p] = c;
        g_in_use += c;
        return p;
    }
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, cap);
    if (e != hipSuccess) {
        // give cached blocks back and retry once
        (void)hipStreamSynchronize(g_stream);
        for (auto& kv : g_free) (void)hipFree(kv.second);
        g_free.clear();
        g_cached = 0;
        e = hipMalloc(&p, cap);
        if (e != hipSuccess) {
            set_error(BH_ENOMEM, "bh_malloc(%zu): %s", nbytes, hipGetErrorString(e));
            return nullptr;
        }
    }
    g_live[p] = cap;
    g_in_use += cap;
    return p;
}

void bh_free(void* dptr) {
    if (!dptr) return;
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_live.find(dptr);
    if (it == g_live.end()) {
        set_error(BH_EINVAL, "bh_free: pointer %p was not handed out by bh_malloc", dptr);
        return;
    }
    size_t c = it->second;
    g_live.erase(it);
    g_in_use -= c;
    g_free.emplace(c, dptr);
    g_cached += c;
}

int bh_cache_release(void) {
    BH_REQUIRE_INIT();
    std::lock_guard<std::mutex> lk(g_mu);
    int rc = check_hip(hipStreamSynchronize(g_stream), "hipStreamSynchronize");
    for (auto& kv : g_free) (void)hipFree(kv.second);
    g_free.clear();
    g_cached = 0;
    return rc;
}

size_t bh_bytes_in_use(void) { return g_in_use; }
size_t bh_bytes_cached(void) { return g_cached; }

struct bh_buffer {
    void* ptr;
    size_t nbytes;
    int refs;
};

bh_buffer_t* bh_buffer_create(size_t nbytes, int zero_fill) {
    void* p = bh_malloc(nbytes);
    if (!p) return nullptr;
    if (zero_fill && bh_memset_zero(p, nbytes) != BH_OK) {
        bh_free(p);
        return nullptr;
    }
    bh_buffer_t* b = new bh_buffer_t{p, nbytes, 1};
    return b;
}
void bh_buffer_ref(bh_buffer_t* b) {
    if (b) b->refs++;
}
void bh_buffer_unref(bh_buffer_t* b) {
    if (!b) return;
    if (--b->refs == 0) {
        bh_free(b->ptr);
        delete b;
    }
}
void* bh_buffer_ptr(const bh_buffer_t* b) { return b ? b->ptr : nullptr; }
size_t bh_buffer_nbytes(const bh_buffer_t* b) { return b ? b->nbytes : 0; }
int bh_buffer_refcount(const bh_buffer_t* b) { return b ? b->refs : 0; }

int bh_memcpy_h2d(void* dst, const void* src, size_t nbytes) {
    BH_REQUIRE_INIT();
    if (nbytes == 0) return BH_OK;
    BH_CHECK_ARG(dst && src, "null pointer");
    // pageable source: the runtime stages it, so the host buffer is reusable on return
    int rc = check_hip(hipMemcpyAsync(dst, src, nbytes, hipMemcpyHostToDevice, g_stream), "memcpy h2d");
    if (rc) return rc;
    return check_hip(hipStreamSynchronize(g_stream), "memcpy h2d sync");
}
int bh_memcpy_d2h(void* dst, const void* src, size_t nbytes) {
    BH_REQUIRE_INIT();
    if (nbytes == 0) return BH_OK;
    BH_CHECK_ARG(dst && src, "null pointer");
    int rc = check_hip(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToHost, g_stream), "memcpy d2h");
    if (rc) return rc;
    return check_hip(hipStreamSynchronize(g_stream), "memcpy d2h sync");
}
void* bh_host_alloc(size_t nbytes) {
    if (!ready() && bh_init() != BH_OK) return nullptr;
    void* p = nullptr;
    if (hipHostMalloc(&p, nbytes ? nbytes : 1, hipHostMallocDefault) != hipSuccess) {
        (void)hipGetLastError();   /* the caller falls back to pageable memory: not an error of the library */
        return nullptr;
    }
    return p;
}
void bh_host_free(void* p) {
    if (p) (void)hipHostFree(p);
}
int bh_memcpy_h2d_async(void* dst, const void* src, size_t nbytes) {
    BH_REQUIRE_INIT();
    if (nbytes == 0) return BH_OK;
    BH_CHECK_ARG(dst && src, "null pointer");
    return check_hip(hipMemcpyAsync(dst, src, nbytes, hipMemcpyHostToDevice, g_stream), "memcpy h2d (queued)");
}
int bh_memcpy_d2h_async(void* dst, const void* src, size_t nbytes) {
    BH_REQUIRE_INIT();
    if (nbytes == 0) return BH_OK;
    BH_CHECK_ARG(dst && src, "null pointer");
    return check_hip(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToHost, g_stream), "memcpy d2h (queued)");
}
int bh_memcpy_d2d(void* dst, const void* src, size_t nbytes) {
    BH_REQUIRE_INIT();
    if (nbytes == 0) return BH_OK;
    BH_CHECK_ARG(dst && src, "null pointer");
    // whole floats go through a copy kernel on the stream: in order with the kernels around it and without the
    // runtime's blit path, whose set-up costs tens of microseconds between two small kernels
    if (((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src) | nbytes) & 3) == 0)
        return bh_copy_f32(static_cast<float*>(dst), static_cast<const float*>(src), (int64_t)(nbytes / 4));
    return check_hip(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToDevice, g_stream), "memcpy d2d");
}

int bh_profile_enable(int max_calls) {
    BH_REQUIRE_INIT();
    std::lock_guard<std::mutex> lk(g_mu);
    (void)hipStreamSynchronize(g_stream);
    for (auto& r : g_prof) {
        g_prof_pool.push_back(r.a);
        if (r.b) g_prof_pool.push_back(r.b);
    }
    g_prof.clear();
    g_prof_depth = 0;
    if (max_calls <= 0) {
        g_prof_on = false;
        for (hipEvent_t e : g_prof_pool) (void)hipEventDestroy(e);
        g_prof_pool.clear();
        return BH_OK;
    }
    while (g_prof_pool.size() < 2 * (size_t)max_calls) {
        hipEvent_t e;
        int rc = check_hip(hipEventCreate(&e), "hipEventCreate");
        if (rc) return rc;
        g_prof_pool.push_back(e);
    }
    g_prof.reserve((size_t)max_calls);
    g_prof_on = true;
    return BH_OK;
}

int bh_profile_read(int cls, double* total_ms, double* total_work, int64_t* calls) {
    BH_REQUIRE_INIT();
    int rc = check_hip(hipStreamSynchronize(g_stream), "hipStreamSynchronize");
    if (rc) return rc;
    double ms = 0.0, work = 0.0;
    int64_t n = 0;
    for (const ProfRec& r : g_prof) {
        if (r.cls != cls || !r.b) continue;
        float t = 0.f;
        if (hipEventElapsedTime(&t, r.a, r.b) != hipSuccess) continue;
        ms += t;
        work += r.work;
        n++;
    }
    if (total_ms) *total_ms = ms;
    if (total_work) *total_work = work;
    if (calls) *calls = n;
    return BH_OK;
}

struct bh_event {
    hipEvent_t ev;
};
bh_event_t* bh_event_create(void) {
    if (!ready() && bh_init() != BH_OK) return nullptr;
    bh_event_t* e = new bh_event_t;
    if (hipEventCreate(&e->ev) != hipSuccess) {
        delete e;
        return nullptr;
    }
    return e;
}
void bh_event_destroy(bh_event_t* e) {
    if (!e) return;
    (void)hipEventDestroy(e->ev);
    delete e;
}
int bh_event_record(bh_event_t* e) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(e, "null event");
    return check_hip(hipEventRecord(e->ev, g_stream), "hipEventRecord");
}
int bh_event_wait(bh_event_t* e) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(e, "null event");
    return check_hip(hipEventSynchronize(e->ev), "hipEventSynchronize");
}
float bh_event_elapsed_ms(bh_event_t* a, bh_event_t* b) {
    if (!a || !b) return -1.f;
    if (hipEventSynchronize(b->ev) != hipSuccess) return -1.f;
    float ms = -1.f;
    if (hipEventElapsedTime(&ms, a->ev, b->ev) != hipSuccess) return -1.f;
    return ms;
}

}  // extern "C"
