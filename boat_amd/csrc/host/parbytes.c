/* parbytes.c - comparing and copying large host buffers on a few threads.
 *
 * A tensor whose data pointer the caller holds (src/core/tensor.c:65-135: the pointer is the storage) is compared with
 * the copy of what was last uploaded before every device read, and copied back after every device write (core.c).  One
 * core moves about 30 GB/s; for the weights of a large layer that is milliseconds per call.  From kParallelMin bytes on
 * the work is cut into page-aligned pieces for three helper threads and the calling thread.  The helpers are started on
 * first use and sleep on a condition variable in between; a process that forked after that (the helpers do not exist
 * in the child) and any failure to start them leave the single-threaded path.
 */
#include "boat_internal.h"

#include <pthread.h>
#include <string.h>
#include <unistd.h>

enum { kHelpers = 3 };
static const size_t kParallelMin = (size_t)2 << 20;

typedef struct {
    const char* a;      /* compare: first operand; copy: source */
    const char* b;      /* compare: second operand; copy: NULL */
    char* dst;          /* copy: destination */
    size_t n;
    bool equal;         /* compare: result */
} piece_t;

static pthread_mutex_t g_mu = PTHREAD_MUTEX_INITIALIZER;
static pthread_cond_t g_go = PTHREAD_COND_INITIALIZER, g_done = PTHREAD_COND_INITIALIZER;
static piece_t g_piece[kHelpers];
static unsigned g_posted[kHelpers], g_taken[kHelpers];   /* a helper runs its piece when posted != taken */
static int g_running = 0;                                /* pieces handed out and not finished */
static int g_state = 0;                                  /* 0 not started, 1 helpers alive, -1 unavailable */
static pid_t g_owner = 0;

static void run_piece(piece_t* p) {
    if (p->b) p->equal = memcmp(p->a, p->b, p->n) == 0;
    else memcpy(p->dst, p->a, p->n);
}

static void* helper_main(void* arg) {
    const int id = (int)(intptr_t)arg;
    pthread_mutex_lock(&g_mu);
    for (;;) {
        while (g_posted[id] == g_taken[id]) pthread_cond_wait(&g_go, &g_mu);
        g_taken[id] = g_posted[id];
        pthread_mutex_unlock(&g_mu);
        run_piece(&g_piece[id]);
        pthread_mutex_lock(&g_mu);
        if (--g_running == 0) pthread_cond_signal(&g_done);
    }
    return NULL;
}

static bool helpers_ready(void) {
    if (g_state == 1 && g_owner != getpid()) g_state = -1;   /* forked: the helpers stayed with the parent */
    if (g_state != 0) return g_state == 1;
    g_state = -1;
    pthread_attr_t attr;
    if (pthread_attr_init(&attr) != 0) return false;
    pthread_attr_setdetachstate(&attr, PTHREAD_CREATE_DETACHED);
    int started = 0;
    for (; started < kHelpers; started++) {
        pthread_t th;
        if (pthread_create(&th, &attr, helper_main, (void*)(intptr_t)started) != 0) break;
    }
    pthread_attr_destroy(&attr);
    /* helpers that did start and are never posted to sleep for good */
    if (started == kHelpers) {
        g_state = 1;
        g_owner = getpid();
    }
    return g_state == 1;
}

/* cut [0, n) into kHelpers + 1 pieces on 4 KiB boundaries, hand the first kHelpers out, run the last one here */
static bool run_parallel(const char* a, const char* b, char* dst, size_t n) {
    const size_t each = (n / (kHelpers + 1)) & ~(size_t)4095;
    piece_t mine = {a + kHelpers * each, b ? b + kHelpers * each : NULL, dst ? dst + kHelpers * each : NULL, n - kHelpers * each, true};
    pthread_mutex_lock(&g_mu);
    for (int i = 0; i < kHelpers; i++) {
        g_piece[i] = (piece_t){a + i * each, b ? b + i * each : NULL, dst ? dst + i * each : NULL, each, true};
        g_posted[i]++;
    }
    g_running = kHelpers;
    pthread_cond_broadcast(&g_go);
    pthread_mutex_unlock(&g_mu);
    run_piece(&mine);
    pthread_mutex_lock(&g_mu);
    while (g_running > 0) pthread_cond_wait(&g_done, &g_mu);
    bool equal = mine.equal;
    for (int i = 0; i < kHelpers; i++) equal = equal && g_piece[i].equal;
    pthread_mutex_unlock(&g_mu);
    return equal;
}

bool bt_bytes_equal(const void* a, const void* b, size_t n) {
    if (n < kParallelMin || !helpers_ready()) return memcmp(a, b, n) == 0;
    return run_parallel((const char*)a, (const char*)b, NULL, n);
}

void bt_bytes_copy(void* dst, const void* src, size_t n) {
    if (n < kParallelMin || !helpers_ready()) {
        memcpy(dst, src, n);
        return;
    }
    run_parallel((const char*)src, NULL, (char*)dst, n);
}
