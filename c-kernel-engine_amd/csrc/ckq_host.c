/*
 * ckq_host.c - host layer of libckernel_quant_hip.so (plain C).
 *
 * Implements the reference engine's kernel symbols for the quantized
 * dequant-dot path (declared in include/ckernel_quant_hip.h, part 1) on top of
 * the device launchers of ckq_launch.h, plus the device-resident `_dev` entry
 * points and the library control calls.
 *
 * Host-pointer calls: activations are copied to the device, the kernel runs on
 * the library's stream, results are copied back and the stream is synchronized
 * before returning (the reference kernels are synchronous).  Weight matrices
 * are uploaded once and stay resident, keyed by host address, size and a
 * sampled fingerprint.  Device pointers are detected and used in place.
 * One mutex serializes the host-pointer entry points, so they may be called
 * from any number of threads (the reference's thread pool calls the same
 * symbol from every worker).
 *
 * There is no CPU fallback: if no gfx950 device is usable every entry point
 * reports the HIP error on stderr and aborts (set CKQ_ABORT_ON_ERROR=0 to get
 * the code from ckq_last_error() instead).
 */
#include <hip/hip_runtime_api.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <strings.h>
#include <time.h>
#include <unistd.h>

#include "ckernel_quant_hip.h"
#include "ckq_launch.h"
#include "ckq_pure.h"

/* ------------------------------------------------------------------------ */
/* State                                                                     */
/* ------------------------------------------------------------------------ */

typedef struct {
    const void *host;
    size_t      bytes;
    uint64_t    fp;
    void       *dev;
    int         pinned;   /* registered by the caller: serves any sub-range, content is not re-checked */
    uint64_t    last_use; /* value of g_use_clock at the last hit (eviction order of unpinned entries) */
} weight_entry;

typedef struct {
    void  *dev;
    size_t cap;
} dev_buf;

enum { BUF_X = 0, BUF_Y, BUF_BIAS, BUF_Q, BUF_GU, BUF_H, BUF_COUNT };

static pthread_mutex_t g_mu = PTHREAD_MUTEX_INITIALIZER;
static int          g_inited = 0;
static int          g_err = 0;            /* accessed with __atomic builtins: any thread may fail */
static int          g_cache_on = 1;
/* Thread-split entry points: 1 = the ith == 0 call computes all rows in one
 * launch and the other threads return (through the reference's 16-thread pool:
 * 53 us per GEMV against 480 us when each thread runs its own row range). */
#define CKQ_PARALLEL_WHOLE_DEFAULT 0
static int          g_parallel_whole = CKQ_PARALLEL_WHOLE_DEFAULT;
static hipStream_t  g_stream = NULL;
static dev_buf      g_buf[BUF_COUNT];
/* Pinned host twins of the staging buffers.  Small transfers (a decode step's
 * activation vector up, its outputs down) go through them: a copy between
 * pageable memory and the device makes the runtime stage and wait inside each
 * hipMemcpyAsync; a twin is device-visible, so the plain copy kernel moves
 * the bytes instead (measured for a 4.6 KB upload, a kernel and a 44 KB
 * download, synchronised once: 24 us pageable, 22 us with pinned copies, 18 us
 * with copy kernels).  Every host-pointer call ends in a stream
 * synchronisation, so a twin is free again when the next call starts. */
enum { PIN_MAX_BYTES = 1 << 20 };
typedef struct {
    void  *host;
    void  *dev;     /* the same memory as the device addresses it */
    size_t cap;
} pin_buf;
static pin_buf      g_pin[BUF_COUNT];
/* Inputs of a decode step (up to DIRECT_MAX_BYTES: an activation vector, a bias)
 * skip even that: MI300-class boards expose their whole memory to the CPU, and a
 * fine-grained allocation is coherent for the GPU, so the CPU copies such an
 * input straight into a device buffer (4.6 KB: 0.4 us of posted PCIe writes) and
 * no upload is launched at all (host-pointer GEMV 23.7 -> 19 us).  The buffers
 * are allocated once and kept until the process ends.  CKQ_DIRECT_UPLOAD=0, or
 * an allocation the CPU cannot address (probed without touching it from user
 * code), leaves the pinned twins in charge. */
enum { DIRECT_MAX_BYTES = 64 << 10 };
static void        *g_direct[BUF_COUNT];
static int          g_direct_ok = -1;      /* -1: not decided yet */
/* Completion word of the host-pointer calls: a dword of pinned memory that the
 * stream writes (hipStreamWriteValue32) once everything enqueued before it has
 * finished.  The caller spins on it for a bounded time instead of entering
 * hipStreamSynchronize, whose wake-up costs several microseconds on a call that
 * is a few tens long; when the word does not arrive in time, or the write cannot
 * be enqueued, the synchronisation call takes over. */
static volatile uint32_t *g_done_host = NULL;
static void              *g_done_dev = NULL;
static uint32_t           g_done_seq = 0;
static int                g_done_ok = 1;       /* cleared for good when the stream write is not available */
static weight_entry *g_w = NULL;
static size_t       g_nw = 0, g_capw = 0;
static size_t       g_cache_max_bytes = (size_t)64 << 30;   /* bound on unpinned resident weights */

/* ------------------------------------------------------------------------ */
/* Errors                                                                    */
/* ------------------------------------------------------------------------ */

const char *ckq_error_string(int code)
{
    switch (code) {
    case 0: return "success";
    case CKQ_EINVAL: return "invalid argument (NULL pointer or non-positive dimension)";
    case CKQ_ESHAPE: return "K is not a multiple of the quantization block size";
    case CKQ_EFORMAT: return "unknown weight format";
    case CKQ_ENODUMP: return "the integer dumps of the exactness tests are built into libckernel_quant_hip_dump.so, not into this library";
    case CKQ_ESCRATCH: return "the call needs more scratch than ckq_gemm_nt_noalloc_dev holds (4 MiB); use ckq_gemm_nt_dev or fewer tokens per call";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
    }
}

int ckq_last_error(void) { return __atomic_load_n(&g_err, __ATOMIC_RELAXED); }
void ckq_clear_error(void) { __atomic_store_n(&g_err, 0, __ATOMIC_RELAXED); }

static int fail(int code, const char *what)
{
    if (code == 0) return 0;
    __atomic_store_n(&g_err, code, __ATOMIC_RELAXED);
    fprintf(stderr, "libckernel_quant_hip: %s failed: %s (%d)\n", what, ckq_error_string(code), code);
    const char *e = getenv("CKQ_ABORT_ON_ERROR");
    if (!e || strcmp(e, "0") != 0) {
        fprintf(stderr, "libckernel_quant_hip: no CPU fallback exists; aborting (CKQ_ABORT_ON_ERROR=0 to continue)\n");
        abort();
    }
    return code;
}

#define HIP_TRY(expr)                                   \
    do {                                                \
        hipError_t e_ = (expr);                         \
        if (e_ != hipSuccess) return fail((int)e_, #expr); \
    } while (0)

/* An error path leaves its do-block after copies from the caller's buffers
 * may have been enqueued: wait for them, so that with CKQ_ABORT_ON_ERROR=0 the
 * call does not return while the device still reads the caller's memory. */
static void drain_after_error(void);

/* ------------------------------------------------------------------------ */
/* Init, buffers, pointer classification                                     */
/* ------------------------------------------------------------------------ */

static int init_locked(void)
{
    if (g_inited) return 0;
    int n = 0;
    HIP_TRY(hipGetDeviceCount(&n));
    if (n <= 0) return fail((int)hipErrorNoDevice, "hipGetDeviceCount");
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, dev));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        fprintf(stderr, "libckernel_quant_hip: device %d is %s; this library holds gfx950 code only\n", dev,
                prop.gcnArchName);
        return fail((int)hipErrorInvalidDeviceFunction, "architecture check");
    }
    HIP_TRY(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
    const char *c = getenv("CKQ_WEIGHT_CACHE");
    if (c && strcmp(c, "0") == 0) g_cache_on = 0;
    const char *mb = getenv("CKQ_WEIGHT_CACHE_MB");
    if (mb && atoll(mb) > 0) g_cache_max_bytes = (size_t)atoll(mb) << 20;
    const char *p = getenv("CKQ_PARALLEL_MODE");
    if (p) g_parallel_whole = strcmp(p, "whole") == 0;
    const char *gp = getenv("CKQ_GEMM_POLICY");
    if (gp && strcmp(gp, "matrix") == 0) ckq_launch_set_gemm_policy(CKQ_GEMM_MATRIX);
    if (gp && strcmp(gp, "stream") == 0) ckq_launch_set_gemm_policy(CKQ_GEMM_STREAM);
    const char *tile = getenv("CKQ_Q4K_TILE");
    if (tile) ckq_launch_set_q4k_tile(atoi(tile));
    const char *q6v = getenv("CKQ_Q6K_VARIANT");
    if (q6v) ckq_launch_set_q6k_variant(atoi(q6v));
    const char *q5v = getenv("CKQ_Q5K_VARIANT");
    if (q5v) ckq_launch_set_q5k_variant(atoi(q5v));
    /* address of the static scratch of the entry point that allocates nothing, for this device */
    {
        const int rc = ckq_launch_noalloc_setup();
        if (rc) return fail(rc, "ckq_launch_noalloc_setup");
    }
    g_inited = 1;
    return 0;
}

static void drain_after_error(void)
{
    if (g_inited && g_stream) {
        (void)hipStreamSynchronize(g_stream);
        (void)hipGetLastError();
    }
}

int ckq_init(void)
{
    pthread_mutex_lock(&g_mu);
    const int rc = init_locked();
    pthread_mutex_unlock(&g_mu);
    return rc;
}

int ckq_synchronize(void)
{
    pthread_mutex_lock(&g_mu);
    int rc = init_locked();
    if (rc == 0) {
        hipError_t e = hipStreamSynchronize(g_stream);
        if (e != hipSuccess) rc = fail((int)e, "hipStreamSynchronize");
    }
    pthread_mutex_unlock(&g_mu);
    return rc;
}

/* A host-pointer call classifies its operands (x, W, y) on every call, and the
 * same buffers come back token after token.  Addresses the runtime has
 * reported as plain host memory are remembered (a small direct-mapped table),
 * so the steady state asks the runtime nothing.  Only "host" is remembered,
 * never "device": should an address change hands, the stale answer makes the
 * CPU copy from it (at worst a host fault), never a kernel dereference it.
 * ckq_weights_clear() and ckq_weights_invalidate() empty the table. */
enum { PTR_CACHE = 64 };
static const void *g_host_ptr[PTR_CACHE];
static void ptr_cache_clear(void) { memset(g_host_ptr, 0, sizeof g_host_ptr); }

static int is_device_ptr(const void *p)
{
    const size_t slot = ((uintptr_t)p >> 6) % PTR_CACHE;
    if (p && g_host_ptr[slot] == p) return 0;
    hipPointerAttribute_t at;
    memset(&at, 0, sizeof(at));
    hipError_t e = hipPointerGetAttributes(&at, p);
    if (e != hipSuccess) {
        (void)hipGetLastError(); /* plain host memory: clear the sticky error */
        g_host_ptr[slot] = p;
        return 0;
    }
    if (at.type == hipMemoryTypeDevice || at.type == hipMemoryTypeManaged) return 1;
    if (at.type == hipMemoryTypeUnregistered) g_host_ptr[slot] = p;
    return 0;
}

/* Waits for the work enqueued on the library's stream so far. */
static int stream_wait(void)
{
    if (g_done_ok && !g_done_host) {
        void *h = NULL;
        if (hipHostMalloc(&h, 64, hipHostMallocDefault) == hipSuccess && hipHostGetDevicePointer(&g_done_dev, h, 0) == hipSuccess) {
            g_done_host = (volatile uint32_t *)h;
            *g_done_host = 0;
        } else {
            (void)hipGetLastError();
            g_done_ok = 0;
        }
    }
    if (g_done_ok) {
        const uint32_t seq = ++g_done_seq;
        if (hipStreamWriteValue32(g_stream, g_done_dev, seq, 0) == hipSuccess) {
            struct timespec t0, t1;
            clock_gettime(CLOCK_MONOTONIC, &t0);
            for (unsigned spins = 0;; ++spins) {
                if (*g_done_host == seq) return 0;
                __builtin_ia32_pause();
                if ((spins & 1023) == 1023) {
                    clock_gettime(CLOCK_MONOTONIC, &t1);
                    if ((t1.tv_sec - t0.tv_sec) * 1000000000L + (t1.tv_nsec - t0.tv_nsec) > 200000L) break;   /* 0.2 ms: a long job */
                }
            }
        } else {
            (void)hipGetLastError();
            g_done_ok = 0;
        }
    }
    HIP_TRY(hipStreamSynchronize(g_stream));
    return 0;
}

static int buf_reserve(int which, size_t bytes, void **out)
{
    dev_buf *b = &g_buf[which];
    if (b->cap < bytes) {
        if (b->dev) {
            HIP_TRY(hipStreamSynchronize(g_stream));
            HIP_TRY(hipFree(b->dev));
            b->dev = NULL;
            b->cap = 0;
        }
        size_t cap = bytes + bytes / 4 + 4096;
        HIP_TRY(hipMalloc(&b->dev, cap));
        b->cap = cap;
    }
    *out = b->dev;
    return 0;
}

/* Pinned twin of staging buffer `which`, at least `bytes` large (bytes <=
 * PIN_MAX_BYTES).  Nothing is in flight on a twin when this is called. */
static int pin_reserve(int which, size_t bytes, void **out)
{
    pin_buf *b = &g_pin[which];
    if (b->cap < bytes) {
        if (b->host) {
            HIP_TRY(hipHostFree(b->host));
            b->host = NULL;
            b->cap = 0;
        }
        size_t cap = bytes < 65536 ? 65536 : bytes + bytes / 4;
        HIP_TRY(hipHostMalloc(&b->host, cap, hipHostMallocDefault));
        b->cap = cap;
        HIP_TRY(hipHostGetDevicePointer(&b->dev, b->host, 0));
    }
    *out = b->host;
    return 0;
}

/* Whether the CPU can read the byte at p: the kernel copies it for us and
 * reports EFAULT instead of raising a signal. */
static int cpu_can_read(const void *p)
{
    int fd[2];
    if (pipe(fd) != 0) return 0;
    const ssize_t n = write(fd[1], p, 1);
    close(fd[0]);
    close(fd[1]);
    return n == 1;
}

/* CPU-writable device buffer for small inputs of staging slot `which`, or NULL. */
static void *direct_buffer(int which)
{
    if (g_direct_ok < 0) {
        const char *e = getenv("CKQ_DIRECT_UPLOAD");
        g_direct_ok = !(e && strcmp(e, "0") == 0);
    }
    if (!g_direct_ok) return NULL;
    if (!g_direct[which]) {
        void *p = NULL;
        if (hipExtMallocWithFlags(&p, DIRECT_MAX_BYTES, hipDeviceMallocFinegrained) != hipSuccess) {
            (void)hipGetLastError();
            g_direct_ok = 0;
            return NULL;
        }
        if (!cpu_can_read(p) || !cpu_can_read((const uint8_t *)p + DIRECT_MAX_BYTES - 1)) {
            g_direct_ok = 0;             /* no CPU mapping of device memory on this system; the buffer is kept, unused */
            return NULL;
        }
        g_direct[which] = p;
    }
    return g_direct[which];
}

/* bytes rounded up to the copy kernel's 16-byte units (every staging buffer
 * and twin is allocated with that much slack) */
static size_t round16(size_t bytes) { return (bytes + 15) & ~(size_t)15; }

/* Device view of an input: device pointers pass through, host memory is
 * copied into staging buffer `which` (small inputs by way of its pinned twin). */
static int stage_in(int which, const void *p, size_t bytes, const void **out)
{
    if (is_device_ptr(p)) {
        *out = p;
        return 0;
    }
    void *d = bytes <= DIRECT_MAX_BYTES ? direct_buffer(which) : NULL;
    if (d) {
        memcpy(d, p, bytes);
#if defined(__x86_64__) || defined(__i386__)
        __builtin_ia32_sfence();         /* write-combined stores leave the CPU before the launch that follows */
#else
        __sync_synchronize();
#endif
        *out = d;
        return 0;
    }
    int rc = buf_reserve(which, bytes, &d);
    if (rc) return rc;
    if (bytes <= PIN_MAX_BYTES) {
        void *h = NULL;
        rc = pin_reserve(which, round16(bytes), &h);
        if (rc) return rc;
        memcpy(h, p, bytes);
        rc = ckq_launch_copy(d, g_pin[which].dev, round16(bytes), g_stream);
        if (rc) return fail(rc, "upload through the pinned twin");
    } else {
        HIP_TRY(hipMemcpyAsync(d, p, bytes, hipMemcpyHostToDevice, g_stream));
    }
    *out = d;
    return 0;
}

/* The contents of staging buffer `which` back to the host and the stream
 * drained: `rows` rows of `w` bytes, `src_pitch` apart on the device,
 * `dst_pitch` apart at `dst`.  Small results come down in one copy into the
 * pinned twin and are scattered by the CPU after the synchronisation. */
static int stage_out_sync(int which, void *dst, size_t dst_pitch, size_t src_pitch, size_t w, size_t rows)
{
    const uint8_t *dev = (const uint8_t *)g_buf[which].dev;
    const size_t span = rows ? (rows - 1) * src_pitch + w : 0;
    if (span && span <= PIN_MAX_BYTES) {
        void *h = NULL;
        int rc = pin_reserve(which, round16(span), &h);
        if (rc) return rc;
        rc = ckq_launch_copy(g_pin[which].dev, dev, round16(span), g_stream);
        if (rc) return fail(rc, "download through the pinned twin");
        rc = stream_wait();
        if (rc) return rc;
        for (size_t r = 0; r < rows; ++r) memcpy((uint8_t *)dst + r * dst_pitch, (const uint8_t *)h + r * src_pitch, w);
        return 0;
    }
    if (rows == 1 || (dst_pitch == w && src_pitch == w)) {
        HIP_TRY(hipMemcpyAsync(dst, dev, rows * w, hipMemcpyDeviceToHost, g_stream));
    } else {
        HIP_TRY(hipMemcpy2DAsync(dst, dst_pitch, dev, src_pitch, w, rows, hipMemcpyDeviceToHost, g_stream));
    }
    HIP_TRY(hipStreamSynchronize(g_stream));
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Weight residency                                                          */
/* ------------------------------------------------------------------------ */

static uint64_t fingerprint(const void *p, size_t bytes) { return ckq_fingerprint(p, bytes); }

/* The table of unpinned entries is bounded: beyond CACHE_MAX_ENTRIES entries
 * or g_cache_max_bytes bytes (CKQ_WEIGHT_CACHE_MB, default 64 GiB) the least
 * recently used unpinned entry is dropped.  Registered regions are never
 * evicted. */
enum { CACHE_MAX_ENTRIES = 4096 };
static uint64_t g_use_clock = 0;
/* g_use_clock when the current call resolved its first weight operand: entries
 * used later than this belong to the call and must stay until its kernels are
 * enqueued (the fused MLP holds W1 while it resolves W2). */
static uint64_t g_call_epoch = 0;

static size_t cache_unpinned_bytes(void)
{
    size_t b = 0;
    for (size_t i = 0; i < g_nw; ++i)
        if (!g_w[i].pinned) b += g_w[i].bytes;
    return b;
}

static void drop_entry(size_t i);

/* Make room for a new unpinned entry of `bytes`: least recently used entries go
 * first, entries of the current call never.  Returns 0 when the bound cannot
 * be met (the caller then serves the operand without caching it). */
static int cache_evict_for(size_t bytes)
{
    for (;;) {
        size_t n_unpinned = 0, lru = (size_t)-1;
        for (size_t i = 0; i < g_nw; ++i) {
            if (g_w[i].pinned) continue;
            ++n_unpinned;
            if (g_w[i].last_use > g_call_epoch) continue;      /* held by this call */
            if (lru == (size_t)-1 || g_w[i].last_use < g_w[lru].last_use) lru = i;
        }
        if (n_unpinned < CACHE_MAX_ENTRIES && cache_unpinned_bytes() + bytes <= g_cache_max_bytes) return 1;
        if (lru == (size_t)-1) return 0;
        drop_entry(lru);
    }
}

static int weights_uncached(int slot, const void *W, size_t bytes, const void **out);

static int weights_lookup(int slot, const void *W, size_t bytes, const void **out)
{
    if (is_device_ptr(W)) {
        *out = W;
        return 0;
    }
    /* registered regions first: any range inside one is resident as it stands */
    for (size_t i = 0; i < g_nw; ++i) {
        const uint8_t *h = (const uint8_t *)g_w[i].host, *w = (const uint8_t *)W;
        if (g_w[i].pinned && w >= h && w + bytes <= h + g_w[i].bytes) {
            *out = (const uint8_t *)g_w[i].dev + (w - h);
            return 0;
        }
    }
    const uint64_t fp = fingerprint(W, bytes);
    for (size_t i = 0; i < g_nw; ++i) {
        if (g_w[i].host == W && g_w[i].bytes == bytes) {
            g_w[i].last_use = ++g_use_clock;
            if (g_w[i].fp == fp) {
                *out = g_w[i].dev;
                return 0;
            }
            /* same address, new content: refresh in place; the old fingerprint
             * stays if the copy cannot be enqueued */
            HIP_TRY(hipMemcpyAsync(g_w[i].dev, W, bytes, hipMemcpyHostToDevice, g_stream));
            g_w[i].fp = fp;
            *out = g_w[i].dev;
            return 0;
        }
    }
    if (!cache_evict_for(bytes)) {
        if (slot < 0) return fail((int)hipErrorOutOfMemory, "registering weights beyond the cache bound");
        return weights_uncached(slot, W, bytes, out);
    }
    if (g_nw == g_capw) {
        size_t nc = g_capw ? g_capw * 2 : 64;
        weight_entry *nw = (weight_entry *)realloc(g_w, nc * sizeof(*nw));
        if (!nw) return fail((int)hipErrorOutOfMemory, "realloc weight table");
        g_w = nw;
        g_capw = nc;
    }
    void *d = NULL;
    HIP_TRY(hipMalloc(&d, bytes));
    hipError_t e = hipMemcpyAsync(d, W, bytes, hipMemcpyHostToDevice, g_stream);
    if (e != hipSuccess) {                       /* no entry for a failed upload */
        (void)hipFree(d);
        return fail((int)e, "upload weights");
    }
    g_w[g_nw].host = W;
    g_w[g_nw].bytes = bytes;
    g_w[g_nw].fp = fp;
    g_w[g_nw].dev = d;
    g_w[g_nw].pinned = 0;
    g_w[g_nw].last_use = ++g_use_clock;
    g_nw++;
    *out = d;
    return 0;
}

/* Uncached weights share no staging buffer with activations: every weight
 * operand of a call gets its own grow-only device buffer (`slot`), so a call
 * with two weight matrices (the fused MLP) keeps both alive until its kernels
 * have been enqueued. */
enum { WTMP_SLOTS = 2 };
static dev_buf g_wtmp[WTMP_SLOTS];
static int weights_uncached(int slot, const void *W, size_t bytes, const void **out)
{
    dev_buf *b = &g_wtmp[slot];
    if (b->cap < bytes) {
        if (b->dev) {
            HIP_TRY(hipStreamSynchronize(g_stream));
            HIP_TRY(hipFree(b->dev));
            b->dev = NULL;
            b->cap = 0;
        }
        HIP_TRY(hipMalloc(&b->dev, bytes));
        b->cap = bytes;
    }
    HIP_TRY(hipMemcpyAsync(b->dev, W, bytes, hipMemcpyHostToDevice, g_stream));
    *out = b->dev;
    return 0;
}

enum { CACHE_MIN_BYTES = 64 * 1024 };
static int in_registered_region(const void *W, size_t bytes)
{
    for (size_t i = 0; i < g_nw; ++i) {
        const uint8_t *h = (const uint8_t *)g_w[i].host, *w = (const uint8_t *)W;
        if (g_w[i].pinned && w >= h && w + bytes <= h + g_w[i].bytes) return 1;
    }
    return 0;
}

/* Device view of weight operand number `slot` (0 or 1) of the current call. */
static int weights_resolve(int slot, const void *W, size_t bytes, const void **out)
{
    if (slot == 0) g_call_epoch = g_use_clock;       /* the first operand opens a call */
    if (is_device_ptr(W)) {
        *out = W;
        return 0;
    }
    if (!g_cache_on) return weights_uncached(slot, W, bytes, out);
    /* Operands under 64 KiB (a single row handed to a vec_dot, a parity
     * harness's scratch matrix) are cheaper to copy than to track: a per-row
     * loop over a large matrix would otherwise leave one allocation per row. */
    if (bytes < CACHE_MIN_BYTES && !in_registered_region(W, bytes)) return weights_uncached(slot, W, bytes, out);
    return weights_lookup(slot, W, bytes, out);
}

static int register_locked(const void *W, size_t bytes)
{
    const void *d;
    g_call_epoch = g_use_clock;
    int rc = weights_lookup(-1, W, bytes, &d);
    if (rc) return rc;
    for (size_t i = 0; i < g_nw; ++i)
        if (g_w[i].host == W && g_w[i].bytes == bytes) g_w[i].pinned = 1;
    return 0;
}

int ckq_weights_register(const void *W, size_t bytes)
{
    if (!W || bytes == 0) return CKQ_EINVAL;
    if (is_device_ptr(W)) return 0;
    pthread_mutex_lock(&g_mu);
    int rc = init_locked();
    if (rc == 0) rc = register_locked(W, bytes);
    if (rc == 0) {
        hipError_t e = hipStreamSynchronize(g_stream);
        if (e != hipSuccess) rc = fail((int)e, "hipStreamSynchronize");
    }
    pthread_mutex_unlock(&g_mu);
    return rc;
}

/* Loader hook: walk a weights manifest (one tensor per line,
 * name|dtype|file_offset|size|runtime_offset, '#' comments and blank lines
 * skipped, numbers in any C base) and register every tensor of a quantized
 * weight format this library computes with, at base + runtime_offset. */
int ckq_weights_register_manifest(const void *base, const char *manifest_path)
{
    if (!base || !manifest_path) return CKQ_EINVAL;
    FILE *mf = fopen(manifest_path, "r");
    if (!mf) return CKQ_EINVAL;
    char line[4096];
    int n = 0, rc = 0, inited = 0;
    while (rc == 0 && fgets(line, sizeof line, mf)) {
        unsigned long long size = 0, off = 0;
        const int kind = ckq_manifest_parse_line(line, &size, &off);
        if (kind < 0) { rc = CKQ_EINVAL; break; }      /* malformed line */
        if (kind == 0) continue;
        pthread_mutex_lock(&g_mu);
        if (!inited) { rc = init_locked(); inited = 1; }
        if (rc == 0) rc = register_locked((const uint8_t *)base + off, (size_t)size);
        pthread_mutex_unlock(&g_mu);
        if (rc == 0) ++n;
    }
    fclose(mf);
    if (rc == 0 && inited) {
        pthread_mutex_lock(&g_mu);
        hipError_t e = hipStreamSynchronize(g_stream);
        if (e != hipSuccess) rc = fail((int)e, "hipStreamSynchronize");
        pthread_mutex_unlock(&g_mu);
    }
    return rc ? rc : n;
}

/* Number of resident weight regions; their total size through *bytes. */
int ckq_weights_resident(size_t *bytes)
{
    pthread_mutex_lock(&g_mu);
    size_t b = 0;
    for (size_t i = 0; i < g_nw; ++i) b += g_w[i].bytes;
    const int n = (int)g_nw;
    pthread_mutex_unlock(&g_mu);
    if (bytes) *bytes = b;
    return n;
}

static void drop_entry(size_t i)
{
    (void)hipStreamSynchronize(g_stream);
    (void)hipFree(g_w[i].dev);
    g_w[i] = g_w[g_nw - 1];
    g_nw--;
}

void ckq_weights_invalidate(const void *W)
{
    pthread_mutex_lock(&g_mu);
    ptr_cache_clear();
    for (size_t i = 0; i < g_nw;) {
        if (g_w[i].host == W) drop_entry(i);
        else ++i;
    }
    pthread_mutex_unlock(&g_mu);
}

void ckq_weights_clear(void)
{
    pthread_mutex_lock(&g_mu);
    ptr_cache_clear();
    while (g_nw) drop_entry(g_nw - 1);
    pthread_mutex_unlock(&g_mu);
}

void ckq_weights_set_limit(size_t bytes)
{
    pthread_mutex_lock(&g_mu);
    g_cache_max_bytes = bytes ? bytes : (size_t)64 << 30;
    g_call_epoch = g_use_clock;
    (void)cache_evict_for(0);
    pthread_mutex_unlock(&g_mu);
}

int ckq_release_stream(void *stream) { return ckq_launch_release_stream(stream); }

void ckq_weights_set_cache(int enabled)
{
    pthread_mutex_lock(&g_mu);
    g_cache_on = enabled != 0;
    pthread_mutex_unlock(&g_mu);
}

void ckq_set_gemm_policy(int policy) { ckq_launch_set_gemm_policy(policy); }
void ckq_set_prefill_variant(int fmt, int variant)
{
    if (fmt == CKQ_FMT_Q4_K) ckq_launch_set_q4k_tile(variant);
    else if (fmt == CKQ_FMT_Q6_K) ckq_launch_set_q6k_variant(variant);
    else if (fmt == CKQ_FMT_Q5_K) ckq_launch_set_q5k_variant(variant);
}

static int g_prefill_grouping = 1;
void ckq_set_prefill_grouping(int enabled)
{
    __atomic_store_n(&g_prefill_grouping, enabled != 0, __ATOMIC_RELAXED);
}

void ckq_set_parallel_whole(int enabled)
{
    pthread_mutex_lock(&g_mu);
    if (enabled < 0) {                       /* back to the default (CKQ_PARALLEL_MODE or the built-in one) */
        const char *p = getenv("CKQ_PARALLEL_MODE");
        __atomic_store_n(&g_parallel_whole, p ? strcmp(p, "whole") == 0 : CKQ_PARALLEL_WHOLE_DEFAULT, __ATOMIC_RELAXED);
    } else {
        __atomic_store_n(&g_parallel_whole, enabled != 0, __ATOMIC_RELAXED);
    }
    pthread_mutex_unlock(&g_mu);
}

/* ------------------------------------------------------------------------ */
/* Shapes                                                                    */
/* ------------------------------------------------------------------------ */

static int fmt_block_elems(int fmt) { return (fmt == CKQ_FMT_Q8_0 || fmt == CKQ_FMT_Q5_0 || fmt == CKQ_KERNEL_Q80_F32) ? 32 : 256; }

static int is_f32act(int fmt) { return fmt == CKQ_KERNEL_Q80_F32 || fmt == CKQ_KERNEL_Q4K_F32 || fmt == CKQ_KERNEL_Q6K_F32; }

static int weight_fmt(int fmt)
{
    return fmt == CKQ_KERNEL_Q80_F32 ? CKQ_FMT_Q8_0 : fmt == CKQ_KERNEL_Q4K_F32 ? CKQ_FMT_Q4_K
         : fmt == CKQ_KERNEL_Q6K_F32 ? CKQ_FMT_Q6_K : fmt;
}

static size_t weight_row_bytes(int fmt, int K)
{
    return ckq_row_bytes(weight_fmt(fmt), K);
}

static size_t act_row_bytes(int fmt, int K)
{
    if (is_f32act(fmt)) return (size_t)K * 4;
    if (fmt == CKQ_FMT_Q8_0 || fmt == CKQ_FMT_Q5_0) return ckq_row_bytes(CKQ_FMT_Q8_0, K);
    return ckq_row_bytes(CKQ_FMT_Q8_K, K);
}

/* ------------------------------------------------------------------------ */
/* Core host-pointer matmul                                                  */
/* ------------------------------------------------------------------------ */

/*
 * C[t*ldc + n] = dot(B[n], A[t]) (+bias[n]) for n in [row0,row1), t < ntok,
 * any mix of host and device pointers; synchronous.
 */
static void matmul_locked(int fmt, const void *A, const void *B, const float *bias, float *C,
                          int ntok, int nrows, int K, long ldc, int row0, int row1)
{
    int done = 0;
    do {
        if (init_locked()) break;
        const void *dB, *dA, *dbias = NULL;
        if (weights_resolve(0, B, (size_t)nrows * weight_row_bytes(fmt, K), &dB)) break;
        if (stage_in(BUF_X, A, (size_t)ntok * act_row_bytes(fmt, K), &dA)) break;
        if (bias && stage_in(BUF_BIAS, bias, (size_t)nrows * sizeof(float), &dbias)) break;
        const int c_on_dev = is_device_ptr(C);
        float *dC = C;
        long   ld = ldc;
        void  *ypin = NULL;      /* small results are written by the kernel straight into the pinned twin */
        if (!c_on_dev) {
            void *t;
            ld = row1 - row0; /* compact staging: only the computed rows */
            const size_t ybytes = (size_t)ntok * (size_t)ld * sizeof(float);
            if (ybytes <= PIN_MAX_BYTES) {
                if (pin_reserve(BUF_Y, round16(ybytes), &ypin)) break;
                t = g_pin[BUF_Y].dev;
            } else if (buf_reserve(BUF_Y, ybytes, &t)) break;
            /* the kernel indexes with absolute rows: bias the base by row0 in integer
             * arithmetic (a pointer in front of its allocation must not be formed) */
            dC = (float *)((uintptr_t)t - (uintptr_t)row0 * sizeof(float));
        }
        int rc = ckq_launch_gemv(fmt, dC, dB, dA, (const float *)dbias, nrows, K, ntok, ld, row0, row1, NULL, g_stream);
        if (rc) { fail(rc, "ckq_launch_gemv"); break; }
        if (ypin) {
            if (stream_wait()) break;
            const size_t w = (size_t)(row1 - row0) * sizeof(float);
            for (int t = 0; t < ntok; ++t) memcpy(C + (size_t)t * ldc + row0, (const uint8_t *)ypin + (size_t)t * w, w);
        } else if (!c_on_dev) {
            if (stage_out_sync(BUF_Y, C + row0, (size_t)ldc * sizeof(float), (size_t)ld * sizeof(float),
                               (size_t)(row1 - row0) * sizeof(float), (size_t)ntok)) break;
        } else {
            hipError_t e = hipStreamSynchronize(g_stream);
            if (e != hipSuccess) { fail((int)e, "hipStreamSynchronize"); break; }
        }
        done = 1;
    } while (0);
    if (!done) drain_after_error();
}

static void host_matmul(int fmt, const void *A, const void *B, const float *bias, float *C,
                        int ntok, int nrows, int K, long ldc, int row0, int row1)
{
    if (!A || !B || !C || ntok <= 0 || nrows <= 0 || K <= 0) return;
    if (K % fmt_block_elems(fmt) != 0) return;
    if (row0 < 0) row0 = 0;
    if (row1 > nrows) row1 = nrows;
    if (row0 >= row1) return;
    pthread_mutex_lock(&g_mu);
    matmul_locked(fmt, A, B, bias, C, ntok, nrows, K, ldc, row0, row1);
    pthread_mutex_unlock(&g_mu);
}

/* Row range of thread ith of nth (reference: gemm_kernels_q4k_q8k.c:226-231). */
static int split_rows(int M, int ith, int nth, int *r0, int *r1)
{
    return ckq_split_rows(M, ith, nth, __atomic_load_n(&g_parallel_whole, __ATOMIC_RELAXED), r0, r1);
}

static void host_gemv_split(int fmt, float *y, const void *W, const void *x, int M, int K, int ith, int nth)
{
    if (!y || !W || !x || M <= 0 || K <= 0) return;
    int r0, r1;
    if (!split_rows(M, ith, nth, &r0, &r1)) return;
    host_matmul(fmt, x, W, NULL, y, 1, M, K, M, r0, r1);
}

/* fp32 [rows x k] -> quantized blocks, any pointer mix, synchronous. */
static void host_quantize(int q8k, const float *x, void *y, int rows, int k)
{
    if (!x || !y || rows <= 0 || k <= 0) return;
    const int be = q8k ? 256 : 32;
    if (k % be) return; /* the reference asserts; a release build would write nothing sensible */
    const size_t in_bytes = (size_t)rows * k * 4;
    const size_t out_bytes = (size_t)rows * ckq_row_bytes(q8k ? CKQ_FMT_Q8_K : CKQ_FMT_Q8_0, k);
    pthread_mutex_lock(&g_mu);
    int done = 0;
    do {
        if (init_locked()) break;
        const void *dx;
        if (stage_in(BUF_X, x, in_bytes, &dx)) break;
        const int y_on_dev = is_device_ptr(y);
        void *dy = y;
        if (!y_on_dev && buf_reserve(BUF_Y, out_bytes, &dy)) break;
        int rc = q8k ? ckq_launch_quantize_q8_k((const float *)dx, dy, rows, k, g_stream)
                     : ckq_launch_quantize_q8_0((const float *)dx, dy, rows, k, g_stream);
        if (rc) { fail(rc, "quantize launch"); break; }
        if (!y_on_dev) {
            if (stage_out_sync(BUF_Y, y, out_bytes, out_bytes, out_bytes, 1)) break;
        } else {
            hipError_t e = hipStreamSynchronize(g_stream);
            if (e != hipSuccess) { fail((int)e, "hipStreamSynchronize"); break; }
        }
        done = 1;
    } while (0);
    if (!done) drain_after_error();
    pthread_mutex_unlock(&g_mu);
}

/* fp32 activations: quantize on the device, then the quantized kernel. */
static void host_matmul_f32act(int fmt, const float *A, const void *B, const float *bias, float *C,
                               int ntok, int nrows, int K, long ldc)
{
    if (!A || !B || !C || ntok <= 0 || nrows <= 0 || K <= 0) return;
    const int q8k = fmt != CKQ_FMT_Q8_0;
    if (K % (q8k ? 256 : 32)) return;
    pthread_mutex_lock(&g_mu);
    void *dq = NULL;
    int done = 0;
    do {
        if (init_locked()) break;
        const void *dA;
        if (stage_in(BUF_X, A, (size_t)ntok * K * 4, &dA)) break;
        if (buf_reserve(BUF_Q, (size_t)ntok * act_row_bytes(fmt, K), &dq)) break;
        int rc = q8k ? ckq_launch_quantize_q8_k((const float *)dA, dq, ntok, K, g_stream)
                     : ckq_launch_quantize_q8_0((const float *)dA, dq, ntok, K, g_stream);
        if (rc) { fail(rc, "quantize launch"); break; }
        /* dq is a device pointer, so the second stage uses it in place; work
         * on one stream runs in order. */
        matmul_locked(fmt, dq, B, bias, C, ntok, nrows, K, ldc, 0, nrows);
        done = 1;
    } while (0);
    if (!done) drain_after_error();
    pthread_mutex_unlock(&g_mu);
}

/* ------------------------------------------------------------------------ */
/* Part 1: drop-in symbols                                                   */
/* ------------------------------------------------------------------------ */

void quantize_row_q8_k(const float *x, void *y, int k) { host_quantize(1, x, y, 1, k); }
void quantize_batch_q8_k(const float *x, void *y, int num_rows, int k) { host_quantize(1, x, y, num_rows, k); }
void quantize_row_q8_0(const float *x, void *y, int k) { host_quantize(0, x, y, 1, k); }
void quantize_batch_q8_0(const float *x, void *y, int num_rows, int k) { host_quantize(0, x, y, num_rows, k); }

#define DEFINE_GEMV_FAMILY(NAME, FMT)                                                                         \
    void gemv_##NAME(float *y, const void *W, const void *x_q8, int M, int K)                                \
    {                                                                                                         \
        host_matmul(FMT, x_q8, W, NULL, y, 1, M, K, M, 0, M);                                                \
    }                                                                                                         \
    void gemv_##NAME##_parallel(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth)    \
    {                                                                                                         \
        host_gemv_split(FMT, y, W, x_q8, M, K, ith, nth);                                                    \
    }                                                                                                         \
    void gemv_##NAME##_parallel_simd(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth) \
    {                                                                                                         \
        host_gemv_split(FMT, y, W, x_q8, M, K, ith, nth);                                                    \
    }

DEFINE_GEMV_FAMILY(q4_k_q8_k, CKQ_FMT_Q4_K)
DEFINE_GEMV_FAMILY(q6_k_q8_k, CKQ_FMT_Q6_K)
DEFINE_GEMV_FAMILY(q8_0_q8_0, CKQ_FMT_Q8_0)

void gemv_q4_k_q8_k_ref(float *y, const void *W, const void *x_q8, int M, int K)
{
    host_matmul(CKQ_FMT_Q4_K, x_q8, W, NULL, y, 1, M, K, M, 0, M);
}

void gemm_q4_k_q8_k(float *Y, const void *W, const void *X_q8, int M, int N, int K)
{
    host_matmul(CKQ_FMT_Q4_K, X_q8, W, NULL, Y, N, M, K, M, 0, M);
}

void gemm_nt_q4_k_q8_k(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K)
{
    host_matmul(CKQ_FMT_Q4_K, A_q8, B, bias, C, M, N, K, N, 0, N);
}

void gemv_q5_k_q8_k(float *y, const void *W, const void *x_q8, int M, int K)
{
    host_matmul(CKQ_FMT_Q5_K, x_q8, W, NULL, y, 1, M, K, M, 0, M);
}

void gemm_nt_q5_k_q8_k(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K)
{
    host_matmul(CKQ_FMT_Q5_K, A_q8, B, bias, C, M, N, K, N, 0, N);
}

void gemv_q5_k(float *y, const void *W, const float *x, int M, int K)
{
    host_matmul_f32act(CKQ_FMT_Q5_K, x, W, NULL, y, 1, M, K, M);
}

void gemm_nt_q5_k(const float *A, const void *B, const float *bias, float *C, int M, int N, int K)
{
    host_matmul_f32act(CKQ_FMT_Q5_K, A, B, bias, C, M, N, K, N);
}

void vec_dot_q6_k_q8_k(int n, float *s, const void *vx, const void *vy)
{
    if (!s || !vx || !vy || n <= 0) return;
    host_matmul(CKQ_FMT_Q6_K, vy, vx, NULL, s, 1, 1, n, 1, 0, 1);
}

void gemm_q6_k_q8_k(float *Y, const void *W, const void *X_q8, int M, int N, int K)
{
    host_matmul(CKQ_FMT_Q6_K, X_q8, W, NULL, Y, N, M, K, M, 0, M);
}

void gemm_nt_q6_k_q8_k(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K)
{
    host_matmul(CKQ_FMT_Q6_K, A_q8, B, bias, C, M, N, K, N, 0, N);
}

void vec_dot_q8_0_q8_0(int n, float *s, const void *vx, const void *vy)
{
    if (!s || !vx || !vy || n <= 0) return;
    host_matmul(CKQ_FMT_Q8_0, vy, vx, NULL, s, 1, 1, n, 1, 0, 1);
}

/* Q5_0 weights (the format of rows too short for K-quants) against Q8_0 activations. */
void vec_dot_q5_0_q8_0(int n, float *s, const void *vx, const void *vy)
{
    if (!s || !vx || !vy || n <= 0) return;
    host_matmul(CKQ_FMT_Q5_0, vy, vx, NULL, s, 1, 1, n, 1, 0, 1);
}

void gemv_q5_0_q8_0(float *y, const void *W, const void *x_q8, int M, int K)
{
    host_matmul(CKQ_FMT_Q5_0, x_q8, W, NULL, y, 1, M, K, M, 0, M);
}

void gemv_q5_0_q8_0_parallel_simd(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth)
{
    host_gemv_split(CKQ_FMT_Q5_0, y, W, x_q8, M, K, ith, nth);
}

void gemm_nt_q5_0_q8_0(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K)
{
    host_matmul(CKQ_FMT_Q5_0, A_q8, B, bias, C, M, N, K, N, 0, N);
}

void gemv_q8_0(float *y, const void *W, const float *x, int M, int K)
{
    host_matmul(CKQ_KERNEL_Q80_F32, x, W, NULL, y, 1, M, K, M, 0, M);
}

void gemm_nt_q8_0_q8_0(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K)
{
    host_matmul(CKQ_FMT_Q8_0, A_q8, B, bias, C, M, N, K, N, 0, N);
}

/* Row dequantizers and quantized embedding lookup, any pointer mix, synchronous.
 * The table is treated like a weight matrix (uploaded once, kept resident). */
static void host_dequant_rows(int fmt, const void *table, size_t table_rows, const int32_t *ids, int vocab,
                              const float *pos, float *out, int n_valid, int n_row, int tokens, int n_out_rows)
{
    if (!table || !out || n_row <= 0 || n_out_rows <= 0) return;
    if (n_row % (fmt == CKQ_FMT_Q8_0 ? 32 : 256)) return;
    if (tokens < 0) tokens = 0;
    if (tokens > n_out_rows) tokens = n_out_rows;
    pthread_mutex_lock(&g_mu);
    int done = 0;
    do {
        if (init_locked()) break;
        const void *dT, *dids = NULL, *dpos = NULL;
        if (weights_resolve(0, table, table_rows * ckq_row_bytes(fmt, n_row), &dT)) break;
        if (ids && tokens > 0 && stage_in(BUF_X, ids, (size_t)tokens * sizeof(int32_t), &dids)) break;
        if (pos && tokens > 0 && stage_in(BUF_BIAS, pos, (size_t)tokens * n_row * sizeof(float), &dpos)) break;
        const size_t out_bytes = (size_t)n_out_rows * n_row * sizeof(float);
        const int on_dev = is_device_ptr(out);
        void *dout = out;
        if (!on_dev && buf_reserve(BUF_Y, out_bytes, &dout)) break;
        int rc = ckq_launch_dequant_rows(fmt, dT, ids ? (const int32_t *)dids : NULL, vocab, (const float *)dpos,
                                         (float *)dout, n_valid, n_row, tokens, n_out_rows, g_stream);
        if (rc) { fail(rc, "ckq_launch_dequant_rows"); break; }
        if (!on_dev) {
            if (stage_out_sync(BUF_Y, out, out_bytes, out_bytes, out_bytes, 1)) break;
        } else {
            hipError_t e = hipStreamSynchronize(g_stream);
            if (e != hipSuccess) { fail((int)e, "hipStreamSynchronize"); break; }
        }
        done = 1;
    } while (0);
    if (!done) drain_after_error();
    pthread_mutex_unlock(&g_mu);
}

void dequant_q4_k_row(const void *src, float *dst, size_t n_elements)
{
    if (n_elements == 0 || n_elements > 0x7fffff00u) return;
    host_dequant_rows(CKQ_FMT_Q4_K, src, 1, NULL, 0, NULL, dst, (int)n_elements, (int)n_elements, 1, 1);
}

void dequant_q6_k_row(const void *src, float *dst, size_t n_elements)
{
    if (n_elements == 0 || n_elements > 0x7fffff00u) return;
    host_dequant_rows(CKQ_FMT_Q6_K, src, 1, NULL, 0, NULL, dst, (int)n_elements, (int)n_elements, 1, 1);
}

void dequant_q8_0_row(const void *src, float *dst, size_t n_elements)
{
    if (n_elements == 0 || n_elements > 0x7fffffe0u) return;
    host_dequant_rows(CKQ_FMT_Q8_0, src, 1, NULL, 0, NULL, dst, (int)n_elements, (int)n_elements, 1, 1);
}

#define DEFINE_EMBEDDING(NAME, FMT)                                                                              \
    void embedding_forward_##NAME(const int32_t *token_ids, int token_count, int vocab_size,                      \
                                  const void *token_embeddings, const float *pos_embeddings, float *output,      \
                                  int embed_dim, int aligned_embed_dim, int context_window, int add_pos)         \
    {                                                                                                             \
        if (!token_ids || !token_embeddings || !output || vocab_size <= 0 || context_window <= 0) return;        \
        host_dequant_rows(FMT, token_embeddings, (size_t)vocab_size, token_ids, vocab_size,                      \
                          add_pos ? pos_embeddings : NULL, output, embed_dim, aligned_embed_dim, token_count,    \
                          context_window);                                                                        \
    }
DEFINE_EMBEDDING(q4_k, CKQ_FMT_Q4_K)
DEFINE_EMBEDDING(q6_k, CKQ_FMT_Q6_K)
DEFINE_EMBEDDING(q8_0, CKQ_FMT_Q8_0)

/* Fused producer: RMSNorm then Q8_K quantization, any pointer mix, synchronous. */
void rmsnorm_q8_k_fused(const float *input, const float *gamma, void *vy, int tokens, int d_model,
                        int aligned_embed_dim, float eps)
{
    if (!input || !gamma || !vy || tokens <= 0 || d_model <= 0 || aligned_embed_dim < d_model) return;
    if (d_model % 256) return;
    const size_t in_bytes = ((size_t)(tokens - 1) * aligned_embed_dim + d_model) * 4;
    const size_t out_bytes = (size_t)tokens * ckq_row_bytes(CKQ_FMT_Q8_K, d_model);
    pthread_mutex_lock(&g_mu);
    int done = 0;
    do {
        if (init_locked()) break;
        const void *dx, *dg;
        if (stage_in(BUF_X, input, in_bytes, &dx)) break;
        if (stage_in(BUF_BIAS, gamma, (size_t)d_model * 4, &dg)) break;
        const int y_on_dev = is_device_ptr(vy);
        void *dy = vy;
        if (!y_on_dev && buf_reserve(BUF_Y, out_bytes, &dy)) break;
        int rc = ckq_launch_rmsnorm_q8_k_fused((const float *)dx, (const float *)dg, dy, tokens, d_model,
                                               aligned_embed_dim, eps, g_stream);
        if (rc) { fail(rc, "rmsnorm_q8_k_fused launch"); break; }
        if (!y_on_dev) {
            if (stage_out_sync(BUF_Y, vy, out_bytes, out_bytes, out_bytes, 1)) break;
        } else {
            hipError_t e = hipStreamSynchronize(g_stream);
            if (e != hipSuccess) { fail((int)e, "hipStreamSynchronize"); break; }
        }
        done = 1;
    } while (0);
    if (!done) drain_after_error();
    pthread_mutex_unlock(&g_mu);
}

/* Fused prefill MLP: Q8_0 quantization, one GEMM over the stacked gate and up
 * rows, SiLU(gate)*up quantized to Q8_K, the down GEMM.  The four kernels run
 * back to back on the library's stream; intermediates never leave the device. */
void fused_mlp_swiglu_prefill_w1w2_quant(const float *x, const void *W1, const float *B1, ckq_ck_dtype w1_dt_e,
                                         const void *W2, const float *B2, ckq_ck_dtype w2_dt_e, float *output,
                                         int seq_len, int embed_dim, int aligned_embed_dim,
                                         int intermediate_dim, int aligned_intermediate_dim, void *scratch)
{
    const int w1_dt = (int)w1_dt_e, w2_dt = (int)w2_dt_e;
    if (!x || !W1 || !W2 || !output || !scratch) return;
    if (seq_len <= 0 || embed_dim <= 0 || aligned_embed_dim <= 0 || intermediate_dim <= 0 ||
        aligned_intermediate_dim <= 0)
        return;
    if (aligned_embed_dim < embed_dim || aligned_intermediate_dim < intermediate_dim) return;
    if (aligned_embed_dim % 32 || aligned_intermediate_dim % 256) return;
    if ((w1_dt != CKQ_CK_DT_Q8_0 && w1_dt != CKQ_CK_DT_Q5_0) || (w2_dt != CKQ_CK_DT_Q4_K && w2_dt != CKQ_CK_DT_Q6_K))
        return;
    const int fmt1 = w1_dt == CKQ_CK_DT_Q8_0 ? CKQ_FMT_Q8_0 : CKQ_FMT_Q5_0;
    const int E = aligned_embed_dim, I = aligned_intermediate_dim;
    const int fmt2 = w2_dt == CKQ_CK_DT_Q4_K ? CKQ_FMT_Q4_K : CKQ_FMT_Q6_K;
    const size_t out_bytes = (size_t)seq_len * E * 4;
    pthread_mutex_lock(&g_mu);
    int done = 0;
    do {
        if (init_locked()) break;
        const void *dx, *dW1, *dW2, *dB1 = NULL, *dB2 = NULL;
        void *dq, *dgu, *dh;
        if (stage_in(BUF_X, x, (size_t)seq_len * E * 4, &dx)) break;
        if (weights_resolve(0, W1, (size_t)2 * I * weight_row_bytes(fmt1, E), &dW1)) break;
        if (weights_resolve(1, W2, (size_t)E * weight_row_bytes(fmt2, I), &dW2)) break;
        /* both biases share the bias staging buffer: B1 first, B2 behind it */
        if (B1 || B2) {
            const int b1_dev = B1 && is_device_ptr(B1), b2_dev = B2 && is_device_ptr(B2);
            void *db = NULL;
            if (((B1 && !b1_dev) || (B2 && !b2_dev)) && buf_reserve(BUF_BIAS, ((size_t)2 * I + E) * 4, &db)) break;
            hipError_t e = hipSuccess;
            if (B1) {
                dB1 = B1;
                if (!b1_dev) { e = hipMemcpyAsync(db, B1, (size_t)2 * I * 4, hipMemcpyHostToDevice, g_stream); dB1 = db; }
            }
            if (e == hipSuccess && B2) {
                dB2 = B2;
                if (!b2_dev) {
                    e = hipMemcpyAsync((float *)db + 2 * (size_t)I, B2, (size_t)E * 4, hipMemcpyHostToDevice, g_stream);
                    dB2 = (float *)db + 2 * (size_t)I;
                }
            }
            if (e != hipSuccess) { fail((int)e, "copy biases to device"); break; }
        }
        if (buf_reserve(BUF_Q, (size_t)seq_len * act_row_bytes(CKQ_FMT_Q8_0, E), &dq)) break;
        if (buf_reserve(BUF_GU, (size_t)seq_len * 2 * I * 4, &dgu)) break;
        if (buf_reserve(BUF_H, (size_t)seq_len * act_row_bytes(fmt2, I), &dh)) break;
        const int out_on_dev = is_device_ptr(output);
        void *dout = output;
        if (!out_on_dev && buf_reserve(BUF_Y, out_bytes, &dout)) break;
        int rc = ckq_launch_quantize_q8_0((const float *)dx, dq, seq_len, E, g_stream);
        if (rc) { fail(rc, "quantize launch"); break; }
        rc = ckq_launch_gemv(fmt1, (float *)dgu, dW1, dq, (const float *)dB1, 2 * I, E, seq_len, 2L * I, 0, 2 * I,
                             NULL, g_stream);
        if (rc) { fail(rc, "gate/up GEMM launch"); break; }
        rc = ckq_launch_swiglu_q8_k((const float *)dgu, (const float *)dgu + I, dh, seq_len, I, 2L * I, g_stream);
        if (rc) { fail(rc, "swiglu launch"); break; }
        rc = ckq_launch_gemv(fmt2, (float *)dout, dW2, dh, (const float *)dB2, E, I, seq_len, (long)E, 0, E, NULL, g_stream);
        if (rc) { fail(rc, "down GEMM launch"); break; }
        if (!out_on_dev) {
            if (stage_out_sync(BUF_Y, output, out_bytes, out_bytes, out_bytes, 1)) break;
        } else {
            hipError_t e = hipStreamSynchronize(g_stream);
            if (e != hipSuccess) { fail((int)e, "hipStreamSynchronize"); break; }
        }
        done = 1;
    } while (0);
    if (!done) drain_after_error();
    pthread_mutex_unlock(&g_mu);
}

/* What the reference asks its callers to provide (tiles of 64 tokens: Q8_0
 * rows, gate and up tiles, Q8_K rows, each rounded up to 64 bytes), so code that
 * sizes its arena with this call allocates the same amount. */
size_t fused_mlp_swiglu_prefill_w1w2_quant_scratch_size(int aligned_embed_dim, int aligned_intermediate_dim)
{
    if (aligned_embed_dim <= 0 || aligned_intermediate_dim <= 0) return 0;
    const size_t tile = 64;
    const size_t q8 = tile * ((size_t)aligned_embed_dim / 32) * 34;
    const size_t gate = tile * (size_t)aligned_intermediate_dim * 4;
    const size_t q8k = tile * ((size_t)aligned_intermediate_dim / 256) * 292;
#define CKQ_UP64(v) (((v) + 63) / 64 * 64)
    return CKQ_UP64(q8) + 2 * CKQ_UP64(gate) + CKQ_UP64(q8k);
#undef CKQ_UP64
}

/* fp32 activations used as they are (no activation quantization). */
void gemv_q4_k(float *y, const void *W, const float *x, int M, int K)
{
    host_matmul(CKQ_KERNEL_Q4K_F32, x, W, NULL, y, 1, M, K, M, 0, M);
}

void gemm_q4_k(float *Y, const void *W, const float *X, int M, int N, int K)
{
    host_matmul(CKQ_KERNEL_Q4K_F32, X, W, NULL, Y, N, M, K, M, 0, M);
}

void gemm_nt_q4_k(const float *A, const void *B, const float *bias, float *C, int M, int N, int K)
{
    host_matmul(CKQ_KERNEL_Q4K_F32, A, B, bias, C, M, N, K, N, 0, N);
}

float dot_q4_k(const void *w_q4k, const float *x, int K)
{
    float r = 0.0f;
    gemv_q4_k(&r, w_q4k, x, 1, K);
    return r;
}

void gemv_q6_k(float *y, const void *W, const float *x, int M, int K)
{
    host_matmul(CKQ_KERNEL_Q6K_F32, x, W, NULL, y, 1, M, K, M, 0, M);
}

void gemm_q6_k(float *Y, const void *W, const float *X, int M, int N, int K)
{
    host_matmul(CKQ_KERNEL_Q6K_F32, X, W, NULL, Y, N, M, K, M, 0, M);
}

void gemm_nt_q6_k(const float *A, const void *B, const float *bias, float *C, int M, int N, int K)
{
    host_matmul(CKQ_KERNEL_Q6K_F32, A, B, bias, C, M, N, K, N, 0, N);
}

void gemm_q8_0(float *Y, const void *W, const float *X, int M, int N, int K)
{
    host_matmul(CKQ_KERNEL_Q80_F32, X, W, NULL, Y, N, M, K, M, 0, M);
}

void gemm_nt_q8_0(const float *A, const void *B, const float *bias, float *C, int M, int N, int K)
{
    host_matmul(CKQ_KERNEL_Q80_F32, A, B, bias, C, M, N, K, N, 0, N);
}

/* Parity-test wrappers (reference: src/ck_parity_api.c). */
void ck_test_quantize_q8_k(const float *src, void *dst, int n) { quantize_row_q8_k(src, dst, n); }
void ck_test_dequant_q4_k(const void *src, float *dst, int n) { if (n > 0) dequant_q4_k_row(src, dst, (size_t)n); }
void ck_test_dequant_q6_k(const void *src, float *dst, int n) { if (n > 0) dequant_q6_k_row(src, dst, (size_t)n); }

void ck_test_gemv_q4_k(const void *w, const float *in, float *out, int cols)
{
    host_matmul_f32act(CKQ_FMT_Q4_K, in, w, NULL, out, 1, 1, cols, 1);
}

void ck_test_gemv_q6_k(const void *w, const float *in, float *out, int cols)
{
    host_matmul_f32act(CKQ_FMT_Q6_K, in, w, NULL, out, 1, 1, cols, 1);
}

void ck_test_gemv_q8_0(const void *w, const float *in, float *out, int rows, int cols)
{
    host_matmul_f32act(CKQ_FMT_Q8_0, in, w, NULL, out, 1, rows, cols, rows);
}

void ck_test_gemv_q8_0_q8_0(const void *w, const float *in, float *out, int rows, int cols)
{
    host_matmul_f32act(CKQ_FMT_Q8_0, in, w, NULL, out, 1, rows, cols, rows);
}

void ck_test_vec_dot_q8_0_q8_0(const void *w, const void *in_q8, float *out, int cols)
{
    vec_dot_q8_0_q8_0(cols, out, w, in_q8);
}

void ck_test_gemm_q4_k(const void *w, const float *in, float *out, int rows, int cols, int n_tokens)
{
    host_matmul_f32act(CKQ_FMT_Q4_K, in, w, NULL, out, n_tokens, rows, cols, rows);
}

void ck_test_gemm_q6_k(const void *w, const float *in, float *out, int rows, int cols, int n_tokens)
{
    host_matmul_f32act(CKQ_FMT_Q6_K, in, w, NULL, out, n_tokens, rows, cols, rows);
}

void ck_test_gemm_q8_0(const void *w, const float *in, float *out, int rows, int cols, int n_tokens)
{
    host_matmul_f32act(CKQ_FMT_Q8_0, in, w, NULL, out, n_tokens, rows, cols, rows);
}

int ck_get_block_q4_k_size(void) { return CKQ_BLOCK_Q4_K_SIZE; }
int ck_get_block_q6_k_size(void) { return CKQ_BLOCK_Q6_K_SIZE; }
int ck_get_block_q8_k_size(void) { return CKQ_BLOCK_Q8_K_SIZE; }
int ck_get_qk_k(void) { return CKQ_QK_K; }

/* ------------------------------------------------------------------------ */
/* Part 2: device-resident entry points                                      */
/* ------------------------------------------------------------------------ */

int ckq_quantize_q8_k_dev(const float *x, void *y, int num_rows, int k, void *stream)
{
    return ckq_launch_quantize_q8_k(x, y, num_rows, k, stream);
}

int ckq_quantize_q8_0_dev(const float *x, void *y, int num_rows, int k, void *stream)
{
    return ckq_launch_quantize_q8_0(x, y, num_rows, k, stream);
}

int ckq_gemm_nt_dev(int fmt, const void *A_q8, const void *B, const float *bias, float *C,
                    int M, int N, int K, long ldc, void *stream)
{
    if (fmt != CKQ_FMT_Q4_K && fmt != CKQ_FMT_Q5_K && fmt != CKQ_FMT_Q6_K && fmt != CKQ_FMT_Q8_0 && fmt != CKQ_FMT_Q5_0)
        return CKQ_EFORMAT;
    return ckq_launch_gemv(fmt, C, B, A_q8, bias, N, K, M, ldc, 0, N, NULL, stream);
}

int ckq_gemm_nt_noalloc_dev(int fmt, const void *A_q8, const void *B, const float *bias, float *C,
                            int M, int N, int K, long ldc, void *stream)
{
    return ckq_launch_gemv_noalloc(fmt, C, B, A_q8, bias, N, K, M, ldc, stream);
}

#define DEFINE_DEV(NAME, FMT)                                                                                   \
    int ckq_gemv_##NAME##_dev(float *y, const void *W, const void *x_q8, int M, int K, void *stream)            \
    {                                                                                                           \
        return ckq_launch_gemv(FMT, y, W, x_q8, NULL, M, K, 1, M, 0, M, NULL, stream);                          \
    }                                                                                                           \
    int ckq_gemm_nt_##NAME##_dev(const void *A_q8, const void *B, const float *bias, float *C, int M, int N,    \
                                 int K, void *stream)                                                           \
    {                                                                                                           \
        return ckq_launch_gemv(FMT, C, B, A_q8, bias, N, K, M, N, 0, N, NULL, stream);                          \
    }

DEFINE_DEV(q4_k_q8_k, CKQ_FMT_Q4_K)
DEFINE_DEV(q5_k_q8_k, CKQ_FMT_Q5_K)
DEFINE_DEV(q6_k_q8_k, CKQ_FMT_Q6_K)
DEFINE_DEV(q8_0_q8_0, CKQ_FMT_Q8_0)

int ckq_gemv_q8_0_dev(float *y, const void *W, const float *x, int M, int K, void *stream)
{
    return ckq_launch_gemv(CKQ_KERNEL_Q80_F32, y, W, x, NULL, M, K, 1, M, 0, M, NULL, stream);
}

int ckq_dequant_rows_dev(int fmt, const void *table, const int32_t *ids, int vocab, const float *pos, float *out,
                         int n_valid, int n_row, int tokens, int n_out_rows, void *stream)
{
    return ckq_launch_dequant_rows(fmt, table, ids, vocab, pos, out, n_valid, n_row, tokens, n_out_rows, stream);
}

int ckq_rmsnorm_q8_k_fused_dev(const float *input, const float *gamma, void *y, int tokens, int d_model,
                               int aligned_embed_dim, float eps, void *stream)
{
    return ckq_launch_rmsnorm_q8_k_fused(input, gamma, y, tokens, d_model, aligned_embed_dim, eps, stream);
}

int ckq_swiglu_q8_k_dev(const float *gate, const float *up, void *y, int rows, int k, long ld, void *stream)
{
    return ckq_launch_swiglu_q8_k(gate, up, y, rows, k, ld, stream);
}

int ckq_gemm_nt_f32act_dev(int fmt, const float *A, const void *B, const float *bias, float *C,
                           int M, int N, int K, long ldc, void *stream)
{
    const int k = fmt == CKQ_FMT_Q4_K ? CKQ_KERNEL_Q4K_F32 : fmt == CKQ_FMT_Q6_K ? CKQ_KERNEL_Q6K_F32
                : fmt == CKQ_FMT_Q8_0 ? CKQ_KERNEL_Q80_F32 : -1;
    if (k < 0) return CKQ_EFORMAT;
    return ckq_launch_gemv(k, C, B, A, bias, N, K, M, ldc, 0, N, NULL, stream);
}

static int ranges_overlap(const void *a, size_t na, const void *b, size_t nb) { return ckq_ranges_overlap(a, na, b, nb); }

/* Entries i and j of a sequence can share a launch when they have one format,
 * input width and token count (their row counts may differ: K and V are
 * narrower than Q under grouped-query attention) and neither writes what the
 * other reads or writes. */
static int ops_independent(const ckq_matmul_op *p, const ckq_matmul_op *q)
{
    if (p->fmt != q->fmt || p->M != q->M || p->K != q->K || q->N <= 0 || q->ldc < q->N || !q->A_q8 || !q->B || !q->C)
        return 0;
    const size_t pc = ((size_t)(p->M - 1) * (size_t)p->ldc + (size_t)p->N) * sizeof(float);
    const size_t qc = ((size_t)(q->M - 1) * (size_t)q->ldc + (size_t)q->N) * sizeof(float);
    const size_t ab = (size_t)p->M * act_row_bytes(p->fmt, p->K);
    const size_t pw = (size_t)p->N * weight_row_bytes(p->fmt, p->K), qw = (size_t)q->N * weight_row_bytes(q->fmt, q->K);
    if (ranges_overlap(p->C, pc, q->C, qc)) return 0;
    if (ranges_overlap(p->C, pc, q->A_q8, ab) || ranges_overlap(q->C, qc, p->A_q8, ab)) return 0;
    if (ranges_overlap(p->C, pc, q->B, qw) || ranges_overlap(q->C, qc, p->B, pw)) return 0;
    if (p->bias && ranges_overlap(q->C, qc, p->bias, (size_t)p->N * sizeof(float))) return 0;
    if (q->bias && ranges_overlap(p->C, pc, q->bias, (size_t)q->N * sizeof(float))) return 0;
    return 1;
}

/* A producer entry of a sequence: the activation quantizer in front of the matmuls that follow. */
static int issue_producer(const ckq_matmul_op *o, void *stream)
{
    if (!o->A_q8 || !o->C || o->M <= 0 || o->K <= 0) return CKQ_EINVAL;
    const long ld = o->ldc ? o->ldc : o->K;
    switch (o->fmt) {
    case CKQ_STEP_QUANTIZE_Q8_K: return ckq_launch_quantize_q8_k((const float *)o->A_q8, o->C, o->M, o->K, stream);
    case CKQ_STEP_QUANTIZE_Q8_0: return ckq_launch_quantize_q8_0((const float *)o->A_q8, o->C, o->M, o->K, stream);
    case CKQ_STEP_RMSNORM_Q8_K:
        if (ld > 0x7fffffff) return CKQ_EINVAL;
        return ckq_launch_rmsnorm_q8_k_fused((const float *)o->A_q8, (const float *)o->B, o->C, o->M, o->K, (int)ld, o->eps, stream);
    case CKQ_STEP_SWIGLU_Q8_K:
        return ckq_launch_swiglu_q8_k((const float *)o->A_q8, (const float *)o->B, o->C, o->M, o->K, ld, stream);
    default: return CKQ_EFORMAT;
    }
}

/* Number of consecutive matmul entries from ops[i] on that can share a launch (1..4). */
static int group_length(const ckq_matmul_op *ops, int i, int nops)
{
    enum { GROUP_MAX = 4 };
    const ckq_matmul_op *o = &ops[i];
    int n = 1;
    const int groupable = o->A_q8 && o->B && o->C && o->M >= 1 && o->N > 0 && o->K > 0 &&
                          o->ldc >= o->N && !is_f32act(o->fmt) && !(o->fmt & CKQ_ACT_F32) && o->K % fmt_block_elems(o->fmt) == 0;
    while (groupable && n < GROUP_MAX && i + n < nops) {
        if (ops[i + n].fmt >= CKQ_STEP_QUANTIZE_Q8_K && ops[i + n].fmt <= CKQ_STEP_SWIGLU_Q8_K) break;
        if (ops[i + n].fmt & CKQ_ACT_F32) break;
        /* beyond eight tokens the matrices share a matrix-core launch, which takes one activation matrix */
        if (o->M > 8 && (ops[i + n].A_q8 != o->A_q8 || !__atomic_load_n(&g_prefill_grouping, __ATOMIC_RELAXED))) break;
        int ok = 1;
        for (int j = 0; j < n && ok; ++j) ok = ops_independent(&ops[i + j], &ops[i + n]);
        if (!ok) break;
        ++n;
    }
    return n;
}

int ckq_matmul_sequence_dev(const ckq_matmul_op *ops, int nops, int repeat, void *stream)
{
    if (!ops || nops <= 0 || repeat <= 0) return CKQ_EINVAL;
    enum { GROUP_MAX = 4 };
    for (int r = 0; r < repeat; ++r)
        for (int i = 0; i < nops;) {
            const ckq_matmul_op *o = &ops[i];
            if (o->fmt >= CKQ_STEP_QUANTIZE_Q8_K && o->fmt <= CKQ_STEP_SWIGLU_Q8_K) {
                const int rc = issue_producer(o, stream);
                if (rc) return rc;
                ++i;
                continue;
            }
            if (o->fmt & CKQ_ACT_F32) {              /* fp32 activations: the dequant-dot kernels, one launch per entry */
                const int rc = ckq_gemm_nt_f32act_dev(o->fmt & ~CKQ_ACT_F32, (const float *)o->A_q8, o->B, o->bias, o->C, o->M,
                                                      o->N, o->K, o->ldc, stream);
                if (rc) return rc;
                ++i;
                continue;
            }
            /* consecutive entries of one shape that do not depend on each other
             * (Q/K/V, gate/up) go out as one launch */
            const int n = group_length(ops, i, nops);
            int rc;
            if (n > 1) {
                float *y[GROUP_MAX];
                const void *W[GROUP_MAX], *X[GROUP_MAX];
                const float *b[GROUP_MAX];
                int rows[GROUP_MAX];
                long ld[GROUP_MAX];
                for (int j = 0; j < n; ++j) {
                    y[j] = ops[i + j].C; W[j] = ops[i + j].B; X[j] = ops[i + j].A_q8; b[j] = ops[i + j].bias;
                    rows[j] = ops[i + j].N; ld[j] = ops[i + j].ldc;
                }
                rc = o->M > 8 ? ckq_launch_gemm_group(o->fmt, n, y, W, o->A_q8, b, rows, ld, o->K, o->M, stream)
                              : ckq_launch_gemv_group(o->fmt, n, y, W, X, b, rows, ld, o->K, o->M, NULL, stream);
                if (rc == CKQ_ENOGROUP) {            /* better one by one (too few tiles, or sizes the streaming kernel serves) */
                    rc = 0;
                    for (int j = 0; j < n && !rc; ++j)
                        rc = ckq_gemm_nt_dev(ops[i + j].fmt, ops[i + j].A_q8, ops[i + j].B, ops[i + j].bias, ops[i + j].C,
                                             ops[i + j].M, ops[i + j].N, ops[i + j].K, ops[i + j].ldc, stream);
                }
            } else {
                rc = ckq_gemm_nt_dev(o->fmt, o->A_q8, o->B, o->bias, o->C, o->M, o->N, o->K, o->ldc, stream);
            }
            if (rc) return rc;
            i += n;
        }
    return 0;
}

int ckq_subblock_dots_dev(int fmt, int32_t *out, const void *W, const void *x_q8, int M, int K, void *stream)
{
    if (!out) return CKQ_EINVAL;
    if (fmt != CKQ_FMT_Q4_K && fmt != CKQ_FMT_Q5_K && fmt != CKQ_FMT_Q6_K && fmt != CKQ_FMT_Q8_0 && fmt != CKQ_FMT_Q5_0)
        return CKQ_EFORMAT;
    return ckq_launch_gemv(fmt, NULL, W, x_q8, NULL, M, K, 1, M, 0, M, out, stream);
}

int ckq_subblock_dots_tokens_dev(int fmt, int32_t *out, const void *W, const void *X_q8, int M, int K, int ntok, void *stream)
{
    if (!out) return CKQ_EINVAL;
    if (fmt != CKQ_FMT_Q4_K && fmt != CKQ_FMT_Q5_K && fmt != CKQ_FMT_Q6_K && fmt != CKQ_FMT_Q8_0 && fmt != CKQ_FMT_Q5_0)
        return CKQ_EFORMAT;
    return ckq_launch_gemv(fmt, NULL, W, X_q8, NULL, M, K, ntok, M, 0, M, out, stream);
}

int ckq_subblock_dots_group_dev(int fmt, int n, int32_t *out, const void *const *W, const void *const *X_q8, const int *rows,
                                int K, int ntok, void *stream)
{
    if (!out) return CKQ_EINVAL;
    if (fmt != CKQ_FMT_Q4_K && fmt != CKQ_FMT_Q5_K && fmt != CKQ_FMT_Q6_K && fmt != CKQ_FMT_Q8_0 && fmt != CKQ_FMT_Q5_0)
        return CKQ_EFORMAT;
    return ckq_launch_gemv_group(fmt, n, NULL, W, X_q8, NULL, rows, NULL, K, ntok, out, stream);
}

int ckq_gemm_block_sums_dev(int fmt, const void *A_q8, const void *B, const float *bias, float *C, int32_t *sums,
                            int M, int N, int K, void *stream)
{
    return ckq_launch_gemm_block_sums(fmt, A_q8, B, bias, C, sums, M, N, K, N, stream);
}

int ckq_copy_dev(void *dst, const void *src, size_t bytes, void *stream)
{
    return ckq_launch_copy(dst, src, bytes, stream);
}

int ckq_read_dev(const void *src, size_t bytes, void *sink, void *stream)
{
    return ckq_launch_read(src, bytes, sink, stream);
}

int ckq_read_tuned_dev(const void *src, size_t bytes, void *sink, int blocks, int unroll, void *stream)
{
    return ckq_launch_read_tuned(src, bytes, sink, blocks, unroll, stream);
}
