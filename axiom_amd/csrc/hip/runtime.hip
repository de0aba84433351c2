// Lifecycle, memory and timing entry points of libaxhip.so.
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include <mutex>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "common.h"

namespace {
thread_local char t_err[512] = "";
thread_local const char *t_kernel = "";
int g_ready = 0;            // 1 once a gfx950-class device was initialised
int g_devices = -1;
char g_name[128] = "";
int g_cu_count = 0;
void *g_ws = nullptr;
size_t g_ws_bytes = 0;
int *g_ctr = nullptr;
size_t g_ctr_n = 0;
float *g_ones = nullptr;
size_t g_ones_n = 0;

// allocation pool: block -> rounded size for everything handed out, and the free blocks per size
std::mutex g_pool_mutex;
std::unordered_map<void *, size_t> g_pool_size;
std::unordered_map<size_t, std::vector<void *>> g_pool_free;
std::unordered_set<void *> g_pool_idle;                  // blocks sitting in g_pool_free: a second free of one is ignored
// what callers asked for and gave back (ax_cuda_alloc_stats, cuda/memory.cu:13-29), and how often the driver was needed
int64_t g_stat_allocs = 0, g_stat_frees = 0, g_stat_bytes_alloc = 0, g_stat_bytes_free = 0, g_stat_driver_allocs = 0;
size_t g_pool_cached = 0;
constexpr size_t kPoolMaxBlock = size_t(1) << 30;        // larger blocks go straight back to the driver
constexpr size_t kPoolMaxCached = size_t(16) << 30;      // bytes the pool may hold back

axhip::Tuning g_tuning = {};

// "64x64" / "128x128" / "256x256" / "128x256" / "64x64k2" or the bare first number; 0 when absent or not one of `allowed`
int parse_tile(const char *name, const int *allowed, int n_allowed) {
    const char *v = getenv(name);
    if (!v || !*v) return 0;
    char *end = nullptr;
    long t = strtol(v, &end, 10);
    if (end == v) return 0;
    if (strstr(v, "k2")) t = t * 10 + 2;
    if (t == 128 && !strcmp(end, "x64")) t = 1264;
    for (int i = 0; i < n_allowed; i++)
        if (allowed[i] == t) return (int)t;
    return 0;
}

// one of `names` exactly: its position + 1, else 0
int parse_choice(const char *name, const char *const *names, int n) {
    const char *v = getenv(name);
    if (!v || !*v) return 0;
    for (int i = 0; i < n; i++)
        if (!strcmp(v, names[i])) return i + 1;
    return 0;
}

int parse_count(const char *name, long lo, long hi) {
    const char *v = getenv(name);
    if (!v || !*v) return 0;
    char *end = nullptr;
    const long t = strtol(v, &end, 10);
    return (end != v && *end == 0 && t >= lo && t <= hi) ? (int)t : 0;
}
}  // namespace

namespace axhip {

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(t_err, sizeof t_err, fmt, ap);
    va_end(ap);
    return code;
}

int cu_count() { return g_cu_count; }

const Tuning &tuning() { return g_tuning; }

// sizes are rounded so that blocks get reused: powers of two up to 1 MiB, then multiples of 1 MiB
size_t pool_class(size_t bytes) {
    if (bytes <= (size_t(1) << 20)) {
        size_t c = 256;
        while (c < bytes) c <<= 1;
        return c;
    }
    const size_t mib = size_t(1) << 20;
    return (bytes + mib - 1) / mib * mib;
}

// returns every cached block to the driver (out of memory, shutdown)
void pool_release_all() {
    std::vector<void *> blocks;
    {
        std::lock_guard<std::mutex> lock(g_pool_mutex);
        for (auto &kv : g_pool_free)
            for (void *p : kv.second) {
                blocks.push_back(p);
                g_pool_size.erase(p);
            }
        g_pool_free.clear();
        g_pool_idle.clear();
        g_pool_cached = 0;
    }
    for (void *p : blocks) (void)hipFree(p);
}

void note_kernel(const char *name) { t_kernel = name; }

int ensure_ready() {
    if (g_ready) return AXHIP_OK;
    return axhip_init();
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(AXHIP_ERR_BACKEND, "%s launch: %s", what, hipGetErrorString(e));
    return AXHIP_OK;
}

void *workspace(size_t bytes) {
    if (bytes <= g_ws_bytes) return g_ws;
    if (g_ws) {
        (void)hipDeviceSynchronize();
        (void)hipFree(g_ws);
        g_ws = nullptr;
        g_ws_bytes = 0;
    }
    size_t want = bytes < (size_t(8) << 20) ? (size_t(8) << 20) : bytes;
    if (hipMalloc(&g_ws, want) != hipSuccess) {
        g_ws = nullptr;
        fail(AXHIP_ERR_ALLOC, "workspace of %zu bytes: out of device memory", want);
        return nullptr;
    }
    g_ws_bytes = want;
    return g_ws;
}

float *ones_vector(size_t n) {
    if (n <= g_ones_n) return g_ones;
    if (g_ones) {
        (void)hipDeviceSynchronize();
        (void)hipFree(g_ones);
        g_ones = nullptr;
        g_ones_n = 0;
    }
    size_t want = n < 65536 ? 65536 : n;
    if (hipMalloc(reinterpret_cast<void **>(&g_ones), want * sizeof(float)) != hipSuccess) {
        g_ones = nullptr;
        fail(AXHIP_ERR_ALLOC, "ones vector (%zu floats): out of device memory", want);
        return nullptr;
    }
    g_ones_n = want;      // set before the fill so a failure below still leaves a consistent size
    if (axhip_fill_f32(g_ones, 1.0f, (int64_t)want) != AXHIP_OK) {
        (void)hipFree(g_ones);
        g_ones = nullptr;
        g_ones_n = 0;
        return nullptr;
    }
    return g_ones;
}

int *strip_counters(size_t n) {
    if (n <= g_ctr_n) return g_ctr;
    if (g_ctr) {
        (void)hipDeviceSynchronize();
        (void)hipFree(g_ctr);
        g_ctr = nullptr;
        g_ctr_n = 0;
    }
    size_t want = n < 4096 ? 4096 : n;
    if (hipMalloc(reinterpret_cast<void **>(&g_ctr), want * sizeof(int)) != hipSuccess ||
        hipMemset(g_ctr, 0, want * sizeof(int)) != hipSuccess) {
        g_ctr = nullptr;
        fail(AXHIP_ERR_ALLOC, "arrival counters (%zu ints): out of device memory", want);
        return nullptr;
    }
    g_ctr_n = want;
    return g_ctr;
}

int strip_counters_reset() {
    if (g_ctr && hipMemsetAsync(g_ctr, 0, g_ctr_n * sizeof(int), kStream) != hipSuccess)
        return fail(AXHIP_ERR_BACKEND, "zero-fill of the arrival counters failed");
    return AXHIP_OK;
}

}  // namespace axhip

using axhip::fail;

extern "C" {

int axhip_device_count(void) {
    if (g_devices >= 0) return g_devices;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) n = 0;
    g_devices = n;
    return n;
}

int axhip_tuning_reload(void) {
    static const int i8_tiles[] = {64, 642, 128, 1264, 256}, f32_tiles[] = {64, 642, 128};
    g_tuning.i8_tile = parse_tile("AX_HIP_I8_TILE", i8_tiles, 5);
    g_tuning.i8_splitk = parse_count("AX_HIP_I8_SPLITK", 1, 16);
    g_tuning.i8_mfma = parse_count("AX_HIP_I8_MFMA", 16, 32);
    if (g_tuning.i8_mfma != 16 && g_tuning.i8_mfma != 32) g_tuning.i8_mfma = 0;
    g_tuning.f32_tile = parse_tile("AX_HIP_F32_TILE", f32_tiles, 3);
    g_tuning.f32_splitk = parse_count("AX_HIP_F32_SPLITK", 1, 4096);
    g_tuning.skinny_blocks = parse_count("AX_HIP_SKINNY_BLOCKS", 1, 65535);
    g_tuning.skinny_form = parse_count("AX_HIP_SKINNY_FORM", 1, 3);
    g_tuning.skinny_kps = parse_count("AX_HIP_SKINNY_KPS", 16, 8192) / 16 * 16;
    g_tuning.nt_walk = parse_count("AX_HIP_NT_WALK", 1, 2);
    static const char *const w8a32_tiles[] = {"128x256", "128x128", "64x128", "32x128", "32x64"};
    g_tuning.w8a32_tile = parse_choice("AX_HIP_W8A32_TILE", w8a32_tiles, 5);
    return (g_tuning.i8_tile != 0) + (g_tuning.i8_splitk != 0) + (g_tuning.f32_tile != 0) + (g_tuning.f32_splitk != 0) +
           (g_tuning.skinny_blocks != 0) + (g_tuning.w8a32_tile != 0) + (g_tuning.skinny_form != 0) + (g_tuning.skinny_kps != 0) + (g_tuning.i8_mfma != 0) + (g_tuning.nt_walk != 0);
}

int axhip_workspace_reserve(size_t bytes, size_t *have) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (bytes > 0 && !axhip::workspace(bytes)) return AXHIP_ERR_ALLOC;
    if (have) *have = g_ws_bytes;
    return AXHIP_OK;
}

int axhip_tuning_get(const char *name) {
    if (!name) return -1;
    if (!strcmp(name, "AX_HIP_I8_TILE")) return g_tuning.i8_tile;
    if (!strcmp(name, "AX_HIP_I8_SPLITK")) return g_tuning.i8_splitk;
    if (!strcmp(name, "AX_HIP_I8_MFMA")) return g_tuning.i8_mfma;
    if (!strcmp(name, "AX_HIP_F32_TILE")) return g_tuning.f32_tile;
    if (!strcmp(name, "AX_HIP_F32_SPLITK")) return g_tuning.f32_splitk;
    if (!strcmp(name, "AX_HIP_SKINNY_BLOCKS")) return g_tuning.skinny_blocks;
    if (!strcmp(name, "AX_HIP_SKINNY_FORM")) return g_tuning.skinny_form;
    if (!strcmp(name, "AX_HIP_SKINNY_KPS")) return g_tuning.skinny_kps;
    if (!strcmp(name, "AX_HIP_NT_WALK")) return g_tuning.nt_walk;
    if (!strcmp(name, "AX_HIP_W8A32_TILE")) return g_tuning.w8a32_tile;
    return -1;
}

int axhip_init(void) {
    if (g_ready) return AXHIP_OK;
    (void)axhip_tuning_reload();
    if (axhip_device_count() <= 0)
        return fail(AXHIP_ERR_BACKEND, "no HIP device visible: libaxhip has no CPU fallback");
    AXHIP_HIP_TRY(hipSetDevice(0), "hipSetDevice");
    hipDeviceProp_t prop;
    AXHIP_HIP_TRY(hipGetDeviceProperties(&prop, 0), "hipGetDeviceProperties");
    snprintf(g_name, sizeof g_name, "%s", prop.gcnArchName);
    g_cu_count = prop.multiProcessorCount;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(AXHIP_ERR_BACKEND, "device 0 is %s; this library holds gfx950 code only",
                    prop.gcnArchName);
    if (int rc = axhip::skinny_setup()) return rc;
    // the shared workspace and the arrival counters exist from the start (64 MiB, 4096 counters): a first
    // call at a new shape then pays no allocation or device-wide wait unless it needs more than that
    if (!axhip::workspace(size_t(64) << 20) || !axhip::strip_counters(4096)) return AXHIP_ERR_ALLOC;
    g_ready = 1;
    return AXHIP_OK;
}

void axhip_shutdown(void) {
    if (!g_ready) return;
    (void)hipDeviceSynchronize();
    axhip::pool_release_all();
    axhip::skinny_teardown();
    if (g_ws) (void)hipFree(g_ws);
    if (g_ctr) (void)hipFree(g_ctr);
    if (g_ones) (void)hipFree(g_ones);
    g_ones = nullptr;
    g_ones_n = 0;
    g_ws = nullptr;
    g_ws_bytes = 0;
    g_ctr = nullptr;
    g_ctr_n = 0;
    g_ready = 0;
}

int axhip_synchronize(void) {
    if (int rc = axhip::ensure_ready()) return rc;
    AXHIP_HIP_TRY(hipDeviceSynchronize(), "hipDeviceSynchronize");
    return AXHIP_OK;
}

const char *axhip_last_error(void) { return t_err; }
const char *axhip_device_name(void) { return g_name; }
const char *axhip_last_kernel(void) { return t_kernel; }

// Device allocations go through a pool: a freed block is kept, keyed by its rounded size, and
// handed out again without a trip to the driver.  hipMalloc costs tens of microseconds and
// hipFree waits for the whole device, which is several times the run time of the bs=1 kernels
// whose outputs the host core allocates and releases on every call.  Reuse is safe because all
// work runs in issue order on one stream: whatever still reads a released block was enqueued
// before whatever writes its next owner.  Blocks above 1 GiB are returned to the driver at once;
// when the driver is out of memory the pool is emptied and the request retried.
static void *pool_take(size_t bytes) {
    if (axhip::ensure_ready()) return nullptr;
    if (bytes == 0) bytes = 4;
    const size_t size = axhip::pool_class(bytes);
    void *p = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_pool_mutex);
        auto it = g_pool_free.find(size);
        if (it != g_pool_free.end() && !it->second.empty()) {
            p = it->second.back();
            it->second.pop_back();
            g_pool_cached -= size;
            g_pool_idle.erase(p);
            g_stat_allocs++;
            g_stat_bytes_alloc += (int64_t)size;
        }
    }
    if (!p) {
        if (hipMalloc(&p, size) != hipSuccess) {
            (void)hipGetLastError();
            axhip::pool_release_all();
            if (hipMalloc(&p, size) != hipSuccess) {
                (void)hipGetLastError();
                fail(AXHIP_ERR_ALLOC, "hipMalloc(%zu) failed", size);
                return nullptr;
            }
        }
        std::lock_guard<std::mutex> lock(g_pool_mutex);
        g_pool_size[p] = size;
        g_stat_allocs++;
        g_stat_driver_allocs++;
        g_stat_bytes_alloc += (int64_t)size;
    }
    return p;
}

void *axhip_malloc_uninit(size_t bytes) { return pool_take(bytes); }

void *axhip_malloc(size_t bytes) {
    void *p = pool_take(bytes);
    if (p && bytes && hipMemsetAsync(p, 0, bytes, axhip::kStream) != hipSuccess) {
        axhip_free(p);
        fail(AXHIP_ERR_BACKEND, "zero-fill of %zu bytes failed", bytes);
        return nullptr;
    }
    return p;
}

void axhip_free(void *p) {
    if (!p) return;
    size_t size = 0;
    {
        std::lock_guard<std::mutex> lock(g_pool_mutex);
        auto it = g_pool_size.find(p);
        if (it == g_pool_size.end() || g_pool_idle.count(p)) return;   // not ours, or freed twice: leave it alone
        size = it->second;
        g_stat_frees++;
        g_stat_bytes_free += (int64_t)size;
        if (size <= kPoolMaxBlock && g_pool_cached + size <= kPoolMaxCached) {
            g_pool_free[size].push_back(p);
            g_pool_idle.insert(p);
            g_pool_cached += size;
            return;
        }
        g_pool_size.erase(it);
    }
    (void)hipFree(p);
}

void axhip_alloc_stats(int64_t *allocs, int64_t *frees, int64_t *bytes_alloc, int64_t *bytes_free,
                       int64_t *driver_allocs, int64_t *bytes_cached) {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    if (allocs) *allocs = g_stat_allocs;
    if (frees) *frees = g_stat_frees;
    if (bytes_alloc) *bytes_alloc = g_stat_bytes_alloc;
    if (bytes_free) *bytes_free = g_stat_bytes_free;
    if (driver_allocs) *driver_allocs = g_stat_driver_allocs;
    if (bytes_cached) *bytes_cached = (int64_t)g_pool_cached;
}

int64_t axhip_device_free_bytes(void) {
    if (axhip::ensure_ready()) return -1;
    size_t free_bytes = 0, total = 0;
    if (hipMemGetInfo(&free_bytes, &total) != hipSuccess) return -1;
    return (int64_t)free_bytes;
}

void axhip_reset_alloc_stats(void) {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    g_stat_allocs = g_stat_frees = g_stat_bytes_alloc = g_stat_bytes_free = g_stat_driver_allocs = 0;
}

int axhip_memset(void *p, int v, size_t bytes) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!p) return fail(AXHIP_ERR_NULL_ARG, "memset: NULL");
    AXHIP_HIP_TRY(hipMemsetAsync(p, v, bytes, axhip::kStream), "hipMemsetAsync");
    return AXHIP_OK;
}

int axhip_memcpy_h2d(void *dst, const void *src, size_t bytes) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!dst || !src) return fail(AXHIP_ERR_NULL_ARG, "memcpy_h2d: NULL");
    AXHIP_HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice), "hipMemcpy h2d");
    return AXHIP_OK;
}

int axhip_memcpy_d2h(void *dst, const void *src, size_t bytes) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!dst || !src) return fail(AXHIP_ERR_NULL_ARG, "memcpy_d2h: NULL");
    AXHIP_HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost), "hipMemcpy d2h");
    return AXHIP_OK;
}

int axhip_memcpy_d2d(void *dst, const void *src, size_t bytes) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!dst || !src) return fail(AXHIP_ERR_NULL_ARG, "memcpy_d2d: NULL");
    AXHIP_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, axhip::kStream),
                  "hipMemcpy d2d");
    return AXHIP_OK;
}

void *axhip_event_create(void) {
    if (axhip::ensure_ready()) return nullptr;
    hipEvent_t ev;
    if (hipEventCreate(&ev) != hipSuccess) return nullptr;
    return (void *)ev;
}

void axhip_event_destroy(void *ev) {
    if (ev) (void)hipEventDestroy((hipEvent_t)ev);
}

int axhip_event_record(void *ev) {
    if (!ev) return fail(AXHIP_ERR_NULL_ARG, "event_record: NULL");
    AXHIP_HIP_TRY(hipEventRecord((hipEvent_t)ev, axhip::kStream), "hipEventRecord");
    return AXHIP_OK;
}

int axhip_event_elapsed_ms(void *start, void *stop, float *ms) {
    if (!start || !stop || !ms) return fail(AXHIP_ERR_NULL_ARG, "event_elapsed: NULL");
    AXHIP_HIP_TRY(hipEventSynchronize((hipEvent_t)stop), "hipEventSynchronize");
    AXHIP_HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop),
                  "hipEventElapsedTime");
    return AXHIP_OK;
}

}  // extern "C"
