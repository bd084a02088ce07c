// Host side of libmk_hip.so: device context, error reporting, the pointer-keyed
// weight cache and the host-slice entry points that stand where the reference's
// Metal calls stand (src/metal.rs:441-451,599-665,874-1017).
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <chrono>
#include <map>
#include <mutex>
#include <set>
#include <tuple>
#include <vector>

#include "mk_common.h"

namespace {

thread_local char g_err[512] = "";
std::mutex g_mu;  // serialises host-level calls (the reference's io mutex)

struct DevBuf {
    void *p = nullptr;
    size_t cap = 0;
    int ensure(size_t bytes) {
        if (bytes <= cap) return MK_OK;
        if (p) hipFree(p);
        p = nullptr;
        cap = 0;
        size_t want = bytes < 4096 ? 4096 : bytes;
        if (mk_check_hip(hipMalloc(&p, want), "hipMalloc(staging)") != MK_OK) return MK_ERR_NOMEM;
        cap = want;
        return MK_OK;
    }
};

struct CachedWeight {
    void *packed = nullptr;  // MXFP4: the nibbles; f32: the matrix
    void *scales = nullptr;  // MXFP4 only
    size_t bytes = 0;
    uint8_t head[16] = {};   // the first bytes as they were at upload time: a hit is re-validated against the host
    size_t nhead = 0;        // bytes without touching the device (src/metal.rs:417-430 re-reads its own shared buffer)
};

struct Ctx {
    bool ready = false;
    int status = MK_ERR_NO_DEVICE;
    int device = -1;
    hipStream_t stream = nullptr;
    size_t cache_cap = 0;  // bytes, 0 = unlimited
    size_t cache_bytes = 0;
    std::map<std::tuple<const void *, size_t, size_t, int>, CachedWeight> cache;  // (host pointer, rows, cols, kind)
    DevBuf x, y, xq, xs, tmp;
    int force_q8 = -1;
    bool prof_on = false;
    mk_prof prof = {};
};
Ctx g_ctx;

int ensure_init() {
    MK_REQUIRE_ENABLED();
    if (g_ctx.ready) return MK_OK;
    return mk_init(0);
}

// HIP's current device is a per-thread setting: every host-level entry point binds the calling thread to the
// library's device before it touches the runtime (called with g_mu held).
int bind_device() { return mk_check_hip(hipSetDevice(g_ctx.device), "hipSetDevice"); }

double now_ms() { return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count(); }

}  // namespace

void mk_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int mk_check_hip(hipError_t e, const char *what) {
    if (e == hipSuccess) return MK_OK;
    mk_set_error("HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
    return MK_ERR_HIP;
}

int mk_launch_status(const char *kernel) {
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return MK_OK;
    mk_set_error("launch of %s failed: %d (%s)", kernel, (int)e, hipGetErrorString(e));
    return MK_ERR_HIP;
}

int mk_env_int(const char *name, int dflt) {
    const char *e = getenv(name);
    return (e && *e) ? atoi(e) : dflt;
}

int mk_lds_opt_in(const void *kernel, int bytes) {
    static std::mutex mu;
    static std::set<std::pair<const void *, int>> done;
    // what this thread has already seen done: the launch path takes no lock after a kernel's first launch
    thread_local const void *seen_kernel[8] = {};
    thread_local int seen_dev[8] = {};
    int dev = 0;
    MK_HIP_TRY(hipGetDevice(&dev));
    const unsigned slot = (unsigned)(((uintptr_t)kernel >> 4) & 7);
    if (seen_kernel[slot] == kernel && seen_dev[slot] == dev) return MK_OK;
    std::lock_guard<std::mutex> lk(mu);
    if (!done.count({kernel, dev})) {
        MK_HIP_TRY(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
        done.insert({kernel, dev});
    }
    seen_kernel[slot] = kernel;
    seen_dev[slot] = dev;
    return MK_OK;
}

extern "C" const char *mk_last_error(void) { return g_err; }

int mk_enabled_state = -1;
int mk_enabled_slow() {
    const char *e = getenv("MK_HIP");
    const int on = !(e && e[0] == '0' && e[1] == 0);
    int expect = -1;
    __atomic_compare_exchange_n(&mk_enabled_state, &expect, on, false, __ATOMIC_RELAXED, __ATOMIC_RELAXED);
    return __atomic_load_n(&mk_enabled_state, __ATOMIC_RELAXED);
}
extern "C" void mk_set_enabled(int on) { __atomic_store_n(&mk_enabled_state, on ? 1 : 0, __ATOMIC_RELAXED); }
extern "C" int mk_enabled_now(void) { return mk_enabled() ? 1 : 0; }

extern "C" int mk_init(int device) {
    MK_REQUIRE_ENABLED();
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_ctx.ready) return MK_OK;
    int n = 0;
    hipError_t ce = hipGetDeviceCount(&n);
    if (ce != hipSuccess || n <= 0) {
        mk_set_error("no HIP device visible (hipGetDeviceCount: %d %s, count %d)", (int)ce, hipGetErrorString(ce), n);
        return g_ctx.status = MK_ERR_NO_DEVICE;
    }
    if (device < 0 || device >= n) {
        mk_set_error("device %d out of range (%d visible)", device, n);
        return g_ctx.status = MK_ERR_NO_DEVICE;
    }
    hipDeviceProp_t prop;
    if (mk_check_hip(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties") != MK_OK) return g_ctx.status = MK_ERR_NO_DEVICE;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        mk_set_error("device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
        return g_ctx.status = MK_ERR_NO_DEVICE;
    }
    if (mk_check_hip(hipSetDevice(device), "hipSetDevice") != MK_OK) return g_ctx.status = MK_ERR_HIP;
    if (mk_check_hip(hipStreamCreate(&g_ctx.stream), "hipStreamCreate") != MK_OK) return g_ctx.status = MK_ERR_HIP;
    if (mk_mla_static_init(nullptr) != MK_OK) {
        // a failed initialisation keeps nothing: the next mk_init starts from the beginning
        hipStreamDestroy(g_ctx.stream);
        g_ctx.stream = nullptr;
        return g_ctx.status = MK_ERR_HIP;
    }
    const char *mb = getenv("MK_GPU_CACHE_MB");
    if (mb && *mb) g_ctx.cache_cap = (size_t)strtoull(mb, nullptr, 10) << 20;
    const char *dbg = getenv("MK_GPU_DEBUG");
    g_ctx.prof_on = dbg && strcmp(dbg, "1") == 0;
    g_ctx.device = device;
    g_ctx.ready = true;
    return g_ctx.status = MK_OK;
}

extern "C" int mk_available(void) { return g_ctx.ready && mk_enabled() ? 1 : 0; }

extern "C" void mk_shutdown(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_ctx.ready) return;
    hipStreamSynchronize(g_ctx.stream);
    for (auto &kv : g_ctx.cache) {
        hipFree(kv.second.packed);
        hipFree(kv.second.scales);
    }
    g_ctx.cache.clear();
    g_ctx.cache_bytes = 0;
    for (DevBuf *b : {&g_ctx.x, &g_ctx.y, &g_ctx.xq, &g_ctx.xs, &g_ctx.tmp}) {
        if (b->p) hipFree(b->p);
        b->p = nullptr;
        b->cap = 0;
    }
    hipStreamDestroy(g_ctx.stream);
    g_ctx.stream = nullptr;
    g_ctx.ready = false;
    g_ctx.status = MK_ERR_NO_DEVICE;
}

extern "C" void mk_set_cache_mb(size_t mb) {
    std::lock_guard<std::mutex> lk(g_mu);
    g_ctx.cache_cap = mb << 20;
}

extern "C" void mk_force_q8(int v) {
    std::lock_guard<std::mutex> lk(g_mu);
    g_ctx.force_q8 = v < 0 ? -1 : (v ? 1 : 0);
}

namespace {
int q8_enabled_locked() {
    if (g_ctx.force_q8 >= 0) return g_ctx.force_q8;
    const char *e = getenv("MICROKIMI_NO_Q8");
    return (e && strcmp(e, "1") == 0) ? 0 : 1;
}
}  // namespace

extern "C" int mk_q8_enabled(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    return q8_enabled_locked();
}

// ------------------------------------------------------------- GpuProf
extern "C" void mk_prof_enable(int on) {
    std::lock_guard<std::mutex> lk(g_mu);
    g_ctx.prof_on = on != 0;
}

extern "C" void mk_prof_reset(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    g_ctx.prof = mk_prof{};
}

extern "C" void mk_prof_get(mk_prof *out) {
    if (!out) return;
    std::lock_guard<std::mutex> lk(g_mu);
    *out = g_ctx.prof;
    out->cache_tensors = g_ctx.cache.size();
    out->cache_bytes = g_ctx.cache_bytes;
}

extern "C" void mk_prof_print(void) {
    mk_prof p;
    mk_prof_get(&p);
    if (p.calls == 0) return;
    const double n = (double)p.calls, hm = (double)(p.hits + p.misses);
    printf("gpu profile: %llu matvec calls | weight cache: %llu hits, %llu misses (%.1f%% hit rate)\n", (unsigned long long)p.calls,
           (unsigned long long)p.hits, (unsigned long long)p.misses, 100.0 * (double)p.hits / (hm > 0 ? hm : 1.0));
    printf("  avg/call: cache %.3f ms | io %.3f ms | launch %.3f ms | wait %.3f ms | readback %.3f ms\n", p.t_cache_ms / n, p.t_io_ms / n,
           p.t_launch_ms / n, p.t_wait_ms / n, p.t_readback_ms / n);
    printf("  weight cache: %zu tensors, %.1f MB on device\n", p.cache_tensors, (double)p.cache_bytes / 1e6);
}

namespace {

// (host pointer, rows, cols) -> device copy, uploaded on first use; a hit is
// re-validated against the first 16 host bytes because a freed host buffer can
// come back at the same address with other contents (src/metal.rs:417-430).  The
// 16 bytes are kept on the host at upload time: a hit costs a memcmp, no device
// traffic.  kind 0: MXFP4 (pb nibble bytes + sb scale bytes), kind 1: f32 matrix
// (pb bytes, sb = 0).
int cached_weight(const void *w0, const void *w1, size_t rows, size_t cols, int kind, size_t pb, size_t sb, CachedWeight *out, bool *hit) {
    auto key = std::make_tuple(w0, rows, cols, kind);
    auto it = g_ctx.cache.find(key);
    *hit = false;
    if (it != g_ctx.cache.end()) {
        if (memcmp(it->second.head, w0, it->second.nhead) == 0) {
            *out = it->second;
            *hit = true;
            return MK_OK;
        }
        hipFree(it->second.packed);
        if (it->second.scales) hipFree(it->second.scales);
        g_ctx.cache_bytes -= it->second.bytes;
        g_ctx.cache.erase(it);
    }
    if (g_ctx.cache_cap && g_ctx.cache_bytes + pb + sb > g_ctx.cache_cap) {
        mk_set_error("device weight cache budget exhausted (%zu MiB)", g_ctx.cache_cap >> 20);
        return MK_ERR_NOMEM;
    }
    CachedWeight w;
    if (mk_check_hip(hipMalloc(&w.packed, pb ? pb : 16), "hipMalloc(weight)") != MK_OK) return MK_ERR_NOMEM;
    if (kind == 0 && mk_check_hip(hipMalloc(&w.scales, sb ? sb : 16), "hipMalloc(weight scales)") != MK_OK) {
        hipFree(w.packed);
        return MK_ERR_NOMEM;
    }
    w.bytes = pb + sb;
    w.nhead = pb < 16 ? pb : 16;
    memcpy(w.head, w0, w.nhead);
    int s = mk_check_hip(hipMemcpyAsync(w.packed, w0, pb, hipMemcpyHostToDevice, g_ctx.stream), "upload weight");
    if (s == MK_OK && kind == 0) s = mk_check_hip(hipMemcpyAsync(w.scales, w1, sb, hipMemcpyHostToDevice, g_ctx.stream), "upload scales");
    if (s == MK_OK) s = mk_check_hip(hipStreamSynchronize(g_ctx.stream), "upload sync");
    if (s != MK_OK) {
        hipFree(w.packed);
        if (w.scales) hipFree(w.scales);
        return s;
    }
    g_ctx.cache[key] = w;
    g_ctx.cache_bytes += w.bytes;
    *out = w;
    return MK_OK;
}

// The phases of a host-level matvec as src/metal.rs:750-870 times them (cache, io = input upload, launch = enqueue,
// wait, readback).  With profiling on, the input upload is synchronised on its own so that the phases separate.
struct Phases {
    double t0, t_cache = 0, t_io = 0, t_launch = 0, t_wait = 0, t_read = 0;
    bool on;
    explicit Phases(bool enabled) : t0(enabled ? now_ms() : 0.0), on(enabled) {}
    void mark(double &slot) {
        if (!on) return;
        const double t = now_ms();
        slot += t - t0;
        t0 = t;
    }
    void commit(bool hit) {
        mk_prof &p = g_ctx.prof;
        p.calls++;
        (hit ? p.hits : p.misses)++;
        p.t_cache_ms += t_cache;
        p.t_io_ms += t_io;
        p.t_launch_ms += t_launch;
        p.t_wait_ms += t_wait;
        p.t_readback_ms += t_read;
    }
};

}  // namespace

extern "C" int mk_mxfp4_matvec(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const float *x, float *out) {
    MK_REQUIRE(packed && scales && x && out, "null pointer");
    MK_REQUIRE(cols % 32 == 0 && cols > 0, "cols must be a positive multiple of 32");
    int s = ensure_init();
    if (s != MK_OK) return s;
    if (rows == 0) return MK_OK;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    Phases ph(g_ctx.prof_on);
    CachedWeight w;
    bool hit = false;
    if ((s = cached_weight(packed, scales, rows, cols, 0, rows * cols / 2, rows * cols / 32, &w, &hit)) != MK_OK) return s;
    ph.mark(ph.t_cache);
    if ((s = g_ctx.x.ensure(cols * 4)) != MK_OK) return s;
    if ((s = g_ctx.y.ensure(rows * 4)) != MK_OK) return s;
    if ((s = g_ctx.xq.ensure(cols)) != MK_OK) return s;
    if ((s = g_ctx.xs.ensure(cols / 32 * 4)) != MK_OK) return s;
    MK_HIP_TRY(hipMemcpyAsync(g_ctx.x.p, x, cols * 4, hipMemcpyHostToDevice, g_ctx.stream));
    if (ph.on) MK_HIP_TRY(hipStreamSynchronize(g_ctx.stream));
    ph.mark(ph.t_io);
    s = mk_dev_mxfp4_matvec((const uint8_t *)w.packed, (const uint8_t *)w.scales, rows, cols, (const float *)g_ctx.x.p, (float *)g_ctx.y.p,
                            q8_enabled_locked() ? MK_MODE_Q8 : MK_MODE_F32, (int8_t *)g_ctx.xq.p, (float *)g_ctx.xs.p, g_ctx.stream);
    if (s != MK_OK) return s;
    ph.mark(ph.t_launch);
    if (ph.on) MK_HIP_TRY(hipStreamSynchronize(g_ctx.stream));
    ph.mark(ph.t_wait);
    std::vector<float> host(rows);  // `out` stays untouched unless everything succeeded
    MK_HIP_TRY(hipMemcpyAsync(host.data(), g_ctx.y.p, rows * 4, hipMemcpyDeviceToHost, g_ctx.stream));
    MK_HIP_TRY(hipStreamSynchronize(g_ctx.stream));
    memcpy(out, host.data(), rows * 4);
    ph.mark(ph.t_read);
    if (ph.on) ph.commit(hit);
    return MK_OK;
}

// metal::gpu_matvec (src/metal.rs:750-870): y = W x for a row-major f32 matrix on host slices, the weight cached on the
// device like the packed ones.
extern "C" int mk_matvec_f32(const float *w, size_t rows, size_t cols, const float *x, float *out) {
    MK_REQUIRE(w && x && out, "null pointer");
    MK_REQUIRE(cols > 0, "cols must be positive");
    int s = ensure_init();
    if (s != MK_OK) return s;
    if (rows == 0) return MK_OK;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    Phases ph(g_ctx.prof_on);
    CachedWeight cw;
    bool hit = false;
    if ((s = cached_weight(w, nullptr, rows, cols, 1, rows * cols * 4, 0, &cw, &hit)) != MK_OK) return s;
    ph.mark(ph.t_cache);
    if ((s = g_ctx.x.ensure(cols * 4)) != MK_OK) return s;
    if ((s = g_ctx.y.ensure(rows * 4)) != MK_OK) return s;
    MK_HIP_TRY(hipMemcpyAsync(g_ctx.x.p, x, cols * 4, hipMemcpyHostToDevice, g_ctx.stream));
    if (ph.on) MK_HIP_TRY(hipStreamSynchronize(g_ctx.stream));
    ph.mark(ph.t_io);
    if ((s = mk_dev_matvec_f32((const float *)cw.packed, rows, cols, (const float *)g_ctx.x.p, 1, (float *)g_ctx.y.p, g_ctx.stream)) != MK_OK) return s;
    ph.mark(ph.t_launch);
    if (ph.on) MK_HIP_TRY(hipStreamSynchronize(g_ctx.stream));
    ph.mark(ph.t_wait);
    std::vector<float> host(rows);
    MK_HIP_TRY(hipMemcpyAsync(host.data(), g_ctx.y.p, rows * 4, hipMemcpyDeviceToHost, g_ctx.stream));
    MK_HIP_TRY(hipStreamSynchronize(g_ctx.stream));
    memcpy(out, host.data(), rows * 4);
    ph.mark(ph.t_read);
    if (ph.on) ph.commit(hit);
    return MK_OK;
}

extern "C" int mk_mxfp4_dequant(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, float *out) {
    MK_REQUIRE(packed && scales && out, "null pointer");
    MK_REQUIRE(cols % 32 == 0, "cols must be a multiple of 32");
    int s = ensure_init();
    if (s != MK_OK) return s;
    if (rows * cols == 0) return MK_OK;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    const size_t pb = rows * cols / 2, sb = rows * cols / 32;
    if ((s = g_ctx.tmp.ensure(pb + sb + 16)) != MK_OK) return s;
    if ((s = g_ctx.y.ensure(rows * cols * 4)) != MK_OK) return s;
    uint8_t *dp = (uint8_t *)g_ctx.tmp.p, *ds = dp + ((pb + 15) & ~(size_t)15);
    MK_HIP_TRY(hipMemcpyAsync(dp, packed, pb, hipMemcpyHostToDevice, g_ctx.stream));
    MK_HIP_TRY(hipMemcpyAsync(ds, scales, sb, hipMemcpyHostToDevice, g_ctx.stream));
    if ((s = mk_dev_mxfp4_dequant(dp, ds, rows, cols, (float *)g_ctx.y.p, g_ctx.stream)) != MK_OK) return s;
    std::vector<float> host(rows * cols);  // `out` stays untouched unless everything succeeded
    MK_HIP_TRY(hipMemcpyAsync(host.data(), g_ctx.y.p, rows * cols * 4, hipMemcpyDeviceToHost, g_ctx.stream));
    MK_HIP_TRY(hipStreamSynchronize(g_ctx.stream));
    memcpy(out, host.data(), rows * cols * 4);
    return MK_OK;
}

extern "C" int mk_quantize_q8(const float *x, size_t n, int8_t *q, float *scales) {
    MK_REQUIRE(x && q && scales, "null pointer");
    MK_REQUIRE(n % 32 == 0, "q8 blocks are 32 wide");
    int s = ensure_init();
    if (s != MK_OK) return s;
    if (n == 0) return MK_OK;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    if ((s = g_ctx.x.ensure(n * 4)) != MK_OK) return s;
    if ((s = g_ctx.xq.ensure(n)) != MK_OK) return s;
    if ((s = g_ctx.xs.ensure(n / 32 * 4)) != MK_OK) return s;
    MK_HIP_TRY(hipMemcpyAsync(g_ctx.x.p, x, n * 4, hipMemcpyHostToDevice, g_ctx.stream));
    if ((s = mk_dev_quantize_q8((const float *)g_ctx.x.p, 1, n, (int8_t *)g_ctx.xq.p, (float *)g_ctx.xs.p, g_ctx.stream)) != MK_OK) return s;
    std::vector<int8_t> hq(n);
    std::vector<float> hs(n / 32);
    MK_HIP_TRY(hipMemcpyAsync(hq.data(), g_ctx.xq.p, n, hipMemcpyDeviceToHost, g_ctx.stream));
    MK_HIP_TRY(hipMemcpyAsync(hs.data(), g_ctx.xs.p, n / 32 * 4, hipMemcpyDeviceToHost, g_ctx.stream));
    MK_HIP_TRY(hipStreamSynchronize(g_ctx.stream));
    memcpy(q, hq.data(), n);
    memcpy(scales, hs.data(), n / 32 * 4);
    return MK_OK;
}

// ------------------------------------------------------------------ Q8Head
struct mk_q8head {
    int8_t *q = nullptr;
    void *scales = nullptr;
    int f16 = 0;
    size_t rows = 0, cols = 0;
    DevBuf x, xq, xs, y, ws, idx;
};

extern "C" void mk_q8head_free(mk_q8head *h) {
    if (!h) return;
    std::lock_guard<std::mutex> lk(g_mu);
    if (h->q) hipFree(h->q);
    if (h->scales) hipFree(h->scales);
    for (DevBuf *b : {&h->x, &h->xq, &h->xs, &h->y, &h->ws, &h->idx})
        if (b->p) hipFree(b->p);
    delete h;
}

namespace {
int q8head_alloc(size_t rows, size_t cols, int f16, mk_q8head **out) {
    mk_q8head *h = new mk_q8head();
    h->rows = rows;
    h->cols = cols;
    h->f16 = f16 ? 1 : 0;
    const size_t nsc = rows * cols / 32;
    if (mk_check_hip(hipMalloc((void **)&h->q, rows * cols + 16), "hipMalloc(q8 head)") != MK_OK ||
        mk_check_hip(hipMalloc(&h->scales, nsc * (f16 ? 2 : 4) + 16), "hipMalloc(q8 head scales)") != MK_OK) {
        if (h->q) hipFree(h->q);
        delete h;
        return MK_ERR_NOMEM;
    }
    *out = h;
    return MK_OK;
}
}  // namespace

extern "C" int mk_q8head_from_f32(const float *w, size_t rows, size_t cols, int scales_f16, mk_q8head **out) {
    MK_REQUIRE(w && out, "null pointer");
    MK_REQUIRE(cols % 32 == 0 && cols > 0 && rows > 0, "cols must be a positive multiple of 32");
    int s = ensure_init();
    if (s != MK_OK) return s;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    mk_q8head *h = nullptr;
    if ((s = q8head_alloc(rows, cols, scales_f16, &h)) != MK_OK) return s;
    // quantize on the device in row chunks of at most 256 MiB of f32
    size_t chunk = (256u << 20) / (cols * 4);
    if (chunk == 0) chunk = 1;
    if (chunk > rows) chunk = rows;
    s = g_ctx.tmp.ensure(chunk * cols * 4);
    for (size_t r0 = 0; s == MK_OK && r0 < rows; r0 += chunk) {
        size_t nr = rows - r0 < chunk ? rows - r0 : chunk;
        s = mk_check_hip(hipMemcpyAsync(g_ctx.tmp.p, w + r0 * cols, nr * cols * 4, hipMemcpyHostToDevice, g_ctx.stream), "upload f32 rows");
        if (s == MK_OK)
            s = mk_dev_q8head_from_f32((const float *)g_ctx.tmp.p, nr, cols, h->q + r0 * cols,
                                       (uint8_t *)h->scales + r0 * (cols / 32) * (scales_f16 ? 2 : 4), scales_f16, g_ctx.stream);
        if (s == MK_OK) s = mk_check_hip(hipStreamSynchronize(g_ctx.stream), "quantize sync");
    }
    if (s != MK_OK) {
        hipFree(h->q);
        hipFree(h->scales);
        delete h;
        return s;
    }
    *out = h;
    return MK_OK;
}

extern "C" int mk_q8head_from_q8(const int8_t *q, const float *scales, size_t rows, size_t cols, int scales_f16, mk_q8head **out) {
    MK_REQUIRE(q && scales && out, "null pointer");
    MK_REQUIRE(cols % 32 == 0 && cols > 0 && rows > 0, "cols must be a positive multiple of 32");
    int s = ensure_init();
    if (s != MK_OK) return s;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    mk_q8head *h = nullptr;
    if ((s = q8head_alloc(rows, cols, scales_f16, &h)) != MK_OK) return s;
    const size_t nsc = rows * cols / 32;
    s = mk_check_hip(hipMemcpyAsync(h->q, q, rows * cols, hipMemcpyHostToDevice, g_ctx.stream), "upload q8 rows");
    std::vector<uint16_t> half;
    if (s == MK_OK) {
        if (scales_f16) {
            half.resize(nsc);
            for (size_t i = 0; i < nsc; i++) {
                _Float16 hv = (_Float16)scales[i];
                memcpy(&half[i], &hv, 2);
            }
            s = mk_check_hip(hipMemcpyAsync(h->scales, half.data(), nsc * 2, hipMemcpyHostToDevice, g_ctx.stream), "upload f16 scales");
        } else {
            s = mk_check_hip(hipMemcpyAsync(h->scales, scales, nsc * 4, hipMemcpyHostToDevice, g_ctx.stream), "upload f32 scales");
        }
    }
    if (s == MK_OK) s = mk_check_hip(hipStreamSynchronize(g_ctx.stream), "upload sync");
    if (s != MK_OK) {
        hipFree(h->q);
        hipFree(h->scales);
        delete h;
        return s;
    }
    *out = h;
    return MK_OK;
}

extern "C" int mk_q8head_matvec(mk_q8head *h, const float *x, size_t batch, float *out, int32_t *argmax_out) {
    MK_REQUIRE(h && x && out, "null pointer");
    MK_REQUIRE(batch >= 1, "batch must be at least 1");
    int s = ensure_init();  // after mk_shutdown the handle's memory is still valid; the stream is not until re-initialised
    if (s != MK_OK) return s;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    if ((s = h->x.ensure(batch * h->cols * 4)) != MK_OK) return s;
    if ((s = h->xq.ensure(batch * h->cols)) != MK_OK) return s;
    if ((s = h->xs.ensure(batch * h->cols / 32 * 4)) != MK_OK) return s;
    if ((s = h->y.ensure(batch * h->rows * 4)) != MK_OK) return s;
    if ((s = h->ws.ensure(2 * batch * 1024 * 4)) != MK_OK) return s;
    if ((s = h->idx.ensure(batch * 4)) != MK_OK) return s;
    MK_HIP_TRY(hipMemcpyAsync(h->x.p, x, batch * h->cols * 4, hipMemcpyHostToDevice, g_ctx.stream));
    if ((s = mk_dev_quantize_q8((const float *)h->x.p, batch, h->cols, (int8_t *)h->xq.p, (float *)h->xs.p, g_ctx.stream)) != MK_OK) return s;
    for (size_t b0 = 0; b0 < batch; b0 += 8) {
        size_t nb = batch - b0 < 8 ? batch - b0 : 8;
        s = mk_dev_q8_matvec(h->q, h->scales, h->f16, h->rows, h->cols, (const int8_t *)h->xq.p + b0 * h->cols,
                             (const float *)h->xs.p + b0 * (h->cols / 32), nb, (float *)h->y.p + b0 * h->rows, g_ctx.stream);
        if (s != MK_OK) return s;
    }
    if (argmax_out) {
        if ((s = mk_dev_argmax((const float *)h->y.p, batch, h->rows, h->ws.p, (int32_t *)h->idx.p, g_ctx.stream)) != MK_OK) return s;
    }
    std::vector<float> host(batch * h->rows);
    std::vector<int32_t> hidx(batch);
    MK_HIP_TRY(hipMemcpyAsync(host.data(), h->y.p, batch * h->rows * 4, hipMemcpyDeviceToHost, g_ctx.stream));
    if (argmax_out) MK_HIP_TRY(hipMemcpyAsync(hidx.data(), h->idx.p, batch * 4, hipMemcpyDeviceToHost, g_ctx.stream));
    MK_HIP_TRY(hipStreamSynchronize(g_ctx.stream));
    memcpy(out, host.data(), batch * h->rows * 4);
    if (argmax_out) memcpy(argmax_out, hidx.data(), batch * 4);
    return MK_OK;
}

// --------------------------------------------------------------- MLA cache
// Two layouts behind one handle:
//   shared latent (mk_mla_cache_new): one q8_0 latent row (L int8 + L/32 f16 scales) and one q8_0 rope row per position,
//     K = V = latent for every head -- the weight-absorbed form of the benchmark configuration;
//   per head (mk_mla_cache_new_heads): MlaCache as the reference keeps it (src/model.rs:765-781): per position and head
//     a K-nope row and a V row (int8 + f32 scales) and one shared f32 rope row.
struct mk_mla_cache {
    int heads_layout = 0;
    int had = 0;  // heads layout: rotated form (kv_hadamard, src/model.rs:1532-1535)
    size_t nh = 0, L = 0, R = 0, vd = 0, cap = 0, n = 0;  // heads layout: L = nope, R = rope
    int8_t *lat_q = nullptr, *rope_q = nullptr;            // heads layout: kq, vq
    void *lat_s = nullptr, *rope_s = nullptr;              // heads layout: ks (f32), vs (f32)
    float *kr = nullptr;                                   // heads layout only
    DevBuf in, q, out, ws;
};

extern "C" void mk_mla_cache_free(mk_mla_cache *c) {
    if (!c) return;
    std::lock_guard<std::mutex> lk(g_mu);
    for (void *p : {(void *)c->lat_q, (void *)c->rope_q, c->lat_s, c->rope_s, (void *)c->kr})
        if (p) hipFree(p);
    for (DevBuf *b : {&c->in, &c->q, &c->out, &c->ws})
        if (b->p) hipFree(b->p);
    delete c;
}

extern "C" int mk_mla_cache_new(size_t nh, size_t L, size_t R, size_t capacity, mk_mla_cache **out) {
    MK_REQUIRE(out, "null pointer");
    // the shapes mk_mla_attn (mk_dev_mla_q8_decode) and mk_mla_cache_push (mk_dev_mla_cache_append) accept
    MK_REQUIRE(nh > 0 && nh <= 65535 && capacity > 0, "bad cache shape");
    MK_REQUIRE(L % 64 == 0 && L >= 64 && L <= 512, "latent width must be a multiple of 64 up to 512");
    MK_REQUIRE(R == 32 || R == 64, "rope width must be 32 or 64");
    int s = ensure_init();
    if (s != MK_OK) return s;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    mk_mla_cache *c = new mk_mla_cache();
    c->nh = nh;
    c->L = L;
    c->R = R;
    c->vd = L;
    c->cap = capacity;
    bool ok = hipMalloc((void **)&c->lat_q, capacity * L + 64) == hipSuccess && hipMalloc(&c->lat_s, capacity * (L / 32) * 2 + 64) == hipSuccess &&
              hipMalloc((void **)&c->rope_q, capacity * R + 64) == hipSuccess && hipMalloc(&c->rope_s, capacity * (R / 32) * 2 + 64) == hipSuccess;
    if (!ok) {
        mk_set_error("hipMalloc(mla cache) failed");
        for (void *p : {(void *)c->lat_q, (void *)c->rope_q, c->lat_s, c->rope_s})
            if (p) hipFree(p);
        delete c;
        return MK_ERR_NOMEM;
    }
    *out = c;
    return MK_OK;
}

extern "C" int mk_mla_cache_new_heads(size_t nh, size_t nope, size_t rope, size_t vd, size_t capacity, mk_mla_cache **out) {
    MK_REQUIRE(out, "null pointer");
    MK_REQUIRE(nh > 0 && nh <= 65535 && capacity > 0, "bad cache shape");
    MK_REQUIRE(nope % 32 == 0 && nope >= 32 && nope <= 256, "latent K width must be a multiple of 32 up to 256");
    MK_REQUIRE(vd % 32 == 0 && vd >= 32 && vd <= 512, "V width must be a multiple of 32 up to 512");
    MK_REQUIRE(rope >= 1 && rope <= 4096, "rope width out of range");
    int s = ensure_init();
    if (s != MK_OK) return s;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    mk_mla_cache *c = new mk_mla_cache();
    c->heads_layout = 1;
    {
        const char *e = getenv("MICROKIMI_KV_HADAMARD");
        c->had = e && strcmp(e, "1") == 0;
    }
    c->nh = nh;
    c->L = nope;
    c->R = rope;
    c->vd = vd;
    c->cap = capacity;
    bool ok = hipMalloc((void **)&c->lat_q, capacity * nh * nope + 64) == hipSuccess &&
              hipMalloc(&c->lat_s, capacity * nh * (nope / 32) * 4 + 64) == hipSuccess &&
              hipMalloc((void **)&c->rope_q, capacity * nh * vd + 64) == hipSuccess &&
              hipMalloc(&c->rope_s, capacity * nh * (vd / 32) * 4 + 64) == hipSuccess &&
              hipMalloc((void **)&c->kr, capacity * rope * 4 + 64) == hipSuccess;
    if (!ok) {
        mk_set_error("hipMalloc(mla cache) failed");
        for (void *p : {(void *)c->lat_q, (void *)c->rope_q, c->lat_s, c->rope_s, (void *)c->kr})
            if (p) hipFree(p);
        delete c;
        return MK_ERR_NOMEM;
    }
    *out = c;
    return MK_OK;
}

extern "C" size_t mk_mla_cache_positions(const mk_mla_cache *c) { return c ? c->n : 0; }

extern "C" int mk_mla_cache_set_hadamard(mk_mla_cache *c, int on) {
    MK_REQUIRE(c, "null pointer");
    std::lock_guard<std::mutex> lk(g_mu);
    MK_REQUIRE(c->heads_layout, "the Hadamard option belongs to the per-head layout (mk_mla_cache_new_heads)");
    MK_REQUIRE(c->n == 0, "the option can change only while the cache is empty");
    c->had = on ? 1 : 0;
    return MK_OK;
}

namespace {
// widths of the two host rows a position is given as: (latent, rope) or (k_row = nh x (nope + rope), v_row = nh x vd)
size_t row0_floats(const mk_mla_cache *c) { return c->heads_layout ? c->nh * (c->L + c->R) : c->L; }
size_t row1_floats(const mk_mla_cache *c) { return c->heads_layout ? c->nh * c->vd : c->R; }

// appends n_new positions given as host rows; chunked through the staging buffer (at most 64 MiB at a time)
int mla_append_host(mk_mla_cache *c, const float *r0, const float *r1, size_t n_new) {
    const size_t w0 = row0_floats(c), w1 = row1_floats(c);
    size_t chunk = (64u << 20) / ((w0 + w1) * 4);
    if (chunk == 0) chunk = 1;
    if (!c->heads_layout) chunk = 1;  // the shared-latent append kernel takes one position
    int s;
    for (size_t j0 = 0; j0 < n_new; j0 += chunk) {
        const size_t nj = n_new - j0 < chunk ? n_new - j0 : chunk;
        if ((s = c->in.ensure(nj * (w0 + w1) * 4)) != MK_OK) return s;
        float *d0 = (float *)c->in.p, *d1 = d0 + nj * w0;
        MK_HIP_TRY(hipMemcpyAsync(d0, r0 + j0 * w0, nj * w0 * 4, hipMemcpyHostToDevice, g_ctx.stream));
        if (w1) MK_HIP_TRY(hipMemcpyAsync(d1, r1 + j0 * w1, nj * w1 * 4, hipMemcpyHostToDevice, g_ctx.stream));
        if (c->heads_layout)
            s = mk_dev_mla_heads_append(d0, d1, nj, c->nh, c->L, c->R, c->vd, c->n, c->had, c->lat_q, (float *)c->lat_s, c->kr, c->rope_q, (float *)c->rope_s,
                                        g_ctx.stream);
        else
            s = mk_dev_mla_cache_append(d0, d1, c->L, c->R, c->n, c->lat_q, c->lat_s, c->rope_q, c->rope_s, g_ctx.stream);
        if (s != MK_OK) return s;
        MK_HIP_TRY(hipStreamSynchronize(g_ctx.stream));  // the staging buffer is reused by the next chunk
        c->n += nj;
    }
    return MK_OK;
}
}  // namespace

extern "C" int mk_mla_cache_push(mk_mla_cache *c, const float *row0, const float *row1) {
    MK_REQUIRE(c && row0 && row1, "null pointer");
    int s = ensure_init();
    if (s != MK_OK) return s;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    if (c->n >= c->cap) {
        mk_set_error("mla cache full (%zu positions)", c->cap);
        return MK_ERR_NOMEM;
    }
    return mla_append_host(c, row0, row1, 1);
}

extern "C" int mk_mla_cache_assign_f32(mk_mla_cache *c, const float *rows0, const float *rows1, size_t n) {
    MK_REQUIRE(c && (n == 0 || (rows0 && rows1)), "null pointer");
    int s = ensure_init();
    if (s != MK_OK) return s;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    if (n > c->cap) {
        mk_set_error("%zu positions do not fit a cache of %zu", n, c->cap);
        return MK_ERR_NOMEM;
    }
    c->n = 0;  // *self = MlaCache::new() (src/model.rs:1681)
    return mla_append_host(c, rows0, rows1, n);
}

extern "C" int mk_mla_cache_to_f32(const mk_mla_cache *c, float *rows0, float *rows1) {
    MK_REQUIRE(c && rows0 && rows1, "null pointer");
    int s = ensure_init();
    if (s != MK_OK) return s;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    const size_t n = c->n, L = c->L, R = c->R;
    if (n == 0) return MK_OK;
    if (c->heads_layout) {
        // dequantized on the device, then one copy per array; staged so that the caller's rows stay untouched on failure
        const size_t w0 = row0_floats(c), w1 = row1_floats(c);
        void *dk = nullptr;
        if (mk_check_hip(hipMalloc(&dk, n * (w0 + w1) * 4), "hipMalloc(to_f32)") != MK_OK) return MK_ERR_NOMEM;
        float *k = (float *)dk, *v = k + n * w0;
        s = mk_dev_mla_heads_to_f32(c->lat_q, (const float *)c->lat_s, c->kr, c->rope_q, (const float *)c->rope_s, n, c->nh, c->L, c->R, c->vd, c->had, k, v,
                                    g_ctx.stream);
        std::vector<float> hk, hv;
        if (s == MK_OK) {
            hk.resize(n * w0);
            hv.resize(n * w1);
            s = mk_check_hip(hipMemcpyAsync(hk.data(), k, n * w0 * 4, hipMemcpyDeviceToHost, g_ctx.stream), "read k");
        }
        if (s == MK_OK) s = mk_check_hip(hipMemcpyAsync(hv.data(), v, n * w1 * 4, hipMemcpyDeviceToHost, g_ctx.stream), "read v");
        if (s == MK_OK) s = mk_check_hip(hipStreamSynchronize(g_ctx.stream), "to_f32 sync");
        hipFree(dk);
        if (s != MK_OK) return s;
        memcpy(rows0, hk.data(), n * w0 * 4);
        memcpy(rows1, hv.data(), n * w1 * 4);
        return MK_OK;
    }
    std::vector<int8_t> lq(n * L), rq(n * R);
    std::vector<uint16_t> ls(n * L / 32), rs(n * R / 32);
    MK_HIP_TRY(hipMemcpyAsync(lq.data(), c->lat_q, n * L, hipMemcpyDeviceToHost, g_ctx.stream));
    MK_HIP_TRY(hipMemcpyAsync(ls.data(), c->lat_s, n * L / 32 * 2, hipMemcpyDeviceToHost, g_ctx.stream));
    MK_HIP_TRY(hipMemcpyAsync(rq.data(), c->rope_q, n * R, hipMemcpyDeviceToHost, g_ctx.stream));
    MK_HIP_TRY(hipMemcpyAsync(rs.data(), c->rope_s, n * R / 32 * 2, hipMemcpyDeviceToHost, g_ctx.stream));
    MK_HIP_TRY(hipStreamSynchronize(g_ctx.stream));
    // the byte-level dequantization q * s of MlaCache::to_f32 (src/model.rs:1641-1646)
    auto h2f = [](uint16_t b) {
        _Float16 h;
        memcpy(&h, &b, 2);
        return (float)h;
    };
    for (size_t i = 0; i < n * L; i++) rows0[i] = (float)lq[i] * h2f(ls[i / 32]);
    for (size_t i = 0; i < n * R; i++) rows1[i] = (float)rq[i] * h2f(rs[i / 32]);
    return MK_OK;
}

namespace {
// m queries against the cache: query i attends positions 0 ..= pos0 + i
int mla_attn_host(mk_mla_cache *c, const float *q, size_t m, size_t pos0, float scale, float *out) {
    int s;
    const size_t qn = m * c->nh * (c->L + c->R), on = m * c->nh * c->vd;
    if ((s = c->q.ensure(qn * 4)) != MK_OK) return s;
    if ((s = c->out.ensure(on * 4)) != MK_OK) return s;
    const size_t need = c->heads_layout ? mk_mla_heads_workspace_bytes(m, c->nh, c->L, c->vd) : mk_mla_decode_workspace_bytes(c->nh, c->L, c->cap);
    if ((s = c->ws.ensure(need)) != MK_OK) return s;
    MK_HIP_TRY(hipMemcpyAsync(c->q.p, q, qn * 4, hipMemcpyHostToDevice, g_ctx.stream));
    if (c->heads_layout) {
        s = mk_dev_mla_heads_q8_attn(c->lat_q, (const float *)c->lat_s, c->kr, c->rope_q, (const float *)c->rope_s, pos0, (const float *)c->q.p, m,
                                     c->nh, c->L, c->R, c->vd, scale, c->had, c->ws.p, (float *)c->out.p, g_ctx.stream);
    } else {
        for (size_t i = 0; i < m && s == MK_OK; i++)
            s = mk_dev_mla_q8_decode(c->lat_q, c->lat_s, c->rope_q, c->rope_s, pos0 + i, (const float *)c->q.p + i * c->nh * (c->L + c->R), c->nh,
                                     c->L, c->R, scale, c->ws.p, (float *)c->out.p + i * c->nh * c->vd, g_ctx.stream);
    }
    if (s != MK_OK) return s;
    std::vector<float> host(on);
    MK_HIP_TRY(hipMemcpyAsync(host.data(), c->out.p, on * 4, hipMemcpyDeviceToHost, g_ctx.stream));
    MK_HIP_TRY(hipStreamSynchronize(g_ctx.stream));
    memcpy(out, host.data(), on * 4);
    return MK_OK;
}
}  // namespace

extern "C" int mk_mla_attn(mk_mla_cache *c, const float *q, float scale, float *out) {
    MK_REQUIRE(c && q && out, "null pointer");
    int s = ensure_init();
    if (s != MK_OK) return s;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    if (c->n == 0) {
        mk_set_error("mla cache is empty");
        return MK_ERR_INVALID;
    }
    return mla_attn_host(c, q, 1, c->n - 1, scale, out);
}

extern "C" int mk_mla_attn_prefill(mk_mla_cache *c, const float *q, size_t m, float scale, float *out) {
    MK_REQUIRE(c && q && out, "null pointer");
    MK_REQUIRE(m >= 1 && m <= 65535, "bad query count");
    int s = ensure_init();
    if (s != MK_OK) return s;
    std::lock_guard<std::mutex> lk(g_mu);
    if ((s = bind_device()) != MK_OK) return s;
    if (c->n < m) {
        mk_set_error("the cache holds %zu positions, fewer than the %zu queries", c->n, m);
        return MK_ERR_INVALID;
    }
    return mla_attn_host(c, q, m, c->n - m, scale, out);
}
