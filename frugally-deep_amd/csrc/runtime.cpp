// Process-wide state of the fdx library: device selection, the library stream, error
// text, device-memory plumbing, a HIP-event stopwatch and the per-kernel-family profile.
#include <cmath>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include "common.hpp"

namespace fdx {

static thread_local std::string g_error;
static hipStream_t g_stream = nullptr;
static bool g_inited = false;
static std::mutex g_mutex;
static hipEvent_t g_t0 = nullptr, g_t1 = nullptr;
// One int in pinned host memory that kernels can reach: a kernel whose bounded wait ran out stores its code there, and
// the calls that wait for the stream (fdx_sync, fdx_d2h) look at it, so a failed exchange comes back as an error from
// the very call that would hand the results out.
static int* g_async_err = nullptr;

static bool g_profile = false;
struct Pending {
    hipEvent_t a, b;
    const char* family;
    double flops, bytes, executed;
};
struct Family {
    uint64_t launches = 0;
    double ms = 0, flops = 0, bytes = 0, executed = 0;
};
static std::vector<Pending> g_pending;
static std::vector<hipEvent_t> g_event_pool;
static std::map<std::string, Family> g_families;
static hipEvent_t g_cur = nullptr;

void set_error(const char* fmt, ...)
{
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_error = buf;
}

fdx_status ensure_init();
hipError_t noalloc_setup(); // decode_kernels.hip: device address of the scratch array of fdx_dense_rows_noalloc_f32
hipStream_t stream()
{
    if (!g_inited)
        (void)ensure_init();
    return g_stream;
}
bool profiling() { return g_profile; }
int* async_error_cell()
{
    if (!g_inited)
        (void)ensure_init();
    return g_async_err;
}
// after the stream has drained: reports and clears what a kernel left in the cell
static fdx_status check_async_error()
{
    if (!g_async_err)
        return FDX_OK;
    const int code = *static_cast<volatile int*>(g_async_err);
    if (code == 0)
        return FDX_OK;
    *g_async_err = 0;
    set_error("a kernel gave up a bounded wait for another workgroup's partial results (code %d): the results of the calls since the last "
              "synchronisation are not valid", code);
    return FDX_ERR_HIP;
}

hipError_t zero_device(void* p, size_t bytes)
{
    hipStream_t s = stream();
    hipError_t e = hipMemsetAsync(p, 0, bytes, s);
    if (e != hipSuccess)
        return e;
    return hipStreamSynchronize(s);
}

static hipEvent_t get_event()
{
    if (!g_event_pool.empty()) {
        hipEvent_t e = g_event_pool.back();
        g_event_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess)
        return nullptr;
    return e;
}

void profile_begin()
{
    if (!g_profile)
        return;
    g_cur = get_event();
    if (g_cur)
        (void)hipEventRecord(g_cur, g_stream);
}

void profile_end(const char* family, double flops, double bytes, double executed_flops)
{
    if (!g_profile || !g_cur)
        return;
    hipEvent_t b = get_event();
    if (!b)
        return;
    (void)hipEventRecord(b, g_stream);
    g_pending.push_back({ g_cur, b, family, flops, bytes, executed_flops < 0 ? flops : executed_flops });
    g_cur = nullptr;
}

static void drain_profile()
{
    if (g_pending.empty())
        return;
    (void)hipStreamSynchronize(g_stream);
    for (auto& p : g_pending) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, p.a, p.b) == hipSuccess) {
            Family& f = g_families[p.family];
            f.launches += 1;
            f.ms += ms;
            f.flops += p.flops;
            f.bytes += p.bytes;
            f.executed += p.executed;
        }
        g_event_pool.push_back(p.a);
        g_event_pool.push_back(p.b);
    }
    g_pending.clear();
}

fdx_status ensure_init()
{
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_inited)
        return FDX_OK;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count == 0) {
        set_error("no HIP device available: the fdx forward path needs an MI355X (gfx950)");
        return FDX_ERR_HIP;
    }
    FDX_HIP(hipSetDevice(0));
    FDX_HIP(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
    FDX_HIP(hipEventCreate(&g_t0));
    FDX_HIP(hipEventCreate(&g_t1));
    FDX_HIP(noalloc_setup());
    FDX_HIP(hipHostMalloc(reinterpret_cast<void**>(&g_async_err), sizeof(int), hipHostMallocDefault));
    *g_async_err = 0;
    g_inited = true;
    return FDX_OK;
}

} // namespace fdx

using namespace fdx;

extern "C" void fdx_set_last_error(const char* text)
{
    fdx::set_error("%s", text ? text : "");
}

extern "C" const char* fdx_last_error(void) { return g_error.c_str(); }

extern "C" fdx_status fdx_init(int device)
{
    FDX_REQUIRE(device == 0, "fdx runs on one GPU: device index must be 0");
    return ensure_init();
}

extern "C" fdx_status fdx_dev_alloc(size_t bytes, void** out)
{
    FDX_REQUIRE(out, "dev_alloc: null out");
    fdx_status st = ensure_init();
    if (st != FDX_OK)
        return st;
    FDX_HIP(hipMalloc(out, bytes ? bytes : 4));
    return FDX_OK;
}

extern "C" fdx_status fdx_dev_free(void* p)
{
    if (p) {
        FDX_HIP(hipStreamSynchronize(g_stream));
        FDX_HIP(hipFree(p));
    }
    return FDX_OK;
}

extern "C" fdx_status fdx_h2d(void* dst, const void* src, size_t bytes)
{
    FDX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_stream));
    FDX_HIP(hipStreamSynchronize(g_stream));
    return FDX_OK;
}

extern "C" fdx_status fdx_d2h(void* dst, const void* src, size_t bytes)
{
    FDX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_stream));
    FDX_HIP(hipStreamSynchronize(g_stream));
    return check_async_error();
}

extern "C" fdx_status fdx_sync(void)
{
    fdx_status st = ensure_init();
    if (st != FDX_OK)
        return st;
    FDX_HIP(hipStreamSynchronize(g_stream));
    return check_async_error();
}

extern "C" fdx_status fdx_dev_mem_info(size_t* free_bytes, size_t* total_bytes)
{
    FDX_REQUIRE(free_bytes && total_bytes, "dev_mem_info: null argument");
    fdx_status st = ensure_init();
    if (st != FDX_OK)
        return st;
    FDX_HIP(hipMemGetInfo(free_bytes, total_bytes));
    return FDX_OK;
}

extern "C" fdx_status fdx_timer_start(void)
{
    fdx_status st = ensure_init();
    if (st != FDX_OK)
        return st;
    FDX_HIP(hipEventRecord(g_t0, g_stream));
    return FDX_OK;
}

extern "C" fdx_status fdx_timer_stop(float* ms)
{
    FDX_REQUIRE(ms, "timer_stop: null out");
    FDX_HIP(hipEventRecord(g_t1, g_stream));
    FDX_HIP(hipEventSynchronize(g_t1));
    FDX_HIP(hipEventElapsedTime(ms, g_t0, g_t1));
    return FDX_OK;
}

extern "C" fdx_status fdx_profile_enable(int on)
{
    fdx_status st = ensure_init();
    if (st != FDX_OK)
        return st;
    drain_profile();
    g_profile = on != 0;
    return FDX_OK;
}

extern "C" fdx_status fdx_profile_reset(void)
{
    drain_profile();
    g_families.clear();
    return FDX_OK;
}

extern "C" fdx_status fdx_profile_get(int index, char* name, size_t name_len, uint64_t* launches, double* total_ms,
    double* flops, double* bytes)
{
    drain_profile();
    FDX_REQUIRE(index >= 0 && name && name_len > 0, "profile_get: bad arguments");
    if (index >= (int)g_families.size()) {
        set_error("profile_get: index out of range");
        return FDX_ERR_INVALID;
    }
    auto it = g_families.begin();
    std::advance(it, index);
    std::strncpy(name, it->first.c_str(), name_len - 1);
    name[name_len - 1] = 0;
    if (launches) *launches = it->second.launches;
    if (total_ms) *total_ms = it->second.ms;
    if (flops) *flops = it->second.flops;
    if (bytes) *bytes = it->second.bytes;
    return FDX_OK;
}

extern "C" fdx_status fdx_profile_get_executed(int index, double* executed_flops)
{
    drain_profile();
    FDX_REQUIRE(index >= 0 && executed_flops, "profile_get_executed: bad arguments");
    if (index >= (int)g_families.size()) {
        set_error("profile_get_executed: index out of range");
        return FDX_ERR_INVALID;
    }
    auto it = g_families.begin();
    std::advance(it, index);
    *executed_flops = it->second.executed;
    return FDX_OK;
}

// include/fdeep/convolution.hpp:320-396 (the non-transposed branch)
extern "C" fdx_status fdx_window_geometry(int in_h, int in_w, int k_h, int k_w, int s_h, int s_w, int padding, int* geom)
{
    FDX_REQUIRE(geom && in_h > 0 && in_w > 0 && k_h > 0 && k_w > 0 && s_h > 0 && s_w > 0, "window_geometry: bad arguments");
    FDX_REQUIRE(padding >= 0 && padding <= 2, "no padding");
    auto ceil_fudge = [](int num, int den) {
        return (int)std::ceil((double)((float)num / (float)den) - 0.001);
    };
    int out_h, out_w, pt = 0, pb = 0, pl = 0, pr = 0;
    if (padding == 1 || padding == 2) {
        out_h = ceil_fudge(in_h, s_h);
        out_w = ceil_fudge(in_w, s_w);
    } else {
        out_h = ceil_fudge(in_h - k_h + 1, s_h);
        out_w = ceil_fudge(in_w - k_w + 1, s_w);
    }
    if (padding == 1) {
        const int ah = in_h % s_h == 0 ? std::max(k_h - s_h, 0) : std::max(k_h - in_h % s_h, 0);
        const int aw = in_w % s_w == 0 ? std::max(k_w - s_w, 0) : std::max(k_w - in_w % s_w, 0);
        pt = ah / 2; pb = ah - pt; pl = aw / 2; pr = aw - pl;
    } else if (padding == 2) {
        pt = k_h - 1;
        pl = k_w - 1;
    }
    FDX_REQUIRE(out_h >= 0 && out_w >= 0, "window_geometry: negative output size");
    geom[0] = pt; geom[1] = pb; geom[2] = pl; geom[3] = pr; geom[4] = out_h; geom[5] = out_w;
    return FDX_OK;
}
