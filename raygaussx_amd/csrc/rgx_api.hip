// Host-only part of the C ABI: version, error strings, per-thread HIP error.
#include "rgx_device.h"

static thread_local int g_last_hip_error = 0;

int rgx_set_hip_error(hipError_t e)
{
    g_last_hip_error = (int)e;
    return RGX_EHIP;
}

DeviceScope::DeviceScope(const void *p)
{
    if (!p) return;
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError(); // not memory the runtime knows: not an error of this call
        return;
    }
    int cur = -1;
    if (attr.type != hipMemoryTypeDevice || hipGetDevice(&cur) != hipSuccess || cur == attr.device) return;
    if (hipSetDevice(attr.device) == hipSuccess) prev = cur;
}

DeviceScope::~DeviceScope()
{
    if (prev >= 0) (void)hipSetDevice(prev);
}

extern "C" int rgx_abi_version(void) { return RGX_ABI_VERSION; }

extern "C" int rgx_last_hip_error(void) { return g_last_hip_error; }

extern "C" const char *rgx_strerror(int code)
{
    switch (code) {
    case RGX_OK: return "ok";
    case RGX_EINVAL: return "invalid argument";
    case RGX_EWORKSPACE: return "workspace too small or misaligned";
    case RGX_EHIP: return "HIP runtime error (see rgx_last_hip_error)";
    case RGX_ELIMIT: return "size beyond the limits of the allocation-free entry point";
    default: return "unknown error";
    }
}

// ---------------------------------------------------------------------------
// Optional per-kernel timing with HIP events on the launch stream (used by the
// benchmark to price the dominant kernels; off by default, no cost when off).
#include <mutex>
#include <vector>

namespace {
struct Span {
    hipEvent_t a, b;
    int id;
};
std::mutex g_mu;
std::vector<Span> g_spans;
bool g_timing = false;
const char *const g_names[RGX_T_COUNT] = {"build", "sh_forward", "pack_prims", "march_forward",
                                          "march_backward", "unpermute_grads", "sh_backward"};
} // namespace

void *rgx_span_begin(int id, hipStream_t s)
{
    if (!g_timing) return nullptr;
    Span *sp = new Span;
    sp->id = id;
    if (hipEventCreate(&sp->a) != hipSuccess || hipEventCreate(&sp->b) != hipSuccess) {
        delete sp;
        return nullptr;
    }
    (void)hipEventRecord(sp->a, s);
    return sp;
}

void rgx_span_end(void *h, hipStream_t s)
{
    if (!h) return;
    Span *sp = (Span *)h;
    (void)hipEventRecord(sp->b, s);
    std::lock_guard<std::mutex> lk(g_mu);
    g_spans.push_back(*sp);
    delete sp;
}

extern "C" int rgx_timing_enable(int on)
{
    std::lock_guard<std::mutex> lk(g_mu);
    g_timing = on != 0;
    return RGX_OK;
}

extern "C" int rgx_timing_reset(void)
{
    std::lock_guard<std::mutex> lk(g_mu);
    for (Span &sp : g_spans) {
        (void)hipEventDestroy(sp.a);
        (void)hipEventDestroy(sp.b);
    }
    g_spans.clear();
    return RGX_OK;
}

extern "C" const char *rgx_timing_name(int id) { return id >= 0 && id < RGX_T_COUNT ? g_names[id] : nullptr; }

extern "C" int rgx_timing_read(int id, double *total_ms, int64_t *launches)
{
    if (!total_ms || !launches || id < 0 || id >= RGX_T_COUNT) return RGX_EINVAL;
    std::lock_guard<std::mutex> lk(g_mu);
    double tot = 0.0;
    int64_t cnt = 0;
    for (Span &sp : g_spans) {
        if (sp.id != id) continue;
        RGX_HIP(hipEventSynchronize(sp.b));
        float ms = 0.f;
        RGX_HIP(hipEventElapsedTime(&ms, sp.a, sp.b));
        tot += ms;
        ++cnt;
    }
    *total_ms = tot;
    *launches = cnt;
    return RGX_OK;
}
