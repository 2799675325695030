// Error text, version and device queries shared by all entry points.
#include "cf_common.h"

#include <stdarg.h>
#include <string.h>

namespace cf {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int hip_failed(hipError_t err, const char *what)
{
    set_error("%s: %s", what, hipGetErrorString(err));
    return CF_ERR_HIP;
}

int device_cu_count()
{
    static thread_local int cached_dev = -1;
    static thread_local int cached_cus = 0;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (dev != cached_dev) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        cached_dev = dev;
        cached_cus = cus;
    }
    return cached_cus;
}

static thread_local double g_launch_share = 1.0;

int persistent_grid_cap(int per_cu)
{
    const int64_t cap = (int64_t)((double)device_cu_count() * per_cu * g_launch_share);
    return (int)(cap < 1 ? 1 : cap);
}

// Live sizes on the device (cf_set_size_header): the header and the capacities it goes with.
static thread_local const int64_t *g_size_header = nullptr;
static thread_local int64_t g_cap_atoms = -1, g_cap_edges = -1;

const int64_t *live_atoms(int64_t N) { return (g_size_header && N == g_cap_atoms) ? g_size_header : nullptr; }
const int64_t *live_edges(int64_t E) { return (g_size_header && E == g_cap_edges) ? g_size_header + 1 : nullptr; }
const int64_t *live_units(int64_t U)
{
    return (g_size_header && 2 * U == g_cap_atoms + g_cap_edges) ? g_size_header + 2 : nullptr;
}
int64_t *size_header_for_layout(int64_t N, int64_t E)
{
    return (g_size_header && N == g_cap_atoms && E == g_cap_edges) ? const_cast<int64_t *>(g_size_header) : nullptr;
}

}  // namespace cf

extern "C" int cf_version(void) { return 101; }

extern "C" int cf_set_size_header(int64_t *header_4, int64_t N_cap, int64_t E_cap)
{
    if (!header_4) {
        cf::g_size_header = nullptr;
        cf::g_cap_atoms = cf::g_cap_edges = -1;
        return CF_OK;
    }
    CF_REQUIRE(N_cap >= 1 && E_cap >= 1 && (N_cap + E_cap) % 2 == 0, CF_ERR_INVALID_ARGUMENT,
               "cf_set_size_header: capacities must be positive with an even sum (got %lld atoms, %lld edges)",
               (long long)N_cap, (long long)E_cap);
    cf::g_size_header = header_4;
    cf::g_cap_atoms = N_cap;
    cf::g_cap_edges = E_cap;
    return CF_OK;
}

extern "C" const int64_t *cf_get_size_header(void) { return cf::g_size_header; }

extern "C" int cf_set_launch_share(double share)
{
    CF_REQUIRE(share > 0.0 && share <= 1.0, CF_ERR_INVALID_ARGUMENT,
               "cf_set_launch_share: share %g outside (0, 1]", share);
    cf::g_launch_share = share;
    return CF_OK;
}

extern "C" double cf_get_launch_share(void) { return cf::g_launch_share; }

extern "C" const char *cf_last_error(void) { return cf::g_error; }

extern "C" int cf_max_translation_range(void) { return cf::MAX_RANGE; }
