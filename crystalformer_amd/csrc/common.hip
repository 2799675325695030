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

}  // namespace cf

extern "C" int cf_version(void) { return 100; }

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
