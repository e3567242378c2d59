// Host-side entry points: initialisation, error text, shard-length rounding.
#include "common.h"
#include <string.h>
#include <vector>

static thread_local char g_err[512] = "";

int hapmi_set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

extern "C" const char *hapmi_last_error(void) { return g_err; }
extern "C" int hapmi_version(void) { return 1; }

extern "C" int hapmi_init(void) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hapmi_set_error(HAPMI_EARCH, "hipGetDevice: %s", hipGetErrorString(e));
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return hapmi_set_error(HAPMI_EARCH, "hipGetDeviceProperties: %s", hipGetErrorString(e));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return hapmi_set_error(HAPMI_EARCH, "device %d is %s; this library holds gfx950 code only", dev,
                               prop.gcnArchName);
    return hapmi_sumsq_static_setup();
}

// Integer shard lengths.  full_length == 1 gives every rank one unit (the
// broadcast case).  Otherwise truncate ratio * n, then hand the missing units
// out one at a time to the rank that is furthest below its ratio; among equal
// deficits the highest rank wins.
extern "C" int hapmi_sharding_round(int64_t full_length, const double *ratios, int64_t n_ranks, int64_t *lengths) {
    HAPMI_REQUIRE(full_length >= 0 && n_ranks > 0 && ratios && lengths, HAPMI_EINVAL, "sharding_round: bad argument");
    if (full_length == 1) {
        for (int64_t i = 0; i < n_ranks; ++i) lengths[i] = 1;
        return HAPMI_OK;
    }
    const double n = (double)full_length;
    int64_t have = 0;
    for (int64_t i = 0; i < n_ranks; ++i) {
        lengths[i] = (int64_t)(ratios[i] * n);
        have += lengths[i];
    }
    HAPMI_REQUIRE(have <= full_length, HAPMI_EINVAL, "sharding_round: ratios sum above 1 (%lld > %lld)",
                  (long long)have, (long long)full_length);
    for (; have < full_length; ++have) {
        int64_t pick = n_ranks - 1;
        double deficit = ratios[pick] - (double)lengths[pick] / n;
        for (int64_t i = n_ranks - 2; i >= 0; --i) {
            const double d = ratios[i] - (double)lengths[i] / n;
            if (d > deficit) {
                deficit = d;
                pick = i;
            }
        }
        lengths[pick] += 1;
    }
    return HAPMI_OK;
}
