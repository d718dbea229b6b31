// Library-wide host services: version, thread-local error text, device probe (and, in the cross-check build only, the
// knob that selects a superseded kernel).
#include <atomic>
#include <mutex>
#include <stdarg.h>
#include <string.h>

#include "cdm_common.h"

namespace {
thread_local char g_err[512] = "";
#ifdef CDM_CROSSCHECK
std::atomic<int> g_variant[2] = {{0}, {0}};
#endif
std::once_flag g_dev_once;
int g_dev_count = 0;

void probe_devices() {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        n = 0;
        (void)hipGetLastError();   // do not leave the probe's error for the next call to find
    }
    g_dev_count = n;
}
}  // namespace

void cdm_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int32_t cdm_require_device(void) {
    std::call_once(g_dev_once, probe_devices);
    if (g_dev_count <= 0) CDM_FAIL(CDM_ERR_NO_DEVICE, "no HIP device visible to this process");
    return CDM_OK;
}

#ifdef CDM_CROSSCHECK
int32_t cdm_get_variant(int which) { return g_variant[which].load(std::memory_order_relaxed); }
#endif

#ifndef CDM_SOURCE_HASH
#define CDM_SOURCE_HASH "unknown"
#endif
// the marker lets a loader read the hash from the file without loading it
static const char kSourceHash[] = "CDM_SRC_HASH=" CDM_SOURCE_HASH;

extern "C" int32_t cdm_version(void) { return 101; }

extern "C" const char* cdm_source_hash(void) { return kSourceHash + 13; }

extern "C" const char* cdm_last_error(void) { return g_err; }

extern "C" int32_t cdm_device_count(void) {
    std::call_once(g_dev_once, probe_devices);
    return g_dev_count;
}

#ifdef CDM_CROSSCHECK
extern "C" int32_t cdm_set_variant(const char* op, int32_t variant) {
    CDM_REQUIRE(op, CDM_ERR_BAD_ARG, "set_variant: null op");
    int which = -1;
    if (strcmp(op, "attn") == 0) which = 0;
    else if (strcmp(op, "gemm") == 0) which = 1;
    CDM_REQUIRE(which >= 0, CDM_ERR_BAD_ARG, "set_variant: unknown op '%s'", op);
    CDM_REQUIRE(variant >= 0 && variant < 64, CDM_ERR_BAD_ARG, "set_variant: variant %d out of range", variant);
    return g_variant[which].exchange(variant);
}
#endif
