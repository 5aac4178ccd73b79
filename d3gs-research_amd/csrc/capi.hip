// Host-side utilities of the C ABI: thread-local error text, version, and the
// bit-length helper the sort's bit range is derived from.
#include <cstdarg>
#include <cstdio>

#include "device_math.h"

namespace d3gs {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

}  // namespace d3gs

extern "C" int d3gs_abi_version(void) { return D3GS_ABI_VERSION; }

extern "C" const char* d3gs_last_error_string(void) { return d3gs::g_error; }

// devsort.py:131-149 returns the bit length of n (0 for n == 0)
extern "C" int d3gs_higher_msb(uint32_t n) {
    int b = 0;
    while (n) {
        ++b;
        n >>= 1;
    }
    return b;
}
