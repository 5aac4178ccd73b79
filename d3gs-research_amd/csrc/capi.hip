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

// Significant bits of the keys d3gs_preprocess_fwd writes to depth_sort_keys (see depth_sort_key()).
extern "C" int d3gs_depth_key_bits(const d3gs_params* p) {
    if (!p) return 32;
    if (p->enable_32bit_sort) return d3gs::kDepthStepBits;
    union { float f; uint32_t u; } far_bits;
    // largest stored value of an accepted gaussian: z_far, or with render_inv_depth 1 / z_near
    if (p->render_inv_depth) {
        if (!(p->z_near > 0.0f)) return 32;
        far_bits.f = 1.0f / p->z_near;
    } else {
        far_bits.f = p->z_far;
    }
    const uint32_t base = d3gs::depth_key_base(*p);
    if (!(p->z_far > 0.0f) || far_bits.u < base) return 1;    // nothing is accepted: every key is 0
    const int bits = d3gs_higher_msb(far_bits.u - base);
    return bits > 0 ? bits : 1;
}
