// Error text and version of the FlashMoE gfx950 library.
#include <stdarg.h>
#include <string.h>

#include <atomic>

#include "fmoe_common.h"

namespace fmoe {
namespace {
thread_local char g_error[512] = {0};
}

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

void clear_error() { g_error[0] = '\0'; }

// Compute units, XCDs (each with its own L2) and L2 size of the current device, asked once per device.  Without a
// device (sizing a workspace on a host without a GPU) or where the runtime reports nothing, an unpartitioned MI355X
// is assumed: 256 compute units in 8 XCDs, 4 MiB of L2 each.
const ChipInfo& chip_info() {
    static const ChipInfo fallback = {256, 8, 4ll << 20};
    static ChipInfo cached[64];
    static std::atomic<int> state[64];                       // 0 = not asked, 1 = being filled, 2 = ready
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();
        return fallback;
    }
    if (state[dev].load(std::memory_order_acquire) == 2) return cached[dev];
    int expected = 0;
    if (!state[dev].compare_exchange_strong(expected, 1)) {
        while (state[dev].load(std::memory_order_acquire) != 2) {}
        return cached[dev];
    }
    ChipInfo info = fallback;
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) info.cus = v;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeNumberOfXccs, dev) == hipSuccess && v > 0) info.xcds = v;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeL2CacheSize, dev) == hipSuccess && v >= (1 << 20)) info.l2_bytes = v;
    (void)hipGetLastError();
    cached[dev] = info;
    state[dev].store(2, std::memory_order_release);
    return cached[dev];
}

}  // namespace fmoe

extern "C" int fmoe_abi_version(void) { return FMOE_ABI_VERSION; }

extern "C" const char* fmoe_last_error(void) { return fmoe::g_error; }
