// Error text and version of the FlashMoE gfx950 library.
#include <stdarg.h>
#include <string.h>

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

}  // namespace fmoe

extern "C" int fmoe_abi_version(void) { return FMOE_ABI_VERSION; }

extern "C" const char* fmoe_last_error(void) { return fmoe::g_error; }
