// Thread-local error text behind aeon_last_error(), and the ABI revision.
#include "common.hpp"

#include <cstring>

namespace aeon355 {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list args;
    va_start(args, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, args);
    va_end(args);
}

}  // namespace aeon355

extern "C" const char* aeon_last_error(void) { return aeon355::g_error; }
extern "C" int aeon_abi_version(void) { return 3; }
