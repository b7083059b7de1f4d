// Error reporting and library identification of libnvalchemi_amd.so.
#include "common.h"

namespace nvamd {

char* error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

int32_t fail(int32_t code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

}  // namespace nvamd

NVAMD_EXPORT int32_t nvamd_abi_version(void) { return NVAMD_ABI_VERSION; }

NVAMD_EXPORT const char* nvamd_last_error(void) { return nvamd::error_buffer(); }
