// Library-wide entry points: version and the per-thread error message.
#include "fm_common.h"

namespace fm {
char *error_buffer() {
    static thread_local char buffer[512] = {0};
    return buffer;
}
}  // namespace fm

extern "C" int fm_version(void) { return FM_VERSION; }

extern "C" const char *fm_last_error(void) { return fm::error_buffer(); }
