// Process-wide pieces of the C ABI: version and the thread-local error string.
#include "common.h"

namespace flyhip {
char* error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}
}  // namespace flyhip

extern "C" int flyhip_version(void) { return 100; }
extern "C" const char* flyhip_last_error(void) { return flyhip::error_buffer(); }
