// Library-wide C-ABI entry points: version and the thread-local error message.
#include "pmoe_common.h"

namespace pmoe {
char *error_buffer() {
    static thread_local char buf[kErrorBufferBytes] = {0};
    return buf;
}
}  // namespace pmoe

extern "C" int pmoe_version(void) { return 1; }

extern "C" const char *pmoe_last_error(void) { return pmoe::error_buffer(); }
