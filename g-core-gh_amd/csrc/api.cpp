// Library-wide entry points: version and the thread-local error string.
#include "lowp_common.h"

namespace lowp {
char *error_buffer()
{
    static thread_local char buf[kErrorBufferSize] = {0};
    return buf;
}
}  // namespace lowp

extern "C" int lp_version(void) { return 100; }

extern "C" const char *lp_last_error(void) { return lowp::error_buffer(); }
