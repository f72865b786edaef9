// The error channel of the C entry points: one message per host thread.
#include "common.h"
#include "leone_hip.h"

namespace leone {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list args;
    va_start(args, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, args);
    va_end(args);
}

}  // namespace leone

extern "C" const char* leone_last_error() { return leone::g_error; }
extern "C" int leone_library_version() { return 1; }
