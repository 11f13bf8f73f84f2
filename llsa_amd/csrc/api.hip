// Library-level entry points: version and the per-thread error string.
#include "llsa_host.h"
#include "../../include/llsa_hip.h"

namespace llsa {
char* error_buffer() {
    static thread_local char buf[512] = "";
    return buf;
}
}  // namespace llsa

extern "C" int llsa_version(void) { return 100; }
extern "C" const char* llsa_last_error_string(void) { return llsa::error_buffer(); }
