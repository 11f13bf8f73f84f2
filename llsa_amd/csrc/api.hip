// Library-level entry points: version and the per-thread error string.
#include "llsa_host.h"
#include "../../include/llsa_hip.h"

namespace llsa {
char* error_buffer() {
    static thread_local char buf[512] = "";
    return buf;
}
}  // namespace llsa

// bumped whenever an argument structure or a signature of include/llsa_hip.h changes; the Python binding checks it
extern "C" int llsa_version(void) { return LLSA_ABI_VERSION; }
extern "C" const char* llsa_last_error_string(void) { return llsa::error_buffer(); }
