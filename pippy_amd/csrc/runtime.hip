// Status reporting shared by every entry point.
#include "common.h"

namespace pp {
char* error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}
}  // namespace pp

extern "C" int pp_abi_version(void) { return 1; }
extern "C" const char* pp_last_error(void) { return pp::error_buffer(); }
