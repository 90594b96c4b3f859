#include "common.hpp"

namespace fmoe {
char *error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}
}  // namespace fmoe

extern "C" const char *fmoe_last_error(void) { return fmoe::error_buffer(); }
extern "C" int fmoe_abi_version(void) { return 3; }
