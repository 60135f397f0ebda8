// Library-wide pieces of the C-ABI: version and the thread-local error message.
#include "common.hip.h"

namespace pcfgnat {
char *error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}
}  // namespace pcfgnat

extern "C" int pcfgnat_abi_version(void) { return 1; }

extern "C" const char *pcfgnat_last_error(void) { return pcfgnat::error_buffer(); }
