// Error text, version and the tile-configuration table.
#include "common.hpp"
#include <string.h>

namespace spx {
char* last_error_buf() {
    static thread_local char buf[512] = {0};
    return buf;
}
}  // namespace spx

extern "C" const char* spx_last_error(void) { return spx::last_error_buf(); }
extern "C" int spx_version(void) { return SPX_VERSION; }
