// Version / error entry points of libti8.
#include "ti8_common.h"

namespace ti8 {
char* err_buf() {
    static thread_local char buf[512] = {0};
    return buf;
}
}  // namespace ti8

extern "C" int ti8_version(void) { return 100; }
extern "C" const char* ti8_last_error(void) { return ti8::err_buf(); }
extern "C" const char* ti8_arch(void) { return "gfx950"; }
