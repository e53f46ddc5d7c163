// Version and error-string entry points of libmdx.
#include "mdx_common.h"

namespace mdx {
char* error_buffer() {
    static thread_local char buf[512] = "";
    return buf;
}
}  // namespace mdx

extern "C" int mdx_version(void) { return MDX_VERSION; }
extern "C" const char* mdx_last_error(void) { return mdx::error_buffer(); }
