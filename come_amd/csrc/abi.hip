// Library-wide pieces of the C ABI: version and the per-thread error message.
#include "come_common.h"

#include <string>

namespace come {
namespace {
thread_local std::string g_last_error;
}

void set_error(const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
}

void clear_error() { g_last_error.clear(); }

}  // namespace come

// 0.2.0: the attention entry points take a `flags` argument (the process-wide scale switch is gone)
// 0.2.1: come_attn_varlen_fwd_qp; come_qk_norm_rope skips a null q or k
extern "C" int come_version(void) { return 201; }

extern "C" const char *come_last_error(void) { return come::g_last_error.c_str(); }
