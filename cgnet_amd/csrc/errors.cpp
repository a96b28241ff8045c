// Thread-local error message of the C ABI and trivial queries.
#include <cstdarg>
#include <cstdio>

#include "common.h"

namespace cgnet {
static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}
void clear_error() { g_err[0] = 0; }
}  // namespace cgnet

extern "C" const char* cgnet_last_error(void) { return cgnet::g_err; }
extern "C" int cgnet_abi_version(void) { return 1; }
extern "C" int cgnet_sparse_maxL(void) { return cgnet::kMaxL; }
