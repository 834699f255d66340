// Error reporting and ABI identification of libpicasso_mesh.
#include "common.h"
#include "../../include/picasso_mesh.h"
#include <cstdarg>
#include <cstdio>

namespace pmesh {

static thread_local char g_err[512] = "";

int fail(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return 1;
}

void clear_error() { g_err[0] = 0; }

}  // namespace pmesh

extern "C" const char *pmesh_last_error(void) { return pmesh::g_err; }
extern "C" int pmesh_abi_version(void) { return 11; }
