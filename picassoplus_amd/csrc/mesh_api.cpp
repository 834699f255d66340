// Error reporting and ABI identification of libpicasso_mesh.
#include "common.h"
#include "../../include/picasso_mesh.h"
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <mutex>

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

static Options g_options;
static bool g_options_loaded = false;
static std::mutex g_options_lock;

static bool env_set(const char *name)
{
    const char *e = getenv(name);
    return e && e[0] == '1';
}

static void load_options()
{
    g_options.f2f_generic = env_set("PMESH_F2F_GENERIC");
    g_options.f2f_bf16x3 = env_set("PMESH_F2F_BF16X3");
    g_options.f2f_half = env_set("PMESH_F2F_HALF");
    g_options.f2v_valu = env_set("PMESH_F2V_VALU");
    g_options.f2v_fp32mfma = env_set("PMESH_F2V_FP32MFMA");
    g_options.point_conv_two_passes = env_set("PMESH_POINT_CONV_TWO_PASSES");
    g_options.dense_fp32mfma = env_set("PMESH_DENSE_FP32MFMA");
    g_options_loaded = true;
}

const Options &options()
{
    std::lock_guard<std::mutex> hold(g_options_lock);
    if (!g_options_loaded) load_options();
    return g_options;
}

}  // namespace pmesh

extern "C" const char *pmesh_last_error(void) { return pmesh::g_err; }
extern "C" int pmesh_abi_version(void) { return 21; }
extern "C" void pmesh_reload_options(void)
{
    std::lock_guard<std::mutex> hold(pmesh::g_options_lock);
    pmesh::load_options();
}
