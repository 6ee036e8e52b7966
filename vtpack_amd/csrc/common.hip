// Error plumbing shared by every entry point of libvtdge.
#include "common.h"

namespace vtdge {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int check_launch(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: kernel launch failed: %s", what, hipGetErrorString(e));
        return VTDGE_ERR_LAUNCH;
    }
    return VTDGE_OK;
}

int compute_units()
{
    // asked once per device; the answer cannot change while the process lives
    static std::once_flag once[16];
    static int count[16];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return 256;
    std::call_once(once[dev], [&] {
        hipDeviceProp_t prop;
        count[dev] = hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0
                         ? prop.multiProcessorCount
                         : 256;
    });
    return count[dev];
}

}  // namespace vtdge

extern "C" int vtdge_version(void) { return 100; }
extern "C" const char *vtdge_last_error(void) { return vtdge::g_err; }
