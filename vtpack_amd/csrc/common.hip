// Error plumbing shared by every entry point of libvtdge.
#include "common.h"
#include <cxxabi.h>
#include <stdlib.h>

namespace vtdge {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

// The kernel of the latest launch made from this thread, for tools that want to tell a caller's entry points from
// the kernels a profiler lists (vtdge_last_kernel).  Only the pointer is kept at launch time; the name is looked up
// and demangled when somebody asks.
static thread_local const void *last_kernel_fn = nullptr;
static thread_local char last_kernel_name[512];

void note_kernel(const void *host_function) { last_kernel_fn = host_function; }

extern "C" const char *vtdge_last_kernel(void)
{
    last_kernel_name[0] = 0;
    if (last_kernel_fn == nullptr) return last_kernel_name;
    const char *mangled = hipKernelNameRefByPtr(last_kernel_fn, nullptr);
    if (mangled == nullptr) return last_kernel_name;
    int status = 1;
    char *plain = abi::__cxa_demangle(mangled, nullptr, nullptr, &status);
    snprintf(last_kernel_name, sizeof(last_kernel_name), "%s", status == 0 && plain ? plain : mangled);
    free(plain);
    return last_kernel_name;
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
