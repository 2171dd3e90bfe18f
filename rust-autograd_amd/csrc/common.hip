// Status handling and geometry helpers of the C ABI.
#include "ag_internal.h"

namespace ag {

static thread_local char g_err[512] = "";

ag_status_t fail(ag_status_t code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

ag_status_t check_hip(hipError_t e, const char *what)
{
    if (e == hipSuccess) return AG_OK;
    return fail(AG_ERR_HIP_BASE + static_cast<int>(e), "%s: %s", what, hipGetErrorString(e));
}

}  // namespace ag

extern "C" {

const char *ag_last_error(void) { return ag::g_err; }

const char *ag_version(void) { return "ag_hip 0.1.0 gfx950"; }

int ag_conv_out_size(int x, int k, int pad, int stride, int dilation)
{
    return (x + 2 * pad - (dilation * (k - 1) + 1)) / stride + 1;
}

int ag_conv_transpose_out_size(int y, int k, int pad, int stride, int dilation)
{
    return stride * (y - 1) - 2 * pad + (dilation * (k - 1) + 1);
}

int ag_pool_out_size(int x, int size, int pad, int stride)
{
    return (x + 2 * pad - size) / stride + 1;
}

int ag_pool_grad_in_size(int y, int size, int pad, int stride)
{
    return stride * (y - 1) - 2 * pad + size;
}

}  // extern "C"

namespace ag {
int device_cus()
{
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            return n;
        return 256;
    }();
    return cus;
}
}  // namespace ag
