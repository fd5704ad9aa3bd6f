// Status strings, version and the per-thread record of the last HIP error.
#include <cstring>
#include <initializer_list>

#include "swc_common.h"

namespace swc {
namespace {
thread_local int g_last_hip_error = 0;
thread_local const char *g_conv_kernel = "";
thread_local char g_forced_tiling[16] = "";
}

const char *forced_conv_tiling() { return g_forced_tiling[0] != '\0' ? g_forced_tiling : nullptr; }

void note_conv_kernel(const char *name) { g_conv_kernel = name; }

int note_hip_error(hipError_t e)
{
    g_last_hip_error = static_cast<int>(e);
    return SWC_ERR_HIP;
}
}  // namespace swc

extern "C" const char *swc_strerror(int status)
{
    switch (status) {
        case SWC_OK: return "ok";
        case SWC_ERR_NULL_POINTER: return "a required pointer is NULL";
        case SWC_ERR_BAD_DIMS: return "a dimension is non-positive, inconsistent or too large";
        case SWC_ERR_BAD_PAD: return "pad_h and pad_w must both be 1";
        case SWC_ERR_HIP: return "the HIP runtime refused the launch (see swc_last_hip_error)";
        case SWC_ERR_BAD_RANK: return "wrong tensor rank or leading dimension";
        case SWC_ERR_UNSUPPORTED: return "this entry point has no kernel for these (valid) arguments";
        case SWC_ERR_TOO_LARGE: return "the arguments need more than this entry point's fixed scratch memory";
        default: return "unknown status";
    }
}

extern "C" int swc_last_hip_error(void) { return swc::g_last_hip_error; }

extern "C" const char *swc_winograd2x2_conv_last_kernel(void) { return swc::g_conv_kernel; }

extern "C" int swc_winograd2x2_conv_force_tiling(const char *name)
{
    if (name == nullptr || name[0] == '\0') {
        swc::g_forced_tiling[0] = '\0';
        return SWC_OK;
    }
    for (const char *known : {"sync", "ring32", "ring16", "tall16", "short16", "wide48", "wide48x64"}) {
        if (std::strcmp(name, known) == 0) {
            std::strcpy(swc::g_forced_tiling, known);
            return SWC_OK;
        }
    }
    return SWC_ERR_UNSUPPORTED;
}

extern "C" const char *swc_version(void) { return "0.1"; }
