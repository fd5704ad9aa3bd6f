// Internal helpers shared by the HIP sources of the Winograd library.
#pragma once

#include <hip/hip_runtime.h>

#include "../../include/winograd2x2.h"

namespace swc {

// Records a failed HIP call for swc_last_hip_error() and maps it to SWC_ERR_HIP.
int note_hip_error(hipError_t e);

// Records which convolution kernel a call chose, for swc_winograd2x2_conv_last_kernel().
void note_conv_kernel(const char *name);

// The tiling set with swc_winograd2x2_conv_force_tiling() on this host thread, or nullptr.
const char *forced_conv_tiling();

inline int check_launch()
{
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? SWC_OK : note_hip_error(e);
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Workgroups are handed to the 8 XCDs round-robin by linear id.  This maps the
// hardware id to a logical id such that consecutive logical ids share an XCD (and
// with it an L2): logical ids [x*per, (x+1)*per) all run on XCD x.
__device__ __forceinline__ unsigned xcd_swizzle(unsigned hw_id, unsigned n_blocks)
{
    constexpr unsigned kXcds = 8;
    const unsigned full = (n_blocks / kXcds) * kXcds;  // ids beyond this keep their place
    if (hw_id >= full) return hw_id;
    return (hw_id % kXcds) * (n_blocks / kXcds) + hw_id / kXcds;
}

}  // namespace swc
