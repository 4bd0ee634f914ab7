// Host-side facts about the device the launch heuristics size their grids by.
#pragma once
#include <hip/hip_runtime.h>

namespace wkv {

// Compute units of the device that is current at the first call (cached for the process: the grids and the
// workspace sizes derived from it must agree between a size query and the launch that follows).  256 on an
// MI355X in its default partition mode; 256 is also the answer where no device can be asked (size queries on a host
// without a GPU).
inline int compute_units() {
    static const int n = [] {
        int dev = 0, cu = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cu <= 0)
            cu = 256;
        (void)hipGetLastError();   // a host without a device leaves an error behind that is not a launch's
        return cu;
    }();
    return n;
}

}  // namespace wkv
