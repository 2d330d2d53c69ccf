// Error reporting and version of the C ABI.
#include "common.hpp"

#include <atomic>

namespace mstf {
static std::atomic<int> g_last_hip_error{0};
void set_last_hip_error(int e) { g_last_hip_error.store(e); }
}  // namespace mstf

extern "C" const char* mstf_strerror(int code)
{
    switch (code) {
        case MSTF_OK: return "ok";
        case MSTF_EINVAL: return "invalid argument (null pointer, non-positive size or inconsistent shape)";
        case MSTF_EALIGN: return "pointer not aligned as required";
        case MSTF_EUNSUPPORTED: return "shape not supported by the gfx950 kernels";
        case MSTF_EWORKSPACE: return "workspace missing or too small";
        case MSTF_ELAUNCH: return "HIP kernel launch failed (see mstf_last_hip_error)";
        case MSTF_ETOOLARGE:
            return "the problem needs more scratch memory than the library's fixed buffer holds (use the entry point "
                   "that takes a workspace)";
        default: return "unknown error code";
    }
}

extern "C" int mstf_last_hip_error(void) { return mstf::g_last_hip_error.load(); }

extern "C" int mstf_version(void) { return 100; }
