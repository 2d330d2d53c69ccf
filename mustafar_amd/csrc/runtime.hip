// Error reporting and version of the C ABI.
#include "common.hpp"

#include <atomic>

namespace mstf {
static std::atomic<int> g_last_hip_error{0};
void set_last_hip_error(int e) { g_last_hip_error.store(e); }

// Polls a one-pass producer's workgroup spends on a wait before it gives up (0 in the atomic = the default).
static std::atomic<uint32_t> g_spin_limit{0u};
static std::atomic<bool> g_spin_limit_set{false};
uint32_t onepass_spin_limit() { return g_spin_limit_set.load() ? g_spin_limit.load() : (1u << 20); }
}  // namespace mstf

extern "C" void mstf_test_set_spin_limit(int64_t polls)
{
    if (polls < 0) {
        mstf::g_spin_limit_set.store(false);
        return;
    }
    mstf::g_spin_limit.store(polls > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)polls);
    mstf::g_spin_limit_set.store(true);
}

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

// ------------------------------------------------------------------ measurement aid
// Streams `bytes` of device memory with 16-byte loads per lane and nothing else (the xor of everything read goes to
// sink[workgroup]): the plain-read time of a buffer, against which the kernels' times are read.
namespace mstf {
__global__ __launch_bounds__(256) void read_probe_kernel(const uint4* __restrict__ src, size_t n16, uint32_t* __restrict__ sink)
{
    uint4 acc = {0u, 0u, 0u, 0u};
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) {
        const uint4 v = src[i];
        acc.x ^= v.x;
        acc.y ^= v.y;
        acc.z ^= v.z;
        acc.w ^= v.w;
    }
    const uint32_t r = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (r == 0x9e3779b9u) sink[blockIdx.x] = r;  // practically never: keeps the loads alive without a store per lane
}
}  // namespace mstf

extern "C" int mstf_probe_read(void* stream, const void* src, size_t bytes, uint32_t* sink, int workgroups)
{
    if (!src || !sink || bytes < 16 || workgroups <= 0) return MSTF_EINVAL;
    if (!mstf::aligned_to(src, 16) || !mstf::aligned_to(sink, 4)) return MSTF_EALIGN;
    hipLaunchKernelGGL(mstf::read_probe_kernel, dim3((unsigned)workgroups), dim3(256), 0, mstf::as_stream(stream),
                       reinterpret_cast<const uint4*>(src), bytes / 16, sink);
    return mstf::check_launch();
}
