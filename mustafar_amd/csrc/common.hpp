// Shared host/device helpers for the gfx950 kernels.  Wave size is 64 throughout.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/mustafar_hip.h"

#define MSTF_LDS __attribute__((address_space(3)))

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x16_t __attribute__((ext_vector_type(16)));
// Same vectors with only dword alignment promised (scalar-memory loads need no more).
typedef u32x4_t u32x4_a4 __attribute__((aligned(4)));
typedef u32x8_t u32x8_a4 __attribute__((aligned(4)));
typedef u32x16_t u32x16_a4 __attribute__((aligned(4)));

namespace mstf {

constexpr int kWave = 64;
constexpr int kTile = 64;  // elements per bitmap tile

// Bit casts always go through by-value helpers: applying __builtin_bit_cast directly to an
// element of an ext_vector (v[i]) reads element 0 with this compiler.
__device__ __forceinline__ h2_t as_h2(uint32_t x) { return __builtin_bit_cast(h2_t, x); }
__device__ __forceinline__ uint32_t as_u32(h2_t x) { return __builtin_bit_cast(uint32_t, x); }
__device__ __forceinline__ uint16_t as_u16(_Float16 x) { return __builtin_bit_cast(uint16_t, x); }
__device__ __forceinline__ _Float16 as_h(uint16_t x) { return __builtin_bit_cast(_Float16, x); }

__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & 63u); }
__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

// Number of set bits of the wave-uniform mask m strictly below this lane.
__device__ __forceinline__ uint32_t rank_below(uint64_t m)
{
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
}
// This lane's bit of the wave-uniform mask m (the mask is used directly as a lane mask).
__device__ __forceinline__ bool lane_bit(uint64_t m) { return __builtin_amdgcn_inverse_ballot_w64(m); }

__device__ __forceinline__ uint64_t u64_of(uint32_t lo, uint32_t hi) { return ((uint64_t)hi << 32) | lo; }

// Tile bitmaps are MSB-first (bit 63-i <=> element i); reversed, bit i <=> lane i.
__device__ __forceinline__ uint64_t lanes_of(uint64_t bmp) { return __builtin_bitreverse64(bmp); }

__device__ __forceinline__ uint32_t lds_addr(const void* p)
{
    return (uint32_t)(uintptr_t)(MSTF_LDS const char*)p;
}
__device__ __forceinline__ _Float16 lds_load_h(uint32_t a) { return *(MSTF_LDS const _Float16*)(uintptr_t)a; }
__device__ __forceinline__ uint32_t lds_load_u32(uint32_t a) { return *(MSTF_LDS const uint32_t*)(uintptr_t)a; }
__device__ __forceinline__ uint32_t lds_load_u16(uint32_t a) { return *(MSTF_LDS const uint16_t*)(uintptr_t)a; }

// lanes whose bit of the wave-uniform mask m is set take `yes`, the others `no`.  Written as one
// v_cndmask on the mask register pair so the compiler keeps the decompression straight-line
// (it otherwise turns the select into an exec-masked branch per tile).
__device__ __forceinline__ uint32_t select_lane(uint64_t m, uint32_t yes, uint32_t no)
{
    uint32_t r;
    asm("v_cndmask_b32 %0, %1, %2, %3" : "=v"(r) : "v"(no), "v"(yes), "s"(m));
    return r;
}

// Issue priority of the wavefront among those of its SIMD (0 .. 3, the instruction takes a constant: callers pass a
// value that is one after unrolling).  The decode kernels lower it from stage to stage of a block's walk, so that of
// the four wavefronts of a SIMD the ones that are behind go first: they stay within a stage of each other and finish
// together.  With the default - the oldest wavefront first - the oldest runs ahead, and the youngest ends up alone on
// its SIMD with nothing to cover its waits (fp16 kernel at 4096 tokens and 70 %: 15.8 -> 14.6 us at batch 8,
// 29.0 -> 27.0 at 16, 53.2 -> 49.4 at 32; priorities that follow the progress over all blocks of a wavefront, or fall
// only every second stage, or fall within a stage, measured the same or worse).
__device__ __forceinline__ void set_wave_priority(int p)
{
    switch (p & 3) {
    case 0: __builtin_amdgcn_s_setprio(0); break;
    case 1: __builtin_amdgcn_s_setprio(1); break;
    case 2: __builtin_amdgcn_s_setprio(2); break;
    default: __builtin_amdgcn_s_setprio(3); break;
    }
}
// The same for a wave-uniform level that is not a constant (loops that are not unrolled): a chain of scalar compares.
__device__ __forceinline__ void set_wave_priority_uniform(uint32_t p)
{
    asm volatile("s_setprio 0\n\ts_cmp_eq_u32 %[p], 0\n\ts_cbranch_scc1 1f\n\t"
                 "s_setprio 1\n\ts_cmp_eq_u32 %[p], 1\n\ts_cbranch_scc1 1f\n\t"
                 "s_setprio 2\n\ts_cmp_eq_u32 %[p], 2\n\ts_cbranch_scc1 1f\n\t"
                 "s_setprio 3\n\t1:" ::[p] "s"(p)
                 : "scc");
}

// ---------------------------------------------------------------- host side
void set_last_hip_error(int e);

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

inline int check_launch()
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_last_hip_error((int)e);
        return MSTF_ELAUNCH;
    }
    return MSTF_OK;
}

inline bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }
inline size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace mstf
