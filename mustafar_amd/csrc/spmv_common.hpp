// Host-side planning and the split-merge kernel shared by the fp16 and the quantised SpMV files.
#pragma once
#include "common.hpp"

namespace mstf {

// Adds the token-split partials of rows [row0, row0+nw) of every KV head and rounds to fp16.
template <int UNUSED = 0>
__global__ __launch_bounds__(256) void value_merge_kernel(const float* __restrict__ part, _Float16* __restrict__ C,
                                                          int nsplit, int D, int rows_per_kv, int row0, int nw,
                                                          size_t total)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const size_t d = i % D;
    const size_t r = i / D;
    const size_t row = (r / nw) * rows_per_kv + row0 + (r % nw);
    float s = 0.f;
    for (int k = 0; k < nsplit; k++) s += part[(row * nsplit + k) * D + d];
    C[row * D + d] = (_Float16)s;
}

// Largest accumulator count with an instantiated kernel that fits in `left`.
inline int pick_nw(int left)
{
    const int opts[] = {32, 16, 8, 4, 2, 1};
    for (int o : opts)
        if (o <= left) return o;
    return 1;
}

// Workgroups are handed to the chip's eight XCDs round-robin by their linear index, and every XCD has an L2 of its
// own: two workgroups that share cache lines - neighbours in memory - fetch them twice when they sit on different
// XCDs.  xcd_contiguous turns the linear index `id` of a launch of xcd_grid(n) workgroups into a logical index such
// that every XCD works through one contiguous eighth of the n logical workgroups; indices >= n are surplus
// workgroups that leave at once.  (Only traffic depends on the round-robin assumption, never results.)
inline int xcd_grid(int n) { return 8 * ((n + 7) / 8); }
#ifdef __HIPCC__
__device__ __forceinline__ int xcd_contiguous(int id, int n) { return (id & 7) * ((n + 7) >> 3) + (id >> 3); }
#endif

struct ValuePlan {
    int waves;   // wavefronts per workgroup
    int nbpw;    // token blocks per wavefront
    int nsplit;  // workgroups along the token axis
};

inline ValuePlan plan_value(int Lc, int D, int Bkv, int nw)
{
    ValuePlan p;
    const int nblk = Lc / 64;
    const long chunks = (long)nblk * (D / 64) * Bkv;
    p.waves = nw > 8 ? 4 : 8;
    // aim at ~4096 resident wavefronts on 256 CUs, at least two token blocks each to pipeline
    long nb = (chunks + 4095) / 4096;
    if (nb < 1) nb = 1;
    if (nb > nblk) nb = nblk;
    p.nbpw = (int)nb;
    p.nsplit = (nblk + p.waves * p.nbpw - 1) / (p.waves * p.nbpw);
    return p;
}

// Launches the merge of rows [row0, row0+nw) of every KV head.
inline void launch_value_merge(hipStream_t st, const float* part, _Float16* C, int nsplit, int D, int rows_per_kv,
                               int row0, int nw, int Bkv)
{
    const size_t total = (size_t)Bkv * nw * D;
    hipLaunchKernelGGL(value_merge_kernel<0>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, part, C, nsplit,
                       D, rows_per_kv, row0, nw, total);
}

// Workspace of a token-split value product (fp32 partials), 0 when no pass splits.
inline size_t value_workspace_bytes(int head_dim, int tokens, int Bq, int groups, int n_rows)
{
    const int rows_per_kv = groups * n_rows;
    size_t worst = 0;
    for (int row0 = 0; row0 < rows_per_kv;) {
        const int nw = pick_nw(rows_per_kv - row0);
        const ValuePlan pl = plan_value(tokens, head_dim, Bq / groups, nw);
        const size_t need = pl.nsplit > 1 ? (size_t)Bq * n_rows * pl.nsplit * head_dim * sizeof(float) : 0;
        if (need > worst) worst = need;
        row0 += nw;
    }
    return round_up(worst, 256);
}

}  // namespace mstf
