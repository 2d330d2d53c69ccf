// Per-token magnitude pruning fused with the bitmap compressor (fp16 format).
//
// Work unit = one (KV head, 64-token block): a 64 x 128 fp16 slab (16 KB, contiguous in x),
// i.e. exactly 128 tiles of either format, whose packed values are contiguous in the output.
// One wavefront owns a unit.  The slab is streamed into LDS with 16-byte loads and stored with
// a padded row stride, so that lane = token can read its own row (and column reads over tokens)
// without bank conflicts.
//
//   count kernel   : row threshold by a 15-step radix select on the fp16 magnitudes held in
//                    registers (lane = token), bitmaps by ballot (key) or in-lane packing (value),
//                    padded counts and their prefix inside the unit.
//   scan kernels   : unit totals -> unit bases per head, head totals -> nz_off.
//   scatter kernel : re-reads the slab, compacts the survivors of each tile into an LDS image of
//                    the unit's output (rank by popcount of the tile bitmap below the lane) and
//                    streams the image out with 16-byte stores.
#include "compress_common.hpp"

namespace mstf {

// ------------------------------------------------------------------------------- count
// grid = B * M/64 units, 64 threads.  Writes bmp, unit-local exclusive offsets into idx[b][t]
// and the unit total into unit_tot[b][tokblk].
template <bool IS_VALUE>
__global__ __launch_bounds__(64) void compress_count_kernel(const _Float16* __restrict__ x, int M, int kth,
                                                            uint64_t* __restrict__ bmp, uint32_t* __restrict__ idx,
                                                            uint32_t* __restrict__ unit_tot)
{
    __shared__ uint32_t slab[kSlabDw];
    const int lane = lane_id();
    const int nblk = M / 64;
    const int unit = (int)blockIdx.x;
    const int b = unit / nblk, tb = unit - b * nblk;
    const size_t T = (size_t)M * kD / 64;
    slab_load(x + (size_t)b * M * kD, (int64_t)tb * 64, (int64_t)M, slab, lane);
    __builtin_amdgcn_wave_barrier();

    uint32_t mag[64];
    const uint32_t thr = row_threshold(slab, lane, kth, mag);
    uint64_t bmA, bmB;  // tiles tb*128 + lane and tb*128 + 64 + lane
    unit_bitmaps<IS_VALUE>(mag, thr, lane, bmA, bmB);
    uint64_t* bo = bmp + (size_t)b * T + (size_t)tb * kD;
    bo[lane] = bmA;
    bo[64 + lane] = bmB;
    const uint32_t cA = padded_units(bmA), cB = padded_units(bmB);
    uint32_t totA, totB;
    const uint32_t eA = wave_excl_scan(cA, lane, totA);
    const uint32_t eB = wave_excl_scan(cB, lane, totB);
    uint32_t* io = idx + (size_t)b * (T + 1) + (size_t)tb * kD;
    io[lane] = eA;
    io[64 + lane] = totA + eB;
    if (lane == 0) unit_tot[(size_t)b * nblk + tb] = totA + totB;
}

// ------------------------------------------------------------------------------- scans
// grid = B, 256 threads: exclusive scan of the head's unit totals, then idx[b][t] += base of
// its unit, idx[b][T] = head total, head_tot[b] = head total (4-byte units).
__global__ __launch_bounds__(256) void scan_units_kernel(const uint32_t* __restrict__ unit_tot,
                                                         uint32_t* __restrict__ idx, uint32_t* __restrict__ head_tot,
                                                         int nblk, int tiles_per_unit)
{
    extern __shared__ uint32_t base[];  // nblk entries
    const int b = (int)blockIdx.x;
    const int tid = (int)threadIdx.x;
    const uint32_t total = units_scan(unit_tot + (size_t)b * nblk, base, nblk);
    const size_t T = (size_t)nblk * tiles_per_unit;
    uint32_t* ib = idx + (size_t)b * (T + 1);
    for (size_t t = tid; t < T; t += 256) ib[t] += base[t / tiles_per_unit];
    if (tid == 0) {
        ib[T] = total;
        head_tot[b] = total;
    }
}

// one workgroup: nz_off[b] = (sum of earlier head totals) / 4 (16-byte units); total in fp16 values.
__global__ __launch_bounds__(1024) void scan_heads_kernel(const uint32_t* __restrict__ head_tot,
                                                          uint32_t* __restrict__ nz_off,
                                                          uint64_t* __restrict__ total_halfs, int B)
{
    heads_scan(head_tot, nz_off, total_halfs, B, 2, 2ull);
}

// ------------------------------------------------------------------------------- scatter
// grid = B * M/64 units, 64 threads.  bmp / idx / nz_off are final.
template <bool IS_VALUE>
__global__ __launch_bounds__(64) void compress_scatter_kernel(const _Float16* __restrict__ x, int M,
                                                              const uint64_t* __restrict__ bmp,
                                                              const uint32_t* __restrict__ idx,
                                                              const uint32_t* __restrict__ nz_off,
                                                              char* __restrict__ nz, uint64_t nz_capacity_halfs)
{
    __shared__ uint32_t slab[kSlabDw];
    __shared__ __attribute__((aligned(16))) char image[64 * kD * 2];
    const int lane = lane_id();
    const int nblk = M / 64;
    const int unit = (int)blockIdx.x;
    const int b = unit / nblk, tb = unit - b * nblk;
    const size_t T = (size_t)M * kD / 64;
    const uint64_t* bmu = bmp + (size_t)b * T + (size_t)tb * kD;
    const uint32_t* ixu = idx + (size_t)b * (T + 1) + (size_t)tb * kD;
    const uint32_t start = ixu[0];
    uint32_t bytes = (ixu[kD] - start) * 4u;
    if (bytes > (uint32_t)sizeof(image)) bytes = (uint32_t)sizeof(image);
    const uint64_t head_half0 = 8ull * nz_off[b];
    if (head_half0 + 2ull * start + bytes / 2 > nz_capacity_halfs) return;  // would not fit: leave untouched

    slab_load(x + (size_t)b * M * kD, (int64_t)tb * 64, (int64_t)M, slab, lane);
    for (uint32_t o = (uint32_t)lane * 16u; o < bytes; o += 1024u)
        *reinterpret_cast<uint4*>(image + o) = make_uint4(0u, 0u, 0u, 0u);
    __builtin_amdgcn_wave_barrier();

    const _Float16* sh = reinterpret_cast<const _Float16*>(slab);
    _Float16* img = reinterpret_cast<_Float16*>(image);
#pragma unroll 1
    for (int tt = 0; tt < kD; tt += 8) {
        const u32x16_t mv = *reinterpret_cast<const u32x16_a4*>(bmu + tt);
        const u32x8_t iv = *reinterpret_cast<const u32x8_a4*>(ixu + tt);
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int t = tt + u;
            const uint64_t m = lanes_of(u64_of(mv[2 * u], mv[2 * u + 1]));
            const uint32_t off = (iv[u] - start) * 2u;  // halfs inside the image
            // element `lane` of tile t: key -> (token lane, channel t); value -> (token t%64, channel (t/64)*64+lane)
            const int row = IS_VALUE ? (t & 63) : lane;
            const int col = IS_VALUE ? ((t >> 6) * 64 + lane) : t;
            const _Float16 v = sh[row * (2 * kRowDw) + col];
            if (lane_bit(m)) img[off + rank_below(m)] = v;
        }
    }
    __builtin_amdgcn_wave_barrier();
    char* dst = nz + (head_half0 + 2ull * start) * 2ull;
    for (uint32_t o = (uint32_t)lane * 16u; o < bytes; o += 1024u)
        *reinterpret_cast<uint4*>(dst + o) = *reinterpret_cast<const uint4*>(image + o);
}

// ------------------------------------------------------------------------------- dense prune
// y = x * (|x| >= kth-th smallest |x| of the row); 64 rows per wavefront.
__global__ __launch_bounds__(64) void prune_rows_kernel(const _Float16* __restrict__ x, _Float16* y, int64_t rows,
                                                        int kth)
{
    __shared__ uint32_t slab[kSlabDw];
    const int lane = lane_id();
    const int64_t row0 = (int64_t)blockIdx.x * 64;
    slab_load(x, row0, rows, slab, lane);
    __builtin_amdgcn_wave_barrier();
    uint32_t mag[64];
#pragma unroll
    for (int j = 0; j < 64; j++) mag[j] = slab[lane * kRowDw + j] & 0x7FFF7FFFu;
    const uint32_t thr = select_kth(mag, kth);
    const us2_t t2 = as_us2(thr | (thr << 16));
#pragma unroll
    for (int j = 0; j < 64; j++) {
        const uint32_t d = us2_u32(as_us2(mag[j]) - t2);  // bit 15 / 31 set <=> pruned
        uint32_t keep = 0x80008000u;                        // the sign always survives (x * 0 = +-0)
        if (!(d & 0x8000u)) keep |= 0x00007FFFu;
        if (!(d & 0x80000000u)) keep |= 0x7FFF0000u;
        slab[lane * kRowDw + j] &= keep;
    }
    __builtin_amdgcn_wave_barrier();
    uint4* dst = reinterpret_cast<uint4*>(y + row0 * kD);
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const int e = j * 64 + lane;
        const int row = e >> 4, c16 = e & 15;
        const uint32_t* s = slab + row * kRowDw + c16 * 4;
        if (row0 + row < rows) dst[e] = make_uint4(s[0], s[1], s[2], s[3]);
    }
}

// ------------------------------------------------------------------------------- host
struct CompressWs {
    uint32_t* unit_tot;
    uint32_t* head_tot;
};

static size_t compress_ws_bytes(int B, int M)
{
    return round_up((size_t)B * (M / 64) * 4, 256) + round_up((size_t)B * 4, 256);
}

static int check_compress_args(const void* x, int B, int M, int N, int kth)
{
    if (!x || B <= 0 || M <= 0 || N <= 0 || kth < 0 || kth > N) return MSTF_EINVAL;
    if (N != kD || M % 64 != 0) return MSTF_EUNSUPPORTED;
    if ((int64_t)B * (M / 64) > 0x7FFFFFFF) return MSTF_EUNSUPPORTED;
    if (M / 64 > 8192) return MSTF_EUNSUPPORTED;  // unit bases of one head live in LDS during the scan
    if (!aligned_to(x, 16)) return MSTF_EALIGN;
    return MSTF_OK;
}

template <bool IS_VALUE>
static int scatter_impl(void* stream, const mstf_half* x, int B, int M, int N, const uint64_t* bmp,
                        const uint32_t* idx, const uint32_t* nz_off, mstf_half* nz, uint64_t cap)
{
    int rc = check_compress_args(x, B, M, N, 0);
    if (rc != MSTF_OK) return rc;
    if (!bmp || !idx || !nz_off || !nz) return MSTF_EINVAL;
    if (!aligned_to(bmp, 8) || !aligned_to(idx, 4) || !aligned_to(nz_off, 4) || !aligned_to(nz, 16)) return MSTF_EALIGN;
    hipLaunchKernelGGL(compress_scatter_kernel<IS_VALUE>, dim3((unsigned)(B * (M / 64))), dim3(64), 0,
                       as_stream(stream), reinterpret_cast<const _Float16*>(x), M, bmp, idx, nz_off,
                       reinterpret_cast<char*>(nz), cap);
    return check_launch();
}

template <bool IS_VALUE>
static int compress_impl(void* stream, const mstf_half* x, int B, int M, int N, int kth, uint64_t* bmp, uint32_t* idx,
                         uint32_t* nz_off, uint64_t* total_halfs, mstf_half* nz, uint64_t cap, void* ws,
                         size_t ws_bytes)
{
    int rc = check_compress_args(x, B, M, N, kth);
    if (rc != MSTF_OK) return rc;
    if (!bmp || !idx || !nz_off || !total_halfs) return MSTF_EINVAL;
    if (!aligned_to(bmp, 8) || !aligned_to(idx, 4) || !aligned_to(nz_off, 4) || !aligned_to(total_halfs, 8))
        return MSTF_EALIGN;
    if (!ws || ws_bytes < compress_ws_bytes(B, M)) return MSTF_EWORKSPACE;
    if (!aligned_to(ws, 256)) return MSTF_EALIGN;
    hipStream_t st = as_stream(stream);
    const int nblk = M / 64;
    uint32_t* unit_tot = reinterpret_cast<uint32_t*>(ws);
    uint32_t* head_tot = reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(ws) + round_up((size_t)B * nblk * 4, 256));
    hipLaunchKernelGGL(compress_count_kernel<IS_VALUE>, dim3((unsigned)(B * nblk)), dim3(64), 0, st,
                       reinterpret_cast<const _Float16*>(x), M, kth, bmp, idx, unit_tot);
    if ((rc = check_launch()) != MSTF_OK) return rc;
    hipLaunchKernelGGL(scan_units_kernel, dim3((unsigned)B), dim3(256), (size_t)nblk * 4, st, unit_tot, idx, head_tot,
                       nblk, kD);
    if ((rc = check_launch()) != MSTF_OK) return rc;
    hipLaunchKernelGGL(scan_heads_kernel, dim3(1), dim3(1024), 0, st, head_tot, nz_off, total_halfs, B);
    if ((rc = check_launch()) != MSTF_OK) return rc;
    if (nz) return scatter_impl<IS_VALUE>(stream, x, B, M, N, bmp, idx, nz_off, nz, cap);
    return MSTF_OK;
}

}  // namespace mstf

using namespace mstf;

extern "C" size_t mstf_compress_workspace_bytes(int B, int M, int N)
{
    if (B <= 0 || M <= 0 || N <= 0 || M % 64 != 0) return 0;
    return compress_ws_bytes(B, M);
}

extern "C" int mstf_compress_key_f16(void* stream, const mstf_half* x, int B, int M, int N, int kth, uint64_t* bmp,
                                     uint32_t* idx, uint32_t* nz_off, uint64_t* total_halfs, mstf_half* nz,
                                     uint64_t nz_capacity_halfs, void* workspace, size_t workspace_bytes)
{
    return compress_impl<false>(stream, x, B, M, N, kth, bmp, idx, nz_off, total_halfs, nz, nz_capacity_halfs,
                                workspace, workspace_bytes);
}

extern "C" int mstf_compress_value_f16(void* stream, const mstf_half* x, int B, int M, int N, int kth, uint64_t* bmp,
                                       uint32_t* idx, uint32_t* nz_off, uint64_t* total_halfs, mstf_half* nz,
                                       uint64_t nz_capacity_halfs, void* workspace, size_t workspace_bytes)
{
    return compress_impl<true>(stream, x, B, M, N, kth, bmp, idx, nz_off, total_halfs, nz, nz_capacity_halfs,
                               workspace, workspace_bytes);
}

extern "C" int mstf_scatter_key_f16(void* stream, const mstf_half* x, int B, int M, int N, const uint64_t* bmp,
                                    const uint32_t* idx, const uint32_t* nz_off, mstf_half* nz,
                                    uint64_t nz_capacity_halfs)
{
    return scatter_impl<false>(stream, x, B, M, N, bmp, idx, nz_off, nz, nz_capacity_halfs);
}

extern "C" int mstf_scatter_value_f16(void* stream, const mstf_half* x, int B, int M, int N, const uint64_t* bmp,
                                      const uint32_t* idx, const uint32_t* nz_off, mstf_half* nz,
                                      uint64_t nz_capacity_halfs)
{
    return scatter_impl<true>(stream, x, B, M, N, bmp, idx, nz_off, nz, nz_capacity_halfs);
}

extern "C" int mstf_prune_rows_f16(void* stream, const mstf_half* x, mstf_half* y, int64_t rows, int D, int kth)
{
    if (!x || !y || rows <= 0 || kth < 1 || kth > D) return MSTF_EINVAL;
    if (D != kD) return MSTF_EUNSUPPORTED;
    if (!aligned_to(x, 16) || !aligned_to(y, 16)) return MSTF_EALIGN;
    const int64_t units = (rows + 63) / 64;
    if (units > 0x7FFFFFFF) return MSTF_EUNSUPPORTED;
    hipLaunchKernelGGL(prune_rows_kernel, dim3((unsigned)units), dim3(64), 0, as_stream(stream),
                       reinterpret_cast<const _Float16*>(x), reinterpret_cast<_Float16*>(y), rows, kth);
    return check_launch();
}
