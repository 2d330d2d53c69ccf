// Quantised variant of the bitmap format: the producer (bitmaps, per-tile scale / zero-point, packed
// 2/4/8-bit codes).  The consumers are in quant_spmv.hip.
//
// Same tiles, bitmaps and work units as the fp16 format; per tile the non-zeros are replaced by
// codes  q = clamp(floor(v / scale + 0.5) + zero, 0, 2^bit - 1)  packed `capacity = 32 / bit` to a
// 4-byte word (code j of a tile at bits bit*(j % capacity) of word j / capacity), and tile_off[b][t]
// is the GLOBAL word offset of the tile inside the flat `packed` buffer.
//
#include "compress_common.hpp"
#include "spmv_common.hpp"

namespace mstf {

#pragma clang fp contract(off)

__device__ __forceinline__ float half_bits_to_float(uint32_t bits) { return (float)as_h((uint16_t)bits); }

// ------------------------------------------------------------------------------- producer: count
// grid = B * M/64 units, 64 threads.  Lane l owns tiles l and 64+l of the unit: bitmap, raw count,
// units, scale, zero; tile_off gets the unit-local exclusive word offset, unit_tot the unit total.
// G32: two (scale, zero) pairs per tile, pair g from the kept elements 32g .. 32g+31 of the tile; scales / zeros are
// then [B][T][2].
template <bool IS_VALUE, bool G32>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2))) void quant_count_kernel(const _Float16* __restrict__ x, int M, int kth, int bit,
                                                         uint64_t* __restrict__ bmp, uint32_t* __restrict__ counts,
                                                         uint32_t* __restrict__ units, uint32_t* __restrict__ tile_off,
                                                         _Float16* __restrict__ scales, _Float16* __restrict__ zeros,
                                                         uint32_t* __restrict__ unit_tot)
{
    __shared__ uint32_t slab[kHalfSlabDw];
    const int lane = lane_id();
    const int nblk = M / 64;
    const int unit = (int)blockIdx.x;
    const int b = unit / nblk, tb = unit - b * nblk;
    const size_t T = (size_t)M * kD / 64;
    uint32_t r[64];  // this lane's token: 128 fp16 values
    unit_rows(x + (size_t)b * M * kD, (int64_t)tb * 64, (int64_t)M, slab, lane, r);

    uint64_t bm[2];
    uint32_t thr;
    {
        uint32_t mag[64];
#pragma unroll
        for (int j = 0; j < 64; j++) mag[j] = r[j] & 0x7FFF7FFFu;
        thr = unit_keep<IS_VALUE>(mag, kth, lane, bm[0], bm[1]);
    }
    // The pruned elements become NaN (exponent and mantissa all ones under the element's own sign), which the
    // minimum / maximum instructions pass over: no per-element test of the bitmap is needed afterwards.
    typedef short s2_t __attribute__((ext_vector_type(2)));
    const us2_t t2 = as_us2(thr | (thr << 16));
#pragma unroll
    for (int j = 0; j < 64; j++) {
        const s2_t d = __builtin_bit_cast(s2_t, (us2_t)(as_us2(r[j] & 0x7FFF7FFFu) - t2));   // < 0 <=> pruned
        r[j] |= __builtin_bit_cast(uint32_t, (s2_t)(d >> 15)) & 0x7FFF7FFFu;
    }
    const _Float16* sh = reinterpret_cast<const _Float16*>(slab);
    const int cap = 32 / bit;
    const float maxq = (float)((1 << bit) - 1);
    const size_t tile0 = (size_t)b * T + (size_t)tb * kD;
    uint32_t u[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        constexpr int NG = G32 ? 2 : 1;
        float mn[NG], mx[NG];
        const uint64_t m = bm[h];
        if (IS_VALUE) {
            // tile (h, token = lane): the lane's own 64 channels, two per register; group g = registers 16g .. 16g+15
            typedef _Float16 h2v_t __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int g = 0; g < NG; g++) {
                h2v_t mn2 = {(_Float16)INFINITY, (_Float16)INFINITY}, mx2 = {(_Float16)-INFINITY, (_Float16)-INFINITY};
#pragma unroll
                for (int j = g * (32 / NG); j < (g + 1) * (32 / NG); j++) {
                    const h2v_t v = __builtin_bit_cast(h2v_t, r[32 * h + j]);
                    mn2 = __builtin_elementwise_min(mn2, v);
                    mx2 = __builtin_elementwise_max(mx2, v);
                }
                mn[g] = fminf((float)mn2[0], (float)mn2[1]);
                mx[g] = fmaxf((float)mx2[0], (float)mx2[1]);
            }
        } else {
            // tile = channel 64h + lane over the 64 tokens: the half-slab back into LDS, the lane walks its column;
            // group g = tokens 32g .. 32g+31
#pragma unroll
            for (int j = 0; j < 32; j++) slab[lane * kHalfRowDw + j] = r[32 * h + j];
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int g = 0; g < NG; g++) {
                float a = INFINITY, z = -INFINITY;
#pragma unroll 8
                for (int i = g * (64 / NG); i < (g + 1) * (64 / NG); i++) {
                    const float v = (float)sh[i * (2 * kHalfRowDw) + lane];
                    a = fminf(a, v);
                    z = fmaxf(z, v);
                }
                mn[g] = a;
                mx[g] = z;
            }
            __builtin_amdgcn_wave_barrier();
        }
        const uint32_t cnt = (uint32_t)__popcll(m);
        const size_t ti = tile0 + (size_t)h * 64 + lane;
#pragma unroll
        for (int g = 0; g < NG; g++) {
            // an empty group leaves the minimum at +inf: scale 1, zero 0, as for an empty tile
            float scale = 1.f, zero = 0.f;
            if (mn[g] <= mx[g]) {
                scale = (mx[g] - mn[g]) / maxq;
                if (scale == 0.f) scale = 1.f;
                zero = floorf(-mn[g] / scale + 0.5f);
            }
            scales[ti * NG + g] = (_Float16)scale;
            zeros[ti * NG + g] = (_Float16)zero;
        }
        bmp[ti] = m;
        counts[ti] = cnt;
        u[h] = (cnt + (uint32_t)cap - 1u) / (uint32_t)cap;
        units[ti] = u[h];
    }
    uint32_t totA, totB;
    const uint32_t eA = wave_excl_scan(u[0], lane, totA);
    const uint32_t eB = wave_excl_scan(u[1], lane, totB);
    tile_off[tile0 + lane] = eA;
    tile_off[tile0 + 64 + lane] = totA + eB;
    if (lane == 0) unit_tot[(size_t)b * nblk + tb] = totA + totB;
}

// grid = B, 256 threads: exclusive scan of the head's unit totals into unit_base; head_base[b] = words of all earlier
// heads (summed from their unit totals, which spares a launch for a scan over heads); the last head's workgroup
// writes the grand total.
__global__ __launch_bounds__(256) void quant_scan_kernel(const uint32_t* __restrict__ unit_tot,
                                                         uint32_t* __restrict__ unit_base,
                                                         uint32_t* __restrict__ head_base,
                                                         uint64_t* __restrict__ total_words, int nblk)
{
    extern __shared__ uint32_t base[];
    const int b = (int)blockIdx.x;
    const uint32_t total = units_scan(unit_tot + (size_t)b * nblk, base, nblk);
    for (int i = (int)threadIdx.x; i < nblk; i += 256) unit_base[(size_t)b * nblk + i] = base[i];
    const uint64_t pre = sum_before(unit_tot, (size_t)b * nblk);
    if (threadIdx.x == 0) {
        head_base[b] = (uint32_t)pre;
        if (b == (int)gridDim.x - 1) *total_words = pre + total;
    }
}

// tile_off[b][t] += head base + unit base  (global word offsets, as the reference returns them); only when no pack
// follows, which does it itself.
__global__ __launch_bounds__(256) void quant_finalize_kernel(uint32_t* __restrict__ tile_off,
                                                             const uint32_t* __restrict__ unit_base,
                                                             const uint32_t* __restrict__ head_base, int nblk, size_t T)
{
    const int b = (int)blockIdx.y;
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= T) return;
    tile_off[(size_t)b * T + t] += head_base[b] + unit_base[(size_t)b * nblk + t / kD];
}

// ------------------------------------------------------------------------------- producer: pack
// grid = B * M/64 units, 64 threads; every lane quantises and packs its two tiles.  tile_off still holds the
// unit-local offsets of the count kernel and is completed here with the unit's and the head's base.
template <bool IS_VALUE, bool G32>
__global__ __launch_bounds__(64) void quant_pack_kernel(const _Float16* __restrict__ x, int M, int bit,
                                                        const uint64_t* __restrict__ bmp,
                                                        const uint32_t* __restrict__ units, uint32_t* tile_off,
                                                        const uint32_t* __restrict__ unit_base,
                                                        const uint32_t* __restrict__ head_base,
                                                        const _Float16* __restrict__ scales,
                                                        const _Float16* __restrict__ zeros,
                                                        uint32_t* __restrict__ packed, uint64_t capacity_words)
{
    __shared__ uint32_t slab[kHalfSlabDw];
    const int lane = lane_id();
    const int nblk = M / 64;
    const int unit = (int)blockIdx.x;
    const int b = unit / nblk, tb = unit - b * nblk;
    const size_t T = (size_t)M * kD / 64;
    const _Float16* sh = reinterpret_cast<const _Float16*>(slab);
    const float maxq = (float)((1 << bit) - 1);
    const size_t tile0 = (size_t)b * T + (size_t)tb * kD;
    const uint32_t ubase = head_base[b] + unit_base[(size_t)b * nblk + tb];
#pragma unroll 1
    for (int h = 0; h < 2; h++) {
        __builtin_amdgcn_wave_barrier();
        half_slab_load(x + (size_t)b * M * kD, (int64_t)tb * 64, (int64_t)M, h, slab, lane);
        __builtin_amdgcn_wave_barrier();
        const size_t ti = tile0 + (size_t)h * 64 + lane;
        const uint64_t m = bmp[ti];
        const uint64_t off = (uint64_t)tile_off[ti] + ubase;
        tile_off[ti] = (uint32_t)off;
        if (off + units[ti] > capacity_words) continue;  // would not fit: leave untouched
        constexpr int NG = G32 ? 2 : 1;
        float scg[NG], zpg[NG];
#pragma unroll
        for (int g = 0; g < NG; g++) {
            scg[g] = (float)scales[ti * NG + g];
            zpg[g] = (float)zeros[ti * NG + g];
            if (scg[g] == 0.f) scg[g] = 1.f;
        }
        uint32_t cur = 0;
        int pos = 0;
        uint32_t w = 0;
        // only the kept elements, first to last: the wavefront loops as often as its fullest tile has non-zeros
        // (about half of 64 at 70 % sparsity), and every round carries a division
        for (uint64_t rem = m; rem != 0ull;) {
            const int i = __builtin_clzll(rem);
            rem &= ~(0x8000000000000000ull >> i);
            const int e = IS_VALUE ? (lane * (2 * kHalfRowDw) + i) : (i * (2 * kHalfRowDw) + lane);
            const float v = (float)sh[e];
            const float sc = (G32 && i >= 32) ? scg[NG - 1] : scg[0];   // the element's position picks the pair
            const float zp = (G32 && i >= 32) ? zpg[NG - 1] : zpg[0];
            float q = floorf(v / sc + 0.5f) + zp;
            q = fminf(fmaxf(q, 0.f), maxq);
            cur |= (uint32_t)q << pos;
            pos += bit;
            if (pos == 32) {
                packed[off + w++] = cur;
                cur = 0;
                pos = 0;
            }
        }
        if (pos > 0) packed[off + w] = cur;
    }
}

// ------------------------------------------------------------------------------- host
static int cap_shift_of(int bit)
{
    switch (bit) {
        case 2: return 4;
        case 4: return 3;
        case 8: return 2;
        default: return -1;
    }
}

// workspace: unit totals, unit bases (both [B][M/64]) and the head bases [B]
static size_t quant_ws_bytes(int B, int M)
{
    return 2 * round_up((size_t)B * (M / 64) * 4, 256) + round_up((size_t)B * 4, 256);
}

template <bool IS_VALUE, bool G32>
static int compress_quant_impl(void* stream, const mstf_half* x, int B, int M, int N, int kth, int bit, uint64_t* bmp,
                               uint32_t* tile_off, uint32_t* counts, uint32_t* units, mstf_half* scales,
                               mstf_half* zeros, uint64_t* total_words, uint32_t* packed, uint64_t cap_words, void* ws,
                               size_t ws_bytes)
{
    if (!x || !bmp || !tile_off || !counts || !units || !scales || !zeros || !total_words) return MSTF_EINVAL;
    if (B <= 0 || M <= 0 || N <= 0 || kth < 0 || kth > N) return MSTF_EINVAL;
    if (cap_shift_of(bit) < 0) return MSTF_EUNSUPPORTED;
    if (N != kD || M % 64 != 0 || M / 64 > 8192 || (int64_t)B * (M / 64) > 0x7FFFFFFF) return MSTF_EUNSUPPORTED;
    if (!aligned_to(x, 16) || !aligned_to(bmp, 8) || !aligned_to(tile_off, 4) || !aligned_to(counts, 4) ||
        !aligned_to(units, 4) || !aligned_to(scales, G32 ? 4 : 2) || !aligned_to(zeros, G32 ? 4 : 2) || !aligned_to(total_words, 8) ||
        (packed && !aligned_to(packed, 4)))
        return MSTF_EALIGN;
    if (!ws || ws_bytes < quant_ws_bytes(B, M)) return MSTF_EWORKSPACE;
    if (!aligned_to(ws, 256)) return MSTF_EALIGN;
    hipStream_t st = as_stream(stream);
    const int nblk = M / 64;
    const size_t T = (size_t)M * kD / 64;
    char* w = reinterpret_cast<char*>(ws);
    const size_t ub = round_up((size_t)B * nblk * 4, 256);
    uint32_t* unit_tot = reinterpret_cast<uint32_t*>(w);
    uint32_t* unit_base = reinterpret_cast<uint32_t*>(w + ub);
    uint32_t* head_base = reinterpret_cast<uint32_t*>(w + 2 * ub);
    const _Float16* xh = reinterpret_cast<const _Float16*>(x);
    int rc;
    hipLaunchKernelGGL((quant_count_kernel<IS_VALUE, G32>), dim3((unsigned)(B * nblk)), dim3(64), 0, st, xh, M, kth, bit, bmp,
                       counts, units, tile_off, reinterpret_cast<_Float16*>(scales), reinterpret_cast<_Float16*>(zeros),
                       unit_tot);
    if ((rc = check_launch()) != MSTF_OK) return rc;
    hipLaunchKernelGGL(quant_scan_kernel, dim3((unsigned)B), dim3(256), (size_t)nblk * 4, st, unit_tot, unit_base,
                       head_base, total_words, nblk);
    if ((rc = check_launch()) != MSTF_OK) return rc;
    if (packed) {
        hipLaunchKernelGGL((quant_pack_kernel<IS_VALUE, G32>), dim3((unsigned)(B * nblk)), dim3(64), 0, st, xh, M, bit, bmp,
                           units, tile_off, unit_base, head_base, reinterpret_cast<const _Float16*>(scales),
                           reinterpret_cast<const _Float16*>(zeros), packed, cap_words);
    } else {
        hipLaunchKernelGGL(quant_finalize_kernel, dim3((unsigned)((T + 255) / 256), (unsigned)B), dim3(256), 0, st,
                           tile_off, unit_base, head_base, nblk, T);
    }
    if ((rc = check_launch()) != MSTF_OK) return rc;
    return MSTF_OK;
}

}  // namespace mstf

using namespace mstf;

extern "C" size_t mstf_compress_quant_workspace_bytes(int B, int M, int N)
{
    if (B <= 0 || M <= 0 || N <= 0 || M % 64 != 0) return 0;
    return quant_ws_bytes(B, M);
}

// group_size 64: one (scale, zero) pair per tile (the reference); 32: two, scales / zeros [B][T][2].
template <bool IS_VALUE>
static int compress_quant_group(int group_size, void* stream, const mstf_half* x, int B, int M, int N, int kth, int bit,
                                uint64_t* bmp, uint32_t* tile_off, uint32_t* counts, uint32_t* units, mstf_half* scales,
                                mstf_half* zeros, uint64_t* total_words, uint32_t* packed, uint64_t cap_words, void* ws,
                                size_t ws_bytes)
{
    if (group_size == 64)
        return compress_quant_impl<IS_VALUE, false>(stream, x, B, M, N, kth, bit, bmp, tile_off, counts, units, scales, zeros,
                                                    total_words, packed, cap_words, ws, ws_bytes);
    if (group_size == 32)
        return compress_quant_impl<IS_VALUE, true>(stream, x, B, M, N, kth, bit, bmp, tile_off, counts, units, scales, zeros,
                                                   total_words, packed, cap_words, ws, ws_bytes);
    return MSTF_EUNSUPPORTED;
}

extern "C" int mstf_compress_key_quant(void* stream, const mstf_half* x, int B, int M, int N, int kth, int bit,
                                       uint64_t* bmp, uint32_t* tile_off, uint32_t* counts, uint32_t* units,
                                       mstf_half* scales, mstf_half* zeros, uint64_t* total_words, uint32_t* packed,
                                       uint64_t packed_capacity_words, void* workspace, size_t workspace_bytes)
{
    return compress_quant_group<false>(64, stream, x, B, M, N, kth, bit, bmp, tile_off, counts, units, scales, zeros,
                                       total_words, packed, packed_capacity_words, workspace, workspace_bytes);
}

extern "C" int mstf_compress_value_quant(void* stream, const mstf_half* x, int B, int M, int N, int kth, int bit,
                                         uint64_t* bmp, uint32_t* tile_off, uint32_t* counts, uint32_t* units,
                                         mstf_half* scales, mstf_half* zeros, uint64_t* total_words, uint32_t* packed,
                                         uint64_t packed_capacity_words, void* workspace, size_t workspace_bytes)
{
    return compress_quant_group<true>(64, stream, x, B, M, N, kth, bit, bmp, tile_off, counts, units, scales, zeros,
                                      total_words, packed, packed_capacity_words, workspace, workspace_bytes);
}

extern "C" int mstf_compress_quant_grouped(void* stream, const mstf_half* x, int is_value, int B, int M, int N, int kth,
                                           int bit, int group_size, uint64_t* bmp, uint32_t* tile_off, uint32_t* counts,
                                           uint32_t* units, mstf_half* scales, mstf_half* zeros, uint64_t* total_words,
                                           uint32_t* packed, uint64_t packed_capacity_words, void* workspace,
                                           size_t workspace_bytes)
{
    if (is_value)
        return compress_quant_group<true>(group_size, stream, x, B, M, N, kth, bit, bmp, tile_off, counts, units, scales,
                                          zeros, total_words, packed, packed_capacity_words, workspace, workspace_bytes);
    return compress_quant_group<false>(group_size, stream, x, B, M, N, kth, bit, bmp, tile_off, counts, units, scales,
                                       zeros, total_words, packed, packed_capacity_words, workspace, workspace_bytes);
}
