// Quantised variant of the bitmap format: producer (bitmaps, per-tile scale / zero-point, packed
// 2/4/8-bit codes) and the key / value SpMVs with dequantisation fused into the decompression.
//
// Same tiles, bitmaps and work units as the fp16 format; per tile the non-zeros are replaced by
// codes  q = clamp(floor(v / scale + 0.5) + zero, 0, 2^bit - 1)  packed `capacity = 32 / bit` to a
// 4-byte word (code j of a tile at bits bit*(j % capacity) of word j / capacity), and tile_off[b][t]
// is the GLOBAL word offset of the tile inside the flat `packed` buffer.
//
// The consumers read the packed words directly from global memory: a tile's codes are at most 64
// bytes (4-bit) and the lanes of a wavefront touch one or two cache lines per tile, so unlike the
// fp16 path there is nothing worth staging; the work per tile is dominated by the unpack and
// dequantise arithmetic.
#include "compress_common.hpp"
#include "spmv_common.hpp"

namespace mstf {

#pragma clang fp contract(off)

__device__ __forceinline__ float half_bits_to_float(uint32_t bits) { return (float)as_h((uint16_t)bits); }

// ------------------------------------------------------------------------------- producer: count
// grid = B * M/64 units, 64 threads.  Lane l owns tiles l and 64+l of the unit: bitmap, raw count,
// units, scale, zero; tile_off gets the unit-local exclusive word offset, unit_tot the unit total.
template <bool IS_VALUE>
__global__ __launch_bounds__(64) void quant_count_kernel(const _Float16* __restrict__ x, int M, int kth, int bit,
                                                         uint64_t* __restrict__ bmp, uint32_t* __restrict__ counts,
                                                         uint32_t* __restrict__ units, uint32_t* __restrict__ tile_off,
                                                         _Float16* __restrict__ scales, _Float16* __restrict__ zeros,
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

    uint64_t bm[2];
    {
        uint32_t mag[64];
        const uint32_t thr = row_threshold(slab, lane, kth, mag);
        unit_bitmaps<IS_VALUE>(mag, thr, lane, bm[0], bm[1]);
    }
    const _Float16* sh = reinterpret_cast<const _Float16*>(slab);
    const int cap = 32 / bit;
    const float maxq = (float)((1 << bit) - 1);
    const size_t tile0 = (size_t)b * T + (size_t)tb * kD;
    uint32_t u[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        // element i of the tile: key -> (token i, channel h*64+lane); value -> (token lane, channel h*64+i)
        float mn = INFINITY, mx = -INFINITY;
        const uint64_t m = bm[h];
        for (int i = 0; i < 64; i++) {
            const int e = IS_VALUE ? (lane * (2 * kRowDw) + h * 64 + i) : (i * (2 * kRowDw) + h * 64 + lane);
            const float v = (float)sh[e];
            if ((m >> (63 - i)) & 1ull) {
                mn = fminf(mn, v);
                mx = fmaxf(mx, v);
            }
        }
        const uint32_t cnt = (uint32_t)__popcll(m);
        float scale = 1.f, zero = 0.f;
        if (cnt > 0) {
            scale = (mx - mn) / maxq;
            if (scale == 0.f) scale = 1.f;
            zero = floorf(-mn / scale + 0.5f);
        }
        const size_t ti = tile0 + (size_t)h * 64 + lane;
        bmp[ti] = m;
        counts[ti] = cnt;
        u[h] = (cnt + (uint32_t)cap - 1u) / (uint32_t)cap;
        units[ti] = u[h];
        scales[ti] = (_Float16)scale;
        zeros[ti] = (_Float16)zero;
    }
    uint32_t totA, totB;
    const uint32_t eA = wave_excl_scan(u[0], lane, totA);
    const uint32_t eB = wave_excl_scan(u[1], lane, totB);
    tile_off[tile0 + lane] = eA;
    tile_off[tile0 + 64 + lane] = totA + eB;
    if (lane == 0) unit_tot[(size_t)b * nblk + tb] = totA + totB;
}

// grid = B, 256 threads: unit totals -> unit bases (in place), head_tot[b].
__global__ __launch_bounds__(256) void quant_scan_units_kernel(uint32_t* __restrict__ unit_tot,
                                                               uint32_t* __restrict__ head_tot, int nblk)
{
    extern __shared__ uint32_t base[];
    const int b = (int)blockIdx.x;
    uint32_t* ut = unit_tot + (size_t)b * nblk;
    const uint32_t total = units_scan(ut, base, nblk);
    for (int i = (int)threadIdx.x; i < nblk; i += 256) ut[i] = base[i];
    if (threadIdx.x == 0) head_tot[b] = total;
}

__global__ __launch_bounds__(1024) void quant_scan_heads_kernel(const uint32_t* __restrict__ head_tot,
                                                                uint32_t* __restrict__ head_base,
                                                                uint64_t* __restrict__ total_words, int B)
{
    heads_scan(head_tot, head_base, total_words, B, 0, 1ull);
}

// tile_off[b][t] += head base + unit base  (global word offsets, as the reference returns them)
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
// grid = B * M/64 units, 64 threads; every lane quantises and packs its two tiles.
template <bool IS_VALUE>
__global__ __launch_bounds__(64) void quant_pack_kernel(const _Float16* __restrict__ x, int M, int bit,
                                                        const uint64_t* __restrict__ bmp,
                                                        const uint32_t* __restrict__ units,
                                                        const uint32_t* __restrict__ tile_off,
                                                        const _Float16* __restrict__ scales,
                                                        const _Float16* __restrict__ zeros,
                                                        uint32_t* __restrict__ packed, uint64_t capacity_words)
{
    __shared__ uint32_t slab[kSlabDw];
    const int lane = lane_id();
    const int nblk = M / 64;
    const int unit = (int)blockIdx.x;
    const int b = unit / nblk, tb = unit - b * nblk;
    const size_t T = (size_t)M * kD / 64;
    slab_load(x + (size_t)b * M * kD, (int64_t)tb * 64, (int64_t)M, slab, lane);
    __builtin_amdgcn_wave_barrier();
    const _Float16* sh = reinterpret_cast<const _Float16*>(slab);
    const float maxq = (float)((1 << bit) - 1);
    const size_t tile0 = (size_t)b * T + (size_t)tb * kD;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const size_t ti = tile0 + (size_t)h * 64 + lane;
        const uint64_t m = bmp[ti];
        const uint64_t off = tile_off[ti];
        if (off + units[ti] > capacity_words) continue;  // would not fit: leave untouched
        float sc = (float)scales[ti];
        const float zp = (float)zeros[ti];
        if (sc == 0.f) sc = 1.f;
        uint32_t cur = 0;
        int pos = 0;
        uint32_t w = 0;
        for (int i = 0; i < 64; i++) {
            if (!((m >> (63 - i)) & 1ull)) continue;
            const int e = IS_VALUE ? (lane * (2 * kRowDw) + h * 64 + i) : (i * (2 * kRowDw) + h * 64 + lane);
            const float v = (float)sh[e];
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

// ------------------------------------------------------------------------------- consumers
// Dequantised element `lane` of a tile (0 when absent), as fp16.
//   m     : the tile's lane mask (bit i <=> element i present), wave-uniform
//   words : the tile's packed words (global memory)
template <int MODE>
__device__ __forceinline__ _Float16 tile_value_q(uint64_t m, const uint32_t* __restrict__ words, uint32_t scale_bits,
                                                 uint32_t zero_bits, int bit, int cap_shift, uint32_t cmask)
{
    const uint32_t r = rank_below(m);
    const bool present = lane_bit(m);
    const uint32_t word = present ? words[r >> cap_shift] : 0u;
    const uint32_t q = (word >> ((r & ((1u << cap_shift) - 1u)) * (uint32_t)bit)) & cmask;
    _Float16 v;
    if (MODE == 1) {
        const _Float16 d = (_Float16)(int)q - as_h((uint16_t)zero_bits);  // fp16 arithmetic, rounded after each step
        v = d * as_h((uint16_t)scale_bits);
    } else {
        v = (_Float16)(((float)q - half_bits_to_float(zero_bits)) * half_bits_to_float(scale_bits));
    }
    return present ? v : (_Float16)0;
}

// acc[n] += sum over the 64 tiles starting at `tile` of D[t][lane] * w[n][t]; w: fp16 pairs through scalar loads.
template <int NW, int MODE>
__device__ __forceinline__ void chunk_accumulate_q(const uint64_t* __restrict__ bm, const uint32_t* __restrict__ toff,
                                                   const uint16_t* __restrict__ sc, const uint16_t* __restrict__ zp,
                                                   const uint32_t* __restrict__ packed, const _Float16* w,
                                                   size_t wstride, int bit, int cap_shift, uint32_t cmask,
                                                   float (&acc)[NW])
{
#pragma unroll 1
    for (int tt = 0; tt < 64; tt += 2) {
        const uint64_t m0 = lanes_of(bm[tt]);
        const uint64_t m1 = lanes_of(bm[tt + 1]);
        h2_t p;
        p.x = tile_value_q<MODE>(m0, packed + toff[tt], sc[tt], zp[tt], bit, cap_shift, cmask);
        p.y = tile_value_q<MODE>(m1, packed + toff[tt + 1], sc[tt + 1], zp[tt + 1], bit, cap_shift, cmask);
#pragma unroll
        for (int n = 0; n < NW; n++) {
            const uint32_t q = *reinterpret_cast<const uint32_t*>(w + (size_t)n * wstride + tt);
            acc[n] = __builtin_amdgcn_fdot2(p, as_h2(q), acc[n], false);
        }
    }
}

// One wavefront per (KV head, token block).
template <int NW, int MODE>
__global__ __launch_bounds__(256) void key_spmv_quant_kernel(
    const uint64_t* __restrict__ bmp, const uint32_t* __restrict__ packed, const uint32_t* __restrict__ tile_off,
    const uint16_t* __restrict__ scales, const uint16_t* __restrict__ zeros, const _Float16* __restrict__ Bm,
    _Float16* __restrict__ C, int Lc, int D, int nblk, int ntasks, int rows_per_kv, int row0, int bit, int cap_shift)
{
    const int lane = lane_id();
    const int task = (int)blockIdx.x * 4 + wave_id();
    if (task >= ntasks) return;
    const int kv = task / nblk, tb = task - kv * nblk;
    const size_t T = (size_t)Lc * D / 64;
    const size_t t0 = (size_t)kv * T + (size_t)tb * D;
    const _Float16* wk = Bm + ((size_t)kv * rows_per_kv + row0) * D;
    const uint32_t cmask = (1u << bit) - 1u;
    float acc[NW];
#pragma unroll
    for (int n = 0; n < NW; n++) acc[n] = 0.f;
    for (int c = 0; c < D / 64; c++)
        chunk_accumulate_q<NW, MODE>(bmp + t0 + c * 64, tile_off + t0 + c * 64, scales + t0 + c * 64,
                                     zeros + t0 + c * 64, packed, wk + c * 64, (size_t)D, bit, cap_shift, cmask, acc);
    _Float16* out = C + ((size_t)kv * rows_per_kv + row0) * Lc + (size_t)tb * 64 + lane;
#pragma unroll
    for (int n = 0; n < NW; n++) out[(size_t)n * Lc] = (_Float16)acc[n];
}

// grid = (token splits, D/64 halves, KV heads), WAVES wavefronts each walking nbpw token blocks.
template <int NW, int WAVES, int MODE>
__global__ __launch_bounds__(WAVES * 64) void value_spmv_quant_kernel(
    const uint64_t* __restrict__ bmp, const uint32_t* __restrict__ packed, const uint32_t* __restrict__ tile_off,
    const uint16_t* __restrict__ scales, const uint16_t* __restrict__ zeros, const _Float16* __restrict__ P,
    _Float16* __restrict__ C, float* __restrict__ part, int Lc, int D, int nblk, int nbpw, int nsplit, int rows_per_kv,
    int row0, int bit, int cap_shift)
{
    __shared__ float red[WAVES][NW * 64];
    const int lane = lane_id();
    const int wave = wave_id();
    const int split = (int)blockIdx.x, half = (int)blockIdx.y, kv = (int)blockIdx.z;
    const size_t T = (size_t)Lc * D / 64;
    const size_t th = (size_t)kv * T + (size_t)half * 64;
    const _Float16* wk = P + ((size_t)kv * rows_per_kv + row0) * Lc;
    const uint32_t cmask = (1u << bit) - 1u;
    float acc[NW];
#pragma unroll
    for (int n = 0; n < NW; n++) acc[n] = 0.f;
    const int first = (split * WAVES + wave) * nbpw;
    int last = first + nbpw;
    if (last > nblk) last = nblk;
    for (int tb = first; tb < last; tb++) {
        const size_t t0 = th + (size_t)tb * D;
        chunk_accumulate_q<NW, MODE>(bmp + t0, tile_off + t0, scales + t0, zeros + t0, packed, wk + (size_t)tb * 64,
                                     (size_t)Lc, bit, cap_shift, cmask, acc);
    }
#pragma unroll
    for (int n = 0; n < NW; n++) red[wave][n * 64 + lane] = acc[n];
    __syncthreads();
    for (int o = (int)threadIdx.x; o < NW * 64; o += WAVES * 64) {
        float s = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; wv++) s += red[wv][o];
        const int n = o >> 6, ch = o & 63;
        const size_t row = (size_t)kv * rows_per_kv + row0 + n;
        if (nsplit == 1)
            C[row * D + (size_t)half * 64 + ch] = (_Float16)s;
        else
            part[(row * nsplit + split) * D + (size_t)half * 64 + ch] = s;
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

static size_t quant_ws_bytes(int B, int M)
{
    return round_up((size_t)B * (M / 64) * 4, 256) + 2 * round_up((size_t)B * 4, 256);
}

template <bool IS_VALUE>
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
        !aligned_to(units, 4) || !aligned_to(scales, 2) || !aligned_to(zeros, 2) || !aligned_to(total_words, 8) ||
        (packed && !aligned_to(packed, 4)))
        return MSTF_EALIGN;
    if (!ws || ws_bytes < quant_ws_bytes(B, M)) return MSTF_EWORKSPACE;
    if (!aligned_to(ws, 256)) return MSTF_EALIGN;
    hipStream_t st = as_stream(stream);
    const int nblk = M / 64;
    const size_t T = (size_t)M * kD / 64;
    char* w = reinterpret_cast<char*>(ws);
    uint32_t* unit_tot = reinterpret_cast<uint32_t*>(w);
    uint32_t* head_tot = reinterpret_cast<uint32_t*>(w + round_up((size_t)B * nblk * 4, 256));
    uint32_t* head_base = reinterpret_cast<uint32_t*>(w + round_up((size_t)B * nblk * 4, 256) + round_up((size_t)B * 4, 256));
    const _Float16* xh = reinterpret_cast<const _Float16*>(x);
    int rc;
    hipLaunchKernelGGL(quant_count_kernel<IS_VALUE>, dim3((unsigned)(B * nblk)), dim3(64), 0, st, xh, M, kth, bit, bmp,
                       counts, units, tile_off, reinterpret_cast<_Float16*>(scales), reinterpret_cast<_Float16*>(zeros),
                       unit_tot);
    if ((rc = check_launch()) != MSTF_OK) return rc;
    hipLaunchKernelGGL(quant_scan_units_kernel, dim3((unsigned)B), dim3(256), (size_t)nblk * 4, st, unit_tot, head_tot,
                       nblk);
    if ((rc = check_launch()) != MSTF_OK) return rc;
    hipLaunchKernelGGL(quant_scan_heads_kernel, dim3(1), dim3(1024), 0, st, head_tot, head_base, total_words, B);
    if ((rc = check_launch()) != MSTF_OK) return rc;
    hipLaunchKernelGGL(quant_finalize_kernel, dim3((unsigned)((T + 255) / 256), (unsigned)B), dim3(256), 0, st, tile_off,
                       unit_tot, head_base, nblk, T);
    if ((rc = check_launch()) != MSTF_OK) return rc;
    if (packed) {
        hipLaunchKernelGGL(quant_pack_kernel<IS_VALUE>, dim3((unsigned)(B * nblk)), dim3(64), 0, st, xh, M, bit, bmp,
                           units, tile_off, reinterpret_cast<const _Float16*>(scales),
                           reinterpret_cast<const _Float16*>(zeros), packed, cap_words);
        if ((rc = check_launch()) != MSTF_OK) return rc;
    }
    return MSTF_OK;
}

static int check_quant_spmv(const void* bmp, const void* packed, const void* tile_off, const void* scales,
                            const void* zeros, const void* Bm, const void* C, int tokens, int head_dim, int Bq,
                            int groups, int n_rows, int bit, int capacity, int dequant_mode)
{
    if (!bmp || !packed || !tile_off || !scales || !zeros || !Bm || !C) return MSTF_EINVAL;
    if (tokens <= 0 || head_dim <= 0 || Bq <= 0 || groups <= 0 || n_rows <= 0 || Bq % groups != 0) return MSTF_EINVAL;
    if (dequant_mode != 0 && dequant_mode != 1) return MSTF_EINVAL;
    if (cap_shift_of(bit) < 0) return MSTF_EUNSUPPORTED;
    if (capacity != 32 / bit) return MSTF_EINVAL;
    if (tokens % 64 != 0 || head_dim % 64 != 0) return MSTF_EUNSUPPORTED;
    if (!aligned_to(bmp, 8) || !aligned_to(packed, 4) || !aligned_to(tile_off, 4) || !aligned_to(scales, 2) ||
        !aligned_to(zeros, 2) || !aligned_to(Bm, 4) || !aligned_to(C, 2))
        return MSTF_EALIGN;
    return MSTF_OK;
}

#define MSTF_Q_KEY(NWV)                                                                                              \
    case NWV:                                                                                                        \
        if (dequant_mode == 1)                                                                                       \
            hipLaunchKernelGGL((key_spmv_quant_kernel<NWV, 1>), grid, dim3(256), 0, st, bmp, packed, tile_off, sc,    \
                               zp, b, c, M, K, nblk, ntasks, rows_per_kv, row0, bit, cs);                             \
        else                                                                                                         \
            hipLaunchKernelGGL((key_spmv_quant_kernel<NWV, 0>), grid, dim3(256), 0, st, bmp, packed, tile_off, sc,    \
                               zp, b, c, M, K, nblk, ntasks, rows_per_kv, row0, bit, cs);                             \
        break;

#define MSTF_Q_VALUE(NWV, WV)                                                                                        \
    case NWV:                                                                                                        \
        if (dequant_mode == 1)                                                                                       \
            hipLaunchKernelGGL((value_spmv_quant_kernel<NWV, WV, 1>), grid, dim3(WV * 64), 0, st, bmp, packed,        \
                               tile_off, sc, zp, p, c, part, K, M, K / 64, pl.nbpw, pl.nsplit, rows_per_kv, row0,     \
                               bit, cs);                                                                             \
        else                                                                                                         \
            hipLaunchKernelGGL((value_spmv_quant_kernel<NWV, WV, 0>), grid, dim3(WV * 64), 0, st, bmp, packed,        \
                               tile_off, sc, zp, p, c, part, K, M, K / 64, pl.nbpw, pl.nsplit, rows_per_kv, row0,     \
                               bit, cs);                                                                             \
        break;

}  // namespace mstf

using namespace mstf;

extern "C" size_t mstf_compress_quant_workspace_bytes(int B, int M, int N)
{
    if (B <= 0 || M <= 0 || N <= 0 || M % 64 != 0) return 0;
    return quant_ws_bytes(B, M);
}

extern "C" int mstf_compress_key_quant(void* stream, const mstf_half* x, int B, int M, int N, int kth, int bit,
                                       uint64_t* bmp, uint32_t* tile_off, uint32_t* counts, uint32_t* units,
                                       mstf_half* scales, mstf_half* zeros, uint64_t* total_words, uint32_t* packed,
                                       uint64_t packed_capacity_words, void* workspace, size_t workspace_bytes)
{
    return compress_quant_impl<false>(stream, x, B, M, N, kth, bit, bmp, tile_off, counts, units, scales, zeros,
                                      total_words, packed, packed_capacity_words, workspace, workspace_bytes);
}

extern "C" int mstf_compress_value_quant(void* stream, const mstf_half* x, int B, int M, int N, int kth, int bit,
                                         uint64_t* bmp, uint32_t* tile_off, uint32_t* counts, uint32_t* units,
                                         mstf_half* scales, mstf_half* zeros, uint64_t* total_words, uint32_t* packed,
                                         uint64_t packed_capacity_words, void* workspace, size_t workspace_bytes)
{
    return compress_quant_impl<true>(stream, x, B, M, N, kth, bit, bmp, tile_off, counts, units, scales, zeros,
                                     total_words, packed, packed_capacity_words, workspace, workspace_bytes);
}

extern "C" int mstf_key_spmv_quant(void* stream, const uint64_t* bmp, const uint32_t* packed, const uint32_t* tile_off,
                                   const uint32_t* counts, const uint32_t* units, const mstf_half* scales,
                                   const mstf_half* zeros, const mstf_half* Bm, mstf_half* C, int M, int K, int Bq,
                                   int groups, int n_rows, int bit, int capacity, int dequant_mode)
{
    (void)counts;  // raw counts and units follow from the bitmaps; accepted for interface compatibility
    (void)units;
    int rc = check_quant_spmv(bmp, packed, tile_off, scales, zeros, Bm, C, M, K, Bq, groups, n_rows, bit, capacity,
                              dequant_mode);
    if (rc != MSTF_OK) return rc;
    hipStream_t st = as_stream(stream);
    const int Bkv = Bq / groups, rows_per_kv = groups * n_rows, cs = cap_shift_of(bit);
    const int nblk = M / 64, ntasks = Bkv * nblk;
    const dim3 grid((unsigned)((ntasks + 3) / 4));
    const _Float16* b = reinterpret_cast<const _Float16*>(Bm);
    _Float16* c = reinterpret_cast<_Float16*>(C);
    const uint16_t* sc = scales;
    const uint16_t* zp = zeros;
    for (int row0 = 0; row0 < rows_per_kv;) {
        int nw = pick_nw(rows_per_kv - row0);
        if (nw > 8) nw = 8;
        switch (nw) {
            MSTF_Q_KEY(8)
            MSTF_Q_KEY(4)
            MSTF_Q_KEY(2)
            MSTF_Q_KEY(1)
        }
        if ((rc = check_launch()) != MSTF_OK) return rc;
        row0 += nw;
    }
    return MSTF_OK;
}

extern "C" size_t mstf_value_spmv_quant_workspace_bytes(int M, int K, int Bq, int groups, int n_rows)
{
    if (M <= 0 || K <= 0 || Bq <= 0 || groups <= 0 || n_rows <= 0 || K % 64 != 0 || M % 64 != 0 || Bq % groups != 0)
        return 0;
    // the quantised passes cover at most 8 accumulators each; their plan never has fewer splits than a wider one
    const ValuePlan pl = plan_value(K, M, Bq / groups, 8);
    return pl.nsplit > 1 ? round_up((size_t)Bq * n_rows * pl.nsplit * M * sizeof(float), 256) : 0;
}

extern "C" int mstf_value_spmv_quant(void* stream, const uint64_t* bmp, const uint32_t* packed,
                                     const uint32_t* tile_off, const uint32_t* counts, const uint32_t* units,
                                     const mstf_half* scales, const mstf_half* zeros, const mstf_half* P, mstf_half* C,
                                     int M, int K, int Bq, int groups, int n_rows, int bit, int capacity,
                                     int dequant_mode, void* workspace, size_t workspace_bytes)
{
    (void)counts;
    (void)units;
    int rc = check_quant_spmv(bmp, packed, tile_off, scales, zeros, P, C, K, M, Bq, groups, n_rows, bit, capacity,
                              dequant_mode);
    if (rc != MSTF_OK) return rc;
    const size_t need = mstf_value_spmv_quant_workspace_bytes(M, K, Bq, groups, n_rows);
    if (need > 0 && (!workspace || workspace_bytes < need)) return MSTF_EWORKSPACE;
    if (workspace && !aligned_to(workspace, 16)) return MSTF_EALIGN;
    hipStream_t st = as_stream(stream);
    const int Bkv = Bq / groups, rows_per_kv = groups * n_rows, cs = cap_shift_of(bit);
    const _Float16* p = reinterpret_cast<const _Float16*>(P);
    _Float16* c = reinterpret_cast<_Float16*>(C);
    float* part = reinterpret_cast<float*>(workspace);
    const uint16_t* sc = scales;
    const uint16_t* zp = zeros;
    const ValuePlan pl = plan_value(K, M, Bkv, 8);
    const dim3 grid((unsigned)pl.nsplit, (unsigned)(M / 64), (unsigned)Bkv);
    for (int row0 = 0; row0 < rows_per_kv;) {
        int nw = pick_nw(rows_per_kv - row0);
        if (nw > 8) nw = 8;
        switch (nw) {
            MSTF_Q_VALUE(8, 8)
            MSTF_Q_VALUE(4, 8)
            MSTF_Q_VALUE(2, 8)
            MSTF_Q_VALUE(1, 8)
        }
        if ((rc = check_launch()) != MSTF_OK) return rc;
        if (pl.nsplit > 1) {
            launch_value_merge(st, part, c, pl.nsplit, M, rows_per_kv, row0, nw, Bkv);
            if ((rc = check_launch()) != MSTF_OK) return rc;
        }
        row0 += nw;
    }
    return MSTF_OK;
}
