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

// tile_off[b][t] += head base + unit base  (global word offsets, as the reference returns them): the sizing-only call.
__global__ __launch_bounds__(256) void quant_finalize_kernel(uint32_t* __restrict__ tile_off,
                                                             const uint32_t* __restrict__ unit_base,
                                                             const uint32_t* __restrict__ head_base, int nblk, size_t T)
{
    const int b = (int)blockIdx.y;
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= T) return;
    tile_off[(size_t)b * T + t] += head_base[b] + unit_base[(size_t)b * nblk + t / kD];
}

// ------------------------------------------------------------------------------- producer: one pass
// Everything with one read of the input, for the calls that produce the packed words: the count kernel's work on the
// rows held in registers, the workgroup's word total published as a status word, the totals of the workgroups in
// front of it added up (the one-pass ordering of the fp16 compressor, compress.hip), then the pack straight from
// the registers - a half goes back into the LDS slab, and every lane quantises and packs its two tiles at their
// final global word offsets.  grid = units / W workgroups of W wavefronts, W divides M / 64.
// total_words reads as all ones when a wait ran out of its polls.
template <bool IS_VALUE, bool G32, int W>
__global__ __launch_bounds__(64 * W) __attribute__((amdgpu_waves_per_eu(4))) void quant_onepass_kernel(
    const _Float16* __restrict__ x, int M, int kth, int bit, uint64_t* __restrict__ bmp, uint32_t* __restrict__ counts,
    uint32_t* __restrict__ units, uint32_t* __restrict__ tile_off, _Float16* __restrict__ scales,
    _Float16* __restrict__ zeros, uint32_t* __restrict__ packed, uint64_t capacity_words,
    uint64_t* __restrict__ total_words, uint64_t* state, int nunits, int groups_total, uint32_t spin_limit)
{
    __shared__ uint32_t slabs[W][kHalfSlabDw];
    __shared__ uint32_t wave_total[W];
    __shared__ uint64_t bases[W][2];
    __shared__ uint32_t coop_words[W][16];  // the packed words of a tile quantised by the whole wavefront (64 * bit / 32 <= 16)
    const int lane = lane_id();
    const int wave = wave_id();
    const int nblk = M / 64;
    const int g = (int)blockIdx.x;
    const int unit = g * W + wave;
    const int b = unit / nblk, tb = unit - b * nblk;
    const size_t T = (size_t)M * kD / 64;
    uint32_t* slab = slabs[wave];
    uint32_t r[64];  // this lane's token: 128 fp16 values
    {
        UnitRaw raw;
        unit_fetch(x + (size_t)b * M * kD, (int64_t)tb * 64, lane, raw);
        unit_rows_parked(raw, slab, lane, r);  // r[32 .. 64) stays in the slab during the search
    }
    uint64_t bm[2];
    uint32_t thr = 1u;
    {
        uint32_t kept[4];
        if (kth > 0) {
            thr = select_kth_planes_parked<true>(r, slab, lane, kth, kept);  // the sign bits become planes the search never looks at
            if (thr == 0u) thr = 1u;
        } else {
            parked_rows_take(slab, lane, r);
            kept_nonzero(r, kept);
        }
        __builtin_amdgcn_wave_barrier();
        if (IS_VALUE) {
            bm[0] = spread_bitmap(kept[0], kept[1]);
            bm[1] = spread_bitmap(kept[2], kept[3]);
        } else {
            key_bitmaps_from_kept(kept, lane, bm[0], bm[1]);
        }
    }
    // pruned elements become NaN, which the minimum / maximum instructions pass over (see quant_count_kernel)
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
    constexpr int NG = G32 ? 2 : 1;
    uint32_t u[2];
    float scg[2][NG], zpg[2][NG];  // the parameters as the consumers will read them: rounded to fp16
#pragma unroll
    for (int h = 0; h < 2; h++) {
        float mn[NG], mx[NG];
        if (IS_VALUE) {
            typedef _Float16 h2v_t __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int gq = 0; gq < NG; gq++) {
                h2v_t mn2 = {(_Float16)INFINITY, (_Float16)INFINITY}, mx2 = {(_Float16)-INFINITY, (_Float16)-INFINITY};
#pragma unroll
                for (int j = gq * (32 / NG); j < (gq + 1) * (32 / NG); j++) {
                    const h2v_t v = __builtin_bit_cast(h2v_t, r[32 * h + j]);
                    mn2 = __builtin_elementwise_min(mn2, v);
                    mx2 = __builtin_elementwise_max(mx2, v);
                }
                mn[gq] = fminf((float)mn2[0], (float)mn2[1]);
                mx[gq] = fmaxf((float)mx2[0], (float)mx2[1]);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 32; j++) slab[lane * kHalfRowDw + j] = r[32 * h + j];
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int gq = 0; gq < NG; gq++) {
                float a = INFINITY, z = -INFINITY;
#pragma unroll 8
                for (int i = gq * (64 / NG); i < (gq + 1) * (64 / NG); i++) {
                    const float v = (float)sh[i * (2 * kHalfRowDw) + lane];
                    a = fminf(a, v);
                    z = fmaxf(z, v);
                }
                mn[gq] = a;
                mx[gq] = z;
            }
            __builtin_amdgcn_wave_barrier();
        }
        const uint32_t cnt = (uint32_t)__popcll(bm[h]);
        const size_t ti = tile0 + (size_t)h * 64 + lane;
#pragma unroll
        for (int gq = 0; gq < NG; gq++) {
            float scale = 1.f, zero = 0.f;
            if (mn[gq] <= mx[gq]) {
                scale = (mx[gq] - mn[gq]) / maxq;
                if (scale == 0.f) scale = 1.f;
                zero = floorf(-mn[gq] / scale + 0.5f);
            }
            const _Float16 s16 = (_Float16)scale, z16 = (_Float16)zero;
            scales[ti * NG + gq] = s16;
            zeros[ti * NG + gq] = z16;
            scg[h][gq] = (float)s16 == 0.f ? 1.f : (float)s16;
            zpg[h][gq] = (float)z16;
        }
        bmp[ti] = bm[h];
        counts[ti] = cnt;
        u[h] = (cnt + (uint32_t)cap - 1u) / (uint32_t)cap;
        units[ti] = u[h];
    }
    uint32_t totA, totB;
    const uint32_t eA = wave_excl_scan(u[0], lane, totA);
    const uint32_t eB = wave_excl_scan(u[1], lane, totB);
    if (lane == 0) wave_total[wave] = totA + totB;
    __syncthreads();
    uint32_t in_group = 0, group_total = 0;
#pragma unroll
    for (int w = 0; w < W; w++) {
        const uint32_t t = wave_total[w];
        in_group += w < wave ? t : 0u;
        group_total += t;
    }
    if (threadIdx.x == 0) agent_store(state + g, kWordReady | group_total);
    {
        uint64_t lo = 0, hi = 0;
        const bool ok0 = wait_for_words<W>(state, 0, 0, g, wave, lane, spin_limit, lo, hi);
        if (lane == 0) {
            bases[wave][0] = hi;
            bases[wave][1] = ok0 ? 1ull : 0ull;
        }
    }
    __syncthreads();
    uint64_t before = in_group;
    bool ok = true;
#pragma unroll
    for (int w = 0; w < W; w++) {
        before += bases[w][0];
        ok = ok && bases[w][1] != 0ull;
    }
    if (!ok && threadIdx.x == 0) mark_gave_up(state + groups_total, total_words, nullptr);
    if (lane == 0 && unit == nunits - 1 && ok)
        atomicMax(reinterpret_cast<unsigned long long*>(total_words), before + totA + totB);
    const uint64_t off_h[2] = {before + eA, before + totA + eB};
    tile_off[tile0 + lane] = (uint32_t)off_h[0];
    tile_off[tile0 + 64 + lane] = (uint32_t)off_h[1];
    if (!ok) return;
#pragma unroll
    for (int h = 0; h < 2; h++) {  // unrolled: everything indexed by h stays in registers
        // the half back into the slab (the pruned elements are NaN there: the bitmap skips them)
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < 32; j++) slab[lane * kHalfRowDw + j] = r[32 * h + j];
        __builtin_amdgcn_wave_barrier();
        const uint64_t m = bm[h];
        const uint64_t off = off_h[h];
        const bool fits = off + u[h] <= capacity_words;  // a tile that would not fit is left untouched
        // Key tiles with many survivors - a channel of outliers keeps all of its 64 tokens - would make the whole
        // wavefront loop as often as they have elements; the few of them (at most kCoopMax, else none) are left to the
        // cooperative pass below, where the 64 lanes quantise the tile's 64 positions together.
        constexpr uint32_t kCoopOver = 48, kCoopMax = 8;
        uint64_t coop = 0;
        if (!IS_VALUE) {
            coop = __ballot(fits && (uint32_t)__popcll(m) > kCoopOver);
            if ((uint32_t)__popcll(coop) > kCoopMax) coop = 0;
        }
        if (fits && ((coop >> lane) & 1ull) == 0ull) {
            uint32_t cur = 0;
            int pos = 0;
            uint32_t w = 0;
            // the kept elements first to last; the coming element is read from LDS while the current one is quantised
            auto at = [&](int i) { return (float)sh[IS_VALUE ? (lane * (2 * kHalfRowDw) + i) : (i * (2 * kHalfRowDw) + lane)]; };
            uint64_t rem = m;
            int i = rem != 0ull ? __builtin_clzll(rem) : 0;
            float v = at(i);
            while (rem != 0ull) {
                rem &= ~(0x8000000000000000ull >> i);
                const int i_next = rem != 0ull ? __builtin_clzll(rem) : i;
                const float v_next = at(i_next);
                const float sc = (G32 && i >= 32) ? scg[h][NG - 1] : scg[h][0];   // the element's position picks the pair
                const float zp = (G32 && i >= 32) ? zpg[h][NG - 1] : zpg[h][0];
                float q = floorf(v / sc + 0.5f) + zp;
                q = fminf(fmaxf(q, 0.f), maxq);
                cur |= (uint32_t)q << pos;
                pos += bit;
                if (pos == 32) {
                    packed[off + w++] = cur;
                    cur = 0;
                    pos = 0;
                }
                v = v_next;
                i = i_next;
            }
            if (pos > 0) packed[off + w] = cur;
        }
        // cooperative pass: lane = token; the tile's bitmap, parameters and word offset come from its owner lane
        while (coop != 0ull) {
            const int c = __builtin_ctzll(coop);
            coop &= coop - 1ull;
            const uint64_t mc = u64_of((uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)m, c),
                                       (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(m >> 32), c));
            const uint64_t offc = u64_of((uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)off, c),
                                         (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(off >> 32), c));
            auto from_owner = [&](float x) {
                return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), c));
            };
            const float sc0 = from_owner(scg[h][0]), zp0 = from_owner(zpg[h][0]);
            const float sc1 = from_owner(scg[h][NG - 1]), zp1 = from_owner(zpg[h][NG - 1]);
            const float sc = (G32 && lane >= 32) ? sc1 : sc0, zp = (G32 && lane >= 32) ? zp1 : zp0;
            const uint64_t ml = lanes_of(mc);                    // bit i <=> token i
            const bool keep = ((ml >> lane) & 1ull) != 0ull;
            const float v = keep ? (float)sh[lane * (2 * kHalfRowDw) + c] : 0.f;
            float q = floorf(v / sc + 0.5f) + zp;
            q = fminf(fmaxf(q, 0.f), maxq);
            const uint32_t rank = rank_below(ml);
            const uint32_t word = rank / (uint32_t)cap, shift = (rank % (uint32_t)cap) * (uint32_t)bit;
            if (lane < 16) coop_words[wave][lane] = 0u;
            __builtin_amdgcn_wave_barrier();
            if (keep) atomicOr(&coop_words[wave][word], (uint32_t)q << shift);
            __builtin_amdgcn_wave_barrier();
            const uint32_t nwords = ((uint32_t)__popcll(mc) + (uint32_t)cap - 1u) / (uint32_t)cap;
            if ((uint32_t)lane < nwords) packed[offc + lane] = coop_words[wave][lane];
            __builtin_amdgcn_wave_barrier();
        }
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
    return 2 * round_up((size_t)B * (M / 64) * 4, 256) + round_up((size_t)B * 4 + 64, 256);  // also the one-pass status words
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
    // tile offsets are 32-bit word offsets into one buffer (the reference's format): the worst case has to fit
    if ((uint64_t)B * (uint64_t)M * (uint64_t)N / 64u * (uint64_t)(64 * bit / 32) > 0xFFFFFFFFull) return MSTF_EUNSUPPORTED;
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
    if (packed) {
        const int units_all = B * nblk;
        const int W = nblk % 4 == 0 ? 4 : (nblk % 2 == 0 ? 2 : 1);
        const int groups = units_all / W;
        uint64_t* state = reinterpret_cast<uint64_t*>(ws);
        const int words = groups + 1;
        const uint32_t spin_limit = onepass_spin_limit();
        hipLaunchKernelGGL(onepass_init_kernel, dim3((unsigned)((words + 255) / 256 < 256 ? (words + 255) / 256 : 256)),
                           dim3(256), 0, st, state, words, total_words, static_cast<uint64_t*>(nullptr));
        if ((rc = check_launch()) != MSTF_OK) return rc;
#define MSTF_QOP(WV)                                                                                                  \
    hipLaunchKernelGGL((quant_onepass_kernel<IS_VALUE, G32, WV>), dim3((unsigned)groups), dim3(64 * WV), 0, st, xh, M, kth, \
                       bit, bmp, counts, units, tile_off, reinterpret_cast<_Float16*>(scales),                          \
                       reinterpret_cast<_Float16*>(zeros), packed, cap_words, total_words, state, units_all, groups,    \
                       spin_limit)
        if (W == 4)
            MSTF_QOP(4);
        else if (W == 2)
            MSTF_QOP(2);
        else
            MSTF_QOP(1);
#undef MSTF_QOP
        return check_launch();
    }
    hipLaunchKernelGGL((quant_count_kernel<IS_VALUE, G32>), dim3((unsigned)(B * nblk)), dim3(64), 0, st, xh, M, kth, bit, bmp,
                       counts, units, tile_off, reinterpret_cast<_Float16*>(scales), reinterpret_cast<_Float16*>(zeros),
                       unit_tot);
    if ((rc = check_launch()) != MSTF_OK) return rc;
    hipLaunchKernelGGL(quant_scan_kernel, dim3((unsigned)B), dim3(256), (size_t)nblk * 4, st, unit_tot, unit_base,
                       head_base, total_words, nblk);
    if ((rc = check_launch()) != MSTF_OK) return rc;
    hipLaunchKernelGGL(quant_finalize_kernel, dim3((unsigned)((T + 255) / 256), (unsigned)B), dim3(256), 0, st, tile_off,
                       unit_base, head_base, nblk, T);
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
