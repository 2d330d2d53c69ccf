// Device helpers shared by the fp16 and the quantised compressors: the staging of one
// (KV head, 64-token block) unit through padded half-slabs in LDS, the per-row radix select and the tile bitmaps.
#pragma once
#include "common.hpp"

namespace mstf {

constexpr int kD = 128;                  // head_dim the slab layout is built for

// Half a slab: channels [64h, 64h+64) of the unit's 64 tokens.  Staging through half-slabs keeps the LDS of a
// wavefront at 8.25 KB (19 wavefronts per CU instead of 9), the rows themselves live in registers.
constexpr int kHalfRowDw = 32 + 1;             // dwords per LDS row: 32 of data + 1 of padding
constexpr int kHalfSlabDw = 64 * kHalfRowDw;   // 8448 bytes

typedef unsigned short us2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ us2_t as_us2(uint32_t x) { return __builtin_bit_cast(us2_t, x); }
__device__ __forceinline__ uint32_t us2_u32(us2_t x) { return __builtin_bit_cast(uint32_t, x); }

// Streams channels [64h, 64h+64) of rows [row0, row0+64) of an fp16 matrix with 128 channels per row and `stride`
// elements between rows (128: a plain [rows, 128] matrix) into the padded half-slab (rows >= rows_valid as
// zeros); afterwards lane = token reads its own 32 dwords with row_of_lane.
__device__ __forceinline__ void half_slab_load(const _Float16* x, int64_t row0, int64_t rows_valid, int h, uint32_t* slab,
                                               int lane, int64_t stride = kD)
{
    const _Float16* src = x + row0 * stride + h * 64;
    // all eight pieces are requested before the first one is staged: the loads are unconditional (a row past the
    // end reads the last valid row instead, row0 < rows_valid) and the zeros are put in afterwards
    uint4 v[8];
    const int64_t last = rows_valid - 1 - row0;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int e = j * 64 + lane;  // 16-byte piece index inside the half-slab: 8 pieces per row
        const int row = e >> 3, c16 = e & 7;
        const int64_t rr = row <= last ? row : last;
        v[j] = *reinterpret_cast<const uint4*>(src + rr * stride + c16 * 8);
    }
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int e = j * 64 + lane;
        const int row = e >> 3, c16 = e & 7;
        if (row > last) v[j] = make_uint4(0u, 0u, 0u, 0u);
        uint32_t* d = slab + row * kHalfRowDw + c16 * 4;
        d[0] = v[j].x;
        d[1] = v[j].y;
        d[2] = v[j].z;
        d[3] = v[j].w;
    }
}
// The 32 dwords (64 channels) of this lane's token out of the staged half-slab, into r[first .. first+32).
template <int N>
__device__ __forceinline__ void row_of_lane(const uint32_t* slab, int lane, uint32_t (&r)[N], int first)
{
#pragma unroll
    for (int j = 0; j < 32; j++) r[first + j] = slab[lane * kHalfRowDw + j];
}
// Both halves of the lane's row (raw fp16 pairs, signs included) through one half-slab buffer.
__device__ __forceinline__ void unit_rows(const _Float16* x, int64_t row0, int64_t rows_valid, uint32_t* slab, int lane,
                                          uint32_t (&r)[64], int64_t stride = kD)
{
#pragma unroll
    for (int h = 0; h < 2; h++) {
        half_slab_load(x, row0, rows_valid, h, slab, lane, stride);
        __builtin_amdgcn_wave_barrier();
        row_of_lane(slab, lane, r, 32 * h);
        __builtin_amdgcn_wave_barrier();
    }
}
// Rows that are not a contiguous [heads, rows, 128] matrix: element (batch entry bt, token t, KV head h, channel c)
// at x[bt * sb + t * st + h * sh + c].  A projection output [batch, tokens, heads * 128] has sb = tokens * heads * 128,
// st = heads * 128, sh = 128.  Heads are numbered b = bt * heads + h.
struct RowsView {
    const _Float16* x;
    int64_t sb, st, sh;
    int heads;
    __device__ __forceinline__ const _Float16* head(int b) const
    {
        const int bt = b / heads;
        return x + bt * sb + (b - bt * heads) * sh;
    }
};

// Rotary position embedding of 8 channels c .. c+7 < 64 of a row (x0) and their partners c+64 .. (x1), with the
// roundings of the half-precision expression (x * cos) + (rotate_half(x) * sin), rotate_half(x) = [-x[64:], x[:64]]:
// both products and the sum are rounded to fp16 one by one (no fused multiply-add).
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void rope_piece(const uint4& x0, const uint4& x1, const uint4& c0, const uint4& c1,
                                           const uint4& s0, const uint4& s1, uint4& o0, uint4& o1)
{
#pragma clang fp contract(off)
    const uint32_t X0[4] = {x0.x, x0.y, x0.z, x0.w}, X1[4] = {x1.x, x1.y, x1.z, x1.w};
    const uint32_t C0[4] = {c0.x, c0.y, c0.z, c0.w}, C1[4] = {c1.x, c1.y, c1.z, c1.w};
    const uint32_t S0[4] = {s0.x, s0.y, s0.z, s0.w}, S1[4] = {s1.x, s1.y, s1.z, s1.w};
    uint32_t O0[4], O1[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const h2_t a = __builtin_bit_cast(h2_t, X0[k]), b = __builtin_bit_cast(h2_t, X1[k]);
        const h2_t p1 = a * __builtin_bit_cast(h2_t, C0[k]);
        const h2_t p2 = (-b) * __builtin_bit_cast(h2_t, S0[k]);
        const h2_t p3 = b * __builtin_bit_cast(h2_t, C1[k]);
        const h2_t p4 = a * __builtin_bit_cast(h2_t, S1[k]);
        O0[k] = __builtin_bit_cast(uint32_t, (h2_t)(p1 + p2));
        O1[k] = __builtin_bit_cast(uint32_t, (h2_t)(p3 + p4));
    }
    o0 = make_uint4(O0[0], O0[1], O0[2], O0[3]);
    o1 = make_uint4(O1[0], O1[1], O1[2], O1[3]);
}

// The same in two steps, for a wavefront that requests its next unit while it works on the current one:
// unit_fetch leaves the 16 KB of a whole unit (64 full rows from row0, all valid) in the registers of the
// wavefront, unit_rows_from turns them into the lane's row.
struct UnitRaw {
    uint4 v[2][8];
};
__device__ __forceinline__ void unit_fetch(const _Float16* x, int64_t row0, int lane, UnitRaw& raw, int64_t stride = kD)
{
    // one wave-uniform base and a 32-bit byte offset per lane: the sixteen loads differ by constants
    const char* base = reinterpret_cast<const char*>(x + row0 * stride);
    const uint32_t row_bytes = (uint32_t)stride * 2u;
    const uint32_t lane_off = (uint32_t)(lane >> 3) * row_bytes + (uint32_t)(lane & 7) * 16u;
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int j = 0; j < 8; j++)
            raw.v[h][j] = *reinterpret_cast<const uint4*>(base + (lane_off + (uint32_t)j * 8u * row_bytes + (uint32_t)h * 128u));
    }
}
__device__ __forceinline__ void unit_rows_from(const UnitRaw& raw, uint32_t* slab, int lane, uint32_t (&r)[64])
{
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int e = j * 64 + lane;
            uint32_t* d = slab + (e >> 3) * kHalfRowDw + (e & 7) * 4;
            d[0] = raw.v[h][j].x;
            d[1] = raw.v[h][j].y;
            d[2] = raw.v[h][j].z;
            d[3] = raw.v[h][j].w;
        }
        __builtin_amdgcn_wave_barrier();
        row_of_lane(slab, lane, r, 32 * h);
        __builtin_amdgcn_wave_barrier();
    }
}

// (m & x) | (~m & y) as one instruction; m is wave-uniform.
__device__ __forceinline__ uint32_t bit_select(uint32_t m, uint32_t x, uint32_t y)
{
    uint32_t d;
    asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(d) : "s"(m), "v"(x), "v"(y));
    return d;
}

// 32x32 bit-matrix transpose in place on r[first .. first+32): afterwards bit i of r[first+p] is bit p of the old
// r[first+i].  Five butterfly stages of 16 exchanges: byte permutes for the distances 16 and 8 (2 instructions per
// pair), shift + bit select for 4, 2 and 1 (4 per pair) - 256 instructions.
template <int N>
__device__ __forceinline__ void bit_transpose32(uint32_t (&r)[N], int first)
{
#define MSTF_BT_PERM(J, SEL_LO, SEL_HI)                                   \
    _Pragma("unroll") for (int k = 0; k < 32; k++)                        \
    {                                                                     \
        if ((k & J) == 0) {                                               \
            const uint32_t a = r[first + k], b = r[first + k + J];        \
            r[first + k] = __builtin_amdgcn_perm(b, a, SEL_LO);           \
            r[first + k + J] = __builtin_amdgcn_perm(b, a, SEL_HI);       \
        }                                                                 \
    }                                                                     \
    __builtin_amdgcn_sched_barrier(0); /* stage by stage: interleaved stages would double the live registers */
#define MSTF_BT_STAGE(J, M)                                               \
    _Pragma("unroll") for (int k = 0; k < 32; k++)                        \
    {                                                                     \
        if ((k & J) == 0) {                                               \
            const uint32_t a = r[first + k], b = r[first + k + J];        \
            r[first + k] = bit_select(M, a, b << J);                      \
            r[first + k + J] = bit_select(M, a >> J, b);                  \
        }                                                                 \
    }                                                                     \
    __builtin_amdgcn_sched_barrier(0);
    MSTF_BT_PERM(16, 0x05040100u, 0x07060302u)   // [a0 a1 b0 b1], [a2 a3 b2 b3] (bytes, low first)
    MSTF_BT_PERM(8, 0x06020400u, 0x07030501u)    // [a0 b0 a2 b2], [a1 b1 a3 b3]
    MSTF_BT_STAGE(4, 0x0F0F0F0Fu)
    MSTF_BT_STAGE(2, 0x33333333u)
    MSTF_BT_STAGE(1, 0x55555555u)
#undef MSTF_BT_STAGE
#undef MSTF_BT_PERM
}

// kth-th smallest (1-based, 1 <= kth <= 128) of the 128 fp16 magnitudes of this lane's row; mag[j] holds two 15-bit
// magnitudes (channel 2j low, 2j+1 high).  The row is turned into bit planes (two 32x32 bit transposes: plane b of
// channels 2j is register b, of channels 2j+1 register 16+b, per half row), then the answer is fixed MSB-first on
// four 32-bit candidate masks: with c0 = #candidates whose bit is 0, the bit of the answer is 1 iff k > c0.  About
// 830 vector instructions against 1900 for a count per candidate value over the packed row.
// kept[w] (if wanted) = elements >= max(answer, 1): channel c sits in word 2*(c/64) + (c&1), bit (c%64)/2.
// The search of select_kth_planes on the bit planes p (see there).
template <bool WANT_KEPT>
__device__ __forceinline__ uint32_t search_planes(const uint32_t (&p)[64], int kth, uint32_t (&kept)[4])
{
    uint32_t alive[4] = {~0u, ~0u, ~0u, ~0u}, greater[4] = {0u, 0u, 0u, 0u};
    uint32_t k = (uint32_t)kth, thr = 0u;
#pragma unroll
    for (int b = 14; b >= 0; b--) {
        const uint32_t pl[4] = {p[b], p[16 + b], p[32 + b], p[48 + b]};
        uint32_t z[4], c0 = 0;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            z[w] = alive[w] & ~pl[w];
            c0 += (uint32_t)__builtin_popcount(z[w]);
        }
        const bool one = k > c0;  // fewer than k candidates have a 0 here: the answer has a 1
        k = one ? k - c0 : k;
        thr = one ? thr | (1u << b) : thr;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const uint32_t o = alive[w] ^ z[w];
            alive[w] = one ? o : z[w];
            if (WANT_KEPT) greater[w] |= one ? 0u : o;
        }
    }
    if (WANT_KEPT) {
#pragma unroll
        for (int w = 0; w < 4; w++) kept[w] = greater[w] | (thr ? alive[w] : 0u);
    }
    return thr;
}
template <bool WANT_KEPT>
__device__ __forceinline__ uint32_t select_kth_planes(const uint32_t (&mag)[64], int kth, uint32_t (&kept)[4])
{
    uint32_t p[64];
#pragma unroll
    for (int j = 0; j < 64; j++) p[j] = mag[j];
    bit_transpose32(p, 0);
    bit_transpose32(p, 32);
    return search_planes<WANT_KEPT>(p, kth, kept);
}

// The same for a wavefront that keeps only the first half of its rows in registers while it searches: after
// unit_rows_parked the second half of every row is still in the slab; it is read once for its bit planes and once
// more, into r[32 .. 64), when the search is over and the planes are dead - 32 registers fewer at the peak, which is
// what lets a kernel that holds a whole unit in registers run four wavefronts per SIMD instead of three.
__device__ __forceinline__ void unit_rows_parked(const UnitRaw& raw, uint32_t* slab, int lane, uint32_t (&r)[64])
{
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int e = j * 64 + lane;
            uint32_t* d = slab + (e >> 3) * kHalfRowDw + (e & 7) * 4;
            d[0] = raw.v[h][j].x;
            d[1] = raw.v[h][j].y;
            d[2] = raw.v[h][j].z;
            d[3] = raw.v[h][j].w;
        }
        __builtin_amdgcn_wave_barrier();
        if (h == 0) {
            row_of_lane(slab, lane, r, 0);
            __builtin_amdgcn_wave_barrier();
        }
    }
}
__device__ __forceinline__ void parked_rows_take(const uint32_t* slab, int lane, uint32_t (&r)[64])
{
    // (the compiler must neither reuse the values of an earlier read of the slab nor move this one up)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    row_of_lane(slab, lane, r, 32);
}
template <bool WANT_KEPT>
__device__ __forceinline__ uint32_t select_kth_planes_parked(uint32_t (&r)[64], const uint32_t* slab, int lane, int kth,
                                                             uint32_t (&kept)[4])
{
    uint32_t p[64];
#pragma unroll
    for (int j = 0; j < 32; j++) p[j] = r[j];
    bit_transpose32(p, 0);
    row_of_lane(slab, lane, p, 32);
    bit_transpose32(p, 32);
    const uint32_t thr = search_planes<WANT_KEPT>(p, kth, kept);
    asm volatile("" : "+v"(kept[0]), "+v"(kept[1]), "+v"(kept[2]), "+v"(kept[3]));  // the search ends here
    parked_rows_take(slab, lane, r);
    return thr;
}
__device__ __forceinline__ uint32_t select_kth(const uint32_t (&mag)[64], int kth)
{
    uint32_t unused[4];
    return select_kth_planes<false>(mag, kth, unused);
}

// bit i of the 16 low bits of x to bit 2i of the result
__device__ __forceinline__ uint32_t spread16(uint32_t x)
{
    x &= 0xFFFFu;
    x = (x | (x << 8)) & 0x00FF00FFu;
    x = (x | (x << 4)) & 0x0F0F0F0Fu;
    x = (x | (x << 2)) & 0x33333333u;
    x = (x | (x << 1)) & 0x55555555u;
    return x;
}
// MSB-first tile bitmap of 64 channels from the keep words of its even (e) and odd (o) channels
// (bit j = channel 2j resp. 2j+1, as select_kth_planes leaves them).
__device__ __forceinline__ uint64_t spread_bitmap(uint32_t e, uint32_t o)
{
    const uint32_t re = __builtin_bitreverse32(e), ro = __builtin_bitreverse32(o);  // bit 31-j = channel 2j (+1)
    const uint32_t lo = (spread16(re) << 1) | spread16(ro);
    const uint32_t hi = (spread16(re >> 16) << 1) | spread16(ro >> 16);
    return u64_of(lo, hi);
}

// One stage of the 64x64 bit-matrix transpose across the wavefront (lane = row, the 64 bits of (lo, hi) = columns):
// lanes l and l ^ D exchange the DxD blocks off the diagonal of every 2Dx2D block.  The partner's word comes through
// a swizzle (no vector-ALU slot), is rotated so that the wanted bits land on their new positions and merged in.
template <int D>
__device__ __forceinline__ void wave_bit_transpose_stage(uint32_t& lo, uint32_t& hi, int lane)
{
    constexpr uint32_t M0 = D == 16 ? 0x0000FFFFu : D == 8 ? 0x00FF00FFu : D == 4 ? 0x0F0F0F0Fu : D == 2 ? 0x33333333u : 0x55555555u;
    const bool up = (lane & D) != 0;
    const uint32_t keep = up ? ~M0 : M0;                       // the positions this lane keeps
    const uint32_t amt = up ? (uint32_t)D : (uint32_t)(32 - D);  // rotate right: down by D, or up by D
    const uint32_t pl = (uint32_t)__builtin_amdgcn_ds_swizzle((int)lo, 0x1F | (D << 10));
    const uint32_t ph = (uint32_t)__builtin_amdgcn_ds_swizzle((int)hi, 0x1F | (D << 10));
    const uint32_t rl = __builtin_amdgcn_alignbit(pl, pl, amt), rh = __builtin_amdgcn_alignbit(ph, ph, amt);
    lo = (lo & keep) | (rl & ~keep);
    hi = (hi & keep) | (rh & ~keep);
}
// Afterwards bit t of lane k's (lo, hi) is what bit k of lane t's was: 21 vector instructions, 10 swizzles and a
// handful of per-lane constants, against two instructions and two lane writes per column for ballots.
__device__ __forceinline__ void wave_bit_transpose64(uint32_t& lo, uint32_t& hi, int lane)
{
    typedef unsigned u2v_t __attribute__((ext_vector_type(2)));
    const u2v_t r = __builtin_amdgcn_permlane32_swap(lo, hi, false, false);  // lo of lanes 32.. <-> hi of lanes ..31
    lo = r[0];
    hi = r[1];
    wave_bit_transpose_stage<16>(lo, hi, lane);
    wave_bit_transpose_stage<8>(lo, hi, lane);
    wave_bit_transpose_stage<4>(lo, hi, lane);
    wave_bit_transpose_stage<2>(lo, hi, lane);
    wave_bit_transpose_stage<1>(lo, hi, lane);
}

// Key tile bitmaps (MSB-first, lane l: tiles l and 64 + l of the unit) from the keep words of the lanes' rows
// (kept[2h + p] bit j of lane t = channel 64h + 2j + p of token t is kept).
__device__ __forceinline__ void key_bitmaps_from_kept(const uint32_t (&kept)[4], int lane, uint64_t& bmA, uint64_t& bmB)
{
    // after the transpose lane k < 32 holds channel 2k of the half, lane 32 + k channel 2k + 1
    const int from = ((lane >> 1) + 32 * (lane & 1)) * 4;
    uint64_t bm[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        uint32_t lo = kept[2 * h], hi = kept[2 * h + 1];
        wave_bit_transpose64(lo, hi, lane);
        lo = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)lo);
        hi = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)hi);
        bm[h] = u64_of(__builtin_bitreverse32(hi), __builtin_bitreverse32(lo));  // token t -> bit 63 - t
    }
    bmA = bm[0];
    bmB = bm[1];
}

// Keep words of an already pruned row: every non-zero magnitude (layout of select_kth_planes' keep words).
__device__ __forceinline__ void kept_nonzero(const uint32_t (&r)[64], uint32_t (&kept)[4])
{
#pragma unroll
    for (int w = 0; w < 4; w++) kept[w] = 0u;
#pragma unroll
    for (int j = 0; j < 64; j++) {
        const uint32_t e = (r[j] & 0x7FFFu) != 0u ? 1u : 0u, o = (r[j] & 0x7FFF0000u) != 0u ? 1u : 0u;
        kept[2 * (j >> 5)] |= e << (j & 31);
        kept[2 * (j >> 5) + 1] |= o << (j & 31);
    }
}

__device__ __forceinline__ uint32_t wave_excl_scan(uint32_t v, int lane, uint32_t& total)
{
    uint32_t inc = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        uint32_t t = __shfl_up(inc, o, 64);
        if (lane >= o) inc += t;
    }
    total = __shfl(inc, 63, 64);
    return inc - v;
}

__device__ __forceinline__ uint32_t padded_units(uint64_t bm)
{
    return (uint32_t)((__popcll(bm) + 7) & ~7) >> 1;  // 4-byte units: nnz padded to 8 halfs
}


// dst with lane LANE (a constant) replaced by the wave-uniform value v.
__device__ __forceinline__ uint32_t write_lane(uint32_t v, int lane_const, uint32_t dst)
{
    asm("v_writelane_b32 %0, %1, %2" : "+v"(dst) : "s"(v), "n"(lane_const));
    return dst;
}

// Keep decision of one unit, as tile bitmaps (MSB-first).  Lane l returns the bitmaps of tiles
// l (bmA) and 64+l (bmB) of the unit:
//   key   : tile c = channel c over the 64 tokens        (ballot across lane = token)
//   value : tile (half, token) with lane = token         (packed inside the lane)
// mag[j] = magnitudes of channels 2j (low half) and 2j+1 (high half) of this lane's token;
// an element is kept when its magnitude is >= thr (thr >= 1, so zeros never are).
template <bool IS_VALUE>
__device__ __forceinline__ void unit_bitmaps(const uint32_t (&mag)[64], uint32_t thr, int lane, uint64_t& bmA,
                                             uint64_t& bmB)
{
    const us2_t t2 = as_us2(thr | (thr << 16));
    if (!IS_VALUE) {
        // one 16-bit compare per channel; the wave-wide result goes into the lane that owns the tile with two
        // v_writelane (the lane index is a compile-time constant)
        uint32_t aLo = 0u, aHi = 0u, bLo = 0u, bHi = 0u;
        const uint16_t t16 = (uint16_t)thr;
#pragma unroll
        for (int j = 0; j < 64; j++) {
            const uint64_t k0 = __builtin_bitreverse64(__ballot((uint16_t)mag[j] >= t16));
            const uint64_t k1 = __builtin_bitreverse64(__ballot((uint16_t)(mag[j] >> 16) >= t16));
            const int c0 = (2 * j) & 63, c1 = (2 * j + 1) & 63;
            if (j < 32) {
                aLo = write_lane((uint32_t)k0, c0, aLo);
                aHi = write_lane((uint32_t)(k0 >> 32), c0, aHi);
                aLo = write_lane((uint32_t)k1, c1, aLo);
                aHi = write_lane((uint32_t)(k1 >> 32), c1, aHi);
            } else {
                bLo = write_lane((uint32_t)k0, c0, bLo);
                bHi = write_lane((uint32_t)(k0 >> 32), c0, bHi);
                bLo = write_lane((uint32_t)k1, c1, bLo);
                bHi = write_lane((uint32_t)(k1 >> 32), c1, bHi);
            }
        }
        bmA = u64_of(aLo, aHi);
        bmB = u64_of(bLo, bHi);
    } else {
        uint32_t w[4] = {0u, 0u, 0u, 0u};  // [half0 hi, half0 lo, half1 hi, half1 lo]
#pragma unroll
        for (int j = 0; j < 64; j++) {
            const uint32_t d = us2_u32(as_us2(mag[j]) - t2);
            const uint32_t two = (((d >> 15) & 1u) << 1 | (d >> 31)) ^ 3u;  // [kept(2j), kept(2j+1)] MSB-first
            const int jj = j & 15;                                        // pair index inside a 32-channel word
            w[j >> 4] |= two << (30 - 2 * jj);
        }
        bmA = u64_of(w[1], w[0]);
        bmB = u64_of(w[3], w[2]);
    }
}

// Keep threshold of this lane's row from its magnitudes (kth == 0: input already pruned, keep the non-zeros).
__device__ __forceinline__ uint32_t threshold_of(const uint32_t (&mag)[64], int kth)
{
    uint32_t thr = 1u;
    if (kth > 0) {
        thr = select_kth(mag, kth);
        if (thr == 0u) thr = 1u;  // zeros are never stored
    }
    return thr;
}

// Threshold and tile bitmaps of one unit in one go (see unit_bitmaps for the meaning of bmA / bmB).  With pruning
// (kth > 0) the bitmaps come from the select's own keep masks, so the magnitudes are dead once the bit planes exist:
// value tiles spread the masks into channel order, key tiles transpose the lanes' masks across the wavefront.
// Returns the row's threshold: an element is kept <=> its magnitude is >= the returned value (>= 1: zeros never are).
template <bool IS_VALUE>
__device__ __forceinline__ uint32_t unit_keep(const uint32_t (&mag)[64], int kth, int lane, uint64_t& bmA, uint64_t& bmB)
{
    if (kth > 0) {
        uint32_t kept[4];
        const uint32_t thr = select_kth_planes<true>(mag, kth, kept);
        if (IS_VALUE) {
            bmA = spread_bitmap(kept[0], kept[1]);
            bmB = spread_bitmap(kept[2], kept[3]);
        } else {
            key_bitmaps_from_kept(kept, lane, bmA, bmB);
        }
        return thr == 0u ? 1u : thr;
    }
    unit_bitmaps<IS_VALUE>(mag, 1u, lane, bmA, bmB);
    return 1u;
}

// Exclusive scan of one head's unit totals (grid.x = head, 256 threads) into LDS `base`
// (nblk entries); returns the head total to every thread.
__device__ __forceinline__ uint32_t units_scan(const uint32_t* ut, uint32_t* base, int nblk)
{
    __shared__ uint32_t carry_sh[4];
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint32_t carry = 0;
    for (int s = 0; s < nblk; s += 256) {
        const int i = s + tid;
        const uint32_t v = i < nblk ? ut[i] : 0u;
        uint32_t wtot;
        const uint32_t e = wave_excl_scan(v, lane, wtot);
        __syncthreads();
        if (lane == 0) carry_sh[wave] = wtot;
        __syncthreads();
        uint32_t pre = carry;
        for (int w = 0; w < wave; w++) pre += carry_sh[w];
        if (i < nblk) base[i] = pre + e;
        carry += carry_sh[0] + carry_sh[1] + carry_sh[2] + carry_sh[3];
    }
    __syncthreads();
    return carry;
}

// Sum of the `before` words in front of a head's unit totals, over one workgroup of 256 threads (16-byte loads,
// four in flight per thread; ut is 256-byte aligned); the result is valid in thread 0.  Every workgroup re-reads
// at most B * nblk small numbers, which spares a launch for the scan over heads.
__device__ __forceinline__ uint64_t sum_before(const uint32_t* ut, size_t before)
{
    __shared__ uint64_t wsum[4];
    const int tid = (int)threadIdx.x;
    uint64_t mine = 0;
    const uint4* ut4 = reinterpret_cast<const uint4*>(ut);
    const size_t n4 = before / 4;
    for (size_t i = tid; i < n4; i += 1024) {
        uint4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) v[u] = i + 256 * u < n4 ? ut4[i + 256 * u] : make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
        for (int u = 0; u < 4; u++) mine += (uint64_t)v[u].x + v[u].y + v[u].z + v[u].w;
    }
    if (tid < (int)(before - 4 * n4)) mine += ut[4 * n4 + tid];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mine += __shfl_xor(mine, o, 64);
    if ((tid & 63) == 0) wsum[tid >> 6] = mine;
    __syncthreads();
    return wsum[0] + wsum[1] + wsum[2] + wsum[3];
}

// ------------------------------------------------------------------------------- one-pass ordering
// Status words of the one-pass producers (compress.hip describes the protocol): cleared by onepass_init_kernel,
// one word per workgroup = bit 63 | total, published with an agent-scope store, polled by the workgroups behind.
constexpr uint32_t kSpinLimit = 1u << 20;  // the default of onepass_spin_limit() (runtime.hip)
// The limit the launchers pass: kSpinLimit unless mstf_test_set_spin_limit (runtime.hip) lowered it - a test's way
// to force the give-up path from the host while every kernel still exits normally.  The environment has no say.
uint32_t onepass_spin_limit();

// Clears the status words and the caller's total (nullable): the kernel raises the total with atomic maxima - the
// last workgroup to the sum, a workgroup that gave up to all ones - so whichever comes last, a give-up stays visible.
static __global__ __launch_bounds__(256) void onepass_init_kernel(uint64_t* __restrict__ state, int n,
                                                                  uint64_t* __restrict__ total,
                                                                  uint64_t* __restrict__ total2 = nullptr)
{
    for (int i = (int)(blockIdx.x * 256 + threadIdx.x); i < n; i += (int)(gridDim.x * 256)) state[i] = 0ull;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        if (total) *total = 0ull;
        if (total2) *total2 = 0ull;
    }
}
// The marker of a workgroup whose wait ran out, from one thread: the flag word behind the status words, all ones in
// the caller's total (compress contract) or bit 1 of the caller's sticky flag (append contract).
constexpr uint32_t kFlagOverflow = 1u, kFlagGaveUp = 2u;
__device__ __forceinline__ void mark_gave_up(uint64_t* flag_word, uint64_t* total, uint32_t* sticky)
{
    __hip_atomic_store(flag_word, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (total) atomicMax(reinterpret_cast<unsigned long long*>(total), ~0ull);
    if (sticky) atomicOr(sticky, kFlagGaveUp);
}

__device__ __forceinline__ uint64_t agent_load(const uint64_t* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void agent_store(uint64_t* p, uint64_t v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t wave_sum_u64(uint64_t v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
constexpr uint64_t kWordReady = 1ull << 63;

// This wavefront's share of the wait for state[first .. g): the windows of 64 words number `wave`, wave + W, ...,
// four of them in flight at a time.  Returns its part of the sums over [first, split) and [split, g)
// (first <= split <= g); false when a wait ran out.
template <int W>
__device__ __forceinline__ bool wait_for_words(const uint64_t* state, int first, int split, int g, int wave, int lane,
                                               uint32_t spin_limit, uint64_t& sum_lo, uint64_t& sum_hi)
{
    constexpr int K = 4;
    uint64_t lo = 0, hi = 0;
    uint32_t polls = 0;
    bool ok = true;
    for (int w0 = first + wave * 64; w0 < g && ok; w0 += 64 * W * K) {
        uint64_t v[K];
        bool got[K];
#pragma unroll
        for (int k = 0; k < K; k++) {
            v[k] = 0ull;
            got[k] = w0 + k * 64 * W + lane >= g;
        }
        for (;;) {
            bool all = true;
#pragma unroll
            for (int k = 0; k < K; k++)
                if (!got[k]) v[k] = agent_load(state + w0 + k * 64 * W + lane);
#pragma unroll
            for (int k = 0; k < K; k++) {
                got[k] = got[k] || (v[k] >> 63) != 0ull;
                all = all && got[k];
            }
            if (__ballot(!all) == 0ull) break;
            if (++polls > spin_limit) {
                ok = false;
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
#pragma unroll
        for (int k = 0; k < K; k++) {
            const int i = w0 + k * 64 * W + lane;
            const uint64_t t = v[k] & ~kWordReady;
            lo += i < split ? t : 0ull;
            hi += i >= split && i < g ? t : 0ull;
        }
    }
    sum_lo = wave_sum_u64(lo);
    sum_hi = wave_sum_u64(hi);
    return ok;
}


}  // namespace mstf
