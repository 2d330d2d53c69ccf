// Per-token magnitude pruning fused with the bitmap compressor (fp16 format).
//
// Work unit = one (KV head, 64-token block): a 64 x 128 fp16 slab (16 KB, contiguous in x),
// i.e. exactly 128 tiles of either format, whose packed values are contiguous in the output.
// One wavefront owns a unit, lane = token.  The slab goes through LDS in two halves of 64 channels
// (padded row stride, so that a lane reads its own row without bank conflicts) into registers: a lane
// holds the 128 values of its token in 64 registers and the wavefront needs 8.25 KB of LDS.
//
//   one-pass kernel: everything with one read of the slab (the calls that produce the packed values): row threshold
//                    by a 15-step radix select on bit planes, bitmaps, padded counts, compaction into an LDS
//                    image, and the unit's place in the output from the totals that the workgroups in front of it
//                    publish in the workspace.
// The two-pass form remains for the sizing-only call, for phase 2 on its own and for the projection layout:
//   count kernel   : threshold, bitmaps by ballot (key) or in-lane packing (value), padded counts and their prefix
//                    inside the unit.
//   scan kernel    : unit totals -> unit bases per head and, summed over the earlier heads, nz_off.
//   scatter kernel : re-reads the slab and compacts the survivors, half a unit (64 tiles) at a time,
//                    into an LDS image of the output that reuses the staging buffer - key: one
//                    rank-addressed 2-byte write per tile straight from the registers; value: every lane
//                    walks the 64 channels of its own tile - and streams the image out with 16-byte stores.
//                    In the fused call it also turns the unit-local tile offsets in idx into final ones.
#include "compress_common.hpp"

namespace mstf {

// ------------------------------------------------------------------------------- count
// grid = ceil(units / upw) with units = B * M/64, 64 threads: the wavefront owns upw consecutive units and has
// the rows of the coming one in flight while it selects and packs the current one.  Writes bmp, unit-local
// exclusive offsets into idx[b][t] and the unit total into unit_tot[b][tokblk].
template <bool IS_VALUE>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2))) void compress_count_kernel(const _Float16* __restrict__ x, int M, int kth,
                                                            uint64_t* __restrict__ bmp, uint32_t* __restrict__ idx,
                                                            uint32_t* __restrict__ unit_tot, int units, int upw)
{
    __shared__ uint32_t slab[kHalfSlabDw];
    const int lane = lane_id();
    const int nblk = M / 64;
    const size_t T = (size_t)M * kD / 64;
    const int unit0 = (int)blockIdx.x * upw;
    int n = units - unit0;
    n = n > upw ? upw : n;
    UnitRaw raw;
    unit_fetch(x, (int64_t)unit0 * 64, lane, raw);  // units are contiguous: unit u = rows [64u, 64u + 64) of [B*M, 128]
#pragma unroll 1
    for (int u = 0; u < n; u++) {
        const int unit = unit0 + u;
        const int b = unit / nblk, tb = unit - b * nblk;
        uint32_t mag[64];
        unit_rows_from(raw, slab, lane, mag);
        if (u + 1 < n) unit_fetch(x, (int64_t)(unit + 1) * 64, lane, raw);
#pragma unroll
        for (int j = 0; j < 64; j++) mag[j] &= 0x7FFF7FFFu;
        uint64_t bmA, bmB;  // tiles tb*128 + lane and tb*128 + 64 + lane
        unit_keep<IS_VALUE>(mag, kth, lane, bmA, bmB);
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
}

// Rows in the layout of a projection output (RowsView), optionally with the rotary embedding applied first: a unit
// rotates its rows on the way in - in the layout of the loads, where a lane holds 8 channels of a row and their
// partners 64 channels on, so that x, cos, sin and the rotated rows all move as 128-byte runs - and writes them to
// rot (same kind of layout; rot.x may be the input itself).  The units below M / 64 do so inside the one-pass
// kernel, the tokens behind them in rope_tail_kernel.
// cos / sin: [batch entry][token][128] fp16 with strides rb, rt.
struct RopeTables {
    const _Float16* cos;
    const _Float16* sin;
    int64_t rb, rt;
};
__device__ __forceinline__ void unit_fetch_rotated(const RowsView& src, const RopeTables& rope, const RowsView& rot, int b,
                                                   int tb, int rows, int lane, UnitRaw& raw)
{
    const int bt = b / src.heads;
    const _Float16* xb = src.head(b);
    _Float16* rb = const_cast<_Float16*>(rot.head(b));
    const _Float16* cb = rope.cos + bt * rope.rb;
    const _Float16* sb = rope.sin + bt * rope.rb;
    // four pieces at a time: all 24 loads of a batch are requested before the first one is used (loads behind a
    // per-piece branch would each wait for the one before); a row past the end reads the last row instead and is
    // neither rotated into the output nor stored
#pragma unroll
    for (int j0 = 0; j0 < 8; j0 += 4) {
        uint4 x0[4], x1[4], c0[4], c1[4], s0[4], s1[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int e = (j0 + k) * 64 + lane;
            int64_t t = (int64_t)tb * 64 + (e >> 3);
            t = t < rows ? t : rows - 1;
            const int c = (e & 7) * 8;
            const _Float16* xp = xb + t * src.st + c;
            const _Float16* cp = cb + t * rope.rt + c;
            const _Float16* sp = sb + t * rope.rt + c;
            x0[k] = *reinterpret_cast<const uint4*>(xp);
            x1[k] = *reinterpret_cast<const uint4*>(xp + 64);
            c0[k] = *reinterpret_cast<const uint4*>(cp);
            c1[k] = *reinterpret_cast<const uint4*>(cp + 64);
            s0[k] = *reinterpret_cast<const uint4*>(sp);
            s1[k] = *reinterpret_cast<const uint4*>(sp + 64);
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int j = j0 + k;
            const int e = j * 64 + lane;
            const int64_t t = (int64_t)tb * 64 + (e >> 3);
            const int c = (e & 7) * 8;
            rope_piece(x0[k], x1[k], c0[k], c1[k], s0[k], s1[k], raw.v[0][j], raw.v[1][j]);
            if (t < rows) {
                _Float16* rp = rb + t * rot.st + c;
                *reinterpret_cast<uint4*>(rp) = raw.v[0][j];
                *reinterpret_cast<uint4*>(rp + 64) = raw.v[1][j];
            } else {
                raw.v[0][j] = make_uint4(0u, 0u, 0u, 0u);
                raw.v[1][j] = make_uint4(0u, 0u, 0u, 0u);
            }
        }
    }
}
// grid = B * tail units (64 tokens each), 64 threads: rotation only, for the tokens behind the compressed ones
// (first_block = M / 64 onwards) of every head.
__global__ __launch_bounds__(64) void rope_tail_kernel(RowsView src, RopeTables rope, RowsView rot, int rows,
                                                       int first_block, int tail_blocks)
{
    const int b = (int)blockIdx.x / tail_blocks;
    const int tb = first_block + (int)blockIdx.x % tail_blocks;
    UnitRaw raw;
    unit_fetch_rotated(src, rope, rot, b, tb, rows, lane_id(), raw);
}

// ------------------------------------------------------------------------------- scans
// grid = B, 256 threads: exclusive scan of the head's unit totals into unit_base, idx[b][T] = head total.
// With nz_off given (the compress entry points) the workgroup also adds up the unit totals of all earlier heads
// (sum_before): nz_off[b] = that sum / 4 (16-byte units), and the last head's workgroup writes the grand total in
// fp16 values.
__global__ __launch_bounds__(256) void scan_units_kernel(const uint32_t* __restrict__ unit_tot,
                                                         uint32_t* __restrict__ unit_base, uint32_t* __restrict__ idx,
                                                         uint32_t* __restrict__ nz_off,
                                                         uint64_t* __restrict__ total_halfs, int nblk,
                                                         int tiles_per_unit)
{
    extern __shared__ uint32_t base[];  // nblk entries
    const int b = (int)blockIdx.x;
    const int tid = (int)threadIdx.x;
    const uint32_t total = units_scan(unit_tot + (size_t)b * nblk, base, nblk);
    for (int i = tid; i < nblk; i += 256) unit_base[(size_t)b * nblk + i] = base[i];
    if (tid == 0) idx[(size_t)b * ((size_t)nblk * tiles_per_unit + 1) + (size_t)nblk * tiles_per_unit] = total;
    if (nz_off) {
        const uint64_t pre = sum_before(unit_tot, (size_t)b * nblk);
        if (tid == 0) {
            nz_off[b] = (uint32_t)(pre >> 2);
            if (b == (int)gridDim.x - 1) *total_halfs = 2ull * (pre + total);
        }
    }
}

// grid = (T / 256, B): idx[b][t] += base of its unit (only when no scatter follows, which does it itself).
__global__ __launch_bounds__(256) void finalize_idx_kernel(uint32_t* __restrict__ idx,
                                                           const uint32_t* __restrict__ unit_base, int nblk,
                                                           int tiles_per_unit)
{
    const int b = (int)blockIdx.y;
    const size_t T = (size_t)nblk * tiles_per_unit;
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (t < T) idx[(size_t)b * (T + 1) + t] += unit_base[(size_t)b * nblk + t / tiles_per_unit];
}

// Compacts half a unit (64 tiles) into the LDS image at `img` and streams it to dst.
//   v      : this lane's token, channels 64h .. 64h+63 (raw fp16 pairs)
//   bm_l   : bitmap of tile 64h + lane;  ix_l: its final offset (4-byte units);  s_h: offset of the half's first tile
//   bytes  : packed size of the half;  dump: LDS address that takes the writes of the lanes that keep nothing
template <bool IS_VALUE>
__device__ __forceinline__ void scatter_half(const uint32_t (&v)[32], uint64_t bm_l, uint32_t ix_l, uint32_t s_h,
                                             uint32_t bytes, uint32_t img, uint32_t dump, char* dst, int lane)
{
    for (uint32_t o = (uint32_t)lane * 16u; o < bytes; o += 1024u)
        *(MSTF_LDS u32x4_t*)(uintptr_t)(img + o) = u32x4_t{0u, 0u, 0u, 0u};  // the padding stays +0.0
    if (!IS_VALUE) {
        // tile c = channel 64h + c over the 64 tokens: lane = token writes its element at the tile's rank
#pragma unroll
        for (int c = 0; c < 64; c++) {
            const uint64_t m = lanes_of(u64_of(__builtin_amdgcn_readlane((uint32_t)bm_l, c),
                                               __builtin_amdgcn_readlane((uint32_t)(bm_l >> 32), c)));
            const uint32_t off = img + (__builtin_amdgcn_readlane(ix_l, c) - s_h) * 4u;
            const uint32_t a = select_lane(m, rank_below(m) * 2u + off, dump);
            const uint32_t w = v[c >> 1];
            *(MSTF_LDS uint16_t*)(uintptr_t)a = (uint16_t)((c & 1) ? (w >> 16) : w);
        }
    } else {
        // tile (h, token = lane): the lane walks its own 64 channels, MSB of the bitmap first
        uint32_t a = img + (ix_l - s_h) * 4u;
        const uint32_t hi = (uint32_t)(bm_l >> 32), lo = (uint32_t)bm_l;
#pragma unroll
        for (int i = 0; i < 64; i++) {
            const uint32_t word = i < 32 ? hi : lo;
            const int32_t keep = (int32_t)(word << (i & 31)) >> 31;  // -1 when channel i is kept
            const uint32_t w = v[i >> 1];
            *(MSTF_LDS uint16_t*)(uintptr_t)((a & (uint32_t)keep) | (dump & ~(uint32_t)keep)) =
                (uint16_t)((i & 1) ? (w >> 16) : w);
            a -= 2 * keep;
        }
    }
    __builtin_amdgcn_wave_barrier();
    for (uint32_t o = (uint32_t)lane * 16u; o < bytes; o += 1024u)
        *reinterpret_cast<u32x4_t*>(dst + o) = *(MSTF_LDS const u32x4_t*)(uintptr_t)(img + o);
    __builtin_amdgcn_wave_barrier();
}

// ------------------------------------------------------------------------------- scatter
// grid = B * M/64 units, 64 threads.  bmp and nz_off are final; idx is final (ADD_BASE false) or still holds
// the unit-local offsets of the count kernel, which are completed here with unit_base (ADD_BASE true).
// head_limit (nullable): end of head b's slab in 16-byte units from nz; a unit whose values would pass it is
// skipped and *overflow is set.
template <bool IS_VALUE, bool ADD_BASE>
__global__ __launch_bounds__(64) void compress_scatter_kernel(const _Float16* __restrict__ x, int M,
                                                              const uint64_t* __restrict__ bmp, uint32_t* idx,
                                                              const uint32_t* __restrict__ unit_base,
                                                              const uint32_t* __restrict__ nz_off,
                                                              char* __restrict__ nz, uint64_t nz_capacity_halfs,
                                                              const uint32_t* __restrict__ head_limit,
                                                              uint32_t* __restrict__ overflow)
{
    // staging buffer of a half-slab, then image of that half's output (at most 64 tiles x 128 bytes);
    // the dword behind the image takes the writes of the lanes that keep nothing
    __shared__ __attribute__((aligned(16))) uint32_t buf[kHalfSlabDw];
    static_assert(kHalfSlabDw * 4 >= 64 * 128 + 4, "image and dump slot fit the staging buffer");
    const int lane = lane_id();
    const int nblk = M / 64;
    const int unit = (int)blockIdx.x;
    const int b = unit / nblk, tb = unit - b * nblk;
    const size_t T = (size_t)M * kD / 64;
    const uint64_t* bmu = bmp + (size_t)b * T + (size_t)tb * kD;
    uint32_t* ixu = idx + (size_t)b * (T + 1) + (size_t)tb * kD;
    // lane l holds the bitmap and the final offset of tiles l and 64 + l
    const uint64_t bmA = bmu[lane], bmB = bmu[64 + lane];
    uint32_t iA = ixu[lane], iB = ixu[64 + lane];
    uint32_t end;
    if (ADD_BASE) {
        const uint32_t base = unit_base[(size_t)b * nblk + tb];
        iA += base;
        iB += base;
        ixu[lane] = iA;
        ixu[64 + lane] = iB;
        const uint32_t last = __builtin_amdgcn_readlane(iB, 63);
        end = last + padded_units(u64_of(__builtin_amdgcn_readlane((uint32_t)bmB, 63),
                                         __builtin_amdgcn_readlane((uint32_t)(bmB >> 32), 63)));
    } else {
        end = ixu[kD];
    }
    const uint32_t start = __builtin_amdgcn_readlane(iA, 0);
    const uint32_t mid = __builtin_amdgcn_readlane(iB, 0);
    const uint64_t head_half0 = 8ull * nz_off[b];
    if (head_half0 + 2ull * end > nz_capacity_halfs) return;  // would not fit: leave untouched (uniform)
    if (head_limit && head_half0 + 2ull * end > 8ull * head_limit[b]) {
        // the head's values would run past the end of its slab: nothing of this unit is written, the caller is told
        if (lane == 0) atomicOr(overflow, 1u);
        return;
    }

    const uint32_t img = lds_addr(buf);
    const uint32_t dump = img + 64u * 128u;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const uint32_t s_h = h == 0 ? start : mid;
        uint32_t bytes = ((h == 0 ? mid : end) - s_h) * 4u;
        if (bytes > 64u * 128u) bytes = 64u * 128u;  // never true for offsets that follow from the bitmaps
        uint32_t v[32];
        half_slab_load(x + (size_t)b * M * kD, (int64_t)tb * 64, (int64_t)M, h, buf, lane);
        __builtin_amdgcn_wave_barrier();
        row_of_lane(buf, lane, v, 0);
        __builtin_amdgcn_wave_barrier();
        scatter_half<IS_VALUE>(v, h == 0 ? bmA : bmB, h == 0 ? iA : iB, s_h, bytes, img, dump,
                               nz + (head_half0 + 2ull * s_h) * 2ull, lane);
        __builtin_amdgcn_wave_barrier();
    }
}

// ------------------------------------------------------------------------------- one pass
// Pruning + compression with a single read of the input, for the calls that produce the packed values: a wavefront
// owns the unit of its workgroup index, selects, builds bitmaps and padded counts, publishes the unit's total,
// compacts the first half of the unit into an LDS image while the units in front of it publish theirs, learns where
// its values start from a decoupled look-back, and streams the two halves out of the rows it still holds in registers.
// While the threshold is searched only the first half of the lane's row is in registers - the second half waits in
// the staging buffer (unit_rows_parked, select_kth_planes_parked) - which keeps the kernel at four wavefronts per
// SIMD; compress_onepass_kv_kernel runs the keys and the values of the same tokens as one grid over this same body.
//
// A workgroup of W wavefronts owns W consecutive units (W divides the units of a head), adds up their totals in LDS
// and publishes one 64-bit word state[g] = bit 63 | total of workgroup g (4-byte units) with an agent-scope store.
// Its first wavefront then polls the words of the workgroups in front of it - all of them in the packed layout, where
// a head's values start behind those of all earlier heads; those of its own head in the pooled layout - 64 per round
// trip, until every word is set, and adds them up; the others wait at the barrier.
// A workgroup publishes its total before it waits for anything and waits only for workgroups of a lower index, which
// the dispatcher has started before it: every wait ends.  The waits are bounded all the same (kSpinLimit polls); a
// workgroup that gives up writes no values and marks the call itself (mark_gave_up): the flag word behind the
// workgroup words, *total_halfs raised to all ones (packed layout: the last workgroup raises it to the sum with the
// same atomic maximum, so the order of the two does not matter) and bit 1 of *overflow (pooled layout).
// onepass_init_kernel clears the words and *total_halfs before the launch.
// Compacts half h of a unit into the LDS image at img (tile offsets relative to the half's first tile).
//   r     : this lane's token, raw fp16 pairs;  kept: its keep words (see select_kth_planes)
//   key   : tile c = channel 64h + c over the 64 tokens - the lanes that keep the channel write at the tile's running
//           offset plus their rank among the keepers; the keepers of a channel are the carry of doubling the
//           bit-reversed keep word (one instruction pops the next channel of all 64 tokens)
//   value : tile = this lane's token - the lane appends its kept channels at its own tile's offset own4 (4-byte units)
template <bool IS_VALUE>
__device__ __forceinline__ void compact_half(const uint32_t (&r)[64], const uint32_t (&kept)[4], int h, uint32_t own4,
                                             uint32_t bytes, uint32_t img, int lane)
{
    for (uint32_t o = (uint32_t)lane * 16u; o < bytes; o += 1024u)
        *(MSTF_LDS u32x4_t*)(uintptr_t)(img + o) = u32x4_t{0u, 0u, 0u, 0u};  // the padding stays +0.0
    uint32_t we = __builtin_bitreverse32(kept[2 * h]), wo = __builtin_bitreverse32(kept[2 * h + 1]);
    const uint64_t all = __builtin_amdgcn_read_exec();  // every statement hands exec back as it found it
    uint64_t m1;
    if (!IS_VALUE) {
        const uint32_t voff = img + own4 * 4u;  // lane c: where tile c of the half starts in the image
        uint32_t t, o0, o1;
        // two channels per statement: doubling pops the channels' keep bits of every token into vcc and a scalar
        // pair, the tiles' offsets come out of lanes c and c + 1, then the keepers of each channel write at the
        // tile's offset plus twice their rank among the keepers
#pragma unroll
        for (int c = 0; c < 64; c += 2) {
            asm volatile("v_add_co_u32 %[we], vcc, %[we], %[we]\n\t"
                         "v_add_co_u32 %[wo], %[m1], %[wo], %[wo]\n\t"
                         "v_readlane_b32 %[o0], %[voff], %[c0]\n\t"
                         "v_readlane_b32 %[o1], %[voff], %[c1]\n\t"
                         "s_mov_b64 exec, vcc\n\t"
                         "v_mbcnt_lo_u32_b32 %[t], exec_lo, 0\n\t"
                         "v_mbcnt_hi_u32_b32 %[t], exec_hi, %[t]\n\t"
                         "v_lshl_add_u32 %[t], %[t], 1, %[o0]\n\t"
                         "ds_write_b16 %[t], %[v]\n\t"
                         "s_mov_b64 exec, %[m1]\n\t"
                         "v_mbcnt_lo_u32_b32 %[t], exec_lo, 0\n\t"
                         "v_mbcnt_hi_u32_b32 %[t], exec_hi, %[t]\n\t"
                         "v_lshl_add_u32 %[t], %[t], 1, %[o1]\n\t"
                         "ds_write_b16_d16_hi %[t], %[v]\n\t"
                         "s_mov_b64 exec, %[all]"
                         : [we] "+v"(we), [wo] "+v"(wo), [t] "=&v"(t), [m1] "=&s"(m1), [o0] "=&s"(o0), [o1] "=&s"(o1)
                         : [v] "v"(r[32 * h + (c >> 1)]), [voff] "v"(voff), [c0] "n"(c), [c1] "n"(c + 1), [all] "s"(all)
                         : "vcc", "memory");
        }
    } else {
        uint32_t a = img + own4 * 4u;
#pragma unroll
        for (int c = 0; c < 64; c += 2) {
            asm volatile("v_add_co_u32 %[we], vcc, %[we], %[we]\n\t"
                         "v_add_co_u32 %[wo], %[m1], %[wo], %[wo]\n\t"
                         "s_mov_b64 exec, vcc\n\t"
                         "ds_write_b16 %[a], %[v]\n\t"
                         "v_add_u32 %[a], 2, %[a]\n\t"
                         "s_mov_b64 exec, %[m1]\n\t"
                         "ds_write_b16_d16_hi %[a], %[v]\n\t"
                         "v_add_u32 %[a], 2, %[a]\n\t"
                         "s_mov_b64 exec, %[all]"
                         : [we] "+v"(we), [wo] "+v"(wo), [a] "+v"(a), [m1] "=&s"(m1)
                         : [v] "v"(r[32 * h + (c >> 1)]), [all] "s"(all)
                         : "vcc", "memory");
        }
    }
    __builtin_amdgcn_wave_barrier();
}
__device__ __forceinline__ void stream_image(uint32_t img, uint32_t bytes, char* dst, int lane)
{
    for (uint32_t o = (uint32_t)lane * 16u; o < bytes; o += 1024u)
        *reinterpret_cast<u32x4_t*>(dst + o) = *(MSTF_LDS const u32x4_t*)(uintptr_t)(img + o);
    __builtin_amdgcn_wave_barrier();
}

// grid = ceil(units / W) workgroups of W wavefronts, units = B * M/64, W divides M/64.
//   packed layout  (dst_off == nullptr): heads back to back, nz_off[b] and *total_halfs are written here;
//   pooled layout  (dst_off given): head b's values start at nz + 16 * dst_off[b] and may not pass
//                  nz + 16 * dst_limit[b] (else *overflow is set and the unit's values are not written).
// SRC: where the rows come from - kSrcMatrix: the contiguous [B, M, 128] matrix x; kSrcView: through `view` (the
// layout of a projection output); kSrcRope: through `view`, rotated on the way in and written to `rot`.
enum { kSrcMatrix = 0, kSrcView = 1, kSrcRope = 2 };
struct ProjArgs {
    RowsView view;
    RopeTables rope;
    RowsView rot;
    int rows;
};
// (0: the whole row in registers during the search - three wavefronts per SIMD; kept for A/B builds)
#ifndef MSTF_COMPRESS_PARK
#define MSTF_COMPRESS_PARK 1
#endif
// The LDS of a workgroup of the one-pass kernels.
template <int W>
struct OnepassLds {
    // per wavefront: staging buffer of a half-slab, then image of half a unit's output (at most 64 tiles x 128 bytes)
    uint32_t bufs[W][kHalfSlabDw] __attribute__((aligned(16)));
    uint32_t wave_total[W];
    uint64_t bases[W][3];  // per wavefront: its part of the sum over the earlier heads, of the sum over the head's
                           // earlier workgroups, and whether its waits ended
};
static_assert(kHalfSlabDw * 4 >= 64 * 128, "the image fits the staging buffer");

// The work of workgroup g of a one-pass launch over one side (keys or values).
template <bool IS_VALUE, int W, int SRC>
__device__ __forceinline__ void onepass_workgroup(
    OnepassLds<W>& lds, int g, const _Float16* __restrict__ x, const ProjArgs& proj, int M, int kth,
    uint64_t* __restrict__ bmp, uint32_t* __restrict__ idx, uint32_t* __restrict__ nz_off,
    uint64_t* __restrict__ total_halfs, const uint32_t* __restrict__ dst_off, const uint32_t* __restrict__ dst_limit,
    uint32_t* __restrict__ overflow, char* __restrict__ nz, uint64_t nz_capacity_halfs, uint64_t* state, int units,
    int groups_total, uint32_t spin_limit)
{
    auto& bufs = lds.bufs;
    auto& wave_total = lds.wave_total;
    auto& bases = lds.bases;
    const int lane = lane_id();
    const int wave = wave_id();
    const int nblk = M / 64;
    const size_t T = (size_t)M * kD / 64;
    uint64_t* gave_up = state + groups_total;
    const int u = g * W + wave;  // all W units are of one head and exist: W divides nblk
    const int b = u / nblk, tb = u - b * nblk;
    uint32_t* buf = bufs[wave];
    uint32_t r[64];  // this lane's token, raw fp16 pairs; they stay in registers until they are compacted
    {
        UnitRaw raw;  // all 16 KB requested at once; M % 64 == 0: every row exists
        if (SRC == kSrcMatrix)
            unit_fetch(x + (size_t)b * M * kD, (int64_t)tb * 64, lane, raw);
        else if (SRC == kSrcView)
            unit_fetch(proj.view.head(b), (int64_t)tb * 64, lane, raw, proj.view.st);
        else
            unit_fetch_rotated(proj.view, proj.rope, proj.rot, b, tb, proj.rows, lane, raw);
        if (MSTF_COMPRESS_PARK)
            unit_rows_parked(raw, buf, lane, r);  // r[32 .. 64) stays in the staging buffer during the search
        else
            unit_rows_from(raw, buf, lane, r);
    }
    uint32_t kept[4];
    if (MSTF_COMPRESS_PARK) {
        if (kth > 0) {
            select_kth_planes_parked<true>(r, buf, lane, kth, kept);
        } else {
            parked_rows_take(buf, lane, r);
            kept_nonzero(r, kept);
        }
        __builtin_amdgcn_wave_barrier();  // the buffer becomes the image of the output next
    } else if (kth > 0) {
        select_kth_planes<true>(r, kth, kept);  // the sign bits become planes the search never looks at
    } else {
        kept_nonzero(r, kept);
    }
    uint64_t bmA, bmB;  // tiles tb*128 + lane and tb*128 + 64 + lane
    if (IS_VALUE) {
        bmA = spread_bitmap(kept[0], kept[1]);
        bmB = spread_bitmap(kept[2], kept[3]);
    } else {
        key_bitmaps_from_kept(kept, lane, bmA, bmB);
    }
    uint32_t totA, totB;
    const uint32_t eA = wave_excl_scan(padded_units(bmA), lane, totA);
    const uint32_t eB = wave_excl_scan(padded_units(bmB), lane, totB);
    const uint32_t total = totA + totB;
    if (lane == 0) wave_total[wave] = total;
    __syncthreads();
    uint32_t in_group = 0, group_total = 0;  // units of the workgroup in front of this one / all of them
#pragma unroll
    for (int w = 0; w < W; w++) {
        const uint32_t t = wave_total[w];
        in_group += w < wave ? t : 0u;
        group_total += t;
    }
    if (threadIdx.x == 0) agent_store(state + g, kWordReady | group_total);

    const uint32_t img = lds_addr(buf);
    compact_half<IS_VALUE>(r, kept, 0, eA, totA * 4u, img, lane);  // while the workgroups in front publish

    // offset of the unit inside its head and, packed layout, of the head
    const int head_first = (b * nblk) / W;  // first workgroup of this head
    {
        uint64_t lo = 0, hi = 0;
        const bool ok0 = wait_for_words<W>(state, dst_off ? head_first : 0, head_first, g, wave, lane, spin_limit, lo, hi);
        if (lane == 0) {
            bases[wave][0] = lo;
            bases[wave][1] = hi;
            bases[wave][2] = ok0 ? 1ull : 0ull;
        }
    }
    __syncthreads();
    uint64_t H = 0, in_head = 0;
    bool ok = true;
#pragma unroll
    for (int w = 0; w < W; w++) {
        H += bases[w][0];
        in_head += bases[w][1];
        ok = ok && bases[w][2] != 0ull;
    }
    if (!ok && threadIdx.x == 0) mark_gave_up(gave_up, total_halfs, overflow);
    const uint32_t base = (uint32_t)in_head + in_group;
    const uint32_t end = base + total;

    uint64_t* bo = bmp + (size_t)b * T + (size_t)tb * kD;
    uint32_t* io = idx + (size_t)b * (T + 1) + (size_t)tb * kD;
    bo[lane] = bmA;
    bo[64 + lane] = bmB;
    io[lane] = base + eA;
    io[64 + lane] = base + totA + eB;
    if (lane == 0) {
        if (tb == nblk - 1) io[kD] = end;
        if (tb == 0 && nz_off) nz_off[b] = (uint32_t)(H >> 2);
        if (u == units - 1 && total_halfs && ok)
            atomicMax(reinterpret_cast<unsigned long long*>(total_halfs), 2ull * (H + end));
    }
    if (!ok) return;
    const uint64_t head_half0 = dst_off ? 8ull * dst_off[b] : 2ull * H;
    if (head_half0 + 2ull * end > nz_capacity_halfs) return;  // would not fit: leave untouched (wave-uniform)
    if (dst_limit && head_half0 + 2ull * end > 8ull * dst_limit[b]) {
        if (lane == 0) atomicOr(overflow, kFlagOverflow);
        return;
    }
    char* dst = nz + (head_half0 + 2ull * base) * 2ull;
    stream_image(img, totA * 4u, dst, lane);
    compact_half<IS_VALUE>(r, kept, 1, eB, totB * 4u, img, lane);
    stream_image(img, totB * 4u, dst + (size_t)totA * 4u, lane);
}

template <bool IS_VALUE, int W, int SRC>
__global__ __launch_bounds__(64 * W) __attribute__((amdgpu_waves_per_eu((MSTF_COMPRESS_PARK && SRC != kSrcRope) ? 4 : 2))) void compress_onepass_kernel(
    const _Float16* __restrict__ x, ProjArgs proj, int M, int kth, uint64_t* __restrict__ bmp, uint32_t* __restrict__ idx,
    uint32_t* __restrict__ nz_off, uint64_t* __restrict__ total_halfs, const uint32_t* __restrict__ dst_off,
    const uint32_t* __restrict__ dst_limit, uint32_t* __restrict__ overflow, char* __restrict__ nz,
    uint64_t nz_capacity_halfs, uint64_t* state, int units, int groups_total, uint32_t spin_limit)
{
    __shared__ OnepassLds<W> lds;
    onepass_workgroup<IS_VALUE, W, SRC>(lds, (int)blockIdx.x, x, proj, M, kth, bmp, idx, nz_off, total_halfs, dst_off,
                                        dst_limit, overflow, nz, nz_capacity_halfs, state, units, groups_total, spin_limit);
}

// Keys and values of the same tokens in one launch: workgroups 0 .. groups_total-1 compress the keys, the next
// groups_total the values, each side with its own status words and outputs.  One launch has twice the generations of
// workgroups of a launch per side, which run less in lockstep (the loads of one generation overlap the arithmetic of
// the one before), and one clearing launch in front instead of two.
struct OnepassSide {
    const _Float16* x;
    int kth;
    uint64_t* bmp;
    uint32_t* idx;
    uint32_t* nz_off;
    uint64_t* total_halfs;
    const uint32_t* dst_off;
    const uint32_t* dst_limit;
    char* nz;
    uint64_t nz_capacity_halfs;
    uint64_t* state;
};
template <int W>
__global__ __launch_bounds__(64 * W) __attribute__((amdgpu_waves_per_eu(4))) void compress_onepass_kv_kernel(
    OnepassSide k, OnepassSide v, int M, uint32_t* __restrict__ overflow, int units, int groups_total, uint32_t spin_limit)
{
    __shared__ OnepassLds<W> lds;
    const int g = (int)blockIdx.x;
    if (g < groups_total)
        onepass_workgroup<false, W, kSrcMatrix>(lds, g, k.x, ProjArgs{}, M, k.kth, k.bmp, k.idx, k.nz_off, k.total_halfs,
                                                k.dst_off, k.dst_limit, overflow, k.nz, k.nz_capacity_halfs, k.state, units,
                                                groups_total, spin_limit);
    else
        onepass_workgroup<true, W, kSrcMatrix>(lds, g - groups_total, v.x, ProjArgs{}, M, v.kth, v.bmp, v.idx, v.nz_off,
                                               v.total_halfs, v.dst_off, v.dst_limit, overflow, v.nz, v.nz_capacity_halfs,
                                               v.state, units, groups_total, spin_limit);
}

// ------------------------------------------------------------------------------- dense prune
// y = x * (|x| >= kth-th smallest |x| of the row); 64 rows per wavefront.
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2))) void prune_rows_kernel(const _Float16* __restrict__ x, _Float16* y, int64_t rows,
                                                        int kth)
{
    __shared__ uint32_t slab[kHalfSlabDw];
    const int lane = lane_id();
    const int64_t row0 = (int64_t)blockIdx.x * 64;
    uint32_t r[64], mag[64];
    unit_rows(x, row0, rows, slab, lane, r);
#pragma unroll
    for (int j = 0; j < 64; j++) mag[j] = r[j] & 0x7FFF7FFFu;
    const uint32_t thr = select_kth(mag, kth);
    const us2_t t2 = as_us2(thr | (thr << 16));
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int j = 0; j < 32; j++) {
            const uint32_t d = us2_u32(as_us2(mag[32 * h + j]) - t2);  // bit 15 / 31 set <=> pruned
            uint32_t keep = 0x80008000u;                                // the sign always survives (x * 0 = +-0)
            if (!(d & 0x8000u)) keep |= 0x00007FFFu;
            if (!(d & 0x80000000u)) keep |= 0x7FFF0000u;
            slab[lane * kHalfRowDw + j] = r[32 * h + j] & keep;
        }
        __builtin_amdgcn_wave_barrier();
        uint4* dst = reinterpret_cast<uint4*>(y + row0 * kD) + h * 8;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int e = j * 64 + lane;
            const int row = e >> 3, c16 = e & 7;
            const uint32_t* sp = slab + row * kHalfRowDw + c16 * 4;
            if (row0 + row < rows) dst[row * 16 + c16] = make_uint4(sp[0], sp[1], sp[2], sp[3]);
        }
        __builtin_amdgcn_wave_barrier();
    }
}

// ------------------------------------------------------------------------------- host
// workspace: unit totals and unit bases (both [B][M/64], 4 bytes) of the two-pass form, or the status words of the
// one-pass kernel (8 bytes per unit, 8 per head, the flag word) - the same bytes
static size_t compress_ws_bytes(int B, int M)
{
    return 2 * round_up((size_t)B * (M / 64) * 4, 256) + round_up((size_t)B * 8 + 64, 256);
}

// The one-pass kernel behind its init kernel.
template <bool IS_VALUE, int SRC = kSrcMatrix>
static int launch_onepass(hipStream_t st, const _Float16* xh, const ProjArgs& proj, int B, int M, int kth, uint64_t* bmp, uint32_t* idx,
                          uint32_t* nz_off, uint64_t* total_halfs, const uint32_t* dst_off, const uint32_t* dst_limit,
                          uint32_t* overflow, mstf_half* nz, uint64_t cap, void* ws)
{
    const int nblk = M / 64, units = B * nblk;
#ifndef MSTF_ONEPASS_W
#define MSTF_ONEPASS_W 4
#endif
    const int W = nblk % MSTF_ONEPASS_W == 0 ? MSTF_ONEPASS_W : (nblk % 2 == 0 ? 2 : 1);
    const int groups = units / W;
    uint64_t* state = reinterpret_cast<uint64_t*>(ws);
    const int words = groups + 1;
    const uint32_t spin_limit = onepass_spin_limit();
    hipLaunchKernelGGL(onepass_init_kernel, dim3((unsigned)((words + 255) / 256 < 256 ? (words + 255) / 256 : 256)),
                       dim3(256), 0, st, state, words, total_halfs, static_cast<uint64_t*>(nullptr));
    int rc = check_launch();
    if (rc != MSTF_OK) return rc;
#define MSTF_OP(WV)                                                                                                   \
    hipLaunchKernelGGL((compress_onepass_kernel<IS_VALUE, WV, SRC>), dim3((unsigned)groups), dim3(64 * WV), 0, st, xh, proj, M, kth, \
                       bmp, idx, nz_off, total_halfs, dst_off, dst_limit, overflow, reinterpret_cast<char*>(nz), cap,  \
                       state, units, groups, spin_limit)
    if (W == MSTF_ONEPASS_W)
        MSTF_OP(MSTF_ONEPASS_W);
    else if (W == 2)
        MSTF_OP(2);
    else
        MSTF_OP(1);
#undef MSTF_OP
    return check_launch();
}

// Keys and values of the same tokens behind one clearing launch (status words of the keys, then of the values).
static int launch_onepass_kv(hipStream_t st, OnepassSide k, OnepassSide v, int B, int M, uint32_t* overflow, void* ws)
{
    const int nblk = M / 64, units = B * nblk;
    const int W = nblk % MSTF_ONEPASS_W == 0 ? MSTF_ONEPASS_W : (nblk % 2 == 0 ? 2 : 1);
    const int groups = units / W;
    const int words = groups + 1;
    k.state = reinterpret_cast<uint64_t*>(ws);
    v.state = k.state + words;
    const uint32_t spin_limit = onepass_spin_limit();
    hipLaunchKernelGGL(onepass_init_kernel, dim3((unsigned)((2 * words + 255) / 256 < 256 ? (2 * words + 255) / 256 : 256)),
                       dim3(256), 0, st, k.state, 2 * words, k.total_halfs, v.total_halfs);
    int rc = check_launch();
    if (rc != MSTF_OK) return rc;
#define MSTF_OPKV(WV)                                                                                            \
    hipLaunchKernelGGL((compress_onepass_kv_kernel<WV>), dim3(2u * (unsigned)groups), dim3(64 * WV), 0, st, k, v, M, \
                       overflow, units, groups, spin_limit)
    if (W == MSTF_ONEPASS_W)
        MSTF_OPKV(MSTF_ONEPASS_W);
    else if (W == 2)
        MSTF_OPKV(2);
    else
        MSTF_OPKV(1);
#undef MSTF_OPKV
    return check_launch();
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
    hipLaunchKernelGGL((compress_scatter_kernel<IS_VALUE, false>), dim3((unsigned)(B * (M / 64))), dim3(64), 0,
                       as_stream(stream), reinterpret_cast<const _Float16*>(x), M, bmp, const_cast<uint32_t*>(idx),
                       (const uint32_t*)nullptr, nz_off, reinterpret_cast<char*>(nz), cap, (const uint32_t*)nullptr,
                       (uint32_t*)nullptr);
    return check_launch();
}

// Units per wavefront of the count kernel: two once that still fills the chip (its loads then overlap its
// arithmetic), one for small inputs.
template <bool IS_VALUE>
static void launch_count(hipStream_t st, const _Float16* xh, int B, int M, int kth, uint64_t* bmp, uint32_t* idx,
                         uint32_t* unit_tot)
{
    const int units = B * (M / 64);
    const int upw = units >= 4096 ? 2 : 1;
    hipLaunchKernelGGL(compress_count_kernel<IS_VALUE>, dim3((unsigned)((units + upw - 1) / upw)), dim3(64), 0, st, xh,
                       M, kth, bmp, idx, unit_tot, units, upw);
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
    const _Float16* xh = reinterpret_cast<const _Float16*>(x);
    if (nz) {
        if (!aligned_to(nz, 16)) return MSTF_EALIGN;
        return launch_onepass<IS_VALUE>(st, xh, ProjArgs{}, B, M, kth, bmp, idx, nz_off, total_halfs, nullptr, nullptr, nullptr, nz,
                                        cap, ws);
    }
    // sizing only: counts, scan, final offsets
    const size_t ub = round_up((size_t)B * nblk * 4, 256);
    uint32_t* unit_tot = reinterpret_cast<uint32_t*>(ws);
    uint32_t* unit_base = reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(ws) + ub);
    launch_count<IS_VALUE>(st, xh, B, M, kth, bmp, idx, unit_tot);
    if ((rc = check_launch()) != MSTF_OK) return rc;
    hipLaunchKernelGGL(scan_units_kernel, dim3((unsigned)B), dim3(256), (size_t)nblk * 4, st, unit_tot, unit_base, idx,
                       nz_off, total_halfs, nblk, kD);
    if ((rc = check_launch()) != MSTF_OK) return rc;
    hipLaunchKernelGGL(finalize_idx_kernel, dim3((unsigned)(((size_t)nblk * kD + 255) / 256), (unsigned)B), dim3(256), 0,
                       st, idx, unit_base, nblk, kD);
    return check_launch();
}

// Compresses a chunk and places head b's packed values at nz + 16 * dst_off[b] (limit: nz + 16 * dst_limit[b]).
template <bool IS_VALUE>
static int append_impl(void* stream, const mstf_half* x, int B, int M, int N, int kth, uint64_t* bmp, uint32_t* idx,
                       const uint32_t* dst_off, const uint32_t* dst_limit, mstf_half* nz, uint32_t* overflow, void* ws,
                       size_t ws_bytes)
{
    int rc = check_compress_args(x, B, M, N, kth);
    if (rc != MSTF_OK) return rc;
    if (!bmp || !idx || !dst_off || !dst_limit || !nz || !overflow) return MSTF_EINVAL;
    if (!aligned_to(bmp, 8) || !aligned_to(idx, 4) || !aligned_to(dst_off, 4) || !aligned_to(dst_limit, 4) ||
        !aligned_to(nz, 16) || !aligned_to(overflow, 4))
        return MSTF_EALIGN;
    if (!ws || ws_bytes < compress_ws_bytes(B, M)) return MSTF_EWORKSPACE;
    if (!aligned_to(ws, 256)) return MSTF_EALIGN;
    return launch_onepass<IS_VALUE>(as_stream(stream), reinterpret_cast<const _Float16*>(x), ProjArgs{}, B, M, kth, bmp, idx, nullptr,
                                    nullptr, dst_off, dst_limit, overflow, nz, ~0ull, ws);
}

// Rows in the layout of a projection output, optionally rotated first.  dst_off == nullptr: the compress contract
// (nz_off and *total_halfs are outputs), else the append contract (dst_off / dst_limit / overflow are inputs).
static int proj_impl(void* stream, const mstf_proj_source* s, int is_value, int M, int N, int kth, uint64_t* bmp,
                     uint32_t* idx, uint32_t* nz_off, uint64_t* total_halfs, const uint32_t* dst_off,
                     const uint32_t* dst_limit, mstf_half* nz, uint64_t cap, uint32_t* overflow, void* ws, size_t ws_bytes)
{
    if (!s || !s->x || s->batch <= 0 || s->heads <= 0 || s->rows <= 0 || M < 0 || M > s->rows || kth < 0 || kth > N)
        return MSTF_EINVAL;
    if (N != kD || M % 64 != 0) return MSTF_EUNSUPPORTED;
    const bool rope = s->cos || s->sin;
    if (rope && (!s->cos || !s->sin || !s->rot || is_value)) return MSTF_EINVAL;
    if (M == 0 && !rope) return MSTF_EINVAL;
    const int64_t strides[] = {s->stride_batch, s->stride_token, s->stride_head, rope ? s->rope_stride_batch : 0,
                               rope ? s->rope_stride_token : 0, rope ? s->rot_stride_batch : 0,
                               rope ? s->rot_stride_token : 0, rope ? s->rot_stride_head : 0};
    for (int64_t v : strides)
        if (v < 0 || v % 8 != 0) return MSTF_EINVAL;
    // the loaders address the 64 rows of a unit with 32-bit byte offsets from the unit's first row
    const int64_t tok_strides[] = {s->stride_token, rope ? s->rope_stride_token : 0, rope ? s->rot_stride_token : 0};
    for (int64_t v : tok_strides)
        if (v * 2 * 64 > 0xFFFFFFFFll) return MSTF_EUNSUPPORTED;
    if (!aligned_to(s->x, 16) || (rope && (!aligned_to(s->cos, 16) || !aligned_to(s->sin, 16) || !aligned_to(s->rot, 16))))
        return MSTF_EALIGN;
    const int64_t B64 = (int64_t)s->batch * s->heads;
    const int64_t units_all = B64 * ((s->rows + 63) / 64);
    if (units_all > 0x7FFFFFFF || M / 64 > 8192) return MSTF_EUNSUPPORTED;
    const int B = (int)B64;
    const int nblk = M / 64;
    hipStream_t st = as_stream(stream);
    const RowsView src{reinterpret_cast<const _Float16*>(s->x), s->stride_batch, s->stride_token, s->stride_head, s->heads};
    const RowsView rot{reinterpret_cast<const _Float16*>(s->rot), s->rot_stride_batch, s->rot_stride_token,
                       s->rot_stride_head, s->heads};
    const RopeTables tab{reinterpret_cast<const _Float16*>(s->cos), reinterpret_cast<const _Float16*>(s->sin),
                         s->rope_stride_batch, s->rope_stride_token};
    if (M > 0) {
        if (!bmp || !idx || !nz) return MSTF_EINVAL;
        if (dst_off ? (!dst_limit || !overflow) : (!nz_off || !total_halfs)) return MSTF_EINVAL;
        if (!aligned_to(bmp, 8) || !aligned_to(idx, 4) || !aligned_to(nz, 16)) return MSTF_EALIGN;
        if (dst_off ? (!aligned_to(dst_off, 4) || !aligned_to(dst_limit, 4) || !aligned_to(overflow, 4))
                    : (!aligned_to(nz_off, 4) || !aligned_to(total_halfs, 8)))
            return MSTF_EALIGN;
        if (!ws || ws_bytes < compress_ws_bytes(B, M)) return MSTF_EWORKSPACE;
        if (!aligned_to(ws, 256)) return MSTF_EALIGN;
        const ProjArgs pa{src, tab, rot, s->rows};
        const uint64_t capacity = dst_off ? ~0ull : cap;
        int rc;
        if (rope)
            rc = launch_onepass<false, kSrcRope>(st, nullptr, pa, B, M, kth, bmp, idx, nz_off, total_halfs, dst_off,
                                                 dst_limit, overflow, nz, capacity, ws);
        else if (is_value)
            rc = launch_onepass<true, kSrcView>(st, nullptr, pa, B, M, kth, bmp, idx, nz_off, total_halfs, dst_off,
                                                dst_limit, overflow, nz, capacity, ws);
        else
            rc = launch_onepass<false, kSrcView>(st, nullptr, pa, B, M, kth, bmp, idx, nz_off, total_halfs, dst_off,
                                                 dst_limit, overflow, nz, capacity, ws);
        if (rc != MSTF_OK) return rc;
    }
    // the tokens behind the compressed ones are only rotated
    const int blocks_all = (s->rows + 63) / 64;
    if (rope && blocks_all > nblk) {
        hipLaunchKernelGGL(rope_tail_kernel, dim3((unsigned)(B * (blocks_all - nblk))), dim3(64), 0, st, src, tab, rot,
                           s->rows, nblk, blocks_all - nblk);
        return check_launch();
    }
    return MSTF_OK;
}

}  // namespace mstf

using namespace mstf;

extern "C" int mstf_append_key_f16(void* stream, const mstf_half* x, int B, int M, int N, int kth, uint64_t* bmp,
                                   uint32_t* idx, const uint32_t* dst_off, const uint32_t* dst_limit, mstf_half* nz,
                                   uint32_t* overflow, void* workspace, size_t workspace_bytes)
{
    return append_impl<false>(stream, x, B, M, N, kth, bmp, idx, dst_off, dst_limit, nz, overflow, workspace,
                              workspace_bytes);
}

extern "C" int mstf_append_value_f16(void* stream, const mstf_half* x, int B, int M, int N, int kth, uint64_t* bmp,
                                     uint32_t* idx, const uint32_t* dst_off, const uint32_t* dst_limit, mstf_half* nz,
                                     uint32_t* overflow, void* workspace, size_t workspace_bytes)
{
    return append_impl<true>(stream, x, B, M, N, kth, bmp, idx, dst_off, dst_limit, nz, overflow, workspace,
                             workspace_bytes);
}

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

extern "C" int mstf_compress_proj_f16(void* stream, const mstf_proj_source* src, int is_value, int M, int N, int kth,
                                      uint64_t* bmp, uint32_t* idx, uint32_t* nz_off, uint64_t* total_halfs,
                                      mstf_half* nz, uint64_t nz_capacity_halfs, void* workspace, size_t workspace_bytes)
{
    return proj_impl(stream, src, is_value, M, N, kth, bmp, idx, nz_off, total_halfs, nullptr, nullptr, nz,
                     nz_capacity_halfs, nullptr, workspace, workspace_bytes);
}

extern "C" int mstf_append_proj_f16(void* stream, const mstf_proj_source* src, int is_value, int M, int N, int kth,
                                    uint64_t* bmp, uint32_t* idx, const uint32_t* dst_off, const uint32_t* dst_limit,
                                    mstf_half* nz, uint32_t* overflow, void* workspace, size_t workspace_bytes)
{
    if (!dst_off) return MSTF_EINVAL;
    return proj_impl(stream, src, is_value, M, N, kth, bmp, idx, nullptr, nullptr, dst_off, dst_limit, nz, 0, overflow,
                     workspace, workspace_bytes);
}

extern "C" size_t mstf_compress_kv_workspace_bytes(int B, int M, int N)
{
    if (B <= 0 || M <= 0 || N <= 0 || M % 64 != 0) return 0;
    return 2 * compress_ws_bytes(B, M);
}

static int kv_side_check(const void* x, int B, int M, int N, int kth, const void* bmp, const void* idx, const void* nz)
{
    int rc = check_compress_args(x, B, M, N, kth);
    if (rc != MSTF_OK) return rc;
    if (!bmp || !idx || !nz) return MSTF_EINVAL;
    if (!aligned_to(bmp, 8) || !aligned_to(idx, 4) || !aligned_to(nz, 16)) return MSTF_EALIGN;
    return MSTF_OK;
}

extern "C" int mstf_compress_kv_f16(void* stream, const mstf_half* k, const mstf_half* v, int B, int M, int N, int kth_k,
                                    int kth_v, uint64_t* k_bmp, uint32_t* k_idx, uint32_t* k_nz_off,
                                    uint64_t* k_total_halfs, mstf_half* k_nz, uint64_t k_capacity_halfs, uint64_t* v_bmp,
                                    uint32_t* v_idx, uint32_t* v_nz_off, uint64_t* v_total_halfs, mstf_half* v_nz,
                                    uint64_t v_capacity_halfs, void* workspace, size_t workspace_bytes)
{
    int rc = kv_side_check(k, B, M, N, kth_k, k_bmp, k_idx, k_nz);
    if (rc == MSTF_OK) rc = kv_side_check(v, B, M, N, kth_v, v_bmp, v_idx, v_nz);
    if (rc != MSTF_OK) return rc;
    if (!k_nz_off || !k_total_halfs || !v_nz_off || !v_total_halfs) return MSTF_EINVAL;
    if (!aligned_to(k_nz_off, 4) || !aligned_to(v_nz_off, 4) || !aligned_to(k_total_halfs, 8) || !aligned_to(v_total_halfs, 8))
        return MSTF_EALIGN;
    if (!workspace || workspace_bytes < mstf_compress_kv_workspace_bytes(B, M, N)) return MSTF_EWORKSPACE;
    if (!aligned_to(workspace, 256)) return MSTF_EALIGN;
    OnepassSide ks = {reinterpret_cast<const _Float16*>(k), kth_k, k_bmp, k_idx, k_nz_off, k_total_halfs, nullptr, nullptr,
                      reinterpret_cast<char*>(k_nz), k_capacity_halfs, nullptr};
    OnepassSide vs = {reinterpret_cast<const _Float16*>(v), kth_v, v_bmp, v_idx, v_nz_off, v_total_halfs, nullptr, nullptr,
                      reinterpret_cast<char*>(v_nz), v_capacity_halfs, nullptr};
    return launch_onepass_kv(as_stream(stream), ks, vs, B, M, nullptr, workspace);
}

extern "C" int mstf_append_kv_f16(void* stream, const mstf_half* k, const mstf_half* v, int B, int M, int N, int kth_k,
                                  int kth_v, uint64_t* k_bmp, uint32_t* k_idx, const uint32_t* k_dst_off,
                                  const uint32_t* k_dst_limit, mstf_half* k_nz, uint64_t* v_bmp, uint32_t* v_idx,
                                  const uint32_t* v_dst_off, const uint32_t* v_dst_limit, mstf_half* v_nz,
                                  uint32_t* overflow, void* workspace, size_t workspace_bytes)
{
    int rc = kv_side_check(k, B, M, N, kth_k, k_bmp, k_idx, k_nz);
    if (rc == MSTF_OK) rc = kv_side_check(v, B, M, N, kth_v, v_bmp, v_idx, v_nz);
    if (rc != MSTF_OK) return rc;
    if (!k_dst_off || !k_dst_limit || !v_dst_off || !v_dst_limit || !overflow) return MSTF_EINVAL;
    if (!aligned_to(k_dst_off, 4) || !aligned_to(k_dst_limit, 4) || !aligned_to(v_dst_off, 4) || !aligned_to(v_dst_limit, 4) ||
        !aligned_to(overflow, 4))
        return MSTF_EALIGN;
    if (!workspace || workspace_bytes < mstf_compress_kv_workspace_bytes(B, M, N)) return MSTF_EWORKSPACE;
    if (!aligned_to(workspace, 256)) return MSTF_EALIGN;
    OnepassSide ks = {reinterpret_cast<const _Float16*>(k), kth_k, k_bmp, k_idx, nullptr, nullptr, k_dst_off, k_dst_limit,
                      reinterpret_cast<char*>(k_nz), ~0ull, nullptr};
    OnepassSide vs = {reinterpret_cast<const _Float16*>(v), kth_v, v_bmp, v_idx, nullptr, nullptr, v_dst_off, v_dst_limit,
                      reinterpret_cast<char*>(v_nz), ~0ull, nullptr};
    return launch_onepass_kv(as_stream(stream), ks, vs, B, M, overflow, workspace);
}
