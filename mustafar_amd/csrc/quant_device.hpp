// Device-side building blocks of the quantised consumers (quant_spmv.hip, fused_quant.hip): staging sizes,
// dequantisation of a staged run of tiles into an fp16 tile image in LDS, expansion of that image.
#pragma once
#include "spmv_device.hpp"

#ifndef MSTF_IMG_STRIDE
#define MSTF_IMG_STRIDE 144
#endif

namespace mstf {

#pragma clang fp contract(off)

template <int BIT>
struct QFmt {
    static constexpr int kCap = 32 / BIT;                       // codes per packed word
    static constexpr int kCapShift = BIT == 2 ? 4 : (BIT == 4 ? 3 : 2);
    static constexpr int kSlots = 64 / kCap;                    // words of a full tile = lanes per tile in a pass
    static constexpr int kTilesPerPass = 64 / kSlots;
    static constexpr int kPasses = kSubTiles / kTilesPerPass;
    static constexpr int kWordsMax = kSubTiles * kSlots;        // words of a stage, every tile full
    static constexpr int kWordBuf = kWordsMax * 4 + 64;         // + room for the lanes past a tile's last word
};
// fp16 image of a stage: 64 two-byte slots per tile, the tiles kImgStride bytes apart.  128 would do; with 144 the
// sixteen-byte writes of the lanes that dequantise different tiles at the same time (tiles 128 bytes apart start in
// one of two banks) and the gathers spread over all LDS banks.
constexpr int kImgStride = MSTF_IMG_STRIDE;
constexpr int kImgBytes = kSubTiles * kImgStride;
// Staged metadata of a stage.  One (scale, zero) pair per tile: 32 word offsets, 32 scales, 32 zero-points (256 bytes,
// one LDS-direct load).  Two pairs per tile (G32: pair g for the elements 32g .. 32g+31): 32 word offsets, 32 x 2
// scales, 32 x 2 zero-points and the upper halves of the 32 bitmaps (their popcount is the number of codes that
// belong to the first pair), 128 bytes each, two LDS-direct loads.
template <bool G32>
constexpr int meta_bytes()
{
    return G32 ? 512 : 256;
}
template <int BIT, bool G32 = false>
constexpr int q_lds_bytes()
{
    return kImgBytes + 16 + 2 * QFmt<BIT>::kWordBuf + 2 * meta_bytes<G32>();
}

__device__ __forceinline__ float half_bits_to_float(uint32_t bits) { return (float)as_h((uint16_t)bits); }

// The literal arithmetic of the two dequantisation modes for one code.
__device__ __forceinline__ _Float16 dequant_exact(uint32_t q, uint32_t scale_bits, uint32_t zero_bits, int mode)
{
    if (mode == 1) {
        const _Float16 d = (_Float16)(int)q - as_h((uint16_t)zero_bits);  // fp16 arithmetic, rounded after each step
        return d * as_h((uint16_t)scale_bits);
    }
    return (_Float16)(((float)q - half_bits_to_float(zero_bits)) * half_bits_to_float(scale_bits));
}

// fp16x2 ( (q_lo - zero) * scale, (q_hi - zero) * scale ) from two codes held in bytes 0 and 2 of `codes`.
__device__ __forceinline__ uint32_t dequant_pair(uint32_t codes, h2_t neg_bias, h2_t scale2)
{
    const h2_t x = as_h2(codes | 0x64006400u);  // (1024 + q_lo, 1024 + q_hi)
    return as_u32((x + neg_bias) * scale2);
}

// One stage: every lane owns one packed word and writes that word's values to the tile image.  A tile's words are
// visited in two halves: first words 0 .. kSlots/2 - 1 of every tile (kSlots/2 lanes per tile: all there is for a tile
// with at most 32 survivors), then - only if some tile of the stage has more words, a wave-uniform test on the word
// offsets - words kSlots/2 .. kSlots - 1.  Lanes past a tile's last word decode whatever follows in the staged buffer
// into image slots no rank ever points to.
//   meta  : LDS address of the staged metadata; words: LDS address of the staged words, word 0 = `start_word`;
//   end_word: where the stage's last tile ends
template <int BIT, bool G32 = false>
__device__ __forceinline__ void dequant_stage(uint32_t meta, uint32_t words, uint32_t img, uint32_t start_word,
                                              uint32_t end_word, int lane, int mode)
{
    using F = QFmt<BIT>;
    typedef short s2_t __attribute__((ext_vector_type(2)));
    constexpr int kHalfSlots = F::kSlots / 2;
    constexpr int kTilesPerHalfPass = 64 / kHalfSlots;
    constexpr int kHalfPasses = kSubTiles / kTilesPerHalfPass;
    static_assert(kSubTiles == 32, "lanes 0..31 test the 32 tiles of the stage");
    // Tiles with more words than the first half covers: a few of them (a key stage typically holds one channel of
    // outliers, which keeps all 64 tokens) are finished one by one after the first half, lane = rank (dequant_tile_by_rank
    // below: a dozen instructions per tile); only with more than kDirectMax of them does the stage take the second half.
    constexpr int kDirectMax = 4;
    uint32_t long_tiles;
    {
        const uint32_t t = (uint32_t)(lane < 32 ? lane : 31);
        const uint32_t o = lds_load_u32(meta + t * 4u);
        const uint32_t nx = lane < 31 ? lds_load_u32(meta + t * 4u + 4u) : end_word;
        long_tiles = (uint32_t)__ballot(lane < 32 && nx - o > (uint32_t)kHalfSlots);
    }
    const bool need_high = __builtin_popcount(long_tiles) > kDirectMax;
#pragma unroll
    for (int hp = 0; hp < 2 * kHalfPasses; hp++) {
        const int half = hp / kHalfPasses, p = hp % kHalfPasses;
        if (half == 1 && !need_high) break;
        const uint32_t tl = (uint32_t)(p * kTilesPerHalfPass + lane / kHalfSlots);
        const uint32_t slot = (uint32_t)(half * kHalfSlots + lane % kHalfSlots);
        const uint32_t off = lds_load_u32(meta + tl * 4u);
        // sc / zp: the pair of the tile (low half) or, G32, both pairs (first in the low half)
        const uint32_t sc = G32 ? lds_load_u32(meta + 128u + tl * 4u) : lds_load_u16(meta + 128u + tl * 2u);
        const uint32_t zp = G32 ? lds_load_u32(meta + 256u + tl * 4u) : lds_load_u16(meta + 192u + tl * 2u);
        // G32: the codes of this word that belong to the first pair, 0 .. kCap (codes are in rank order over the whole
        // tile; the first popcount(upper bitmap half) of them sit in elements 0 .. 31)
        int kb = F::kCap;
        if (G32) {
            const int c0 = __builtin_popcount(lds_load_u32(meta + 384u + tl * 4u));
            kb = c0 - (int)slot * F::kCap;
            kb = kb < 0 ? 0 : (kb > F::kCap ? F::kCap : kb);
        }
        const uint32_t w = lds_load_u32(words + (off - start_word + slot) * 4u);
        const uint32_t dst = img + tl * (uint32_t)kImgStride + slot * (uint32_t)(F::kCap * 2);
        const bool small_zero = G32 ? ((zp & 0x7fffu) <= 0x6400u && ((zp >> 16) & 0x7fffu) <= 0x6400u)
                                    : ((zp & 0x7fffu) <= 0x6400u);
        if (small_zero) {
            const _Float16 nb = (_Float16)(-1024.0f) - as_h((uint16_t)zp);  // exact: |zero| <= 1024
            const _Float16 sh = as_h((uint16_t)sc);
            const h2_t nb_a = {nb, nb};
            const h2_t sc_a = {sh, sh};
            uint32_t nb_b = 0u, sc_b = 0u, kb2 = 0u;
            if (G32) {
                const _Float16 nb1 = (_Float16)(-1024.0f) - as_h((uint16_t)(zp >> 16));
                const _Float16 sh1 = as_h((uint16_t)(sc >> 16));
                nb_b = as_u32(h2_t{nb1, nb1});
                sc_b = as_u32(h2_t{sh1, sh1});
                kb2 = (uint32_t)kb | ((uint32_t)kb << 16);
            }
            // dequantises codes 2n, 2n+1 of the word (held in bytes 0 and 2 of `codes`); G32: each of the two takes the
            // first pair if its index is below kb - a packed 16-bit subtract and arithmetic shift give the halfword
            // masks, two bit-field inserts the parameters
            auto deq = [&](uint32_t codes, int n) -> uint32_t {
                if (!G32) return dequant_pair(codes, nb_a, sc_a);
                const s2_t d = __builtin_bit_cast(s2_t, (uint32_t)(2 * n) | ((uint32_t)(2 * n + 1) << 16)) -
                               __builtin_bit_cast(s2_t, kb2);                       // < 0 <=> first pair
                const uint32_t m = __builtin_bit_cast(uint32_t, (s2_t)(d >> 15));
                const uint32_t nbx = (m & as_u32(nb_a)) | (~m & nb_b);
                const uint32_t scx = (m & as_u32(sc_a)) | (~m & sc_b);
                return dequant_pair(codes, as_h2(nbx), as_h2(scx));
            };
            if (BIT == 2) {
                // E[k % 4] holds code k in byte k / 4
                const uint32_t e0 = w & 0x03030303u, e1 = (w >> 2) & 0x03030303u;
                const uint32_t e2 = (w >> 4) & 0x03030303u, e3 = (w >> 6) & 0x03030303u;
                u32x4_t lo, hi;
                lo[0] = deq(__builtin_amdgcn_perm(e1, e0, 0x0c040c00u), 0);  // codes 0, 1
                lo[1] = deq(__builtin_amdgcn_perm(e3, e2, 0x0c040c00u), 1);  // codes 2, 3
                lo[2] = deq(__builtin_amdgcn_perm(e1, e0, 0x0c050c01u), 2);
                lo[3] = deq(__builtin_amdgcn_perm(e3, e2, 0x0c050c01u), 3);
                hi[0] = deq(__builtin_amdgcn_perm(e1, e0, 0x0c060c02u), 4);
                hi[1] = deq(__builtin_amdgcn_perm(e3, e2, 0x0c060c02u), 5);
                hi[2] = deq(__builtin_amdgcn_perm(e1, e0, 0x0c070c03u), 6);
                hi[3] = deq(__builtin_amdgcn_perm(e3, e2, 0x0c070c03u), 7);
                *(MSTF_LDS u32x4_t*)(uintptr_t)dst = lo;
                *(MSTF_LDS u32x4_t*)(uintptr_t)(dst + 16u) = hi;
            } else if (BIT == 4) {
                // e0 holds codes 0, 2, 4, 6 in its bytes, e1 codes 1, 3, 5, 7
                const uint32_t e0 = w & 0x0f0f0f0fu, e1 = (w >> 4) & 0x0f0f0f0fu;
                u32x4_t v;
                v[0] = deq(__builtin_amdgcn_perm(e1, e0, 0x0c040c00u), 0);
                v[1] = deq(__builtin_amdgcn_perm(e1, e0, 0x0c050c01u), 1);
                v[2] = deq(__builtin_amdgcn_perm(e1, e0, 0x0c060c02u), 2);
                v[3] = deq(__builtin_amdgcn_perm(e1, e0, 0x0c070c03u), 3);
                *(MSTF_LDS u32x4_t*)(uintptr_t)dst = v;
            } else {
                u32x2_t v;
                v[0] = deq(__builtin_amdgcn_perm(w, w, 0x0c010c00u), 0);
                v[1] = deq(__builtin_amdgcn_perm(w, w, 0x0c030c02u), 1);
                *(MSTF_LDS u32x2_t*)(uintptr_t)dst = v;
            }
        } else {
#pragma unroll 1
            for (int k = 0; k < F::kCap; k++) {
                const uint32_t q = (w >> (k * BIT)) & ((1u << BIT) - 1u);
                const uint32_t sel = (G32 && k >= kb) ? 16u : 0u;
                *(MSTF_LDS _Float16*)(uintptr_t)(dst + 2u * (uint32_t)k) =
                    dequant_exact(q, (sc >> sel) & 0xffffu, (zp >> sel) & 0xffffu, mode);
            }
        }
    }
    if (need_high) return;
    // the long tiles one by one: lane = rank r reads code r of the tile and writes image slot r (the slots of the first
    // half are written again with the same values; ranks beyond the tile's count land in slots no gather points to)
    while (long_tiles != 0u) {
        const uint32_t tl = (uint32_t)__builtin_ctz(long_tiles);
        long_tiles &= long_tiles - 1u;
        const uint32_t off = lds_load_u32(meta + tl * 4u);
        const uint32_t sc = G32 ? lds_load_u32(meta + 128u + tl * 4u) : lds_load_u16(meta + 128u + tl * 2u);
        const uint32_t zp = G32 ? lds_load_u32(meta + 256u + tl * 4u) : lds_load_u16(meta + 192u + tl * 2u);
        const uint32_t r = (uint32_t)lane;
        const uint32_t w = lds_load_u32(words + (off - start_word + (r >> F::kCapShift)) * 4u);
        const uint32_t q = (w >> ((r & (uint32_t)(F::kCap - 1)) * (uint32_t)BIT)) & ((1u << BIT) - 1u);
        uint32_t sel = 0u;  // G32: the first popcount(upper bitmap half) codes belong to the first pair
        if (G32) sel = r >= (uint32_t)__builtin_popcount(lds_load_u32(meta + 384u + tl * 4u)) ? 16u : 0u;
        const uint32_t s1 = (sc >> sel) & 0xffffu, z1 = (zp >> sel) & 0xffffu;
        _Float16 val;
        if ((z1 & 0x7fffu) <= 0x6400u) {
            const _Float16 nb = (_Float16)(-1024.0f) - as_h((uint16_t)z1);  // exact: |zero| <= 1024
            val = (as_h((uint16_t)(0x6400u | q)) + nb) * as_h((uint16_t)s1);
        } else {
            val = dequant_exact(q, s1, z1, mode);
        }
        *(MSTF_LDS _Float16*)(uintptr_t)(img + tl * (uint32_t)kImgStride + r * 2u) = val;
    }
}

// LDS-direct loads of a stage's packed words without control flow (see sub_issue_flat in spmv_device.hpp): piece i
// of lane l is word 64 * i + l of src, issued for the lanes with 64 * i + l < nw by setting exec by hand; the
// wavefront must have all 64 lanes active.  dst_lds: LDS byte address of the word buffer; lane4 = lane * 4.
template <int PIECES>
__device__ __forceinline__ void words_issue_flat(const uint32_t* src, uint32_t nw, uint32_t dst_lds, uint32_t lane,
                                                 uint32_t lane4)
{
    static_assert(PIECES == 2 || PIECES == 4 || PIECES == 8, "pieces of 64 words");
    uint32_t t, m0_kept;
    uint64_t sv;  // exec as found, handed back
#define MSTF_WPIECE(I)                                                     \
    "s_sub_i32 %[t], %[n], " #I " * 64\n\t"                                \
    "v_cmp_gt_i32 vcc, %[t], %[l]\n\t"                                     \
    "s_mov_b64 exec, vcc\n\t"                                              \
    "global_load_lds_dword %[l4], %[src] offset:" #I " * 256\n\t"
#define MSTF_WHEAD "s_mov_b32 %[keep], m0\n\ts_mov_b64 %[sv], exec\n\ts_mov_b32 m0, %[dst]\n\t"
#define MSTF_WTAIL "s_mov_b64 exec, %[sv]\n\ts_mov_b32 m0, %[keep]"
#define MSTF_WOPS                                                                                      \
    : [t] "=&s"(t), [keep] "=&s"(m0_kept), [sv] "=&s"(sv)                                              \
    : [dst] "s"(dst_lds), [n] "s"(nw), [l] "v"(lane), [l4] "v"(lane4), [src] "s"(src)                  \
    : "vcc", "scc", "memory"
    if constexpr (PIECES == 2)
        asm volatile(MSTF_WHEAD MSTF_WPIECE(0) MSTF_WPIECE(1) MSTF_WTAIL MSTF_WOPS);
    else if constexpr (PIECES == 4)
        asm volatile(MSTF_WHEAD MSTF_WPIECE(0) MSTF_WPIECE(1) MSTF_WPIECE(2) MSTF_WPIECE(3) MSTF_WTAIL MSTF_WOPS);
    else
        asm volatile(MSTF_WHEAD MSTF_WPIECE(0) MSTF_WPIECE(1) MSTF_WPIECE(2) MSTF_WPIECE(3) MSTF_WPIECE(4)
                         MSTF_WPIECE(5) MSTF_WPIECE(6) MSTF_WPIECE(7) MSTF_WTAIL MSTF_WOPS);
#undef MSTF_WPIECE
#undef MSTF_WHEAD
#undef MSTF_WTAIL
#undef MSTF_WOPS
}

// Where a lane fetches its 4 bytes of a stage's metadata from (lanes 0..31 the word offsets of the 32 tiles, 32..47
// the scales, 48..63 the zero-points, two per lane): the address for tile 0 and the shift that turns a tile index
// into the lane's byte offset, formed once, so that a stage needs one shift and one 64-bit add.
struct MetaLane {
    const char* p0;
    uint32_t shift;
    __device__ __forceinline__ const void* at(uint32_t t) const { return p0 + ((size_t)t << shift); }
};
__device__ __forceinline__ MetaLane meta_lane(const uint32_t* off_dma, const uint16_t* scales, const uint16_t* zeros, int lane)
{
    MetaLane m;
    m.p0 = lane < 32 ? reinterpret_cast<const char*>(off_dma + lane)
                     : lane < 48 ? reinterpret_cast<const char*>(reinterpret_cast<const uint32_t*>(scales) + (lane - 32))
                                 : reinterpret_cast<const char*>(reinterpret_cast<const uint32_t*>(zeros) + (lane - 48));
    m.shift = lane < 32 ? 2u : 1u;
    return m;
}
// Two pairs per tile: two loads.  First: lanes 0..31 the word offsets, 32..63 the scales (4 bytes per tile).  Second:
// lanes 0..31 the zero-points (4 bytes per tile), 32..63 the upper halves of the bitmaps (elements 0 .. 31 of a tile
// are bits 63 .. 32, i.e. the second 4 bytes of the little-endian 8).
struct MetaLanes {
    MetaLane a, b;
};
__device__ __forceinline__ MetaLanes meta_lanes_g32(const uint32_t* off_dma, const uint16_t* scales, const uint16_t* zeros,
                                                    const uint64_t* bmp, int lane)
{
    MetaLanes m;
    const int l = lane & 31;
    m.a.p0 = lane < 32 ? reinterpret_cast<const char*>(off_dma + l)
                       : reinterpret_cast<const char*>(reinterpret_cast<const uint32_t*>(scales) + l);
    m.a.shift = 2u;
    m.b.p0 = lane < 32 ? reinterpret_cast<const char*>(reinterpret_cast<const uint32_t*>(zeros) + l)
                       : reinterpret_cast<const char*>(bmp + l) + 4;
    m.b.shift = lane < 32 ? 2u : 3u;
    return m;
}
// Issues the metadata of the stage starting at tile t (relative to the pointers the lanes were built from).
template <bool G32>
__device__ __forceinline__ void meta_issue(const MetaLanes& m, uint32_t t, char* metabuf)
{
    dma4(m.a.at(t), metabuf);
    if (G32) dma4(m.b.at(t), metabuf + 256);
}
template <bool G32>
__device__ __forceinline__ MetaLanes meta_lanes(const uint32_t* off_dma, const uint16_t* scales, const uint16_t* zeros,
                                                const uint64_t* bmp, int lane)
{
    if (G32) return meta_lanes_g32(off_dma, scales, zeros, bmp, lane);
    MetaLanes m;
    m.a = meta_lane(off_dma, scales, zeros, lane);
    m.b = m.a;
    return m;
}

// batch_step_img_exec (below) for one accumulator group in the form without packing (batch_step_dual in
// spmv_device.hpp: even tiles into the low halves, odd ones into the high halves of their registers, two sets of sums,
// the weights in MSTF_GB0_3); the gather registers are cleared by two 16-byte reads of the zero slot here - this kernel's
// vector unit is the busier one, vector moves measured slower.
template <bool PREFETCH, int BOFF, int IMG, int WOFF>
__device__ __forceinline__ void batch_step_img_dual(const u32x16_t& mv, u32x16_t& nxt, const uint64_t* bm, uint32_t img,
                                                    uint32_t zaddr, uint32_t wbase, f4_t& acc, f4_t& acc2)
{
#define MSTF_TILE(I, LD, H, A)                                   \
    "s_brev_b64 exec, %[m" #I "]\n\t"                            \
    "v_mbcnt_lo_u32_b32 " A ", exec_lo, 0\n\t"                   \
    "v_mbcnt_hi_u32_b32 " A ", exec_hi, " A "\n\t"               \
    "v_lshl_add_u32 " A ", " A ", 1, %[img]\n\t"                 \
    LD " " H ", " A " offset:%[i" #I "]\n\t"
#define MSTF_LO "ds_read_u16"
#define MSTF_HI "ds_read_u16_d16_hi"
#define MSTF_QCLEAR "ds_read_b128 " MSTF_GV0_3 ", %[z]\n\tds_read_b128 " MSTF_GV4_7 ", %[z]\n\t"
#define MSTF_GATHER                                                                                                  \
    "ds_read_b128 " MSTF_GB0_3 ", %[wa] offset:%[woff]\n\t"                                                          \
    MSTF_QCLEAR \
    MSTF_TILE(0, MSTF_LO, MSTF_GV0, MSTF_GV8) MSTF_TILE(1, MSTF_HI, MSTF_GV2, MSTF_GV9)                              \
    MSTF_TILE(2, MSTF_LO, MSTF_GV1, MSTF_GV10) MSTF_TILE(3, MSTF_HI, MSTF_GV3, MSTF_GV11)                            \
    MSTF_TILE(4, MSTF_LO, MSTF_GV4, MSTF_GV12) MSTF_TILE(5, MSTF_HI, MSTF_GV6, MSTF_GV13)                            \
    MSTF_TILE(6, MSTF_LO, MSTF_GV5, MSTF_GV14) MSTF_TILE(7, MSTF_HI, MSTF_GV7, MSTF_GV15)                            \
    "s_mov_b64 exec, -1\n\t"                                                                                         \
    "s_waitcnt lgkmcnt(4)\n\t"                                                                                       \
    "v_mfma_f32_4x4x4_16b_f16 %[aa], " MSTF_GV0_1 ", " MSTF_GB0_1 ", %[aa]\n\t"                                      \
    "v_mfma_f32_4x4x4_16b_f16 %[ab], " MSTF_GV2_3 ", " MSTF_GB0_1 ", %[ab]\n\t"                                      \
    "s_waitcnt lgkmcnt(0)\n\t"                                                                                       \
    "v_mfma_f32_4x4x4_16b_f16 %[aa], " MSTF_GV4_5 ", " MSTF_GB2_3 ", %[aa]\n\t"                                      \
    "v_mfma_f32_4x4x4_16b_f16 %[ab], " MSTF_GV6_7 ", " MSTF_GB2_3 ", %[ab]\n\t"                                      \
    "s_nop 4"
#define MSTF_IN                                                                                                      \
    [m0] "s"(u64_of(mv[0], mv[1])), [m1] "s"(u64_of(mv[2], mv[3])), [m2] "s"(u64_of(mv[4], mv[5])),                  \
        [m3] "s"(u64_of(mv[6], mv[7])), [m4] "s"(u64_of(mv[8], mv[9])), [m5] "s"(u64_of(mv[10], mv[11])),            \
        [m6] "s"(u64_of(mv[12], mv[13])), [m7] "s"(u64_of(mv[14], mv[15])), [img] "s"(img), [wa] "v"(wbase),         \
        [woff] "i"(WOFF), [i0] "i"(IMG), [i1] "i"(IMG + kImgStride), [i2] "i"(IMG + 2 * kImgStride),                 \
        [i3] "i"(IMG + 3 * kImgStride), [i4] "i"(IMG + 4 * kImgStride), [i5] "i"(IMG + 5 * kImgStride),              \
        [i6] "i"(IMG + 6 * kImgStride), [i7] "i"(IMG + 7 * kImgStride), [z] "v"(zaddr)
#define MSTF_CLOBBER MSTF_GV_CLOBBER, MSTF_GB_CLOBBER, "memory"
    if constexpr (PREFETCH) {
        asm volatile("s_load_dwordx16 %[nm], %[nb], %[boff]\n\t" MSTF_GATHER
                     : [aa] "+v"(acc), [ab] "+v"(acc2), [nm] "=&s"(nxt)
                     : MSTF_IN, [nb] "s"(bm), [boff] "i"(BOFF)
                     : MSTF_CLOBBER);
    } else {
        asm volatile(MSTF_GATHER : [aa] "+v"(acc), [ab] "+v"(acc2) : MSTF_IN : MSTF_CLOBBER);
        nxt = mv;
    }
#undef MSTF_TILE
#undef MSTF_LO
#undef MSTF_HI
#undef MSTF_QCLEAR
#undef MSTF_GATHER
#undef MSTF_IN
#undef MSTF_CLOBBER
}

// Expands 8 tiles of the image and accumulates them, the gather under the tile's exec mask (see batch_step_exec in
// spmv_device.hpp for the statement and the MFMA layout): one statement per batch of 8 tiles on fixed registers
// (MSTF_GV0 .. 15 of spmv_device.hpp); the image slots of tile i sit at img + IMG + kImgStride * i, so the tile's
// base is an immediate offset of the LDS read.  PREFETCH: the bitmaps of the coming batch (bm + BOFF bytes) are
// requested first and completed by the statement's wait.
template <int NM, bool PREFETCH, int BOFF, int IMG, int WOFF>
__device__ __forceinline__ void batch_step_img_exec(const u32x16_t& mv, u32x16_t& nxt, const uint64_t* bm, uint32_t img,
                                                    uint32_t zaddr, uint32_t wbase, uint32_t wgroup, f4_t (&acc)[NM],
                                                    f4_t (&acc2)[NM])
{
    if constexpr (NM == 1 && MSTF_DUAL_ACC) {
        batch_step_img_dual<PREFETCH, BOFF, IMG, WOFF>(mv, nxt, bm, img, zaddr, wbase, acc[0], acc2[0]);
        return;
    }
    u32x4_t qm[NM];
#pragma unroll
    for (int m = 1; m < NM; m++) qm[m] = *(MSTF_LDS const u32x4_t*)(uintptr_t)(wbase + (uint32_t)WOFF + (uint32_t)m * wgroup);
    uint32_t v0, v1, v2, v3;
    uint64_t sv;  // exec as found, handed back
#define MSTF_TILE(I, H, A)                                       \
    "s_brev_b64 exec, %[m" #I "]\n\t"                            \
    "v_mbcnt_lo_u32_b32 " A ", exec_lo, 0\n\t"                   \
    "v_mbcnt_hi_u32_b32 " A ", exec_hi, " A "\n\t"               \
    "v_lshl_add_u32 " A ", " A ", 1, %[img]\n\t"                 \
    "ds_read_u16 " H ", " A " offset:%[i" #I "]\n\t"
#define MSTF_GATHER                                                                                  \
    "s_mov_b64 %[sv], exec\n\t"                                                                      \
    "ds_read_b128 %[qm], %[wa] offset:%[woff]\n\t"                                                   \
    "ds_read_b128 " MSTF_GV0_3 ", %[z]\n\t"                                                                  \
    "ds_read_b128 " MSTF_GV4_7 ", %[z]\n\t"                                                                  \
    MSTF_TILE(0, MSTF_GV0, MSTF_GV8) MSTF_TILE(1, MSTF_GV1, MSTF_GV9) MSTF_TILE(2, MSTF_GV2, MSTF_GV10) MSTF_TILE(3, MSTF_GV3, MSTF_GV11)      \
    MSTF_TILE(4, MSTF_GV4, MSTF_GV12) MSTF_TILE(5, MSTF_GV5, MSTF_GV13) MSTF_TILE(6, MSTF_GV6, MSTF_GV14) MSTF_TILE(7, MSTF_GV7, MSTF_GV15)      \
    "s_mov_b64 exec, %[sv]\n\t"                                                                      \
    "s_waitcnt lgkmcnt(0)\n\t"                                                                       \
    "v_lshl_or_b32 %[v0], " MSTF_GV1 ", 16, " MSTF_GV0 "\n\t"                                                        \
    "v_lshl_or_b32 %[v1], " MSTF_GV3 ", 16, " MSTF_GV2 "\n\t"                                                        \
    "v_lshl_or_b32 %[v2], " MSTF_GV5 ", 16, " MSTF_GV4 "\n\t"                                                        \
    "v_lshl_or_b32 %[v3], " MSTF_GV7 ", 16, " MSTF_GV6
#define MSTF_IN                                                                                                      \
    [m0] "s"(u64_of(mv[0], mv[1])), [m1] "s"(u64_of(mv[2], mv[3])), [m2] "s"(u64_of(mv[4], mv[5])),                  \
        [m3] "s"(u64_of(mv[6], mv[7])), [m4] "s"(u64_of(mv[8], mv[9])), [m5] "s"(u64_of(mv[10], mv[11])),            \
        [m6] "s"(u64_of(mv[12], mv[13])), [m7] "s"(u64_of(mv[14], mv[15])), [img] "s"(img), [wa] "v"(wbase),         \
        [woff] "i"(WOFF), [z] "v"(zaddr), [i0] "i"(IMG), [i1] "i"(IMG + kImgStride), [i2] "i"(IMG + 2 * kImgStride),        \
        [i3] "i"(IMG + 3 * kImgStride), [i4] "i"(IMG + 4 * kImgStride), [i5] "i"(IMG + 5 * kImgStride),                 \
        [i6] "i"(IMG + 6 * kImgStride), [i7] "i"(IMG + 7 * kImgStride)
#define MSTF_CLOBBER                                                                                                 \
    MSTF_GV_CLOBBER, "memory"
    if constexpr (PREFETCH) {
        asm volatile("s_load_dwordx16 %[nm], %[nb], %[boff]\n\t" MSTF_GATHER
                     : [v0] "=&v"(v0), [v1] "=&v"(v1), [v2] "=&v"(v2), [v3] "=&v"(v3), [qm] "=&v"(qm[0]), [sv] "=&s"(sv),
                       [nm] "=&s"(nxt)
                     : MSTF_IN, [nb] "s"(bm), [boff] "i"(BOFF)
                     : MSTF_CLOBBER);
    } else {
        asm volatile(MSTF_GATHER
                     : [v0] "=&v"(v0), [v1] "=&v"(v1), [v2] "=&v"(v2), [v3] "=&v"(v3), [qm] "=&v"(qm[0]), [sv] "=&s"(sv)
                     : MSTF_IN
                     : MSTF_CLOBBER);
        nxt = mv;
    }
#undef MSTF_TILE
#undef MSTF_GATHER
#undef MSTF_IN
#undef MSTF_CLOBBER
#pragma unroll
    for (int m = 0; m < NM; m++) {
        acc[m] = __builtin_amdgcn_mfma_f32_4x4x4f16(as_h4(v0, v1), as_h4(qm[m][0], qm[m][1]), acc[m], 0, 0, 0);
        acc[m] = __builtin_amdgcn_mfma_f32_4x4x4f16(as_h4(v2, v3), as_h4(qm[m][2], qm[m][3]), acc[m], 0, 0, 0);
        asm volatile("" : "+v"(acc[m]));  // pins the products here (see batch_step_exec)
    }
}

// The kSubTiles tiles of one dequantised stage.  The bitmaps of the first batch come out of the registers in which
// lane l < 32 already holds bitmap l of the stage (bm_lo, bm_hi: the coalesced load that pulled the stage's bitmaps
// into L2 one stage ahead) - the dequantisation in front has lane-dependent branches, so nothing scalar is carried
// across it, and a scalar load here would be waited for on the spot; the other batches are requested one batch ahead.
// img: LDS address of the stage's image; wbase: LDS address of w[lane & 3][first tile of the stage].
// acc2: the second set of sums of the form without packing (one accumulator group): the caller adds it to acc when
// its walk is over (dual_settle first).
template <int NM>
__device__ __forceinline__ void stage_img_exec(const uint64_t* bm, uint32_t bm_lo, uint32_t bm_hi, uint32_t img,
                                               uint32_t zaddr, uint32_t wbase, uint32_t wgroup, f4_t (&acc)[NM],
                                               f4_t (&acc2)[NM])
{
    constexpr int G = kSubTiles / 8;
    u32x16_t cur;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        cur[2 * i] = (uint32_t)__builtin_amdgcn_readlane((int)bm_lo, i);
        cur[2 * i + 1] = (uint32_t)__builtin_amdgcn_readlane((int)bm_hi, i);
    }
    static_for<G>([&](auto gc) {
        constexpr int g = decltype(gc)::value;
        u32x16_t nxt;
        batch_step_img_exec<NM, (g + 1 < G), (g + 1) * 64, g * 8 * kImgStride, g * 16>(cur, nxt, bm, img, zaddr, wbase, wgroup,
                                                                                       acc, acc2);
        cur = nxt;
    });
}

}  // namespace mstf
