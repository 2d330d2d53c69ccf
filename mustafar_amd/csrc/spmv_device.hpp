// Device-side building blocks shared by the SpMV kernels (spmv.hip) and the fused decode kernel
// (fused.hip): LDS-direct staging, tile decompression and the MFMA accumulation of a sub-chunk.
#pragma once
#include <utility>
#include "common.hpp"

namespace mstf {

#ifndef MSTF_SUB_TILES
#define MSTF_SUB_TILES 32
#endif
constexpr int kSubTiles = MSTF_SUB_TILES;      // tiles per staged piece ("sub-chunk"): 16 or 32
constexpr int kSubBytes = kSubTiles * 64 * 2;  // worst case: every tile full
constexpr int kNzLds = 2 * kSubBytes + 16;     // value double buffer + zero slot (read by lanes whose bit is clear)

#define MSTF_GLOBAL __attribute__((address_space(1)))

// The sixteen fixed vector registers of the gather statements (batch_step_exec and its quantised counterpart): the top
// of the register budget the kernels are built for - 128 registers with four wavefronts per SIMD, 80 with six.
// MSTF_GV(k): register k as a string, MSTF_GV0_3 / MSTF_GV4_7: the two aligned quads the zero reads fill,
// MSTF_GV0_1 ..: their aligned pairs (A operands of the form without packing), MSTF_GB0_3: the four registers below
// them that take that form's weights.
#ifndef MSTF_GATHER_TOP
#define MSTF_GATHER_TOP 128
#endif
#if MSTF_GATHER_TOP == 128
#define MSTF_GV0 "v112"
#define MSTF_GV1 "v113"
#define MSTF_GV2 "v114"
#define MSTF_GV3 "v115"
#define MSTF_GV4 "v116"
#define MSTF_GV5 "v117"
#define MSTF_GV6 "v118"
#define MSTF_GV7 "v119"
#define MSTF_GV8 "v120"
#define MSTF_GV9 "v121"
#define MSTF_GV10 "v122"
#define MSTF_GV11 "v123"
#define MSTF_GV12 "v124"
#define MSTF_GV13 "v125"
#define MSTF_GV14 "v126"
#define MSTF_GV15 "v127"
#define MSTF_GV0_3 "v[112:115]"
#define MSTF_GV4_7 "v[116:119]"
#define MSTF_GV0_1 "v[112:113]"
#define MSTF_GV2_3 "v[114:115]"
#define MSTF_GV4_5 "v[116:117]"
#define MSTF_GV6_7 "v[118:119]"
#define MSTF_GB0_3 "v[108:111]"
#define MSTF_GB0_1 "v[108:109]"
#define MSTF_GB2_3 "v[110:111]"
#define MSTF_GB_CLOBBER "v108", "v109", "v110", "v111"
#elif MSTF_GATHER_TOP == 80
#define MSTF_GV0 "v64"
#define MSTF_GV1 "v65"
#define MSTF_GV2 "v66"
#define MSTF_GV3 "v67"
#define MSTF_GV4 "v68"
#define MSTF_GV5 "v69"
#define MSTF_GV6 "v70"
#define MSTF_GV7 "v71"
#define MSTF_GV8 "v72"
#define MSTF_GV9 "v73"
#define MSTF_GV10 "v74"
#define MSTF_GV11 "v75"
#define MSTF_GV12 "v76"
#define MSTF_GV13 "v77"
#define MSTF_GV14 "v78"
#define MSTF_GV15 "v79"
#define MSTF_GV0_3 "v[64:67]"
#define MSTF_GV4_7 "v[68:71]"
#define MSTF_GV0_1 "v[64:65]"
#define MSTF_GV2_3 "v[66:67]"
#define MSTF_GV4_5 "v[68:69]"
#define MSTF_GV6_7 "v[70:71]"
#define MSTF_GB0_3 "v[60:63]"
#define MSTF_GB0_1 "v[60:61]"
#define MSTF_GB2_3 "v[62:63]"
#define MSTF_GB_CLOBBER "v60", "v61", "v62", "v63"
#else
#error "MSTF_GATHER_TOP: 128 or 80"
#endif
#define MSTF_GV_CLOBBER                                                                                            \
    MSTF_GV0, MSTF_GV1, MSTF_GV2, MSTF_GV3, MSTF_GV4, MSTF_GV5, MSTF_GV6, MSTF_GV7, MSTF_GV8, MSTF_GV9, MSTF_GV10, \
        MSTF_GV11, MSTF_GV12, MSTF_GV13, MSTF_GV14, MSTF_GV15

typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef float f4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ h4_t as_h4(uint32_t lo, uint32_t hi)
{
    const u32x2_t v = {lo, hi};
    return __builtin_bit_cast(h4_t, v);
}

__device__ __forceinline__ void wait_vm0() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void wait_lgkm0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// LDS-direct loads: data goes from global memory straight into LDS without passing through
// registers; lane l of the instruction writes `size` bytes at dst + l*size.  Completion is
// tracked by vmcnt only, the caller waits with wait_vm0() before reading the LDS.
__device__ __forceinline__ void dma16(const void* src, void* dst_wave_uniform)
{
    __builtin_amdgcn_global_load_lds((MSTF_GLOBAL const void*)src, (MSTF_LDS void*)dst_wave_uniform, 16, 0, 0);
}
__device__ __forceinline__ void dma4(const void* src, void* dst_wave_uniform)
{
    __builtin_amdgcn_global_load_lds((MSTF_GLOBAL const void*)src, (MSTF_LDS void*)dst_wave_uniform, 4, 0, 0);
}

// (16-bit LDS loads cannot merge into one register here: with SRAM ECC they clear the other half,
// hence the explicit pack of two tiles into one fp16x2 register.)
__device__ __forceinline__ uint32_t pack_h2(_Float16 lo, _Float16 hi)
{
    h2_t p;
    p.x = lo;
    p.y = hi;
    return as_u32(p);
}

// Bitmaps and tile offsets of 8 consecutive tiles, in scalar registers (two scalar loads).
struct Batch {
    u32x16_t mv;  // 8 bitmaps as (lo, hi) pairs
    u32x8_t ov;   // idx of the 8 tiles (4-byte units from the start of the KV head's values)
};

#ifndef MSTF_DUAL_ACC
#define MSTF_DUAL_ACC 1
#endif

// batch_step_exec (below) for one accumulator group (at most four query heads per KV head), without the packing of
// two tiles into one register: the tiles with an even index are gathered into the low half of their register, the odd
// ones into the high half (ds_read_u16_d16_hi; the other half of every register is zero, from the clearing move for
// the lanes without an element and from the load itself or that move for the others).  A register pair of two even
// tiles then is the A operand (t0, 0, t2, 0), a pair of two odd ones (0, t1, 0, t3), and both multiply the same B
// operand (w0, w1, w2, w3): two products where the packed form needs one, but no vector instruction to pack.  The
// products of the even tiles add up in acc, those of the odd ones in acc2 (the caller adds the two when the walk is
// over), so that two products on the same accumulator are always two instructions apart, which is what the matrix
// pipeline asks for, and the first four tiles are multiplied while the last four are still on their way from LDS
// (LDS reads return in order, and the scalar loads of the coming batch, on the same counter, can only make that
// first wait longer).  The statement ends with the wait states the matrix pipeline's results need before an ordinary
// vector instruction may read them: the compiler cannot see the products in here, and under register pressure it does
// put such reads - copies of the sums - right behind the statement (results then differ from run to run).  The
// gather registers are cleared by four 64-bit vector moves instead of two 16-byte LDS reads of a zero slot (the LDS
// pipe moves 16 bytes per lane for each of those); the weights arrive in four more fixed registers (MSTF_GB0_3).
// Same-run comparisons at batch 8 for the fused kernel: 18.6 us with the packed form, 18.1 us with this one, 17.3 us
// with the wait states at its end (the copies the compiler placed there stalled on the matrix pipeline before).
template <bool PREFETCH, int BOFF, int IOFF, int WOFF>
__device__ __forceinline__ void batch_step_dual(const Batch& b, Batch& nxt, const uint64_t* nbm, const uint32_t* nix,
                                                uint32_t rel, uint32_t wbase, f4_t& acc, f4_t& acc2)
{
    uint32_t t;
#define MSTF_TILE(I, LD, H, A)                                   \
    "s_brev_b64 exec, %[m" #I "]\n\t"                            \
    "v_mbcnt_lo_u32_b32 " A ", exec_lo, 0\n\t"                   \
    "v_mbcnt_hi_u32_b32 " A ", exec_hi, " A "\n\t"               \
    "s_lshl2_add_u32 %[t], %[o" #I "], %[rel]\n\t"               \
    "v_lshl_add_u32 " A ", " A ", 1, %[t]\n\t"                   \
    LD " " H ", " A "\n\t"
#define MSTF_LO "ds_read_u16"
#define MSTF_HI "ds_read_u16_d16_hi"
#define MSTF_CLEAR8                                                                                                  \
    "v_mov_b64 " MSTF_GV0_1 ", 0\n\tv_mov_b64 " MSTF_GV2_3 ", 0\n\tv_mov_b64 " MSTF_GV4_5 ", 0\n\tv_mov_b64 " MSTF_GV6_7 ", 0\n\t"
#define MSTF_GATHER                                                                                                  \
    "ds_read_b128 " MSTF_GB0_3 ", %[wa] offset:%[woff]\n\t"                                                          \
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
#define MSTF_GATHER_IN                                                                                               \
    [m0] "s"(u64_of(b.mv[0], b.mv[1])), [m1] "s"(u64_of(b.mv[2], b.mv[3])), [m2] "s"(u64_of(b.mv[4], b.mv[5])),      \
        [m3] "s"(u64_of(b.mv[6], b.mv[7])), [m4] "s"(u64_of(b.mv[8], b.mv[9])), [m5] "s"(u64_of(b.mv[10], b.mv[11])), \
        [m6] "s"(u64_of(b.mv[12], b.mv[13])), [m7] "s"(u64_of(b.mv[14], b.mv[15])), [o0] "s"(b.ov[0]),               \
        [o1] "s"(b.ov[1]), [o2] "s"(b.ov[2]), [o3] "s"(b.ov[3]), [o4] "s"(b.ov[4]), [o5] "s"(b.ov[5]),               \
        [o6] "s"(b.ov[6]), [o7] "s"(b.ov[7]), [rel] "s"(rel), [wa] "v"(wbase), [woff] "i"(WOFF)
#define MSTF_GATHER_CLOBBER MSTF_GV_CLOBBER, MSTF_GB_CLOBBER, "scc", "memory"
    if constexpr (PREFETCH) {
        asm volatile(MSTF_CLEAR8 "s_load_dwordx16 %[nm], %[nb], %[boff]\n\t"
                     "s_load_dwordx8 %[no], %[ni], %[ioff]\n\t" MSTF_GATHER
                     : [aa] "+v"(acc), [ab] "+v"(acc2), [t] "=&s"(t), [nm] "=&s"(nxt.mv), [no] "=&s"(nxt.ov)
                     : MSTF_GATHER_IN, [nb] "s"(nbm), [ni] "s"(nix), [boff] "i"(BOFF), [ioff] "i"(IOFF)
                     : MSTF_GATHER_CLOBBER);
    } else {
        asm volatile(MSTF_CLEAR8 MSTF_GATHER
                     : [aa] "+v"(acc), [ab] "+v"(acc2), [t] "=&s"(t)
                     : MSTF_GATHER_IN
                     : MSTF_GATHER_CLOBBER);
        nxt = b;
    }
#undef MSTF_TILE
#undef MSTF_LO
#undef MSTF_HI
#undef MSTF_CLEAR8
#undef MSTF_GATHER
#undef MSTF_GATHER_IN
#undef MSTF_GATHER_CLOBBER
}
// The sums a chain of batch_step_dual statements left in acc and acc2 are read by ordinary vector instructions next:
// the matrix pipeline's results are not interlocked against those, hence the wait states here (once per walk).  The
// sums pass through the statement, so that none of their readers can be scheduled in front of it.
__device__ __forceinline__ void dual_settle(f4_t& acc, f4_t& acc2)
{
    asm volatile("s_nop 7" : "+v"(acc), "+v"(acc2)::"memory");
}

// Decompresses 8 staged tiles and accumulates them.  For every group of 4 tiles the lane builds its own
// four values D[t..t+3][lane] (A operand) and reads the four weights of "its" accumulator (lane & 3) of each
// accumulator group from LDS (B operand); v_mfma_f32_4x4x4f16 then yields, in lane 4b+j, the sums of
// positions 4b..4b+3 for accumulator 4m+j:
//     acc[m][r] += sum_t D[t][4b + r] * w[4m + j][t]
//   rel    : LDS byte address of the staged values minus 4 * idx of the first staged tile
//   zaddr  : LDS address of 16 zero bytes
//   wgroup : bytes between groups of 4 weight rows
// The gather runs with the wavefront's exec mask set to each tile's bitmap in turn: only the lanes whose element is
// present compute a rank and read LDS, the others keep the zero their destination was cleared to (four destinations
// per 16-byte LDS read of the zero slot at zaddr; LDS reads of a wavefront return in order, so the gathers land on
// top), so the select instruction disappears - per tile one s_brev_b64 into exec, two v_mbcnt on exec, the
// scalar base, one v_lshl_add and the LDS read.  It is one statement on fixed registers (MSTF_GV0 .. 15: v112-v127, the top of the
// budget of a kernel that runs four wavefronts per SIMD, listed as clobbered) because nothing of the compiler's may
// be scheduled while exec is partial.  The statement saves the exec mask it is entered with and hands it back, but
// between the two every tile runs under its own bitmap: callers sit in wave-uniform control flow with all 64 lanes
// active (every kernel that uses it is launched with a multiple of 64 threads and branches only on wave-uniform values
// around it).  The scalar loads of the coming batch (PREFETCH) are part of the
// statement: requested first, completed by its one wait - the compiler, which cannot see that wait, would otherwise
// put one of its own in front of the statement and expose the round trip of a request it has just made.
//   nbm + BOFF bytes, nix + IOFF bytes : bitmaps and offsets of the coming batch
//   wbase + WOFF                      : LDS byte address of w[lane & 3][first tile of the batch]
template <int NM, bool PREFETCH, int BOFF, int IOFF, int WOFF>
__device__ __forceinline__ void batch_step_exec(const Batch& b, Batch& nxt, const uint64_t* nbm, const uint32_t* nix,
                                                uint32_t rel, uint32_t zaddr, uint32_t wbase, uint32_t wgroup,
                                                f4_t (&acc)[NM], f4_t (&acc2)[NM])
{
    // acc2: second set of sums, used (and to be added to acc by the caller) only in the form without packing
    if constexpr (NM == 1 && MSTF_DUAL_ACC) {
        batch_step_dual<PREFETCH, BOFF, IOFF, WOFF>(b, nxt, nbm, nix, rel, wbase, acc[0], acc2[0]);
        return;
    }
    u32x4_t qm[NM];
#pragma unroll
    for (int m = 1; m < NM; m++) qm[m] = *(MSTF_LDS const u32x4_t*)(uintptr_t)(wbase + (uint32_t)WOFF + (uint32_t)m * wgroup);
    uint32_t v0, v1, v2, v3, t;
    uint64_t sv;  // the exec mask the statement was entered with, handed back at its end
#define MSTF_TILE(I, H, A)                                       \
    "s_brev_b64 exec, %[m" #I "]\n\t"                            \
    "v_mbcnt_lo_u32_b32 " A ", exec_lo, 0\n\t"                   \
    "v_mbcnt_hi_u32_b32 " A ", exec_hi, " A "\n\t"               \
    "s_lshl2_add_u32 %[t], %[o" #I "], %[rel]\n\t"               \
    "v_lshl_add_u32 " A ", " A ", 1, %[t]\n\t"                   \
    "ds_read_u16 " H ", " A "\n\t"
#define MSTF_GATHER                                                                                                  \
    "s_mov_b64 %[sv], exec\n\t"                                                                                      \
    "ds_read_b128 %[qm], %[wa] offset:%[woff]\n\t"                                                                   \
    "ds_read_b128 " MSTF_GV0_3 ", %[z]\n\t"                                                                                  \
    "ds_read_b128 " MSTF_GV4_7 ", %[z]\n\t"                                                                                  \
    MSTF_TILE(0, MSTF_GV0, MSTF_GV8) MSTF_TILE(1, MSTF_GV1, MSTF_GV9) MSTF_TILE(2, MSTF_GV2, MSTF_GV10) MSTF_TILE(3, MSTF_GV3, MSTF_GV11)                              \
    MSTF_TILE(4, MSTF_GV4, MSTF_GV12) MSTF_TILE(5, MSTF_GV5, MSTF_GV13) MSTF_TILE(6, MSTF_GV6, MSTF_GV14) MSTF_TILE(7, MSTF_GV7, MSTF_GV15)                              \
    "s_mov_b64 exec, %[sv]\n\t"                                                                                      \
    "s_waitcnt lgkmcnt(0)\n\t"                                                                                       \
    "v_lshl_or_b32 %[v0], " MSTF_GV1 ", 16, " MSTF_GV0 "\n\t"                                                                          \
    "v_lshl_or_b32 %[v1], " MSTF_GV3 ", 16, " MSTF_GV2 "\n\t"                                                                          \
    "v_lshl_or_b32 %[v2], " MSTF_GV5 ", 16, " MSTF_GV4 "\n\t"                                                                          \
    "v_lshl_or_b32 %[v3], " MSTF_GV7 ", 16, " MSTF_GV6
#define MSTF_GATHER_IN                                                                                               \
    [m0] "s"(u64_of(b.mv[0], b.mv[1])), [m1] "s"(u64_of(b.mv[2], b.mv[3])), [m2] "s"(u64_of(b.mv[4], b.mv[5])),      \
        [m3] "s"(u64_of(b.mv[6], b.mv[7])), [m4] "s"(u64_of(b.mv[8], b.mv[9])), [m5] "s"(u64_of(b.mv[10], b.mv[11])), \
        [m6] "s"(u64_of(b.mv[12], b.mv[13])), [m7] "s"(u64_of(b.mv[14], b.mv[15])), [o0] "s"(b.ov[0]),               \
        [o1] "s"(b.ov[1]), [o2] "s"(b.ov[2]), [o3] "s"(b.ov[3]), [o4] "s"(b.ov[4]), [o5] "s"(b.ov[5]),               \
        [o6] "s"(b.ov[6]), [o7] "s"(b.ov[7]), [rel] "s"(rel), [wa] "v"(wbase), [woff] "i"(WOFF), [z] "v"(zaddr)
#define MSTF_GATHER_CLOBBER                                                                                          \
    MSTF_GV_CLOBBER, "scc", "memory"
    if constexpr (PREFETCH) {
        asm volatile("s_load_dwordx16 %[nm], %[nb], %[boff]\n\t"
                     "s_load_dwordx8 %[no], %[ni], %[ioff]\n\t" MSTF_GATHER
                     : [v0] "=&v"(v0), [v1] "=&v"(v1), [v2] "=&v"(v2), [v3] "=&v"(v3), [qm] "=&v"(qm[0]), [t] "=&s"(t),
                       [sv] "=&s"(sv), [nm] "=&s"(nxt.mv), [no] "=&s"(nxt.ov)
                     : MSTF_GATHER_IN, [nb] "s"(nbm), [ni] "s"(nix), [boff] "i"(BOFF), [ioff] "i"(IOFF)
                     : MSTF_GATHER_CLOBBER);
    } else {
        asm volatile(MSTF_GATHER
                     : [v0] "=&v"(v0), [v1] "=&v"(v1), [v2] "=&v"(v2), [v3] "=&v"(v3), [qm] "=&v"(qm[0]), [t] "=&s"(t),
                       [sv] "=&s"(sv)
                     : MSTF_GATHER_IN
                     : MSTF_GATHER_CLOBBER);
        nxt = b;
    }
#undef MSTF_TILE
#undef MSTF_GATHER
#undef MSTF_GATHER_IN
#undef MSTF_GATHER_CLOBBER
#pragma unroll
    for (int m = 0; m < NM; m++) {
        acc[m] = __builtin_amdgcn_mfma_f32_4x4x4f16(as_h4(v0, v1), as_h4(qm[m][0], qm[m][1]), acc[m], 0, 0, 0);
        acc[m] = __builtin_amdgcn_mfma_f32_4x4x4f16(as_h4(v2, v3), as_h4(qm[m][2], qm[m][3]), acc[m], 0, 0, 0);
        // pins the products here: left free, they may all be sunk to the first use of the sums, with every
        // batch's operands kept in registers until then
        asm volatile("" : "+v"(acc[m]));
    }
}

// The first batch of a chain for batch_step_exec: requested and waited for in one statement, so that the values are
// in scalar registers whatever the compiler makes of other loads through the same pointers.
__device__ __forceinline__ Batch load_batch_scalar(const uint64_t* bm, const uint32_t* ix)
{
    Batch b;
    asm volatile("s_load_dwordx16 %0, %2, 0\n\ts_load_dwordx8 %1, %3, 0\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(b.mv), "=&s"(b.ov)
                 : "s"(bm), "s"(ix)
                 : "memory");
    return b;
}

// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{}): a loop whose index is a
// constant expression in the body (immediate operands of the statement above).
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f)
{
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}


__device__ __forceinline__ uint32_t sub_bytes(uint32_t start, uint32_t end)
{
    const uint32_t b = (end - start) * 4u;
    return b > (uint32_t)kSubBytes ? (uint32_t)kSubBytes : b;  // a well-formed sub-chunk never exceeds this
}

// The decompression reads bitmaps and tile offsets through the scalar cache.  So that those loads find
// their lines in L2 instead of waiting for HBM, every lane also touches one bitmap / one offset of the
// coming sub-chunk with a coalesced vector load, issued together with the value stream of that sub-chunk
// and completed by the same wait.
struct Touch {
    uint2 bm;
    uint32_t ix;
};
// Waits for every outstanding vector-memory operation (LDS-direct loads included).
__device__ __forceinline__ void wait_vm0_keep(Touch& t)
{
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(t.bm.x), "+v"(t.bm.y), "+v"(t.ix)::"memory");
}

// sub_issue and touch_sub without control flow, for a caller that keeps scalar state (the coming batch) in
// registers across them: a lane predicate written as a branch splits the block there, and values that live
// across such a split may end up in vector registers.  The four (two for 16-tile stages) pieces are issued with exec set by hand
// (piece i: the lanes with lane*16 + i*1024 < bytes; an empty exec issues nothing) - one compare, one exec write
// and the load per piece, where the branches cost ten instructions; the wavefront must have all 64 lanes active.
//   dst_lds : LDS byte address of the buffer (wave-uniform);  lane16 = lane * 16
__device__ __forceinline__ void sub_issue_flat(const char* src, uint32_t bytes, uint32_t dst_lds, uint32_t lane16)
{
    static_assert(kSubBytes == 4096 || kSubBytes == 2048, "four or two 1 KB pieces");
    uint32_t t, m0_kept;  // m0 is the compiler's to manage: handed back as it was found
    // exec is set by hand per piece and handed back as all ones (what the caller has, see above); the pieces behind
    // the stage's last byte are jumped over (the byte count is wave-uniform), typically two of the four
#define MSTF_SHEAD                   \
    "s_mov_b32 %[keep], m0\n\t"      \
    "s_mov_b32 m0, %[dst]\n\t"       \
    "v_cmp_gt_i32 vcc, %[b], %[l]\n\t" \
    "s_mov_b64 exec, vcc\n\t"        \
    "global_load_lds_dwordx4 %[l], %[src]\n\t"
#define MSTF_SPIECE(HEX, OFF)                \
    "s_cmp_le_i32 %[b], " HEX "\n\t"         \
    "s_cbranch_scc1 9f\n\t"                  \
    "s_sub_i32 %[t], %[b], " HEX "\n\t"      \
    "v_cmp_gt_i32 vcc, %[t], %[l]\n\t"       \
    "s_mov_b64 exec, vcc\n\t"                \
    "global_load_lds_dwordx4 %[l], %[src] offset:" OFF "\n\t"
#define MSTF_STAIL "9:\n\ts_mov_b64 exec, -1\n\ts_mov_b32 m0, %[keep]"
#define MSTF_SOPS                                                           \
    : [t] "=&s"(t), [keep] "=&s"(m0_kept)                                   \
    : [dst] "s"(dst_lds), [b] "s"(bytes), [l] "v"(lane16), [src] "s"(src)   \
    : "vcc", "scc", "memory"
    if constexpr (kSubBytes == 4096)
        asm volatile(MSTF_SHEAD MSTF_SPIECE("0x400", "1024") MSTF_SPIECE("0x800", "2048") MSTF_SPIECE("0xc00", "3072")
                         MSTF_STAIL MSTF_SOPS);
    else
        asm volatile(MSTF_SHEAD MSTF_SPIECE("0x400", "1024") MSTF_STAIL MSTF_SOPS);
#undef MSTF_SHEAD
#undef MSTF_SPIECE
#undef MSTF_STAIL
#undef MSTF_SOPS
}
// Every lane touches one bitmap and one offset of the sub-chunk; the lanes beyond it repeat the last one.
//   off8 = min(lane, kSubTiles - 1) * 8, off4 = min(lane, kSubTiles) * 4
__device__ __forceinline__ Touch touch_sub_flat(const uint64_t* bm, const uint32_t* ix, uint32_t off8, uint32_t off4)
{
    Touch t;
    t.bm = *reinterpret_cast<const uint2*>(reinterpret_cast<const char*>(bm) + off8);
    t.ix = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const char*>(ix) + off4);
    return t;
}

// Walks `nsubs` sub-chunks of one KV head with a two-deep pipeline: while sub-chunk n is being
// decompressed out of one LDS buffer, sub-chunk n+1 streams from HBM into the other.
//   tile_of(n)    : first tile of sub-chunk n
//   stage_w(n)    : issues the LDS-direct loads of the weights sub-chunk n needs (may be a no-op)
//   waddr_of(n)   : LDS byte address of w[lane & 3][first tile of sub-chunk n]
template <int NM, class TileOf, class StageW, class WAddrOf>
__device__ __forceinline__ void walk_subs(int nsubs, TileOf tile_of, StageW stage_w, WAddrOf waddr_of, uint32_t wgroup,
                                          const uint64_t* bmk, const uint32_t* ixk, const char* nzk, char* my, int lane,
                                          f4_t (&acc)[NM])
{
    // stage_w must be free of lane-dependent branches: the coming scalar batch is live across it (see sub_issue_flat)
    const uint32_t lbase = lds_addr(my);
    const uint32_t zaddr = lbase + 2 * kSubBytes;
    if (lane < 4) reinterpret_cast<uint32_t*>(my + 2 * kSubBytes)[lane] = 0u;
    if (nsubs <= 0) return;
    const uint32_t lane16 = (uint32_t)lane * 16u;
    const uint32_t off8 = (uint32_t)(lane < kSubTiles ? lane : kSubTiles - 1) * 8u;
    const uint32_t off4 = (uint32_t)(lane <= kSubTiles ? lane : kSubTiles) * 4u;
    size_t t_cur = tile_of(0);
    // (the offsets may come back through a vector load; the statements below want them in scalar registers)
    auto uni = [](uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); };
    const uint32_t s0 = uni(ixk[t_cur]);
    sub_issue_flat(nzk + (size_t)s0 * 4u, sub_bytes(s0, uni(ixk[t_cur + kSubTiles])), lbase, lane16);
    stage_w(0);
    Touch touch = touch_sub_flat(bmk + t_cur, ixk + t_cur, off8, off4);
    size_t t_nxt = nsubs > 1 ? tile_of(1) : t_cur;
    uint32_t s_nxt = uni(ixk[t_nxt]), e_nxt = uni(ixk[t_nxt + kSubTiles]);
    Batch cur = load_batch_scalar(bmk + t_cur, ixk + t_cur);
    constexpr int G = kSubTiles / 8;
    f4_t acc2[NM];  // second set of sums of the form without packing (batch_step_dual)
#pragma unroll
    for (int m = 0; m < NM; m++) acc2[m] = f4_t{0.f, 0.f, 0.f, 0.f};
    for (int n = 0; n < nsubs; n++) {
        set_wave_priority_uniform(3u - ((uint32_t)n & 3u));  // falls from stage to stage (see set_wave_priority)
        wait_vm0_keep(touch);  // sub-chunk n (values, weights) has landed
        // Buffer (n+1)&1 is refilled now.  Its last reader was sub-chunk n-1, and every LDS read of that sub-chunk
        // fed an MFMA issued before this point, so the reads have returned.
        __builtin_amdgcn_sched_barrier(0);
        if (n + 1 < nsubs) {
            sub_issue_flat(nzk + (size_t)s_nxt * 4u, sub_bytes(s_nxt, e_nxt), lbase + (uint32_t)((n + 1) & 1) * kSubBytes,
                           lane16);
            stage_w(n + 1);
            touch = touch_sub_flat(bmk + t_nxt, ixk + t_nxt, off8, off4);
        }
        const size_t t_now = t_cur;
        t_cur = t_nxt;
        if (n + 2 < nsubs) {
            t_nxt = tile_of(n + 2);
            s_nxt = uni(ixk[t_nxt]);
            e_nxt = uni(ixk[t_nxt + kSubTiles]);
        }
        const uint32_t rel = lbase + (uint32_t)(n & 1) * kSubBytes - cur.ov[0] * 4u;
        const uint32_t wbase = waddr_of(n);
        const uint64_t* bm_now = bmk + t_now;
        const uint32_t* ix_now = ixk + t_now;
        static_for<G>([&](auto gc) {
            constexpr int g = decltype(gc)::value;
            Batch nxt;
            if constexpr (g + 1 < G)
                batch_step_exec<NM, true, (g + 1) * 64, (g + 1) * 32, g * 16>(cur, nxt, bm_now, ix_now, rel, zaddr, wbase,
                                                                             wgroup, acc, acc2);
            else  // the first batch of the coming sub-chunk (of this one again after the last: loaded, never used)
                batch_step_exec<NM, true, 0, 0, g * 16>(cur, nxt, bmk + t_cur, ixk + t_cur, rel, zaddr, wbase, wgroup, acc,
                                                        acc2);
            cur = nxt;
        });
        __builtin_amdgcn_sched_barrier(0);
    }
    wait_lgkm0();
    if constexpr (NM == 1 && MSTF_DUAL_ACC) {
        dual_settle(acc[0], acc2[0]);
        acc[0] += acc2[0];
    }
}

}  // namespace mstf
