// Key / value SpMV over the quantised bitmap format, with dequantisation fused into the decompression.
//
// Same work decomposition, LDS-direct staging and MFMA accumulation as the fp16 kernels (spmv.hip); what
// differs is how a staged run of 32 tiles becomes fp16 values:
//   1. the run's packed words (contiguous in `packed`) and its per-tile metadata (word offsets, scales,
//      zero-points) stream HBM -> LDS one stage ahead;
//   2. dequantisation happens in the packed domain: one lane per packed word unpacks its 16 / 8 / 4 codes
//      and writes the fp16 values, in rank order, into a fixed-stride tile image in LDS (128 bytes per
//      tile), so the cost is per non-zero word, not per dense position;
//   3. the image is expanded exactly like the fp16 format (bitmap rank -> LDS gather -> MFMA), with the
//      tile base a constant instead of idx.
// Dequantised value = fp16( (q - zero) * scale ).  For |zero| <= 1024 this is computed with packed fp16
// arithmetic and is the same number the reference's fp32 (dequant_mode 0) and fp16 (dequant_mode 1)
// sequences give: 0x6400 | q is the fp16 number 1024 + q, subtracting 1024 + zero is exact, and the one
// remaining multiplication by scale rounds the exact product once.  Tiles with a larger zero-point take
// the literal per-mode arithmetic.
#include "quant_device.hpp"
#include "spmv_common.hpp"

namespace mstf {

#pragma clang fp contract(off)

// Pointers of one KV-head-agnostic quantised cache.  `off_dma`, `scales`, `zeros`, `packed` feed LDS-direct
// loads; `off` is the same array as `off_dma`, kept as a separate, never-escaping pointer so that the stage
// boundaries are still fetched with scalar loads.
struct QCache {
    const uint64_t* bmp;
    const uint32_t* off;
    const uint32_t* off_dma;
    const uint16_t* scales;
    const uint16_t* zeros;
    const uint32_t* packed;
};

// Walks `nsubs` stages of 32 tiles with a two-deep pipeline (see walk_subs).  Tile indices are global
// (KV head included): tile_off / scales / zeros / bmp are flat over [Bkv, T].
template <int NM, int BIT, bool G32, class TileOf, class StageW, class WAddrOf>
__device__ __forceinline__ void walk_subs_q(int nsubs, TileOf tile_of, StageW stage_w, WAddrOf waddr_of, uint32_t wgroup,
                                            const QCache& c, char* my, int lane, int mode, f4_t (&acc)[NM])
{
    using F = QFmt<BIT>;
    const uint32_t lbase = lds_addr(my);
    const uint32_t zaddr = lbase + kImgBytes;
    char* wordbuf = my + kImgBytes + 16;
    char* metabuf = wordbuf + 2 * F::kWordBuf;
    if (lane < 4) reinterpret_cast<uint32_t*>(my + kImgBytes)[lane] = 0u;
    if (nsubs <= 0) return;

    // words of the stage starting at tile t: [tile_off[t], tile_off[t + 31] + words of tile t + 31)
    auto bounds = [&](size_t t, uint32_t& s, uint32_t& e) {
        s = c.off[t];
        const uint32_t cnt = (uint32_t)__builtin_popcountll(c.bmp[t + kSubTiles - 1]);
        e = c.off[t + kSubTiles - 1] + ((cnt + (uint32_t)F::kCap - 1u) >> F::kCapShift);
    };
    constexpr int kMetaBytes = meta_bytes<G32>();
    const MetaLanes meta = meta_lanes<G32>(c.off_dma, c.scales, c.zeros, c.bmp, lane);
    const uint32_t lane4 = (uint32_t)lane * 4u;
    const uint32_t touch8 = (uint32_t)(lane < kSubTiles ? lane : kSubTiles - 1) * 8u;
    const uint32_t wordbuf_lds = lds_addr(wordbuf);
    auto uni = [](uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); };
    // (no lane-dependent branches in the word and metadata loads: exec set by hand, clamped touch address)
    auto issue = [&](int n, size_t t, uint32_t s, uint32_t e) {
        uint32_t nw = uni(e) - uni(s);
        nw = nw > (uint32_t)F::kWordsMax ? (uint32_t)F::kWordsMax : nw;  // never true for a well-formed cache
        words_issue_flat<F::kWordsMax / 64>(c.packed + uni(s), nw, wordbuf_lds + (uint32_t)(n & 1) * F::kWordBuf,
                                            (uint32_t)lane, lane4);
        // metadata: lanes 0..31 the word offsets, 32..47 the scales, 48..63 the zero-points (two per lane); two loads
        // when a tile has two (scale, zero) pairs
        meta_issue<G32>(meta, (uint32_t)t, metabuf + (n & 1) * kMetaBytes);
        stage_w(n);
        // pulls the stage's bitmaps into L2 ahead of the scalar loads of the expansion
        return *reinterpret_cast<const uint2*>(reinterpret_cast<const char*>(c.bmp + t) + touch8);
    };

    f4_t acc2[NM];  // second set of sums of the gather statements (batch_step_img_dual)
#pragma unroll
    for (int m = 0; m < NM; m++) acc2[m] = f4_t{0.f, 0.f, 0.f, 0.f};
    size_t t_cur = tile_of(0);
    uint32_t s_cur, e_cur;
    bounds(t_cur, s_cur, e_cur);
    uint2 touch = issue(0, t_cur, s_cur, e_cur);
    size_t t_nxt = nsubs > 1 ? tile_of(1) : t_cur;
    uint32_t s_nxt, e_nxt;
    bounds(t_nxt, s_nxt, e_nxt);
    for (int n = 0; n < nsubs; n++) {
        set_wave_priority_uniform(3u - ((uint32_t)n & 3u));  // falls from stage to stage (see set_wave_priority)
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(touch.x), "+v"(touch.y)::"memory");  // stage n has landed
        const uint2 bits = touch;  // lane l < 32: bitmap l of stage n
        if (n + 1 < nsubs) touch = issue(n + 1, t_nxt, s_nxt, e_nxt);
        const size_t t_now = t_cur;
        const uint32_t s_now = s_cur, e_now = e_cur;
        t_cur = t_nxt;
        s_cur = s_nxt;
        e_cur = e_nxt;
        if (n + 2 < nsubs) {
            t_nxt = tile_of(n + 2);
            bounds(t_nxt, s_nxt, e_nxt);
        }
        dequant_stage<BIT, G32>(lds_addr(metabuf) + (uint32_t)(n & 1) * kMetaBytes,
                           lds_addr(wordbuf) + (uint32_t)(n & 1) * F::kWordBuf, lbase, s_now, uni(e_now), lane, mode);
        const uint64_t* bm = c.bmp + t_now;
        const uint32_t waddr = waddr_of(n);
        stage_img_exec<NM>(bm, bits.x, bits.y, lbase, zaddr, waddr, wgroup, acc, acc2);
        wait_lgkm0();  // every read of the image and of the staged buffers is done before they are rewritten
    }
    if constexpr (NM == 1 && MSTF_DUAL_ACC) {
        dual_settle(acc[0], acc2[0]);
        acc[0] += acc2[0];
    }
}

// ------------------------------------------------------------------------------- key
// One wavefront per (KV head, token block); see key_spmv_kernel.
template <int NW, int BIT, bool G32>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4))) void key_spmv_quant_kernel(
    const uint64_t* __restrict__ bmp, const uint32_t* packed, const uint32_t* __restrict__ tile_off,
    const uint32_t* tile_off_dma, const uint16_t* scales, const uint16_t* zeros, const _Float16* Bm,
    _Float16* __restrict__ C, int Lc, int D, int nblk, int ntasks, int rows_per_kv, int row0, int mode)
{
    constexpr int NM = (NW + 3) / 4;
    constexpr int kMaxD = 128;
    constexpr int kQ = q_lds_bytes<BIT, G32>();
    constexpr int kWaveLds = kQ + NM * 4 * kMaxD * 2;
    __shared__ __attribute__((aligned(16))) char lds[4][kWaveLds];
    const int lane = lane_id();
    const int wave = wave_id();
    // neighbouring token blocks on the same XCD: their packed words share cache lines
    const int task = xcd_contiguous((int)blockIdx.x, (ntasks + 3) / 4) * 4 + wave;
    if (task >= ntasks) return;
    const int kv = task / nblk;
    const int tb = task - kv * nblk;
    const size_t T = (size_t)Lc * D / 64;
    const QCache c = {bmp, tile_off, tile_off_dma, scales, zeros, packed};
    const char* wsrc = reinterpret_cast<const char*>(Bm + ((size_t)kv * rows_per_kv + row0) * D);
    char* my = lds[wave];
    char* wl = my + kQ;  // [4*NM rows][D] fp16; rows >= NW stay unwritten
    const uint32_t wbytes = (uint32_t)NW * D * 2u;

    f4_t acc[NM];
#pragma unroll
    for (int m = 0; m < NM; m++) acc[m] = f4_t{0.f, 0.f, 0.f, 0.f};
    const size_t tile0 = (size_t)kv * T + (size_t)tb * D;
    const uint32_t wrow = lds_addr(wl) + (uint32_t)(lane & 3) * (uint32_t)D * 2u;
    walk_subs_q<NM, BIT, G32>(
        D / kSubTiles, [=](int n) { return tile0 + (size_t)n * kSubTiles; },
        [=](int n) {
            if (n != 0) return;  // the query rows are staged once per task
#pragma unroll
            for (int i = 0; i < (NW * kMaxD * 2 + 1023) / 1024; i++) {
                const uint32_t o = (uint32_t)(i * 64 + lane) * 16u;
                if (o < wbytes) dma16(wsrc + o, wl + i * 1024);
            }
        },
        [=](int n) { return wrow + (uint32_t)n * kSubTiles * 2u; }, (uint32_t)D * 8u, c, my, lane, mode, acc);
    // lane 4b+j holds tokens 4b..4b+3 of accumulator 4m+j
    const int j = lane & 3;
    _Float16* out = C + ((size_t)kv * rows_per_kv + row0) * Lc + (size_t)tb * 64 + (lane & ~3);
#pragma unroll
    for (int m = 0; m < NM; m++) {
        if (4 * m + j < NW) {
            h4_t o;
            o[0] = (_Float16)acc[m][0];
            o[1] = (_Float16)acc[m][1];
            o[2] = (_Float16)acc[m][2];
            o[3] = (_Float16)acc[m][3];
            *reinterpret_cast<h4_t*>(out + (size_t)(4 * m + j) * Lc) = o;
        }
    }
}

// ------------------------------------------------------------------------------- value
// grid = xcd_grid(token splits x D/64 halves x KV heads), halves fastest in the logical index: the two halves of a
// token range read the same weights and interleaved cache lines, so they run on the same XCD; see value_spmv_kernel.
template <int NW, int WAVES, int BIT, bool G32>
__global__ __launch_bounds__(WAVES * 64) void value_spmv_quant_kernel(
    const uint64_t* __restrict__ bmp, const uint32_t* packed, const uint32_t* __restrict__ tile_off,
    const uint32_t* tile_off_dma, const uint16_t* scales, const uint16_t* zeros, const _Float16* P,
    _Float16* __restrict__ C, float* __restrict__ part, int Lc, int D, int nblk, int nbpw, int nsplit, int rows_per_kv,
    int row0, int mode, int nwg)
{
    constexpr int NM = (NW + 3) / 4;
    constexpr int kWRow = kSubTiles * 2;
    constexpr int kWBuf = NM * 4 * kWRow;
    constexpr int kQ = q_lds_bytes<BIT, G32>();
    constexpr int kNeed = kQ + 2 * kWBuf;
    constexpr int kWaveLds = kNeed > NW * 256 ? kNeed : NW * 256;  // the per-wave sums are parked here at the end
    __shared__ __attribute__((aligned(16))) char lds[WAVES][kWaveLds];
    const int lane = lane_id();
    const int wave = wave_id();
    const int nhalf = D / 64;
    const int logical = xcd_contiguous((int)blockIdx.x, nwg);
    if (logical >= nwg) return;  // (the whole workgroup: no barrier is left waiting)
    const int half = logical % nhalf;
    const int split = (logical / nhalf) % nsplit;
    const int kv = logical / (nhalf * nsplit);
    const size_t T = (size_t)Lc * D / 64;
    const QCache c = {bmp, tile_off, tile_off_dma, scales, zeros, packed};
    const _Float16* wk = P + ((size_t)kv * rows_per_kv + row0) * Lc;
    char* my = lds[wave];
    char* wl = my + kQ;

    f4_t acc[NM];
#pragma unroll
    for (int m = 0; m < NM; m++) acc[m] = f4_t{0.f, 0.f, 0.f, 0.f};

    const int first = (split * WAVES + wave) * nbpw;
    int last = first + nbpw;
    if (last > nblk) last = nblk;
    constexpr int subs_per_blk = 64 / kSubTiles;
    const uint32_t wrow = lds_addr(wl) + (uint32_t)(lane & 3) * kWRow;
    const size_t thead = (size_t)kv * T + (size_t)half * 64;
    walk_subs_q<NM, BIT, G32>(
        (last - first) * subs_per_blk,
        [=](int n) { return thead + (size_t)(first + n / subs_per_blk) * D + (size_t)(n % subs_per_blk) * kSubTiles; },
        [=](int n) {
            constexpr int kDwPerRow = kSubTiles / 2, kRowsPer = 64 / kDwPerRow;
            const size_t tok0 = (size_t)(first + n / subs_per_blk) * 64 + (size_t)(n % subs_per_blk) * kSubTiles;
#pragma unroll
            for (int i = 0; i < (NM * 4 + kRowsPer - 1) / kRowsPer; i++) {
                const int row = kRowsPer * i + lane / kDwPerRow;
                if (row < NW) dma4(wk + (size_t)row * Lc + tok0 + 2 * (lane % kDwPerRow), wl + (n & 1) * kWBuf + i * 256);
            }
        },
        [=](int n) { return wrow + (uint32_t)(n & 1) * kWBuf; }, 4u * kWRow, c, my, lane, mode, acc);
    // workgroup reduction: every wavefront parks its sums [accumulator][channel] in its own LDS area
    __syncthreads();
    float* mine = reinterpret_cast<float*>(my);
    const int j = lane & 3;
#pragma unroll
    for (int m = 0; m < NM; m++) {
        if (4 * m + j < NW) *reinterpret_cast<f4_t*>(mine + (4 * m + j) * 64 + (lane & ~3)) = acc[m];
    }
    __syncthreads();
    for (int o = (int)threadIdx.x; o < NW * 64; o += WAVES * 64) {
        float s = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; wv++) s += reinterpret_cast<const float*>(lds[wv])[o];
        const int n = o >> 6, ch = o & 63;
        const size_t row = (size_t)kv * rows_per_kv + row0 + n;
        if (nsplit == 1)
            C[row * D + (size_t)half * 64 + ch] = (_Float16)s;
        else
            part[(row * nsplit + split) * D + (size_t)half * 64 + ch] = s;
    }
}

// ------------------------------------------------------------------------------- host
static int check_quant_spmv(const void* bmp, const void* packed, const void* tile_off, const void* scales,
                            const void* zeros, const void* Bm, const void* C, int tokens, int head_dim, int Bq,
                            int groups, int n_rows, int bit, int capacity, int dequant_mode)
{
    if (!bmp || !packed || !tile_off || !scales || !zeros || !Bm || !C) return MSTF_EINVAL;
    if (tokens <= 0 || head_dim <= 0 || Bq <= 0 || groups <= 0 || n_rows <= 0 || Bq % groups != 0) return MSTF_EINVAL;
    if (dequant_mode != 0 && dequant_mode != 1) return MSTF_EINVAL;
    if (bit != 2 && bit != 4 && bit != 8) return MSTF_EUNSUPPORTED;
    if (capacity != 32 / bit) return MSTF_EINVAL;
    if (tokens % 64 != 0 || head_dim % 64 != 0 || head_dim > 128) return MSTF_EUNSUPPORTED;
    if (!aligned_to(bmp, 8) || !aligned_to(packed, 4) || !aligned_to(tile_off, 4) || !aligned_to(scales, 4) ||
        !aligned_to(zeros, 4) || !aligned_to(Bm, 4) || !aligned_to(C, 2))
        return MSTF_EALIGN;
    return MSTF_OK;
}

struct QArgs {
    const uint64_t* bmp;
    const uint32_t* packed;
    const uint32_t* tile_off;
    const uint16_t* scales;
    const uint16_t* zeros;
    int mode;
    int group_size;  // 64: one (scale, zero) pair per tile; 32: two
};

template <int NW, int BIT>
static void launch_key_q(hipStream_t st, const QArgs& a, const _Float16* Bm, _Float16* C, int Lc, int D, int Bkv,
                         int rows_per_kv, int row0)
{
    const int nblk = Lc / 64;
    const int ntasks = Bkv * nblk;
    if (a.group_size == 32)
        hipLaunchKernelGGL((key_spmv_quant_kernel<NW, BIT, true>), dim3(xcd_grid((ntasks + 3) / 4)), dim3(256), 0, st, a.bmp, a.packed,
                           a.tile_off, a.tile_off, a.scales, a.zeros, Bm, C, Lc, D, nblk, ntasks, rows_per_kv, row0, a.mode);
    else
        hipLaunchKernelGGL((key_spmv_quant_kernel<NW, BIT, false>), dim3(xcd_grid((ntasks + 3) / 4)), dim3(256), 0, st, a.bmp, a.packed,
                           a.tile_off, a.tile_off, a.scales, a.zeros, Bm, C, Lc, D, nblk, ntasks, rows_per_kv, row0, a.mode);
}
template <int NW>
static void launch_key_q_bit(int bit, hipStream_t st, const QArgs& a, const _Float16* Bm, _Float16* C, int Lc, int D,
                             int Bkv, int rows_per_kv, int row0)
{
    if (bit == 2)
        launch_key_q<NW, 2>(st, a, Bm, C, Lc, D, Bkv, rows_per_kv, row0);
    else if (bit == 4)
        launch_key_q<NW, 4>(st, a, Bm, C, Lc, D, Bkv, rows_per_kv, row0);
    else
        launch_key_q<NW, 8>(st, a, Bm, C, Lc, D, Bkv, rows_per_kv, row0);
}

template <int NW, int WAVES, int BIT>
static void launch_value_q(hipStream_t st, const ValuePlan& pl, const QArgs& a, const _Float16* P, _Float16* C,
                           float* part, int Lc, int D, int Bkv, int rows_per_kv, int row0)
{
    const int nwg = pl.nsplit * (D / 64) * Bkv;
    if (a.group_size == 32)
        hipLaunchKernelGGL((value_spmv_quant_kernel<NW, WAVES, BIT, true>), dim3(xcd_grid(nwg)), dim3(WAVES * 64), 0,
                           st, a.bmp, a.packed, a.tile_off, a.tile_off, a.scales, a.zeros, P, C, part, Lc, D, Lc / 64,
                           pl.nbpw, pl.nsplit, rows_per_kv, row0, a.mode, nwg);
    else
        hipLaunchKernelGGL((value_spmv_quant_kernel<NW, WAVES, BIT, false>), dim3(xcd_grid(nwg)), dim3(WAVES * 64), 0,
                           st, a.bmp, a.packed, a.tile_off, a.tile_off, a.scales, a.zeros, P, C, part, Lc, D, Lc / 64,
                           pl.nbpw, pl.nsplit, rows_per_kv, row0, a.mode, nwg);
}
template <int NW, int WAVES>
static void launch_value_q_bit(int bit, hipStream_t st, const ValuePlan& pl, const QArgs& a, const _Float16* P,
                               _Float16* C, float* part, int Lc, int D, int Bkv, int rows_per_kv, int row0)
{
    if (bit == 2)
        launch_value_q<NW, WAVES, 2>(st, pl, a, P, C, part, Lc, D, Bkv, rows_per_kv, row0);
    else if (bit == 4)
        launch_value_q<NW, WAVES, 4>(st, pl, a, P, C, part, Lc, D, Bkv, rows_per_kv, row0);
    else
        launch_value_q<NW, WAVES, 8>(st, pl, a, P, C, part, Lc, D, Bkv, rows_per_kv, row0);
}

}  // namespace mstf

using namespace mstf;

static int key_spmv_quant_impl(void* stream, const uint64_t* bmp, const uint32_t* packed, const uint32_t* tile_off,
                               const mstf_half* scales, const mstf_half* zeros, const mstf_half* Bm, mstf_half* C, int M,
                               int K, int Bq, int groups, int n_rows, int bit, int capacity, int dequant_mode,
                               int group_size)
{
    if (group_size != 64 && group_size != 32) return MSTF_EUNSUPPORTED;
    int rc = check_quant_spmv(bmp, packed, tile_off, scales, zeros, Bm, C, M, K, Bq, groups, n_rows, bit, capacity,
                              dequant_mode);
    if (rc != MSTF_OK) return rc;
    hipStream_t st = as_stream(stream);
    const int Bkv = Bq / groups, rows_per_kv = groups * n_rows;
    const _Float16* b = reinterpret_cast<const _Float16*>(Bm);
    _Float16* c = reinterpret_cast<_Float16*>(C);
    const QArgs a = {bmp, packed, tile_off, scales, zeros, dequant_mode, group_size};
    for (int row0 = 0; row0 < rows_per_kv;) {
        const int nw = pick_nw(rows_per_kv - row0);
        switch (nw) {
            case 32: launch_key_q_bit<32>(bit, st, a, b, c, M, K, Bkv, rows_per_kv, row0); break;
            case 16: launch_key_q_bit<16>(bit, st, a, b, c, M, K, Bkv, rows_per_kv, row0); break;
            case 8: launch_key_q_bit<8>(bit, st, a, b, c, M, K, Bkv, rows_per_kv, row0); break;
            case 4: launch_key_q_bit<4>(bit, st, a, b, c, M, K, Bkv, rows_per_kv, row0); break;
            case 2: launch_key_q_bit<2>(bit, st, a, b, c, M, K, Bkv, rows_per_kv, row0); break;
            default: launch_key_q_bit<1>(bit, st, a, b, c, M, K, Bkv, rows_per_kv, row0); break;
        }
        if ((rc = check_launch()) != MSTF_OK) return rc;
        row0 += nw;
    }
    return MSTF_OK;
}

extern "C" int mstf_key_spmv_quant(void* stream, const uint64_t* bmp, const uint32_t* packed, const uint32_t* tile_off,
                                   const uint32_t* counts, const uint32_t* units, const mstf_half* scales,
                                   const mstf_half* zeros, const mstf_half* Bm, mstf_half* C, int M, int K, int Bq,
                                   int groups, int n_rows, int bit, int capacity, int dequant_mode)
{
    (void)counts;  // raw counts and units follow from the bitmaps; accepted for interface compatibility
    (void)units;
    return key_spmv_quant_impl(stream, bmp, packed, tile_off, scales, zeros, Bm, C, M, K, Bq, groups, n_rows, bit, capacity,
                               dequant_mode, 64);
}

extern "C" int mstf_key_spmv_quant_grouped(void* stream, const uint64_t* bmp, const uint32_t* packed,
                                           const uint32_t* tile_off, const mstf_half* scales, const mstf_half* zeros,
                                           const mstf_half* Bm, mstf_half* C, int M, int K, int Bq, int groups, int n_rows,
                                           int bit, int capacity, int dequant_mode, int group_size)
{
    return key_spmv_quant_impl(stream, bmp, packed, tile_off, scales, zeros, Bm, C, M, K, Bq, groups, n_rows, bit, capacity,
                               dequant_mode, group_size);
}

extern "C" size_t mstf_value_spmv_quant_workspace_bytes(int M, int K, int Bq, int groups, int n_rows)
{
    if (M <= 0 || K <= 0 || Bq <= 0 || groups <= 0 || n_rows <= 0 || K % 64 != 0 || M % 64 != 0 || Bq % groups != 0)
        return 0;
    return value_workspace_bytes(M, K, Bq, groups, n_rows);
}

static int value_spmv_quant_impl(void* stream, const uint64_t* bmp, const uint32_t* packed, const uint32_t* tile_off,
                                 const mstf_half* scales, const mstf_half* zeros, const mstf_half* P, mstf_half* C, int M,
                                 int K, int Bq, int groups, int n_rows, int bit, int capacity, int dequant_mode,
                                 int group_size, void* workspace, size_t workspace_bytes)
{
    if (group_size != 64 && group_size != 32) return MSTF_EUNSUPPORTED;
    // M = head_dim, K = compressed tokens (the operator's GEMM naming)
    int rc = check_quant_spmv(bmp, packed, tile_off, scales, zeros, P, C, K, M, Bq, groups, n_rows, bit, capacity,
                              dequant_mode);
    if (rc != MSTF_OK) return rc;
    const size_t need = mstf_value_spmv_quant_workspace_bytes(M, K, Bq, groups, n_rows);
    if (need > 0 && (!workspace || workspace_bytes < need)) return MSTF_EWORKSPACE;
    if (workspace && !aligned_to(workspace, 16)) return MSTF_EALIGN;
    hipStream_t st = as_stream(stream);
    const int Bkv = Bq / groups, rows_per_kv = groups * n_rows;
    const _Float16* p = reinterpret_cast<const _Float16*>(P);
    _Float16* c = reinterpret_cast<_Float16*>(C);
    float* part = reinterpret_cast<float*>(workspace);
    const QArgs a = {bmp, packed, tile_off, scales, zeros, dequant_mode, group_size};
    for (int row0 = 0; row0 < rows_per_kv;) {
        const int nw = pick_nw(rows_per_kv - row0);
        const ValuePlan pl = plan_value(K, M, Bkv, nw);
        switch (nw) {
            case 32: launch_value_q_bit<32, 4>(bit, st, pl, a, p, c, part, K, M, Bkv, rows_per_kv, row0); break;
            case 16: launch_value_q_bit<16, 4>(bit, st, pl, a, p, c, part, K, M, Bkv, rows_per_kv, row0); break;
            case 8: launch_value_q_bit<8, 8>(bit, st, pl, a, p, c, part, K, M, Bkv, rows_per_kv, row0); break;
            case 4: launch_value_q_bit<4, 8>(bit, st, pl, a, p, c, part, K, M, Bkv, rows_per_kv, row0); break;
            case 2: launch_value_q_bit<2, 8>(bit, st, pl, a, p, c, part, K, M, Bkv, rows_per_kv, row0); break;
            default: launch_value_q_bit<1, 8>(bit, st, pl, a, p, c, part, K, M, Bkv, rows_per_kv, row0); break;
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

extern "C" int mstf_value_spmv_quant(void* stream, const uint64_t* bmp, const uint32_t* packed,
                                     const uint32_t* tile_off, const uint32_t* counts, const uint32_t* units,
                                     const mstf_half* scales, const mstf_half* zeros, const mstf_half* P, mstf_half* C,
                                     int M, int K, int Bq, int groups, int n_rows, int bit, int capacity,
                                     int dequant_mode, void* workspace, size_t workspace_bytes)
{
    (void)counts;
    (void)units;
    return value_spmv_quant_impl(stream, bmp, packed, tile_off, scales, zeros, P, C, M, K, Bq, groups, n_rows, bit, capacity,
                                 dequant_mode, 64, workspace, workspace_bytes);
}

extern "C" int mstf_value_spmv_quant_grouped(void* stream, const uint64_t* bmp, const uint32_t* packed,
                                             const uint32_t* tile_off, const mstf_half* scales, const mstf_half* zeros,
                                             const mstf_half* P, mstf_half* C, int M, int K, int Bq, int groups, int n_rows,
                                             int bit, int capacity, int dequant_mode, int group_size, void* workspace,
                                             size_t workspace_bytes)
{
    return value_spmv_quant_impl(stream, bmp, packed, tile_off, scales, zeros, P, C, M, K, Bq, groups, n_rows, bit, capacity,
                                 dequant_mode, group_size, workspace, workspace_bytes);
}
