// Fused sparse decode attention over the quantised format: key SpMV -> scale + softmax -> value SpMV in one
// launch, with the work decomposition, softmax and combine of the fp16 kernel (fused.hip) and the staged
// dequantisation of the quantised SpMVs (quant_spmv.hip).
//
// One wavefront owns one (KV head, 64-token block): four stages of 32 key tiles, then four stages of 32 value
// tiles.  A stage's packed words and metadata arrive by LDS-direct loads one stage ahead (double buffers); the
// stage is dequantised into the wavefront's fp16 tile image and expanded from there.
#include "fused_common.hpp"
#include "step_device.hpp"

#ifndef MSTF_QPAD
#define MSTF_QPAD 16
#endif
#include "quant_device.hpp"

namespace mstf {

#pragma clang fp contract(off)

// One side (keys or values) of a quantised cache; `off_dma` is `off` again, kept apart so that `off` stays a
// pointer that never reaches an LDS-direct load and is read with scalar loads.
struct QSide {
    const uint64_t* bmp;
    const uint32_t* packed;
    const uint32_t* off;
    const uint32_t* off_dma;
    const uint16_t* scales;
    const uint16_t* zeros;
};

// grid = (token splits, KV heads), kFusedWaves wavefronts; see decode_attention_kernel.  STEP: the launch is a whole
// decode step (st, the last argument; QuantKernargs mirrors the argument list and tells where it sits in the
// kernel-argument segment; step_device.hpp).
struct QuantKernargs {
    const void* first_ptrs[4];
    size_t tstride;
    const void* tokens_dev;
    int nblk, heads_fastest;
    const void* ptrs[12];
    int groups, nsplit, write_final;
    float sqrt_d;
    int mode;
    StepArgs st;
};
constexpr size_t kQuantStepArgsAt = offsetof(QuantKernargs, st);
template <int NM, int BIT, bool G32, bool STEP = false>
__global__ __launch_bounds__(kFusedWaves * 64) void decode_attention_quant_kernel(
    const uint32_t* __restrict__ k_off, const uint32_t* __restrict__ v_off, const uint64_t* __restrict__ k_bmp,
    const uint64_t* __restrict__ v_bmp, size_t tstride, const int* __restrict__ tokens_dev, int nblk, int heads_fastest,
    const uint32_t* k_packed, const uint32_t* k_off_dma, const uint16_t* k_scales, const uint16_t* k_zeros,
    const uint32_t* v_packed, const uint32_t* v_off_dma, const uint16_t* v_scales, const uint16_t* v_zeros,
    const _Float16* q, _Float16* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml, int groups,
    int nsplit, int write_final, float sqrt_d, int mode, StepArgs st)
{
    // Argument order: the first fourteen 32-bit words - what a wavefront's first loads need - are in scalar registers
    // when it starts (kernel-argument preload, a compile option of this library).
    // tstride: tiles between the per-tile rows of two heads - the tile count of the cached tokens unless the arrays are
    // pre-allocated for more.  tokens_dev (nullable): the number of cached tokens is read from device memory, at most
    // nblk blocks of it; the launch is then sized for the capacity and the wavefronts beyond the valid blocks leave
    // neutral partials.  heads_fastest: the heads vary fastest over the workgroup index, so that the workgroups beyond
    // the valid blocks are dispatched last instead of standing in front of working ones.
    if (tokens_dev) {
        const int valid = *tokens_dev / 64;
        nblk = valid < nblk ? valid : nblk;
    }
    using F = QFmt<BIT>;
    constexpr int D = kFusedD;
    // query and weight rows sit 16 bytes further apart than their length: the four rows that the lanes of a group read
    // together then start in different LDS banks
    constexpr int kQRow = D * 2 + MSTF_QPAD;
    constexpr int kQLds = NM * 4 * kQRow;
    constexpr int kPRow = 64 * 2 + MSTF_QPAD;
    constexpr int kPLds = NM * 4 * kPRow;
    constexpr int kMetaBytes = meta_bytes<G32>();
    constexpr int kStage = q_lds_bytes<BIT, G32>();  // image, zero slot, two word buffers, two metadata buffers
    constexpr int kNeed = kStage + kQLds + kPLds;
    constexpr int kPark = NM * 4 * D * 4 + 64;
    constexpr int kWaveLds = kNeed > kPark ? kNeed : kPark;
    // one array on purpose (LDS-direct loads into several LDS objects make the compiler serialise them)
    __shared__ __attribute__((aligned(16))) char lds_all[kFusedWaves * kWaveLds];
    const int lane = lane_id();
    const int wave = wave_id();
    const int split = heads_fastest ? (int)blockIdx.y : (int)blockIdx.x;
    const int kv = heads_fastest ? (int)blockIdx.x : (int)blockIdx.y;
    const int tb = split * kFusedWaves + wave;
    const bool active = tb < nblk;  // wave-uniform
    const int j = lane & 3;
    const size_t T = tstride;
    char* my = lds_all + wave * kWaveLds;
    char* wordbuf = my + kImgBytes + 16;
    char* metabuf = wordbuf + 2 * F::kWordBuf;
    char* ql = my + kStage;
    char* pl = ql + kQLds;
    const uint32_t lbase = lds_addr(my);
    const uint32_t zaddr = lbase + kImgBytes;

    f4_t acc_v[NM][2];
    float m_run[NM], l_run[NM];
#pragma unroll
    for (int m = 0; m < NM; m++) {
        acc_v[m][0] = f4_t{0.f, 0.f, 0.f, 0.f};
        acc_v[m][1] = f4_t{0.f, 0.f, 0.f, 0.f};
        m_run[m] = -INFINITY;
        l_run[m] = 0.f;
    }

    if (active) {
        const size_t tile0 = (size_t)kv * T + (size_t)tb * D;  // tile_off / scales / zeros / bmp are flat over [Bkv, T]
        constexpr size_t kPairs = G32 ? 2 : 1;  // (scale, zero) pairs per tile
        const QSide K = {k_bmp + tile0, k_packed, k_off + tile0, k_off_dma + tile0, k_scales + tile0 * kPairs,
                         k_zeros + tile0 * kPairs};
        const QSide V = {v_bmp + tile0, v_packed, v_off + tile0, v_off_dma + tile0, v_scales + tile0 * kPairs,
                         v_zeros + tile0 * kPairs};
        if (lane < 4) reinterpret_cast<uint32_t*>(my + kImgBytes)[lane] = 0u;
        // word offsets at the stage boundaries of both sides by one vector load (lanes 0.. keys, 16.. values); the
        // block's last stage ends where its last tile's words end
        uint32_t bnd = 0u;
        if (lane < kKeySubs) bnd = K.off[lane * kSubTiles];
        else if (lane >= 16 && lane < 16 + kValSubs) bnd = V.off[(lane - 16) * kSubTiles];
        auto words_of = [](uint64_t bm) {
            return ((uint32_t)__builtin_popcountll(bm) + (uint32_t)F::kCap - 1u) >> F::kCapShift;
        };
        const uint32_t endK = K.off[D - 1] + words_of(K.bmp[D - 1]);
        const uint32_t endV = V.off[D - 1] + words_of(V.bmp[D - 1]);
        auto start_of = [&](int n) -> uint32_t {
            return __builtin_amdgcn_readlane(bnd, n < kKeySubs ? n : 16 + n - kKeySubs);
        };
        auto end_of = [&](int n) -> uint32_t {
            if (n == kKeySubs - 1) return endK;
            if (n == kKeySubs + kValSubs - 1) return endV;
            return start_of(n + 1);
        };
        const MetaLanes metaK = meta_lanes<G32>(K.off_dma, K.scales, K.zeros, K.bmp, lane);
        const MetaLanes metaV = meta_lanes<G32>(V.off_dma, V.scales, V.zeros, V.bmp, lane);
        const uint32_t lane4 = (uint32_t)lane * 4u;
        const uint32_t touch8 = (uint32_t)(lane < kSubTiles ? lane : kSubTiles - 1) * 8u;
        const uint32_t wordbuf_lds = lds_addr(wordbuf);
        // (no lane-dependent branches: every piece is issued with exec set by hand or from a clamped address)
        auto issue = [&](int n) {
            const QSide& S = n < kKeySubs ? K : V;
            const MetaLanes& ML = n < kKeySubs ? metaK : metaV;
            const int t = (n < kKeySubs ? n : n - kKeySubs) * kSubTiles;
            const uint32_t s = start_of(n);
            uint32_t nw = end_of(n) - s;
            nw = nw > (uint32_t)F::kWordsMax ? (uint32_t)F::kWordsMax : nw;  // never true for a well-formed cache
            words_issue_flat<F::kWordsMax / 64>(S.packed + s, nw, wordbuf_lds + (uint32_t)(n & 1) * F::kWordBuf,
                                                (uint32_t)lane, lane4);
            // metadata: lanes 0..31 the word offsets, 32..47 the scales, 48..63 the zero-points (two per lane)
            meta_issue<G32>(ML, (uint32_t)t, metabuf + (n & 1) * kMetaBytes);
            // pulls the stage's bitmaps into L2 ahead of the scalar loads of the expansion
            return *reinterpret_cast<const uint2*>(reinterpret_cast<const char*>(S.bmp + t) + touch8);
        };

        // the query rows of this KV head: groups x D fp16, contiguous (STEP: rotated out of the projection output)
        if constexpr (STEP) {
            stage_query_rotated<kQRow>(ql, st, kv, groups, lane);
        } else {
            const char* qsrc = reinterpret_cast<const char*>(q + (size_t)kv * groups * D);
            // a row per load: sixteen lanes fetch the 256 bytes of query row `row`, four rows per pass
            const int row_in_pass = lane >> 4;
#pragma unroll
            for (int i = 0; i < NM; i++) {
                const int row = i * 4 + row_in_pass;
                const uint4 v = row < groups ? *reinterpret_cast<const uint4*>(qsrc + row * (D * 2) + (lane & 15) * 16)
                                             : make_uint4(0u, 0u, 0u, 0u);
                *reinterpret_cast<uint4*>(ql + row * kQRow + (lane & 15) * 16) = v;
            }
        }
        uint2 touch = issue(0);

        f4_t acc_k[NM];
#pragma unroll
        for (int m = 0; m < NM; m++) acc_k[m] = f4_t{0.f, 0.f, 0.f, 0.f};
        const uint32_t qrow = lds_addr(ql) + (uint32_t)j * kQRow;
        const uint32_t prow = lds_addr(pl) + (uint32_t)j * kPRow;

        constexpr bool kDual = NM == 1 && MSTF_DUAL_ACC;
        f4_t acc2[NM];  // second set of sums of the gather statements (batch_step_img_dual), folded in per phase
#pragma unroll
        for (int m = 0; m < NM; m++) acc2[m] = f4_t{0.f, 0.f, 0.f, 0.f};
        auto stage = [&](int n, uint2 bits, uint32_t waddr, uint32_t wgroup, f4_t (&acc)[NM]) {
            const QSide& S = n < kKeySubs ? K : V;
            const int t = (n < kKeySubs ? n : n - kKeySubs) * kSubTiles;
            dequant_stage<BIT, G32>(lds_addr(metabuf) + (uint32_t)(n & 1) * kMetaBytes,
                               lds_addr(wordbuf) + (uint32_t)(n & 1) * F::kWordBuf, lbase, start_of(n), end_of(n), lane, mode);
            stage_img_exec<NM>(S.bmp + t, bits.x, bits.y, lbase, zaddr, waddr, wgroup, acc, acc2);
        };

#pragma unroll
        for (int n = 0; n < kKeySubs + kValSubs; n++) {
            // 3, 2, 1, 0 over the key stages and again over the value stages (keeping the wavefronts that also take a
            // block of the dense window at 3, as the fp16 kernel does, measured slower here: one block per wavefront)
            set_wave_priority(3 - n % 4);
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(touch.x), "+v"(touch.y)::"memory");  // stage n has landed
            const uint2 bits = touch;  // lane l < 32: bitmap l of stage n
            if (n + 1 < kKeySubs + kValSubs) touch = issue(n + 1);
            if (n < kKeySubs) {
                stage(n, bits, qrow + (uint32_t)n * kSubTiles * 2u, 4u * kQRow, acc_k);
            } else {
                if (n == kKeySubs) {
                    if constexpr (kDual) {
                        dual_settle(acc_k[0], acc2[0]);
                        acc_k[0] += acc2[0];
                        acc2[0] = f4_t{0.f, 0.f, 0.f, 0.f};
                    }
                    block_softmax<NM, kPRow>(acc_k, sqrt_d, 64, pl, lane, m_run, l_run);
                }
                const int vs = n - kKeySubs;  // value stage: half = vs / 2, tokens (vs % 2) * 32..
                constexpr int kSubsPerHalf = 64 / kSubTiles;
                const int half = vs / kSubsPerHalf;
                f4_t tmp[NM];
#pragma unroll
                for (int m = 0; m < NM; m++) tmp[m] = acc_v[m][half];
                stage(n, bits, prow + (uint32_t)(vs % kSubsPerHalf) * kSubTiles * 2u, 4u * kPRow, tmp);
                if (kDual && vs % kSubsPerHalf == kSubsPerHalf - 1) {  // the half is complete
                    dual_settle(tmp[0], acc2[0]);
                    tmp[0] += acc2[0];
                    acc2[0] = f4_t{0.f, 0.f, 0.f, 0.f};
                }
#pragma unroll
                for (int m = 0; m < NM; m++) acc_v[m][half] = tmp[m];
            }
            wait_lgkm0();  // every read of the image and of the staged buffers is done before they are rewritten
        }
    }
    if constexpr (STEP) {
        // The dense window: block i goes to wavefront i / ns of split i % ns, behind its compressed block (see
        // decode_attention_kernel); the value rows pass through the room of the tile image, eight at a time.  The
        // step's arguments are fetched again here, through a pointer the compiler cannot see through, so that they
        // hold no scalar registers above.
        static_assert(2 * 8 * D * 2 <= kImgBytes, "two buffers of eight value rows in the room of the image");
        const StepArgs __attribute__((address_space(4)))* sp = (const StepArgs __attribute__((address_space(4)))*)(
            (const char __attribute__((address_space(4)))*)__builtin_amdgcn_kernarg_segment_ptr() + kQuantStepArgsAt);
        asm volatile("" : "+s"(sp));
        StepArgs sw;
        sw.q_in = sp->q_in, sw.k_in = sp->k_in, sw.v_in = sp->v_in;
        sw.q_stride = sp->q_stride, sw.k_stride = sp->k_stride, sw.v_stride = sp->v_stride;
        sw.cos = sp->cos, sw.sin = sp->sin, sw.rope_stride = sp->rope_stride;
        sw.k_win = sp->k_win, sw.v_win = sp->v_win, sw.win_len_dev = sp->win_len_dev, sw.overflow = sp->overflow;
        sw.win_len = sp->win_len, sw.win_stride = sp->win_stride, sw.n_kv = sp->n_kv, sw.ns = sp->ns;
        const int wblk = wave * sw.ns + split;
        if (wblk < (sw.win_len + 63) / 64) {
            if (!active) stage_query_rotated<kQRow>(ql, sw, kv, groups, lane);
            step_window_wave<NM, kQRow, kPRow, 8>(my, ql, pl, sw, part_o, part_ml, kv, groups, nsplit, wblk, sqrt_d, lane);
        }
    }
    workgroup_combine<NM>(lds_all, kWaveLds, wave, lane, acc_v, m_run, l_run, kv, groups, split, nsplit, write_final, out,
                          part_o, part_ml);
}

template <int NM, int BIT>
static void launch_decode_quant(hipStream_t st, dim3 grid, const uint64_t* k_bmp, const uint32_t* k_packed,
                                const uint32_t* k_off, const uint16_t* k_scales, const uint16_t* k_zeros,
                                const uint64_t* v_bmp, const uint32_t* v_packed, const uint32_t* v_off,
                                const uint16_t* v_scales, const uint16_t* v_zeros, const _Float16* q, _Float16* out,
                                float* part_o, float* part_ml, int tokens, int groups, int ns, int write_final, float sq,
                                int mode, int group_size, size_t tstride, const int32_t* tokens_dev, int heads_fastest,
                                const StepArgs* step)
{
    const StepArgs sa = step ? *step : StepArgs{};
    if (step)  // (group_size is 64 there: quant_launch has checked it)
        hipLaunchKernelGGL((decode_attention_quant_kernel<NM, BIT, false, true>), grid, dim3(kFusedWaves * 64), 0, st, k_off,
                           v_off, k_bmp, v_bmp, tstride, tokens_dev, tokens / 64, heads_fastest, k_packed, k_off, k_scales,
                           k_zeros, v_packed, v_off, v_scales, v_zeros, q, out, part_o, part_ml, groups, ns, write_final,
                           sq, mode, sa);
    else if (group_size == 32)
        hipLaunchKernelGGL((decode_attention_quant_kernel<NM, BIT, true>), grid, dim3(kFusedWaves * 64), 0, st, k_off,
                           v_off, k_bmp, v_bmp, tstride, tokens_dev, tokens / 64, heads_fastest, k_packed, k_off, k_scales,
                           k_zeros, v_packed, v_off, v_scales, v_zeros, q, out, part_o, part_ml, groups, ns, write_final,
                           sq, mode, sa);
    else
        hipLaunchKernelGGL((decode_attention_quant_kernel<NM, BIT, false>), grid, dim3(kFusedWaves * 64), 0, st, k_off,
                           v_off, k_bmp, v_bmp, tstride, tokens_dev, tokens / 64, heads_fastest, k_packed, k_off, k_scales,
                           k_zeros, v_packed, v_off, v_scales, v_zeros, q, out, part_o, part_ml, groups, ns, write_final,
                           sq, mode, sa);
}

}  // namespace mstf

using namespace mstf;

// Shared argument checks of the quantised fused entry points.
static int quant_check(const void* k_bmp, const void* k_packed, const void* k_tile_off, const void* k_scales,
                       const void* k_zeros, const void* v_bmp, const void* v_packed, const void* v_tile_off,
                       const void* v_scales, const void* v_zeros, const void* q, int tokens, int head_dim, int Bq,
                       int groups, int bit, int capacity, int dequant_mode)
{
    if (!k_bmp || !k_packed || !k_tile_off || !k_scales || !k_zeros || !v_bmp || !v_packed || !v_tile_off || !v_scales ||
        !v_zeros || !q)
        return MSTF_EINVAL;
    if (tokens <= 0 || Bq <= 0 || groups <= 0 || Bq % groups != 0) return MSTF_EINVAL;
    if (dequant_mode != 0 && dequant_mode != 1) return MSTF_EINVAL;
    if (bit != 2 && bit != 4 && bit != 8) return MSTF_EUNSUPPORTED;
    if (capacity != 32 / bit) return MSTF_EINVAL;
    if (head_dim != kFusedD || tokens % 64 != 0 || groups > 8) return MSTF_EUNSUPPORTED;
    if (!aligned_to(k_bmp, 8) || !aligned_to(v_bmp, 8) || !aligned_to(k_packed, 4) || !aligned_to(v_packed, 4) ||
        !aligned_to(k_tile_off, 4) || !aligned_to(v_tile_off, 4) || !aligned_to(k_scales, 4) || !aligned_to(v_scales, 4) ||
        !aligned_to(k_zeros, 4) || !aligned_to(v_zeros, 4) || !aligned_to(q, 16))
        return MSTF_EALIGN;
    return MSTF_OK;
}

// The quantised kernel over the compressed tokens: fills split slots 0 .. fused_nsplit(tokens)-1 of a workspace
// with nst slots per query row (or writes the final output when write_final).
static int quant_launch(hipStream_t st, const uint64_t* k_bmp, const uint32_t* k_packed, const uint32_t* k_tile_off,
                        const mstf_half* k_scales, const mstf_half* k_zeros, const uint64_t* v_bmp,
                        const uint32_t* v_packed, const uint32_t* v_tile_off, const mstf_half* v_scales,
                        const mstf_half* v_zeros, const mstf_half* q, mstf_half* out, int tokens, int head_dim, int Bq,
                        int groups, int bit, int dequant_mode, void* workspace, int nst, int write_final,
                        int group_size = 64, size_t tile_stride = 0, const int32_t* tokens_dev = nullptr,
                        const StepArgs* step = nullptr)
{
    // step: the launch is a whole decode step; its window blocks are dealt out over the wavefronts of a head
    if (step && (group_size != 64 || window_blocks(step->win_len) > fused_nsplit(tokens) * kFusedWaves))
        return MSTF_EUNSUPPORTED;
    // tile_stride / tokens_dev: a cache pre-allocated for `tokens` tokens that holds *tokens_dev of them (see the kernel)
    const int Bkv = Bq / groups, ns = fused_nsplit(tokens);
    float* part_o = reinterpret_cast<float*>(workspace);
    float* part_ml = part_o + (size_t)Bq * nst * head_dim;
    const int heads_fastest = tokens_dev ? 1 : 0;
    const dim3 grid = heads_fastest ? dim3((unsigned)Bkv, (unsigned)ns) : dim3((unsigned)ns, (unsigned)Bkv);
    const size_t tstride = tile_stride ? tile_stride : (size_t)tokens * head_dim / 64;
    const _Float16* qh = reinterpret_cast<const _Float16*>(q);
    _Float16* oh = reinterpret_cast<_Float16*>(out);
    const float sq = sqrtf((float)head_dim);
    const uint16_t* ks = reinterpret_cast<const uint16_t*>(k_scales);
    const uint16_t* kz = reinterpret_cast<const uint16_t*>(k_zeros);
    const uint16_t* vs = reinterpret_cast<const uint16_t*>(v_scales);
    const uint16_t* vz = reinterpret_cast<const uint16_t*>(v_zeros);
#define MSTF_FQ(NMV, BITV)                                                                                             \
    launch_decode_quant<NMV, BITV>(st, grid, k_bmp, k_packed, k_tile_off, ks, kz, v_bmp, v_packed, v_tile_off, vs, vz, \
                                   qh, oh, part_o, part_ml, tokens, groups, nst, write_final, sq, dequant_mode, group_size, \
                                   tstride, tokens_dev, heads_fastest, step)
    if (groups <= 4) {
        if (bit == 2) MSTF_FQ(1, 2); else if (bit == 4) MSTF_FQ(1, 4); else MSTF_FQ(1, 8);
    } else {
        if (bit == 2) MSTF_FQ(2, 2); else if (bit == 4) MSTF_FQ(2, 4); else MSTF_FQ(2, 8);
    }
#undef MSTF_FQ
    return check_launch();
}

static int decode_attention_quant_impl(void* stream, const uint64_t* k_bmp, const uint32_t* k_packed,
                                       const uint32_t* k_tile_off, const mstf_half* k_scales, const mstf_half* k_zeros,
                                       const uint64_t* v_bmp, const uint32_t* v_packed, const uint32_t* v_tile_off,
                                       const mstf_half* v_scales, const mstf_half* v_zeros, const mstf_half* q,
                                       mstf_half* out, float* lse_out, int tokens, int head_dim, int Bq, int groups,
                                       int bit, int capacity, int dequant_mode, int group_size, void* workspace,
                                       size_t workspace_bytes)
{
    if (!out) return MSTF_EINVAL;
    if (group_size != 64 && group_size != 32) return MSTF_EUNSUPPORTED;
    int rc = quant_check(k_bmp, k_packed, k_tile_off, k_scales, k_zeros, v_bmp, v_packed, v_tile_off, v_scales, v_zeros, q,
                         tokens, head_dim, Bq, groups, bit, capacity, dequant_mode);
    if (rc != MSTF_OK) return rc;
    if (!aligned_to(out, 2) || (lse_out && !aligned_to(lse_out, 4))) return MSTF_EALIGN;
    const size_t need = mstf_decode_attention_workspace_bytes(tokens, head_dim, Bq, groups);
    if (!workspace || workspace_bytes < need) return MSTF_EWORKSPACE;
    if (!aligned_to(workspace, 16)) return MSTF_EALIGN;
    hipStream_t st = as_stream(stream);
    const int ns = fused_nsplit(tokens);
    // with one split and no (max, sum) requested the kernel writes the final output itself
    const int write_final = (ns == 1 && !lse_out) ? 1 : 0;
    rc = quant_launch(st, k_bmp, k_packed, k_tile_off, k_scales, k_zeros, v_bmp, v_packed, v_tile_off, v_scales, v_zeros, q,
                      out, tokens, head_dim, Bq, groups, bit, dequant_mode, workspace, ns, write_final, group_size);
    if (rc != MSTF_OK || write_final) return rc;
    return merge_splits(st, workspace, out, lse_out, ns, head_dim, Bq);
}

extern "C" int mstf_decode_attention_quant(void* stream, const uint64_t* k_bmp, const uint32_t* k_packed,
                                           const uint32_t* k_tile_off, const mstf_half* k_scales,
                                           const mstf_half* k_zeros, const uint64_t* v_bmp, const uint32_t* v_packed,
                                           const uint32_t* v_tile_off, const mstf_half* v_scales,
                                           const mstf_half* v_zeros, const mstf_half* q, mstf_half* out, float* lse_out,
                                           int tokens, int head_dim, int Bq, int groups, int bit, int capacity,
                                           int dequant_mode, void* workspace, size_t workspace_bytes)
{
    return decode_attention_quant_impl(stream, k_bmp, k_packed, k_tile_off, k_scales, k_zeros, v_bmp, v_packed, v_tile_off,
                                       v_scales, v_zeros, q, out, lse_out, tokens, head_dim, Bq, groups, bit, capacity,
                                       dequant_mode, 64, workspace, workspace_bytes);
}

extern "C" int mstf_decode_attention_quant_grouped(void* stream, const uint64_t* k_bmp, const uint32_t* k_packed,
                                                   const uint32_t* k_tile_off, const mstf_half* k_scales,
                                                   const mstf_half* k_zeros, const uint64_t* v_bmp,
                                                   const uint32_t* v_packed, const uint32_t* v_tile_off,
                                                   const mstf_half* v_scales, const mstf_half* v_zeros,
                                                   const mstf_half* q, mstf_half* out, float* lse_out, int tokens,
                                                   int head_dim, int Bq, int groups, int bit, int capacity,
                                                   int dequant_mode, int group_size, void* workspace,
                                                   size_t workspace_bytes)
{
    return decode_attention_quant_impl(stream, k_bmp, k_packed, k_tile_off, k_scales, k_zeros, v_bmp, v_packed, v_tile_off,
                                       v_scales, v_zeros, q, out, lse_out, tokens, head_dim, Bq, groups, bit, capacity,
                                       dequant_mode, group_size, workspace, workspace_bytes);
}

extern "C" int mstf_decode_attention_window_quant(
    void* stream, const uint64_t* k_bmp, const uint32_t* k_packed, const uint32_t* k_tile_off, const mstf_half* k_scales,
    const mstf_half* k_zeros, const uint64_t* v_bmp, const uint32_t* v_packed, const uint32_t* v_tile_off,
    const mstf_half* v_scales, const mstf_half* v_zeros, const mstf_half* q, const mstf_half* k_win,
    const mstf_half* v_win, int win_len, const int32_t* win_len_dev, int win_stride, mstf_half* out, float* lse_out,
    int tokens, int head_dim, int Bq, int groups, int bit, int capacity, int dequant_mode, void* workspace,
    size_t workspace_bytes)
{
    if (!q || !k_win || !v_win || !out) return MSTF_EINVAL;
    if (tokens < 0 || win_len <= 0 || win_stride < win_len || Bq <= 0 || groups <= 0 || Bq % groups != 0)
        return MSTF_EINVAL;
    if (head_dim != kFusedD || tokens % 64 != 0 || groups > 8) return MSTF_EUNSUPPORTED;
    if (!aligned_to(q, 16) || !aligned_to(k_win, 16) || !aligned_to(v_win, 16) || !aligned_to(out, 2) ||
        (lse_out && !aligned_to(lse_out, 4)) || (win_len_dev && !aligned_to(win_len_dev, 4)))
        return MSTF_EALIGN;
    const size_t need = mstf_decode_attention_window_workspace_bytes(tokens, win_len, head_dim, Bq, groups);
    if (!workspace || workspace_bytes < need) return MSTF_EWORKSPACE;
    if (!aligned_to(workspace, 16)) return MSTF_EALIGN;
    hipStream_t st = as_stream(stream);
    const int ns = tokens > 0 ? fused_nsplit(tokens) : 0, nst = ns + window_blocks(win_len);
    int rc;
    if (tokens > 0) {
        rc = quant_check(k_bmp, k_packed, k_tile_off, k_scales, k_zeros, v_bmp, v_packed, v_tile_off, v_scales, v_zeros, q,
                         tokens, head_dim, Bq, groups, bit, capacity, dequant_mode);
        if (rc != MSTF_OK) return rc;
        rc = quant_launch(st, k_bmp, k_packed, k_tile_off, k_scales, k_zeros, v_bmp, v_packed, v_tile_off, v_scales,
                          v_zeros, q, nullptr, tokens, head_dim, Bq, groups, bit, dequant_mode, workspace, nst, 0);
        if (rc != MSTF_OK) return rc;
    }
    if ((rc = window_launch(st, k_win, v_win, q, workspace, win_len, win_len_dev, win_stride, head_dim, Bq, groups, nst,
                            ns)) != MSTF_OK)
        return rc;
    return merge_splits(st, workspace, out, lse_out, nst, head_dim, Bq);
}

extern "C" int mstf_decode_attention_window_quant_pool(
    void* stream, const uint64_t* k_bmp, const uint32_t* k_packed, const uint32_t* k_tile_off, const mstf_half* k_scales,
    const mstf_half* k_zeros, const uint64_t* v_bmp, const uint32_t* v_packed, const uint32_t* v_tile_off,
    const mstf_half* v_scales, const mstf_half* v_zeros, const mstf_half* q, const mstf_half* k_win,
    const mstf_half* v_win, int win_len, const int32_t* win_len_dev, int win_stride, mstf_half* out, float* lse_out,
    int max_tokens, const int32_t* tokens_dev, int64_t tile_capacity, int head_dim, int Bq, int groups, int bit,
    int capacity, int dequant_mode, void* workspace, size_t workspace_bytes)
{
    if (!q || !k_win || !v_win || !out || !tokens_dev) return MSTF_EINVAL;
    if (max_tokens <= 0 || win_len <= 0 || win_stride < win_len || Bq <= 0 || groups <= 0 || Bq % groups != 0)
        return MSTF_EINVAL;
    if (head_dim != kFusedD || max_tokens % 64 != 0 || groups > 8) return MSTF_EUNSUPPORTED;
    if (tile_capacity < (int64_t)max_tokens * head_dim / 64) return MSTF_EINVAL;
    if (!aligned_to(q, 16) || !aligned_to(k_win, 16) || !aligned_to(v_win, 16) || !aligned_to(out, 2) ||
        (lse_out && !aligned_to(lse_out, 4)) || (win_len_dev && !aligned_to(win_len_dev, 4)) || !aligned_to(tokens_dev, 4))
        return MSTF_EALIGN;
    // rows of the per-tile arrays start tile_capacity entries apart: the two-byte ones keep their four-byte alignment
    if (tile_capacity % 2 != 0) return MSTF_EALIGN;
    const size_t need = mstf_decode_attention_window_workspace_bytes(max_tokens, win_len, head_dim, Bq, groups);
    if (!workspace || workspace_bytes < need) return MSTF_EWORKSPACE;
    if (!aligned_to(workspace, 16)) return MSTF_EALIGN;
    hipStream_t st = as_stream(stream);
    const int ns = fused_nsplit(max_tokens), nst = ns + window_blocks(win_len);
    int rc = quant_check(k_bmp, k_packed, k_tile_off, k_scales, k_zeros, v_bmp, v_packed, v_tile_off, v_scales, v_zeros, q,
                         max_tokens, head_dim, Bq, groups, bit, capacity, dequant_mode);
    if (rc != MSTF_OK) return rc;
    rc = quant_launch(st, k_bmp, k_packed, k_tile_off, k_scales, k_zeros, v_bmp, v_packed, v_tile_off, v_scales, v_zeros, q,
                      nullptr, max_tokens, head_dim, Bq, groups, bit, dequant_mode, workspace, nst, 0, 64,
                      (size_t)tile_capacity, tokens_dev);
    if (rc != MSTF_OK) return rc;
    if ((rc = window_launch(st, k_win, v_win, q, workspace, win_len, win_len_dev, win_stride, head_dim, Bq, groups, nst,
                            ns)) != MSTF_OK)
        return rc;
    return merge_splits(st, workspace, out, lse_out, nst, head_dim, Bq);
}

extern "C" int mstf_decode_step_quant_pool(
    void* stream, const uint64_t* k_bmp, const uint32_t* k_packed, const uint32_t* k_tile_off, const mstf_half* k_scales,
    const mstf_half* k_zeros, const uint64_t* v_bmp, const uint32_t* v_packed, const uint32_t* v_tile_off,
    const mstf_half* v_scales, const mstf_half* v_zeros, const mstf_half* q_in, int64_t q_stride, const mstf_half* k_in,
    int64_t k_stride, const mstf_half* v_in, int64_t v_stride, int bs, int n_q, int n_kv, const mstf_half* cos,
    const mstf_half* sin, int64_t rope_stride, mstf_half* k_win, mstf_half* v_win, int win_stride, int win_len,
    const int32_t* win_len_dev, uint32_t* overflow, mstf_half* out, float* lse_out, int max_tokens,
    const int32_t* tokens_dev, int64_t tile_capacity, int head_dim, int bit, int capacity, int dequant_mode,
    void* workspace, size_t workspace_bytes)
{
    if (!q_in || !k_in || !v_in || !k_win || !v_win || !out || !tokens_dev) return MSTF_EINVAL;
    if ((cos == nullptr) != (sin == nullptr)) return MSTF_EINVAL;
    if (bs <= 0 || n_q <= 0 || n_kv <= 0 || n_q % n_kv != 0) return MSTF_EINVAL;
    if (max_tokens <= 0 || win_len <= 0 || win_stride < win_len) return MSTF_EINVAL;
    const int groups = n_q / n_kv;
    const int64_t Bq64 = (int64_t)bs * n_q;
    if (Bq64 > 0x7FFFFFF0) return MSTF_EUNSUPPORTED;
    const int Bq = (int)Bq64;
    if (head_dim != kFusedD || max_tokens % 64 != 0 || groups > 8) return MSTF_EUNSUPPORTED;
    if (tile_capacity < (int64_t)max_tokens * head_dim / 64) return MSTF_EINVAL;
    if (tile_capacity % 2 != 0) return MSTF_EALIGN;  // (rows of the two-byte per-tile arrays stay four-byte aligned)
    if (q_stride % 8 != 0 || k_stride % 8 != 0 || v_stride % 8 != 0 || rope_stride % 8 != 0) return MSTF_EALIGN;
    if (!aligned_to(q_in, 16) || !aligned_to(k_in, 16) || !aligned_to(v_in, 16) || !aligned_to(cos, 16) ||
        !aligned_to(sin, 16) || !aligned_to(k_win, 16) || !aligned_to(v_win, 16) || !aligned_to(out, 2) ||
        (lse_out && !aligned_to(lse_out, 4)) || (win_len_dev && !aligned_to(win_len_dev, 4)) ||
        !aligned_to(tokens_dev, 4) || !aligned_to(overflow, 4))
        return MSTF_EALIGN;
    const size_t need = mstf_decode_attention_window_workspace_bytes(max_tokens, win_len, head_dim, Bq, groups);
    if (!workspace || workspace_bytes < need) return MSTF_EWORKSPACE;
    if (!aligned_to(workspace, 16)) return MSTF_EALIGN;
    int rc = quant_check(k_bmp, k_packed, k_tile_off, k_scales, k_zeros, v_bmp, v_packed, v_tile_off, v_scales, v_zeros,
                         q_in, max_tokens, head_dim, Bq, groups, bit, capacity, dequant_mode);
    if (rc != MSTF_OK) return rc;
    hipStream_t st = as_stream(stream);
    const int ns = fused_nsplit(max_tokens), nst = ns + window_blocks(win_len);
    StepArgs sa = {};
    sa.q_in = reinterpret_cast<const _Float16*>(q_in);
    sa.k_in = reinterpret_cast<const _Float16*>(k_in);
    sa.v_in = reinterpret_cast<const _Float16*>(v_in);
    sa.q_stride = q_stride;
    sa.k_stride = k_stride;
    sa.v_stride = v_stride;
    sa.cos = reinterpret_cast<const _Float16*>(cos);
    sa.sin = reinterpret_cast<const _Float16*>(sin);
    sa.rope_stride = rope_stride;
    sa.k_win = reinterpret_cast<_Float16*>(k_win);
    sa.v_win = reinterpret_cast<_Float16*>(v_win);
    sa.win_len_dev = win_len_dev;
    sa.overflow = overflow;
    sa.win_len = win_len;
    sa.win_stride = win_stride;
    sa.n_kv = n_kv;
    sa.ns = ns;
    rc = quant_launch(st, k_bmp, k_packed, k_tile_off, k_scales, k_zeros, v_bmp, v_packed, v_tile_off, v_scales, v_zeros,
                      q_in, nullptr, max_tokens, head_dim, Bq, groups, bit, dequant_mode, workspace, nst, 0, 64,
                      (size_t)tile_capacity, tokens_dev, &sa);
    if (rc != MSTF_OK) return rc;
    return merge_splits(st, workspace, out, lse_out, nst, head_dim, Bq);
}
