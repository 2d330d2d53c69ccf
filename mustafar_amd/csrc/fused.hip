// Fused sparse decode attention: key SpMV -> scale + softmax -> value SpMV in one launch.
//
// One wavefront owns one (KV head, 64-token block).  It streams the block's 128 key tiles and then
// its 128 value tiles through the same LDS double buffer (the first value loads are issued while
// the last key tiles are still being decompressed - they do not depend on the scores):
//   key phase   : lane = token, MFMA accumulators hold q.K^T for the block's 64 tokens x the
//                 GQA query heads of the KV head;
//   softmax     : scores are rounded to fp16, divided by sqrt(d) in fp16 (as the reference's glue
//                 does), the block maximum and the sum of exp(w - max) are reduced over the wavefront,
//                 and the un-normalised weights exp(w - max) go to LDS as the fp16 B operand;
//   value phase : lane = channel, MFMA accumulators hold sum_t weight[t] * V[t][channel].
// The wavefronts of a workgroup (consecutive token blocks of one KV head) then combine their
// (max, sum, output) triples through LDS; token splits across workgroups are combined by a small
// merge kernel.  Scores and probabilities never touch HBM.
#include "fused_common.hpp"
#include "step_device.hpp"

#include <atomic>

namespace mstf {

// grid = (token splits, KV heads), kFusedWaves wavefronts; wavefront w of split s owns the bpw consecutive token
// blocks (s*kFusedWaves + w)*bpw ...  NM = accumulator groups of four query heads (groups <= 4*NM).
// MULTI = false: bpw is 1.  MULTI = true: the wavefront walks its blocks one after the other - the first value
// stream, the boundaries and the first scalar batch of the coming block are requested while the current block is
// still being decompressed, so only the first block of a wavefront waits for memory - and folds every block's
// (max, sum, output) into running ones before the workgroup combine.
//   write_final (only with one split) : out[(kv*groups + h)*D + d] fp16 final
//   otherwise   : part_o[((kv*groups + h)*nsplit + split)*D + d], part_ml[..][2] = (max, sum)
// STEP: the launch is a whole decode step (StepArgs above, the last argument; DecodeKernargs mirrors the argument list
// and tells where it sits in the kernel-argument segment): the query rows come rotated out of the projection output
// instead of q, and the wavefronts also take the blocks of the dense window.
struct DecodeKernargs {
    const void* first_ptrs[4];
    size_t tstride;
    const void* tokens_dev;
    int nblk, bpw;
    const void* ptrs[8];
    int groups, nsplit, write_final;
    float sqrt_d;
    StepArgs st;
};
constexpr size_t kStepArgsAt = offsetof(DecodeKernargs, st);
template <int NM, bool MULTI, bool STEP = false>
__global__ __launch_bounds__(kFusedWaves * 64) __attribute__((amdgpu_waves_per_eu(MSTF_FUSED_OCCUPANCY))) void decode_attention_kernel(
    const uint32_t* __restrict__ k_idx, const uint32_t* __restrict__ v_idx, const uint32_t* __restrict__ k_nz_off,
    const uint32_t* __restrict__ v_nz_off, size_t tstride, const int* __restrict__ tokens_dev, int nblk, int bpw,
    const uint64_t* __restrict__ k_bmp, const char* __restrict__ k_nz, const uint64_t* __restrict__ v_bmp,
    const char* __restrict__ v_nz, const _Float16* __restrict__ q, _Float16* __restrict__ out,
    float* __restrict__ part_o, float* __restrict__ part_ml, int groups, int nsplit, int write_final, float sqrt_d,
    StepArgs st)
{
    // Argument order: the first fourteen 32-bit words - what the first load of a wavefront, the stage boundaries,
    // needs - are in scalar registers when the wavefront starts (kernel-argument preload, a compile option of this
    // library); the others are fetched from the argument segment while that load is on its way.
    // tstride: tiles between the bitmap rows of two heads (offsets: one more), which is the tile count of the cached
    // tokens unless the cache is pre-allocated for more.  tokens_dev (nullable): the number of cached tokens is read
    // from device memory, at most nblk blocks of it; the launch is then sized for the capacity and the wavefronts
    // beyond the valid blocks leave neutral partials, so a recorded launch stays valid while the cache grows.
    constexpr int D = kFusedD;
    if (tokens_dev) {
        const int valid = *tokens_dev / 64;
        nblk = valid < nblk ? valid : nblk;
        // the launch is sized for one block per wavefront at full capacity; the blocks a wavefront walks follow from
        // the tokens that are there now, as a launch sized for exactly them would choose (fused_blocks_per_wave), and
        // the workgroups behind the last block leave neutral partials
        if (MULTI) {
            const int r = ((int)gridDim.y * nblk + kFusedResident - 1) / kFusedResident;
            bpw = r < 1 ? 1 : (r > kFusedMaxBpw ? kFusedMaxBpw : r);
        }
    }
    constexpr int kQLds = NM * 4 * D * 2;          // query rows [4*NM][D] fp16
    constexpr int kPRow = 64 * 2;                  // one row of block weights: 64 tokens fp16
    constexpr int kPLds = NM * 4 * kPRow;
    constexpr int kNeed = kNzLds + kQLds + kPLds;
    constexpr int kPark = NM * 4 * D * 4 + 64;     // per-wave (output, max, sum) parked for the workgroup combine
    constexpr int kWaveLds = kNeed > kPark ? kNeed : kPark;
    constexpr int kStages = kKeySubs + kValSubs;
    static_assert(kStages % 2 == 0, "the first stage of the coming block lands in buffer 0");
    __shared__ __attribute__((aligned(16))) char lds[kFusedWaves][kWaveLds];
    const int lane = lane_id();
    const int wave = wave_id();
    const int split = (int)blockIdx.x;
    const int kv = (int)blockIdx.y;
    const int tb = (split * kFusedWaves + wave) * (MULTI ? bpw : 1);  // first token block of this wavefront
    int nb = nblk - tb;                                                // its blocks (wave-uniform)
    if (MULTI) nb = nb > bpw ? bpw : nb;
    const bool active = nb > 0;
    // STEP: a wavefront that also has a block of the dense window to do keeps the highest issue priority through its
    // walk (it has the longest way to go; see set_wave_priority)
    uint32_t prio_boost = 0u;
    if constexpr (STEP) prio_boost = step_window_boost(st, wave, split);
    const int j = lane & 3;
    const size_t T = tstride;
    char* my = lds[wave];
    char* ql = my + kNzLds;
    char* pl = ql + kQLds;
    const uint32_t lbase = lds_addr(my);
    const uint32_t zaddr = lbase + 2 * kSubBytes;

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
        const uint64_t* bmK = k_bmp + (size_t)kv * T + (size_t)tb * D;
        const uint32_t* ixK = k_idx + (size_t)kv * (T + 1) + (size_t)tb * D;
        const uint64_t* bmV = v_bmp + (size_t)kv * T + (size_t)tb * D;
        const uint32_t* ixV = v_idx + (size_t)kv * (T + 1) + (size_t)tb * D;
        if (lane < 4) reinterpret_cast<uint32_t*>(my + 2 * kSubBytes)[lane] = 0u;
        const char *nzK = nullptr, *nzV = nullptr;  // the head's value streams (set below, from the boundary load)

        // sub-chunk n of a block's walk: n < kKeySubs -> key tiles n*32.., else value tiles (n-kKeySubs)*32..
        auto bm_of = [&](int n) { return n < kKeySubs ? bmK + n * kSubTiles : bmV + (n - kKeySubs) * kSubTiles; };
        auto ix_of = [&](int n) { return n < kKeySubs ? ixK + n * kSubTiles : ixV + (n - kKeySubs) * kSubTiles; };
        auto nz_of = [&](int n) { return n < kKeySubs ? nzK : nzV; };
        // idx at the boundaries of all sub-chunks of a block, fetched by one vector load (lanes 0.. hold the key
        // boundaries, lanes 16.. the value boundaries): no stage then waits for a scalar load from HBM
        // before it can issue its value stream
        static_assert(kKeySubs < 16 && kValSubs < 48, "boundary lanes");
        // (one unconditional load from a selected address: a branch here would split the block while the coming
        // scalar batch is live)
        const bool bnd_v = lane >= 16 && lane <= 16 + kValSubs;
        const int bnd_i = bnd_v ? (lane - 16) * kSubTiles : (lane <= kKeySubs ? lane * kSubTiles : 0);
        // Lanes 62 and 63 fetch the head's entries of v_nz_off and k_nz_off in the same load: fetched on their own
        // they are a round trip of their own in front of this one (the compiler waits for them where the value
        // streams' addresses are formed, which is before it issues this load).
        const uint32_t* const off_p = lane == 63 ? k_nz_off + kv : v_nz_off + kv;
        auto boundaries = [&](const uint32_t* ik, const uint32_t* iv) {
            const uint32_t* p = (bnd_v ? iv : ik) + bnd_i;
            p = lane >= 62 ? off_p : p;
            return *p;
        };
        uint32_t bnd = boundaries(ixK, ixV);
        __builtin_amdgcn_sched_barrier(0);  // (the load goes out before anything waits for the other arguments)
        // every other argument in registers now: left alone, the compiler fetches them where they are first used,
        // dependent round trips in front of the first load of data
        asm volatile("" ::"s"(k_bmp), "s"(k_nz), "s"(v_bmp), "s"(v_nz), "s"(q), "s"(out), "s"(part_o), "s"(part_ml),
                     "s"(groups), "s"(nsplit), "s"(write_final), "s"(sqrt_d));
        uint32_t bnd_next = bnd;  // MULTI: boundaries of the coming block
        const uint32_t lane16 = (uint32_t)lane * 16u;
        const uint32_t off8 = (uint32_t)(lane < kSubTiles ? lane : kSubTiles - 1) * 8u;
        const uint32_t off4 = (uint32_t)(lane <= kSubTiles ? lane : kSubTiles) * 4u;
        auto issue = [&](int n) {
            const int bl = n < kKeySubs ? n : 16 + n - kKeySubs;
            const uint32_t s0 = __builtin_amdgcn_readlane(bnd, bl);
            const uint32_t s1 = __builtin_amdgcn_readlane(bnd, bl + 1);
            sub_issue_flat(nz_of(n) + (size_t)s0 * 4u, sub_bytes(s0, s1), lbase + (uint32_t)(n & 1) * kSubBytes, lane16);
            return touch_sub_flat(bm_of(n), ix_of(n), off8, off4);
        };
        // first key sub-chunk of the coming block (adv = D tiles ahead; adv = 0 and no bytes after the last block)
        auto issue_coming = [&](int adv) {
            const uint32_t s0 = __builtin_amdgcn_readlane(bnd_next, 0);
            const uint32_t s1 = __builtin_amdgcn_readlane(bnd_next, 1);
            sub_issue_flat(nzK + (size_t)s0 * 4u, adv ? sub_bytes(s0, s1) : 0u, lbase, lane16);
            return touch_sub_flat(bmK + adv, ixK + adv, off8, off4);
        };

        // the query rows of this KV head: groups x D fp16, contiguous (STEP: rotated out of the projection output)
        if constexpr (STEP) {
            stage_query_rotated(ql, st, kv, groups, lane);
        } else {
            const char* qsrc = reinterpret_cast<const char*>(q + (size_t)kv * groups * D);
            const uint32_t qbytes = (uint32_t)groups * D * 2u;
#pragma unroll
            for (int i = 0; i < (kQLds + 1023) / 1024; i++) {
                const uint32_t o = (uint32_t)(i * 64 + lane) * 16u;
                if (o < qbytes) dma16(qsrc + o, ql + i * 1024);
            }
        }
        nzK = k_nz + (size_t)(uint32_t)__builtin_amdgcn_readlane(bnd, 63) * 16u;
        nzV = v_nz + (size_t)(uint32_t)__builtin_amdgcn_readlane(bnd, 62) * 16u;
        Touch touch = issue(0);

        const uint32_t qrow = lds_addr(ql) + (uint32_t)j * D * 2u;
        const uint32_t prow = lds_addr(pl) + (uint32_t)j * kPRow;

        // Bitmaps and tile offsets come in batches of 8 tiles through scalar loads, each requested one batch
        // ahead; the chain runs across the stages, from the key tiles into the value tiles and (MULTI) into the
        // coming block.
        constexpr int kBatches = kSubTiles / 8, kSideBatches = D / 8;
        Batch cur = load_batch_scalar(bmK, ixK);
        // nc, woffc: stage index and byte offset of the stage's first weight from wbase, as constants (they end up in
        // immediate operands)
        auto stage_batches = [&](auto nc, uint32_t buf, uint32_t wbase, auto woffc, uint32_t wgroup, f4_t (&acc)[NM],
                                 f4_t (&acc2)[NM], int adv) {
            constexpr int n = decltype(nc)::value;
            constexpr int woff = decltype(woffc)::value;
            const uint32_t rel = buf - cur.ov[0] * 4u;  // idx counts 4-byte units from the start of the head's values
            static_for<kBatches>([&](auto gc) {
                constexpr int g = decltype(gc)::value;
                constexpr int g1 = n * kBatches + g + 1;  // the coming batch, counted over key then value tiles
                constexpr int wo = woff + g * 16;
                Batch nxt;
                if constexpr (g1 < kSideBatches)
                    batch_step_exec<NM, true, g1 * 64, g1 * 32, wo>(cur, nxt, bmK, ixK, rel, zaddr, wbase, wgroup, acc, acc2);
                else if constexpr (g1 < 2 * kSideBatches)
                    batch_step_exec<NM, true, (g1 - kSideBatches) * 64, (g1 - kSideBatches) * 32, wo>(
                        cur, nxt, bmV, ixV, rel, zaddr, wbase, wgroup, acc, acc2);
                else if constexpr (MULTI)
                    batch_step_exec<NM, true, 0, 0, wo>(cur, nxt, bmK + adv, ixK + adv, rel, zaddr, wbase, wgroup, acc, acc2);
                else
                    batch_step_exec<NM, false, 0, 0, wo>(cur, nxt, bmK, ixK, rel, zaddr, wbase, wgroup, acc, acc2);
                cur = nxt;
            });
        };

#pragma unroll 1
        for (int r = 0; r < (MULTI ? nb : 1); r++) {
            const int adv = (MULTI && r + 1 < nb) ? D : 0;  // tiles to the coming block of this wavefront
            f4_t acc_k[NM], blk_v[NM][2];
            f4_t acc2[NM];  // the second set of sums of the gather statements (batch_step_dual), folded in per phase
            float m_blk[NM], l_blk[NM];
            constexpr bool kDual = NM == 1 && MSTF_DUAL_ACC;
#pragma unroll
            for (int m = 0; m < NM; m++) {
                acc2[m] = f4_t{0.f, 0.f, 0.f, 0.f};
                acc_k[m] = f4_t{0.f, 0.f, 0.f, 0.f};
                blk_v[m][0] = f4_t{0.f, 0.f, 0.f, 0.f};
                blk_v[m][1] = f4_t{0.f, 0.f, 0.f, 0.f};
            }
            static_for<kStages>([&](auto nc) {
                constexpr int n = decltype(nc)::value;
                // 3, 2, 1, 0 over the key stages and again over the value stages
                if constexpr (STEP) set_wave_priority_uniform(prio_boost | (uint32_t)(3 - n % 4));
                else set_wave_priority(3 - n % 4);
                wait_vm0_keep(touch);  // sub-chunk n has landed (with the query rows for the first one)
                // The buffer of sub-chunk n-1 is refilled now: every LDS read of that sub-chunk fed an MFMA that was
                // issued before this point, so the reads have returned.
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (n + 1 < kStages) touch = issue(n + 1);
                else if constexpr (MULTI) touch = issue_coming(adv);
                const uint32_t buf = lbase + (uint32_t)(n & 1) * kSubBytes;
                if constexpr (n < kKeySubs) {
                    stage_batches(nc, buf, qrow, std::integral_constant<int, n * kSubTiles * 2>{}, (uint32_t)D * 8u, acc_k,
                                  acc2, adv);
                } else {
                    if constexpr (n == kKeySubs) {
                        if constexpr (kDual) {
                            dual_settle(acc_k[0], acc2[0]);
                            acc_k[0] += acc2[0];
                            acc2[0] = f4_t{0.f, 0.f, 0.f, 0.f};
                        }
                        block_softmax<NM>(acc_k, sqrt_d, 64, pl, lane, m_blk, l_blk);
                        // its latency is covered by the value phase; the wait of the next stage completes it
                        if (MULTI) bnd_next = boundaries(ixK + adv, ixV + adv);
                    }
                    constexpr int vs = n - kKeySubs;              // value sub-chunk: half = vs / 2, tokens (vs % 2)*32..
                    constexpr int kSubsPerHalf = 64 / kSubTiles;
                    constexpr int half = vs / kSubsPerHalf;
                    f4_t tmp[NM];
#pragma unroll
                    for (int m = 0; m < NM; m++) tmp[m] = blk_v[m][half];
                    stage_batches(nc, buf, prow, std::integral_constant<int, (vs % kSubsPerHalf) * kSubTiles * 2>{},
                                  4u * kPRow, tmp, acc2, adv);
                    if constexpr (kDual && vs % kSubsPerHalf == kSubsPerHalf - 1) {  // the half is complete
                        dual_settle(tmp[0], acc2[0]);
                        tmp[0] += acc2[0];
                        acc2[0] = f4_t{0.f, 0.f, 0.f, 0.f};
                    }
#pragma unroll
                    for (int m = 0; m < NM; m++) blk_v[m][half] = tmp[m];
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            if (!MULTI) {
#pragma unroll
                for (int m = 0; m < NM; m++) {
                    acc_v[m][0] = blk_v[m][0];
                    acc_v[m][1] = blk_v[m][1];
                    m_run[m] = m_blk[m];
                    l_run[m] = l_blk[m];
                }
            } else {
                // fold the block into the running triple of this wavefront (lane 4b+j: head 4m+j in every register)
#pragma unroll
                for (int m = 0; m < NM; m++) {
                    const float mn = fmaxf(m_run[m], m_blk[m]);
                    const float fa = m_run[m] == -INFINITY ? 0.f : __expf(m_run[m] - mn);
                    const float fb = m_blk[m] == -INFINITY ? 0.f : __expf(m_blk[m] - mn);
#pragma unroll
                    for (int h = 0; h < 2; h++)
#pragma unroll
                        for (int c = 0; c < 4; c++) acc_v[m][h][c] = acc_v[m][h][c] * fa + blk_v[m][h][c] * fb;
                    l_run[m] = l_run[m] * fa + l_blk[m] * fb;
                    m_run[m] = mn;
                }
                bmK += adv;
                ixK += adv;
                bmV += adv;
                ixV += adv;
                bnd = bnd_next;
            }
        }
        wait_vm0();
        wait_lgkm0();
    }

    if constexpr (STEP) {
        // The dense window: its 64-token blocks are dealt out over the wavefronts of the head's workgroups - block i to
        // wavefront i / ns of split i % ns - which take them behind their compressed blocks, so the window costs no
        // workgroup of its own (a ninth workgroup per head would find no free slot on a full chip and run behind the
        // others).  The query rows are still in LDS; the value buffers and the weight rows are free again.
        // (the step's arguments are fetched again here, through a pointer the compiler cannot see through: kept in
        // scalar registers across the walk above they would push other values out)
        const StepArgs __attribute__((address_space(4)))* sp = (const StepArgs __attribute__((address_space(4)))*)(
            (const char __attribute__((address_space(4)))*)__builtin_amdgcn_kernarg_segment_ptr() + kStepArgsAt);
        asm volatile("" : "+s"(sp));
        StepArgs sw;
        sw.q_in = sp->q_in, sw.k_in = sp->k_in, sw.v_in = sp->v_in;
        sw.q_stride = sp->q_stride, sw.k_stride = sp->k_stride, sw.v_stride = sp->v_stride;
        sw.cos = sp->cos, sw.sin = sp->sin, sw.rope_stride = sp->rope_stride;
        sw.k_win = sp->k_win, sw.v_win = sp->v_win, sw.win_len_dev = sp->win_len_dev, sw.overflow = sp->overflow;
        sw.win_len = sp->win_len, sw.win_stride = sp->win_stride, sw.n_kv = sp->n_kv, sw.ns = sp->ns;
        const int wblk = wave * sw.ns + split;
        if (wblk < (sw.win_len + 63) / 64) {
            if (!active) stage_query_rotated(ql, sw, kv, groups, lane);
            step_window_wave<NM>(my, ql, pl, sw, part_o, part_ml, kv, groups, nsplit, wblk, sqrt_d, lane);
        }
    }
    workgroup_combine<NM>(&lds[0][0], kWaveLds, wave, lane, acc_v, m_run, l_run, kv, groups, split, nsplit, write_final,
                          out, part_o, part_ml);
}

// grid = Bq, 128 threads: log-sum-exp combine of the token splits.  The splits are taken eight at a time: the
// (max, sum) pairs and the partial outputs of a group are requested together, so a group costs one memory round
// trip, and the groups are folded into running (max, output, sum) values.
__global__ __launch_bounds__(128) void decode_merge_kernel(const float* __restrict__ part_o,
                                                           const float* __restrict__ part_ml,
                                                           _Float16* __restrict__ out, float* __restrict__ lse_out,
                                                           int nsplit, int D)
{
    constexpr int G = 8;
    const size_t row = blockIdx.x;
    const int c = (int)threadIdx.x < D ? (int)threadIdx.x : D - 1;
    const float2* ml = reinterpret_cast<const float2*>(part_ml) + row * nsplit;
    const float* po = part_o + row * nsplit * D + c;
    float M = -INFINITY, so = 0.f, sl = 0.f;
    for (int s0 = 0; s0 < nsplit; s0 += G) {
        float2 m[G];
        float o[G];
#pragma unroll
        for (int u = 0; u < G; u++) {
            const int s = s0 + u < nsplit ? s0 + u : nsplit - 1;  // clamped: the loads stay unconditional
            m[u] = ml[s];
            o[u] = po[(size_t)s * D];
        }
        float gm = M;
#pragma unroll
        for (int u = 0; u < G; u++)
            if (s0 + u < nsplit) gm = fmaxf(gm, m[u].x);
        const float fr = M == -INFINITY ? 0.f : __expf(M - gm);
        so *= fr;
        sl *= fr;
#pragma unroll
        for (int u = 0; u < G; u++) {
            const float f = (s0 + u < nsplit && m[u].x != -INFINITY) ? __expf(m[u].x - gm) : 0.f;
            so += f * o[u];
            sl += f * m[u].y;
        }
        M = gm;
    }
    if ((int)threadIdx.x < D) out[row * D + c] = (_Float16)(so / sl);
    if (lse_out && threadIdx.x == 0) {
        lse_out[row * 2] = M;
        lse_out[row * 2 + 1] = sl;
    }
}

// Dense local window of the decode step (the tokens that are not compressed yet,
// models/llama_mustafar_kernel.py:391-441): one wavefront per (KV head, 64-token block of the window) leaves the
// same (max, sum, un-normalised output) triple as a split of the compressed tokens, in split slot split0 + block,
// so that the merge kernel combines compressed tokens and window under one softmax.
// A dense block is handled as 128 full tiles of each format with the accumulation of the compressed path:
//   key phase   : the K block [64 tokens][128] goes through registers into an LDS slab with a padded row stride, so
//                 that lane = token reads column `channel` without bank conflicts (immediate offsets, no address
//                 arithmetic); MFMA against the query rows as in the compressed path;
//   value phase : the V block arrives by LDS-direct loads; lane = channel reads row `token`.
// k_win, v_win: [Bkv][win_stride][D] fp16, the first win_len tokens of every head valid; rows beyond are never read.
template <int NM>
__global__ __launch_bounds__(64) void window_attention_kernel(const _Float16* __restrict__ k_win, const _Float16* v_win,
                                                              const _Float16* q, float* __restrict__ part_o,
                                                              float* __restrict__ part_ml, int win_len,
                                                              const int* __restrict__ win_len_dev, int win_stride,
                                                              int groups, int nsplit, int split0, float sqrt_d)
{
    constexpr int D = kFusedD;
    constexpr int kKRow = D * 2 + 4;             // bytes per slab row: 256 of data + 4 of padding
    constexpr int kKSlab = 64 * kKRow;
    constexpr int kVBlk = 64 * D * 2;
    constexpr int kZero = 128;                   // a row half of zeros for the tokens beyond the window
    constexpr int kQLds = NM * 4 * D * 2;
    constexpr int kPRow = 64 * 2;
    constexpr int kPLds = NM * 4 * kPRow;
    // one array on purpose (LDS-direct loads into several LDS objects make the compiler serialise them)
    __shared__ __attribute__((aligned(16))) char lds[kKSlab + kVBlk + kZero + kQLds + kPLds];
    const int lane = lane_id();
    // heads vary fastest: the blocks beyond the valid length (a launch sized for the buffer) are dispatched last and do
    // not stand in the queue in front of working ones
    const int blk = (int)blockIdx.y, kv = (int)blockIdx.x;
    const int j = lane & 3;
    // the valid length may live in device memory (a captured graph replays with a growing window); the launch is
    // then sized for the buffer and a block beyond the window leaves a neutral triple
    if (win_len_dev) win_len = *win_len_dev < win_len ? *win_len_dev : win_len;
    if (blk * 64 >= win_len) {
#pragma unroll
        for (int m = 0; m < NM; m++) {
            const int h = 4 * m + j;
            if (h < groups) {
                const size_t slot = ((size_t)kv * groups + h) * nsplit + split0 + blk;
                *reinterpret_cast<f4_t*>(part_o + slot * D + (lane & ~3)) = f4_t{0.f, 0.f, 0.f, 0.f};
                *reinterpret_cast<f4_t*>(part_o + slot * D + 64 + (lane & ~3)) = f4_t{0.f, 0.f, 0.f, 0.f};
                if (lane < 4) {
                    part_ml[slot * 2] = -INFINITY;
                    part_ml[slot * 2 + 1] = 0.f;
                }
            }
        }
        return;
    }
    int nt = win_len - blk * 64;
    nt = nt > 64 ? 64 : nt;
    char* kslab = lds;
    char* vblk = lds + kKSlab;
    char* zero = vblk + kVBlk;
    char* ql = zero + kZero;
    char* pl = ql + kQLds;
    const size_t row0 = (size_t)kv * win_stride + (size_t)blk * 64;

    // ---- staging: V rows and the query rows by LDS-direct loads, K rows through registers into the padded slab
    {
        const char* vsrc = reinterpret_cast<const char*>(v_win + row0 * D);
#pragma unroll
        for (int i = 0; i < kVBlk / 1024; i++) {
            const int row = i * 4 + (lane >> 4);  // 16 lanes per 256-byte row
            if (row < nt) dma16(vsrc + (size_t)(i * 64 + lane) * 16, vblk + i * 1024);
        }
        const char* qsrc = reinterpret_cast<const char*>(q + (size_t)kv * groups * D);
        const uint32_t qbytes = (uint32_t)groups * D * 2u;
#pragma unroll
        for (int i = 0; i < (kQLds + 1023) / 1024; i++) {
            const uint32_t o = (uint32_t)(i * 64 + lane) * 16u;
            if (o < qbytes) dma16(qsrc + o, ql + i * 1024);
        }
        if (lane < kZero / 4) reinterpret_cast<uint32_t*>(zero)[lane] = 0u;
        // all sixteen row pieces are requested before any is stored (a load under a branch would be waited for on
        // the spot): rows beyond the window re-read the last valid row and are cleared in registers
        const u32x4_t* ksrc = reinterpret_cast<const u32x4_t*>(k_win + row0 * D);
        u32x4_t kreg[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int e = i * 64 + lane;  // 16-byte piece: row e / 16, piece e % 16
            const int row = e >> 4, c16 = e & 15;
            const int src_row = row < nt ? row : nt - 1;
            kreg[i] = ksrc[src_row * 16 + c16];
        }
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int e = i * 64 + lane;
            const int row = e >> 4, c16 = e & 15;
            const uint32_t keep = row < nt ? 0xFFFFFFFFu : 0u;
            uint32_t* d = reinterpret_cast<uint32_t*>(kslab + row * kKRow + c16 * 16);
            d[0] = kreg[i][0] & keep;
            d[1] = kreg[i][1] & keep;
            d[2] = kreg[i][2] & keep;
            d[3] = kreg[i][3] & keep;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();

    // ---- key phase: tile c = channel c over the 64 tokens, lane = token
    f4_t acc_k[NM];
#pragma unroll
    for (int m = 0; m < NM; m++) acc_k[m] = f4_t{0.f, 0.f, 0.f, 0.f};
    const uint32_t kcol = lds_addr(kslab) + (uint32_t)lane * kKRow;
    const uint32_t qrow = lds_addr(ql) + (uint32_t)j * D * 2u;
    // the gathers of the next eight channels are issued before the current eight are consumed: with one wavefront
    // per SIMD nothing else would cover the LDS round trip
    auto key_gather = [&](int c8, _Float16 (&h)[8], u32x4_t (&w)[NM]) {
#pragma unroll
        for (int i = 0; i < 8; i++) h[i] = lds_load_h(kcol + (uint32_t)(c8 * 8 + i) * 2u);
#pragma unroll
        for (int m = 0; m < NM; m++)
            w[m] = *(MSTF_LDS const u32x4_t*)(uintptr_t)(qrow + (uint32_t)c8 * 16u + (uint32_t)m * (D * 8u));
    };
    {
        _Float16 hc[8], hn[8];
        u32x4_t wc[NM], wn[NM];
        key_gather(0, hc, wc);
#pragma unroll
        for (int c8 = 0; c8 < D / 8; c8++) {
            if (c8 + 1 < D / 8) key_gather(c8 + 1, hn, wn);
            __builtin_amdgcn_sched_barrier(0);
            const uint32_t v0 = pack_h2(hc[0], hc[1]), v1 = pack_h2(hc[2], hc[3]);
            const uint32_t v2 = pack_h2(hc[4], hc[5]), v3 = pack_h2(hc[6], hc[7]);
#pragma unroll
            for (int m = 0; m < NM; m++) {
                acc_k[m] = __builtin_amdgcn_mfma_f32_4x4x4f16(as_h4(v0, v1), as_h4(wc[m][0], wc[m][1]), acc_k[m], 0, 0, 0);
                acc_k[m] = __builtin_amdgcn_mfma_f32_4x4x4f16(as_h4(v2, v3), as_h4(wc[m][2], wc[m][3]), acc_k[m], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 8; i++) hc[i] = hn[i];
#pragma unroll
            for (int m = 0; m < NM; m++) wc[m] = wn[m];
        }
    }
    // ---- block statistics and fp16 weights; tokens beyond the window get weight 0
    float m_run[NM], l_run[NM];
    block_softmax<NM>(acc_k, sqrt_d, nt, pl, lane, m_run, l_run);
    // ---- value phase: tile (half, token) = 64 channels of one token, lane = channel of the half
    f4_t acc_v[NM][2];
    const uint32_t prow = lds_addr(pl) + (uint32_t)j * kPRow;
    const uint32_t vcol = lds_addr(vblk) + (uint32_t)lane * 2u;
    const uint32_t zcol = lds_addr(zero) + (uint32_t)lane * 2u;
    auto value_gather = [&](int g, _Float16 (&h)[8], u32x4_t (&w)[NM]) {  // g = half * 8 + group of eight tokens
        const int half = g >> 3, t8 = g & 7;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int t = t8 * 8 + i;  // a token beyond the window reads zeros: its weight is 0 but its row is not staged
            h[i] = lds_load_h(t < nt ? vcol + (uint32_t)(t * D * 2 + half * 128) : zcol);
        }
#pragma unroll
        for (int m = 0; m < NM; m++)
            w[m] = *(MSTF_LDS const u32x4_t*)(uintptr_t)(prow + (uint32_t)t8 * 16u + (uint32_t)m * (4u * kPRow));
    };
#pragma unroll
    for (int m = 0; m < NM; m++) acc_v[m][0] = acc_v[m][1] = f4_t{0.f, 0.f, 0.f, 0.f};
    {
        _Float16 hc[8], hn[8];
        u32x4_t wc[NM], wn[NM];
        value_gather(0, hc, wc);
#pragma unroll
        for (int g = 0; g < 16; g++) {
            if (g + 1 < 16) value_gather(g + 1, hn, wn);
            __builtin_amdgcn_sched_barrier(0);
            const int half = g >> 3;
            const uint32_t v0 = pack_h2(hc[0], hc[1]), v1 = pack_h2(hc[2], hc[3]);
            const uint32_t v2 = pack_h2(hc[4], hc[5]), v3 = pack_h2(hc[6], hc[7]);
#pragma unroll
            for (int m = 0; m < NM; m++) {
                acc_v[m][half] = __builtin_amdgcn_mfma_f32_4x4x4f16(as_h4(v0, v1), as_h4(wc[m][0], wc[m][1]),
                                                                    acc_v[m][half], 0, 0, 0);
                acc_v[m][half] = __builtin_amdgcn_mfma_f32_4x4x4f16(as_h4(v2, v3), as_h4(wc[m][2], wc[m][3]),
                                                                    acc_v[m][half], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 8; i++) hc[i] = hn[i];
#pragma unroll
            for (int m = 0; m < NM; m++) wc[m] = wn[m];
        }
    }
    // lane 4b+j holds channels 4b..4b+3 of both halves for head 4m+j
#pragma unroll
    for (int m = 0; m < NM; m++) {
        const int h = 4 * m + j;
        if (h < groups) {
            const size_t slot = ((size_t)kv * groups + h) * nsplit + split0 + blk;
            *reinterpret_cast<f4_t*>(part_o + slot * D + (lane & ~3)) = acc_v[m][0];
            *reinterpret_cast<f4_t*>(part_o + slot * D + 64 + (lane & ~3)) = acc_v[m][1];
            if (lane < 4) {
                part_ml[slot * 2] = m_run[m];
                part_ml[slot * 2 + 1] = l_run[m];
            }
        }
    }
}

}  // namespace mstf

using namespace mstf;

extern "C" size_t mstf_decode_attention_workspace_bytes(int tokens, int head_dim, int Bq, int groups)
{
    if (tokens <= 0 || head_dim != kFusedD || Bq <= 0 || groups <= 0 || tokens % 64 != 0 || Bq % groups != 0) return 0;
    const int ns = fused_nsplit(tokens);
    return round_up((size_t)Bq * ns * (head_dim + 2) * sizeof(float), 256);
}

// Shared argument checks of the fused entry points.
constexpr size_t kWorkspaceIsOurs = ~(size_t)0;
static int decode_check(const void* k_bmp, const void* k_nz, const void* k_idx, const void* k_nz_off, const void* v_bmp,
                        const void* v_nz, const void* v_idx, const void* v_nz_off, const void* q, int tokens,
                        int head_dim, int Bq, int groups, const void* workspace, size_t workspace_bytes)
{
    if (!k_bmp || !k_nz || !k_idx || !k_nz_off || !v_bmp || !v_nz || !v_idx || !v_nz_off || !q) return MSTF_EINVAL;
    if (tokens <= 0 || Bq <= 0 || groups <= 0 || Bq % groups != 0) return MSTF_EINVAL;
    if (head_dim != kFusedD || tokens % 64 != 0 || groups > 8) return MSTF_EUNSUPPORTED;
    if (!aligned_to(k_bmp, 8) || !aligned_to(v_bmp, 8) || !aligned_to(k_nz, 16) || !aligned_to(v_nz, 16) ||
        !aligned_to(k_idx, 4) || !aligned_to(v_idx, 4) || !aligned_to(k_nz_off, 4) || !aligned_to(v_nz_off, 4) ||
        !aligned_to(q, 16))
        return MSTF_EALIGN;
    if (workspace_bytes == kWorkspaceIsOurs) return MSTF_OK;  // the library's own buffer: nothing of the caller's to check
    const size_t need = mstf_decode_attention_workspace_bytes(tokens, head_dim, Bq, groups);
    if (!workspace || workspace_bytes < need) return MSTF_EWORKSPACE;
    if (!aligned_to(workspace, 16)) return MSTF_EALIGN;
    return MSTF_OK;
}

// Launches the fp16 kernel over the compressed tokens; returns through *ns_out the split slots it fills
// (slots 0 .. ns-1 of every query row; nsplit_total slots per row when a dense window adds its own behind them).
static int decode_launch(hipStream_t st, const uint64_t* k_bmp, const mstf_half* k_nz, const uint32_t* k_idx,
                         const uint32_t* k_nz_off, const uint64_t* v_bmp, const mstf_half* v_nz, const uint32_t* v_idx,
                         const uint32_t* v_nz_off, const mstf_half* q, mstf_half* out, int tokens, int head_dim, int Bq,
                         int groups, void* workspace, int write_final, int nsplit_total = 0, size_t tile_stride = 0,
                         const int32_t* tokens_dev = nullptr, const StepArgs* step = nullptr)
{
    const size_t tstride = tile_stride ? tile_stride : (size_t)tokens * head_dim / 64;
    const int Bkv = Bq / groups, nblk = tokens / 64;
    // token count in device memory: as many splits as any count up to `tokens` needs, the kernel works out the blocks
    // per wavefront itself
    const int bpw = tokens_dev ? 0 : fused_blocks_per_wave(tokens, Bkv);
    const int ns = tokens_dev ? fused_nsplit_capacity(tokens, Bkv) : fused_nsplit(tokens, bpw);
    const int nst = nsplit_total > 0 ? nsplit_total : ns;
    float* part_o = reinterpret_cast<float*>(workspace);
    float* part_ml = part_o + (size_t)Bq * nst * head_dim;
    StepArgs sa = {};
    if (step) {
        sa = *step;
        sa.ns = ns;
        // the window's blocks are dealt out over the ns * kFusedWaves wavefronts of a head
        if (window_blocks(sa.win_len) > ns * kFusedWaves) return MSTF_EUNSUPPORTED;
    }
    const dim3 grid((unsigned)ns, (unsigned)Bkv);
    const char* knz = reinterpret_cast<const char*>(k_nz);
    const char* vnz = reinterpret_cast<const char*>(v_nz);
    const _Float16* qh = reinterpret_cast<const _Float16*>(q);
    _Float16* oh = reinterpret_cast<_Float16*>(out);
    const float sq = sqrtf((float)head_dim);
#define MSTF_FD(NMV, MULTIV)                                                                                         \
    hipLaunchKernelGGL((decode_attention_kernel<NMV, MULTIV>), grid, dim3(kFusedWaves * 64), 0, st, k_idx, v_idx,   \
                       k_nz_off, v_nz_off, tstride, tokens_dev, nblk, bpw, k_bmp, knz, v_bmp, vnz, qh, oh, part_o,  \
                       part_ml, groups, nst, write_final, sq, sa)
    if (step) {  // (token count in device memory: the MULTI form)
        if (groups <= 4)
            hipLaunchKernelGGL((decode_attention_kernel<1, true, true>), grid, dim3(kFusedWaves * 64), 0, st, k_idx,
                               v_idx, k_nz_off, v_nz_off, tstride, tokens_dev, nblk, bpw, k_bmp, knz, v_bmp, vnz, qh, oh,
                               part_o, part_ml, groups, nst, write_final, sq, sa);
        else
            hipLaunchKernelGGL((decode_attention_kernel<2, true, true>), grid, dim3(kFusedWaves * 64), 0, st, k_idx,
                               v_idx, k_nz_off, v_nz_off, tstride, tokens_dev, nblk, bpw, k_bmp, knz, v_bmp, vnz, qh, oh,
                               part_o, part_ml, groups, nst, write_final, sq, sa);
    } else if (groups <= 4) {
        if (bpw == 1) MSTF_FD(1, false); else MSTF_FD(1, true);
    } else {
        if (bpw == 1) MSTF_FD(2, false); else MSTF_FD(2, true);
    }  // (bpw == 0: the kernel decides, MULTI form)
#undef MSTF_FD
    return check_launch();
}

// Merge of ns split slots per query row (layout of the partial entry point); shared with the quantised kernel.
int mstf::merge_splits(hipStream_t st, const void* workspace, mstf_half* out, float* lse_out, int ns, int head_dim,
                       int Bq)
{
    const float* part_o = reinterpret_cast<const float*>(workspace);
    const float* part_ml = part_o + (size_t)Bq * ns * head_dim;
    hipLaunchKernelGGL(decode_merge_kernel, dim3((unsigned)Bq), dim3(128), 0, st, part_o, part_ml,
                       reinterpret_cast<_Float16*>(out), lse_out, ns, head_dim);
    return check_launch();
}

int mstf::window_launch(hipStream_t st, const mstf_half* k_win, const mstf_half* v_win, const mstf_half* q,
                        void* workspace, int win_len, const int32_t* win_len_dev, int win_stride, int head_dim, int Bq,
                        int groups, int nst, int split0)
{
    float* part_o = reinterpret_cast<float*>(workspace);
    float* part_ml = part_o + (size_t)Bq * nst * head_dim;
    const _Float16* kw = reinterpret_cast<const _Float16*>(k_win);
    const _Float16* vw = reinterpret_cast<const _Float16*>(v_win);
    const _Float16* qh = reinterpret_cast<const _Float16*>(q);
    const float sq = sqrtf((float)head_dim);
    const dim3 grid((unsigned)(Bq / groups), (unsigned)window_blocks(win_len));
    if (groups <= 4)
        hipLaunchKernelGGL(window_attention_kernel<1>, grid, dim3(64), 0, st, kw, vw, qh, part_o, part_ml, win_len,
                           win_len_dev, win_stride, groups, nst, split0, sq);
    else
        hipLaunchKernelGGL(window_attention_kernel<2>, grid, dim3(64), 0, st, kw, vw, qh, part_o, part_ml, win_len,
                           win_len_dev, win_stride, groups, nst, split0, sq);
    return check_launch();
}

static int splits_of(int tokens, int Bq, int groups)
{
    return fused_nsplit(tokens, fused_blocks_per_wave(tokens, Bq / groups));
}

extern "C" int mstf_decode_attention_splits(int tokens, int head_dim, int Bq, int groups)
{
    if (tokens <= 0 || head_dim != kFusedD || Bq <= 0 || groups <= 0 || tokens % 64 != 0 || Bq % groups != 0) return 0;
    return splits_of(tokens, Bq, groups);
}

extern "C" int mstf_decode_attention_partial_f16(void* stream, const uint64_t* k_bmp, const mstf_half* k_nz,
                                                 const uint32_t* k_idx, const uint32_t* k_nz_off,
                                                 const uint64_t* v_bmp, const mstf_half* v_nz, const uint32_t* v_idx,
                                                 const uint32_t* v_nz_off, const mstf_half* q, int tokens, int head_dim,
                                                 int Bq, int groups, void* workspace, size_t workspace_bytes)
{
    const int rc = decode_check(k_bmp, k_nz, k_idx, k_nz_off, v_bmp, v_nz, v_idx, v_nz_off, q, tokens, head_dim, Bq,
                                groups, workspace, workspace_bytes);
    if (rc != MSTF_OK) return rc;
    return decode_launch(as_stream(stream), k_bmp, k_nz, k_idx, k_nz_off, v_bmp, v_nz, v_idx, v_nz_off, q, nullptr,
                         tokens, head_dim, Bq, groups, workspace, 0);
}

extern "C" int mstf_decode_attention_merge_f16(void* stream, const void* workspace, size_t workspace_bytes,
                                               mstf_half* out, float* lse_out, int tokens, int head_dim, int Bq,
                                               int groups)
{
    if (!out) return MSTF_EINVAL;
    if (tokens <= 0 || Bq <= 0 || groups <= 0 || Bq % groups != 0) return MSTF_EINVAL;
    if (head_dim != kFusedD || tokens % 64 != 0 || groups > 8) return MSTF_EUNSUPPORTED;
    const size_t need = mstf_decode_attention_workspace_bytes(tokens, head_dim, Bq, groups);
    if (!workspace || workspace_bytes < need) return MSTF_EWORKSPACE;
    if (!aligned_to(workspace, 16) || !aligned_to(out, 2) || (lse_out && !aligned_to(lse_out, 4))) return MSTF_EALIGN;
    return merge_splits(as_stream(stream), workspace, out, lse_out, splits_of(tokens, Bq, groups), head_dim, Bq);
}

extern "C" int mstf_decode_attention_f16(void* stream, const uint64_t* k_bmp, const mstf_half* k_nz,
                                         const uint32_t* k_idx, const uint32_t* k_nz_off, const uint64_t* v_bmp,
                                         const mstf_half* v_nz, const uint32_t* v_idx, const uint32_t* v_nz_off,
                                         const mstf_half* q, mstf_half* out, float* lse_out, int tokens, int head_dim,
                                         int Bq, int groups, void* workspace, size_t workspace_bytes)
{
    if (!out) return MSTF_EINVAL;
    int rc = decode_check(k_bmp, k_nz, k_idx, k_nz_off, v_bmp, v_nz, v_idx, v_nz_off, q, tokens, head_dim, Bq, groups,
                          workspace, workspace_bytes);
    if (rc != MSTF_OK) return rc;
    if (!aligned_to(out, 2) || (lse_out && !aligned_to(lse_out, 4))) return MSTF_EALIGN;
    // with one split and no (max, sum) requested the kernel writes the final output itself
    const int write_final = (splits_of(tokens, Bq, groups) == 1 && !lse_out) ? 1 : 0;
    rc = decode_launch(as_stream(stream), k_bmp, k_nz, k_idx, k_nz_off, v_bmp, v_nz, v_idx, v_nz_off, q, out, tokens,
                       head_dim, Bq, groups, workspace, write_final);
    if (rc != MSTF_OK || write_final) return rc;
    return mstf_decode_attention_merge_f16(stream, workspace, workspace_bytes, out, lse_out, tokens, head_dim, Bq,
                                           groups);
}


// ------------------------------------------------------------------ the entry point that allocates nothing
// mstf_decode_attention_f16 with the split partials in a buffer the library itself holds: a file-scope device array
// (one copy per GPU, held until the process ends).  In host code the array's name is only a handle for
// hipGetSymbolAddress; the device address it yields - looked up once per device, with that device current - is what the
// kernels get.
constexpr size_t kStaticScratchBytes = MSTF_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kStaticMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kStaticMaxDevices];

static int static_scratch(void** ptr)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kStaticMaxDevices) {
        set_last_hip_error((int)(e != hipSuccess ? e : hipErrorInvalidDevice));
        return MSTF_ELAUNCH;
    }
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            set_last_hip_error((int)(e != hipSuccess ? e : hipErrorInvalidSymbol));
            return MSTF_ELAUNCH;
        }
        g_scratch_ptr[dev].store(p, std::memory_order_release);  // every thread finds the same address
    }
    *ptr = p;
    return MSTF_OK;
}

extern "C" int mstf_decode_attention_static_f16(void* stream, const uint64_t* k_bmp, const mstf_half* k_nz,
                                                const uint32_t* k_idx, const uint32_t* k_nz_off, const uint64_t* v_bmp,
                                                const mstf_half* v_nz, const uint32_t* v_idx, const uint32_t* v_nz_off,
                                                const mstf_half* q, mstf_half* out, float* lse_out, int tokens,
                                                int head_dim, int Bq, int groups)
{
    if (!out) return MSTF_EINVAL;
    // sizes first, on the host alone: a problem whose partials do not fit is refused before anything touches the GPU
    if (tokens <= 0 || Bq <= 0 || groups <= 0 || Bq % groups != 0) return MSTF_EINVAL;
    if (head_dim != kFusedD || tokens % 64 != 0 || groups > 8) return MSTF_EUNSUPPORTED;
    const size_t need = mstf_decode_attention_workspace_bytes(tokens, head_dim, Bq, groups);
    if (need == 0 || need > kStaticScratchBytes) return MSTF_ETOOLARGE;
    void* ws = nullptr;
    int rc = decode_check(k_bmp, k_nz, k_idx, k_nz_off, v_bmp, v_nz, v_idx, v_nz_off, q, tokens, head_dim, Bq, groups,
                          nullptr, kWorkspaceIsOurs);
    if (rc != MSTF_OK) return rc;
    if (!aligned_to(out, 2) || (lse_out && !aligned_to(lse_out, 4))) return MSTF_EALIGN;
    if ((rc = static_scratch(&ws)) != MSTF_OK) return rc;
    // every split slot of every row is written by the partial kernel before the merge reads it: nothing to clear
    const int write_final = (splits_of(tokens, Bq, groups) == 1 && !lse_out) ? 1 : 0;
    rc = decode_launch(as_stream(stream), k_bmp, k_nz, k_idx, k_nz_off, v_bmp, v_nz, v_idx, v_nz_off, q, out, tokens,
                       head_dim, Bq, groups, ws, write_final);
    if (rc != MSTF_OK || write_final) return rc;
    return merge_splits(as_stream(stream), ws, out, lse_out, splits_of(tokens, Bq, groups), head_dim, Bq);
}

extern "C" size_t mstf_decode_attention_window_workspace_bytes(int tokens, int max_window, int head_dim, int Bq,
                                                               int groups)
{
    if (tokens < 0 || max_window <= 0 || head_dim != kFusedD || Bq <= 0 || groups <= 0 || tokens % 64 != 0 ||
        Bq % groups != 0)
        return 0;
    const int nst = fused_nsplit(tokens) + window_blocks(max_window);
    return round_up((size_t)Bq * nst * (head_dim + 2) * sizeof(float), 256);
}

extern "C" int mstf_decode_attention_window_f16(void* stream, const uint64_t* k_bmp, const mstf_half* k_nz,
                                                const uint32_t* k_idx, const uint32_t* k_nz_off, const uint64_t* v_bmp,
                                                const mstf_half* v_nz, const uint32_t* v_idx, const uint32_t* v_nz_off,
                                                const mstf_half* q, const mstf_half* k_win, const mstf_half* v_win,
                                                int win_len, const int32_t* win_len_dev, int win_stride, mstf_half* out,
                                                float* lse_out, int tokens,
                                                int head_dim, int Bq, int groups, void* workspace,
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
    const int ns = tokens > 0 ? splits_of(tokens, Bq, groups) : 0, nwb = window_blocks(win_len), nst = ns + nwb;
    int rc;
    if (tokens > 0) {
        // the compressed tokens fill split slots 0 .. ns-1 of every row
        rc = decode_check(k_bmp, k_nz, k_idx, k_nz_off, v_bmp, v_nz, v_idx, v_nz_off, q, tokens, head_dim, Bq, groups,
                          workspace, workspace_bytes);
        if (rc != MSTF_OK) return rc;
        rc = decode_launch(as_stream(stream), k_bmp, k_nz, k_idx, k_nz_off, v_bmp, v_nz, v_idx, v_nz_off, q, nullptr,
                           tokens, head_dim, Bq, groups, workspace, 0, nst);
        if (rc != MSTF_OK) return rc;
    }
    if ((rc = window_launch(as_stream(stream), k_win, v_win, q, workspace, win_len, win_len_dev, win_stride, head_dim, Bq,
                            groups, nst, ns)) != MSTF_OK)
        return rc;
    return merge_splits(as_stream(stream), workspace, out, lse_out, nst, head_dim, Bq);
}

extern "C" int mstf_decode_attention_window_pool_f16(void* stream, const uint64_t* k_bmp, const mstf_half* k_nz,
                                                     const uint32_t* k_idx, const uint32_t* k_nz_off,
                                                     const uint64_t* v_bmp, const mstf_half* v_nz, const uint32_t* v_idx,
                                                     const uint32_t* v_nz_off, const mstf_half* q, const mstf_half* k_win,
                                                     const mstf_half* v_win, int win_len, const int32_t* win_len_dev,
                                                     int win_stride, mstf_half* out, float* lse_out, int max_tokens,
                                                     const int32_t* tokens_dev, int64_t tile_capacity, int head_dim,
                                                     int Bq, int groups, void* workspace, size_t workspace_bytes)
{
    if (!q || !k_win || !v_win || !out || !tokens_dev) return MSTF_EINVAL;
    if (max_tokens <= 0 || win_len <= 0 || win_stride < win_len || Bq <= 0 || groups <= 0 || Bq % groups != 0)
        return MSTF_EINVAL;
    if (head_dim != kFusedD || max_tokens % 64 != 0 || groups > 8) return MSTF_EUNSUPPORTED;
    if (tile_capacity < (int64_t)max_tokens * head_dim / 64) return MSTF_EINVAL;
    if (!aligned_to(q, 16) || !aligned_to(k_win, 16) || !aligned_to(v_win, 16) || !aligned_to(out, 2) ||
        (lse_out && !aligned_to(lse_out, 4)) || (win_len_dev && !aligned_to(win_len_dev, 4)) || !aligned_to(tokens_dev, 4))
        return MSTF_EALIGN;
    const size_t need = mstf_decode_attention_window_workspace_bytes(max_tokens, win_len, head_dim, Bq, groups);
    if (!workspace || workspace_bytes < need) return MSTF_EWORKSPACE;
    if (!aligned_to(workspace, 16)) return MSTF_EALIGN;
    const int ns = fused_nsplit_capacity(max_tokens, Bq / groups), nst = ns + window_blocks(win_len);
    int rc = decode_check(k_bmp, k_nz, k_idx, k_nz_off, v_bmp, v_nz, v_idx, v_nz_off, q, max_tokens, head_dim, Bq, groups,
                          workspace, workspace_bytes);
    if (rc != MSTF_OK) return rc;
    rc = decode_launch(as_stream(stream), k_bmp, k_nz, k_idx, k_nz_off, v_bmp, v_nz, v_idx, v_nz_off, q, nullptr, max_tokens,
                       head_dim, Bq, groups, workspace, 0, nst, (size_t)tile_capacity, tokens_dev);
    if (rc != MSTF_OK) return rc;
    if ((rc = window_launch(as_stream(stream), k_win, v_win, q, workspace, win_len, win_len_dev, win_stride, head_dim, Bq,
                            groups, nst, ns)) != MSTF_OK)
        return rc;
    return merge_splits(as_stream(stream), workspace, out, lse_out, nst, head_dim, Bq);
}

extern "C" int mstf_decode_step_pool_f16(void* stream, const uint64_t* k_bmp, const mstf_half* k_nz, const uint32_t* k_idx,
                                         const uint32_t* k_nz_off, const uint64_t* v_bmp, const mstf_half* v_nz,
                                         const uint32_t* v_idx, const uint32_t* v_nz_off, const mstf_half* q_in,
                                         int64_t q_stride, const mstf_half* k_in, int64_t k_stride, const mstf_half* v_in,
                                         int64_t v_stride, int bs, int n_q, int n_kv, const mstf_half* cos,
                                         const mstf_half* sin, int64_t rope_stride, mstf_half* k_win, mstf_half* v_win,
                                         int win_stride, int win_len, const int32_t* win_len_dev, uint32_t* overflow,
                                         mstf_half* out, float* lse_out, int max_tokens, const int32_t* tokens_dev,
                                         int64_t tile_capacity, int head_dim, void* workspace, size_t workspace_bytes)
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
    if (q_stride % 8 != 0 || k_stride % 8 != 0 || v_stride % 8 != 0 || rope_stride % 8 != 0) return MSTF_EALIGN;
    if (!aligned_to(q_in, 16) || !aligned_to(k_in, 16) || !aligned_to(v_in, 16) || !aligned_to(cos, 16) ||
        !aligned_to(sin, 16) || !aligned_to(k_win, 16) || !aligned_to(v_win, 16) || !aligned_to(out, 2) ||
        (lse_out && !aligned_to(lse_out, 4)) || (win_len_dev && !aligned_to(win_len_dev, 4)) ||
        !aligned_to(tokens_dev, 4) || !aligned_to(overflow, 4))
        return MSTF_EALIGN;
    const size_t need = mstf_decode_attention_window_workspace_bytes(max_tokens, win_len, head_dim, Bq, groups);
    if (!workspace || workspace_bytes < need) return MSTF_EWORKSPACE;
    if (!aligned_to(workspace, 16)) return MSTF_EALIGN;
    int rc = decode_check(k_bmp, k_nz, k_idx, k_nz_off, v_bmp, v_nz, v_idx, v_nz_off, q_in, max_tokens, head_dim, Bq, groups,
                          workspace, workspace_bytes);
    if (rc != MSTF_OK) return rc;
    const int ns = fused_nsplit_capacity(max_tokens, Bq / groups), nst = ns + window_blocks(win_len);
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
    rc = decode_launch(as_stream(stream), k_bmp, k_nz, k_idx, k_nz_off, v_bmp, v_nz, v_idx, v_nz_off, q_in, nullptr, max_tokens,
                       head_dim, Bq, groups, workspace, 0, nst, (size_t)tile_capacity, tokens_dev, &sa);
    if (rc != MSTF_OK) return rc;
    return merge_splits(as_stream(stream), workspace, out, lse_out, nst, head_dim, Bq);
}
