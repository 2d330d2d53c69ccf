// Device code of the decode step that runs inside the launch of the compressed tokens (fused.hip, fused_quant.hip):
// rotation of the new query / key heads, append of the new key / value row to the dense window, attention over the
// window's 64-token blocks.
#pragma once
#include "compress_common.hpp"
#include "fused_common.hpp"

namespace mstf {

// ------------------------------------------------------------------ the whole decode step in one launch
// The new token of a decode step for the launch that does everything the caller has to do per layer and step on the
// cache side (models/llama_mustafar_kernel.py:363-374, 391-441): rotary embedding of the new query and key heads, the
// append of the new key / value row to the dense window, attention over the compressed tokens and over the window.
// The workgroups of a KV head are the splits of the compressed tokens (the kernel below as it is, with the query rows
// rotated on their way into LDS); behind their compressed blocks, some of their wavefronts take one 64-token block of
// the window each, and the wavefront whose block holds the new row rotates / appends it.
struct StepArgs {
    const _Float16* q_in;  // projection outputs of the new token: [bs][n_q * 128], [bs][n_kv * 128] x 2, not rotated
    const _Float16* k_in;
    const _Float16* v_in;
    int64_t q_stride, k_stride, v_stride;  // halfs between two batch entries
    const _Float16* cos;                   // [bs][128] (rope_stride halfs apart; 0: one position for all), or null
    const _Float16* sin;
    int64_t rope_stride;
    _Float16* k_win;  // [Bkv][win_stride][128]
    _Float16* v_win;
    const int32_t* win_len_dev;  // valid rows AFTER this step, the new token included (null: win_len)
    uint32_t* overflow;          // sticky: a count outside 1 .. win_stride appends nothing
    int win_len, win_stride, n_kv, ns;
};

// 3 for a wavefront that step_window_wave gives a block of the dense window (block wave * ns + split of the rows that
// are valid after this step), else 0: OR-ed into the issue priority of its walk over the compressed tokens.
__device__ __forceinline__ uint32_t step_window_boost(const StepArgs& sa, int wave, int split)
{
    int wlen = sa.win_len_dev ? *sa.win_len_dev : sa.win_len;
    wlen = wlen < sa.win_len ? wlen : sa.win_len;
    const int has = wave * sa.ns + split < (wlen + 63) / 64;
    return (uint32_t)__builtin_amdgcn_readfirstlane(has ? 3 : 0);
}

// The query rows of KV head kv into LDS (ql: [4*NM][128] fp16), rotated: eight lanes per query head, a lane holds
// channels c .. c+7 and their partners 64 channels on.
template <int QROW = kFusedD * 2>
__device__ __forceinline__ void stage_query_rotated(char* ql, const StepArgs& sa, int kv, int groups, int lane)
{
    const int b = kv / sa.n_kv, hk = kv - b * sa.n_kv;
    const int h = lane >> 3, c = (lane & 7) * 8;
    if (h < groups) {
        const _Float16* xp = sa.q_in + b * sa.q_stride + (int64_t)(hk * groups + h) * kFusedD + c;
        uint4 o0 = *reinterpret_cast<const uint4*>(xp);
        uint4 o1 = *reinterpret_cast<const uint4*>(xp + 64);
        if (sa.cos) {
            const _Float16* cp = sa.cos + b * sa.rope_stride + c;
            const _Float16* sp = sa.sin + b * sa.rope_stride + c;
            const uint4 c0 = *reinterpret_cast<const uint4*>(cp), c1 = *reinterpret_cast<const uint4*>(cp + 64);
            const uint4 s0 = *reinterpret_cast<const uint4*>(sp), s1 = *reinterpret_cast<const uint4*>(sp + 64);
            const uint4 x0 = o0, x1 = o1;
            rope_piece(x0, x1, c0, c1, s0, s1, o0, o1);
        }
        *reinterpret_cast<uint4*>(ql + h * QROW + c * 2) = o0;
        *reinterpret_cast<uint4*>(ql + h * QROW + c * 2 + 128) = o1;
    }
}

// One 64-token block (wblk) of the dense window of KV head kv, by one wavefront; leaves the block's (max, sum,
// un-normalised output) in split slot sa.ns + wblk of every query row of the head, like a split of the compressed
// tokens.  my: the wavefront's LDS (two value buffers of VROWS rows first), ql: the rotated query rows (QROW bytes
// apart), pl: room for the block's weights (rows PROW bytes apart).
//   key phase   : lane = token holds its whole key row in registers (sixteen 16-byte loads; the lane of the new row
//                 reads the projection output instead, rotates it and stores it to the window), so the A operands of
//                 the products are register pairs as they are;
//   value phase : VROWS rows at a time go through LDS (LDS-direct loads, double buffered; the new row is patched in
//                 from registers), lane = channel reads them column-wise.
template <int NM, int QROW = kFusedD * 2, int PROW = 64 * 2, int VROWS = 16>
__device__ __forceinline__ void step_window_wave(char* my, char* ql, char* pl, const StepArgs& sa, float* part_o,
                                                 float* part_ml, int kv, int groups, int nst, int wblk, float sqrt_d,
                                                 int lane)
{
    constexpr int D = kFusedD;
    constexpr int kPRow = PROW;
    constexpr int kVBuf = VROWS * D * 2;  // bytes of one of the two value buffers
    static_assert(VROWS == 16 || VROWS == 8, "value rows per LDS buffer");
    const int j = lane & 3;
    int wlen = sa.win_len_dev ? *sa.win_len_dev : sa.win_len;
    const bool fits = wlen >= 1 && wlen <= sa.win_stride;
    if (!fits && sa.overflow && lane == 0 && wblk == 0) *sa.overflow = 1u;
    const int new_row = fits ? wlen - 1 : -1;
    wlen = wlen < 0 ? 0 : (wlen > sa.win_stride ? sa.win_stride : wlen);
    if (sa.win_len < wlen) wlen = sa.win_len;  // (the launch and the split slots are sized for win_len)
    const int row0 = wblk * 64;
    auto slot_of = [&](int h) { return ((size_t)kv * groups + h) * nst + sa.ns + wblk; };
    if (row0 >= wlen) {
#pragma unroll
        for (int m = 0; m < NM; m++) {
            const int h = 4 * m + j;
            if (h < groups) {
                const size_t slot = slot_of(h);
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
    const int nt = wlen - row0 > 64 ? 64 : wlen - row0;
    const int b = kv / sa.n_kv, hk = kv - b * sa.n_kv;
    const bool has_new = new_row >= row0 && new_row < row0 + 64;  // wave-uniform
    const bool is_new = row0 + lane == new_row;

    // ---- the first two pieces of the value rows are requested up front: they do not depend on the scores, both
    // buffers are free, and they land while the keys are multiplied
    const char* vsrc = reinterpret_cast<const char*>(sa.v_win + ((size_t)kv * sa.win_stride + row0) * D);
    auto issue_rows = [&](int qd) {
#pragma unroll
        for (int i = 0; i < VROWS / 4; i++) {
            const int row = qd * VROWS + i * 4 + (lane >> 4);
            if (row < nt) dma16(vsrc + (size_t)row * (D * 2) + (lane & 15) * 16, my + (qd & 1) * kVBuf + i * 1024);
        }
    };
    issue_rows(0);
    if (VROWS < nt) issue_rows(1);
    // the rows of the later pieces are pulled into the L2 cache meanwhile (one 4-byte load per 128-byte line, result
    // unused): their LDS-direct loads, which have to wait for a free buffer, then find them there
    uint32_t warm = 0u, warm2 = 0u;
    {
        const int wrow = 2 * VROWS + lane / 2;
        if (wrow < nt) warm = *reinterpret_cast<const uint32_t*>(vsrc + (size_t)(2 * VROWS) * (D * 2) + (size_t)lane * 128);
        if (2 * VROWS + 32 < 64 && wrow + 32 < (nt < 64 ? nt : 64))  // (eight rows per piece: rows 48 .. 63 as well)
            warm2 = *reinterpret_cast<const uint32_t*>(vsrc + (size_t)(2 * VROWS + 32) * (D * 2) + (size_t)lane * 128);
    }

    // ---- key rows into registers
    uint4 kr[16];
    {
        const int t = lane < nt ? lane : nt - 1;
        const _Float16* krow = is_new ? sa.k_in + b * sa.k_stride + (int64_t)hk * D
                                      : sa.k_win + ((size_t)kv * sa.win_stride + row0 + t) * D;
#pragma unroll
        for (int i = 0; i < 16; i++) kr[i] = *reinterpret_cast<const uint4*>(krow + 8 * i);
    }
    if (has_new) {
        if (sa.cos) {
            // every lane runs the rotation on its row, the lane of the new row keeps the result
            const _Float16* cp = sa.cos + b * sa.rope_stride;
            const _Float16* sp = sa.sin + b * sa.rope_stride;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const uint4 c0 = *reinterpret_cast<const uint4*>(cp + 8 * i), c1 = *reinterpret_cast<const uint4*>(cp + 64 + 8 * i);
                const uint4 s0 = *reinterpret_cast<const uint4*>(sp + 8 * i), s1 = *reinterpret_cast<const uint4*>(sp + 64 + 8 * i);
                uint4 o0, o1;
                rope_piece(kr[i], kr[i + 8], c0, c1, s0, s1, o0, o1);
                if (is_new) {
                    kr[i] = o0;
                    kr[i + 8] = o1;
                }
            }
        }
        if (is_new) {
            _Float16* dst = sa.k_win + ((size_t)kv * sa.win_stride + new_row) * D;
#pragma unroll
            for (int i = 0; i < 16; i++) *reinterpret_cast<uint4*>(dst + 8 * i) = kr[i];
        }
    }
    if (lane >= nt) {
#pragma unroll
        for (int i = 0; i < 16; i++) kr[i] = make_uint4(0u, 0u, 0u, 0u);
    }

    // ---- scores: channel c of the row x the query rows (B operand: the weights of accumulator lane & 3)
    f4_t acc_k[NM];
#pragma unroll
    for (int m = 0; m < NM; m++) acc_k[m] = f4_t{0.f, 0.f, 0.f, 0.f};
    const uint32_t qrow = lds_addr(ql) + (uint32_t)j * (uint32_t)QROW;
#pragma unroll
    for (int i = 0; i < 16; i++) {
#pragma unroll
        for (int m = 0; m < NM; m++) {
            const u32x4_t w = *(MSTF_LDS const u32x4_t*)(uintptr_t)(qrow + (uint32_t)i * 16u + (uint32_t)m * (4u * QROW));
            acc_k[m] = __builtin_amdgcn_mfma_f32_4x4x4f16(as_h4(kr[i].x, kr[i].y), as_h4(w[0], w[1]), acc_k[m], 0, 0, 0);
            acc_k[m] = __builtin_amdgcn_mfma_f32_4x4x4f16(as_h4(kr[i].z, kr[i].w), as_h4(w[2], w[3]), acc_k[m], 0, 0, 0);
        }
    }
    float m_run[NM], l_run[NM];
    block_softmax<NM, PROW>(acc_k, sqrt_d, nt, pl, lane, m_run, l_run);

    // ---- values: VROWS rows at a time through LDS
    f4_t acc_v[NM][2];
#pragma unroll
    for (int m = 0; m < NM; m++) acc_v[m][0] = acc_v[m][1] = f4_t{0.f, 0.f, 0.f, 0.f};
    uint4 vnew = make_uint4(0u, 0u, 0u, 0u);
    if (has_new) {
        vnew = *reinterpret_cast<const uint4*>(sa.v_in + b * sa.v_stride + (int64_t)hk * D + (lane & 15) * 8);
        if (lane < 16) *reinterpret_cast<uint4*>(sa.v_win + ((size_t)kv * sa.win_stride + new_row) * D + lane * 8) = vnew;
    }
    const uint32_t prow = lds_addr(pl) + (uint32_t)j * kPRow;
#pragma unroll
    for (int qd = 0; qd < 64 / VROWS; qd++) {
        if (qd * VROWS >= nt) break;  // wave-uniform
        wait_vm0();
        wait_lgkm0();  // the reads of the other buffer (two pieces back) are done before it is filled again
        __builtin_amdgcn_sched_barrier(0);
        if (qd >= 1 && qd + 1 < 64 / VROWS) issue_rows(qd + 1);  // (piece 1 is on its way since the start)
        char* buf = my + (qd & 1) * kVBuf;
        // the new row is not in the window buffer yet as far as this wavefront's loads can tell: from registers
        if (has_new && new_row - row0 >= qd * VROWS && new_row - row0 < qd * VROWS + VROWS && lane < 16)
            *reinterpret_cast<uint4*>(buf + (new_row - row0 - qd * VROWS) * (D * 2) + lane * 16) = vnew;
        // rows behind the window's end have weight 0, but what LDS holds there may be anything: zeros
        for (int r = nt > qd * VROWS ? nt : qd * VROWS; r < qd * VROWS + VROWS; r++)
            if (lane < 16) *reinterpret_cast<uint4*>(buf + (r - qd * VROWS) * (D * 2) + lane * 16) = make_uint4(0u, 0u, 0u, 0u);
        const uint32_t vcol = lds_addr(buf) + (uint32_t)lane * 2u;
#pragma unroll
        for (int half = 0; half < 2; half++) {
#pragma unroll
            for (int g4 = 0; g4 < VROWS / 4; g4++) {
                _Float16 h[4];
#pragma unroll
                for (int i = 0; i < 4; i++) h[i] = lds_load_h(vcol + (uint32_t)((g4 * 4 + i) * D * 2 + half * 128));
                const uint32_t v0 = pack_h2(h[0], h[1]), v1 = pack_h2(h[2], h[3]);
#pragma unroll
                for (int m = 0; m < NM; m++) {
                    const u32x2_t w = *(MSTF_LDS const u32x2_t*)(uintptr_t)(prow + (uint32_t)(qd * VROWS + g4 * 4) * 2u +
                                                                             (uint32_t)m * (4u * kPRow));
                    acc_v[m][half] = __builtin_amdgcn_mfma_f32_4x4x4f16(as_h4(v0, v1), as_h4(w[0], w[1]), acc_v[m][half], 0, 0, 0);
                }
            }
        }
    }
    wait_vm0();
    asm volatile("" ::"v"(warm), "v"(warm2));  // (kept until here: a load must not land in a register given to something else)
    // lane 4b+j holds channels 4b..4b+3 of both halves for head 4m+j
#pragma unroll
    for (int m = 0; m < NM; m++) {
        const int h = 4 * m + j;
        if (h < groups) {
            const size_t slot = slot_of(h);
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
