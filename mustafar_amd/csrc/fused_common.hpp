// Pieces shared by the fused decode-attention kernels (fused.hip: fp16 format and dense window; fused_quant.hip:
// quantised format): block softmax statistics, the workgroup combine and the layout of the split partials.
#pragma once
#include "spmv_common.hpp"
#include "spmv_device.hpp"

namespace mstf {

constexpr int kFusedD = 128;
#ifndef MSTF_FUSED_WAVES
#define MSTF_FUSED_WAVES 8
#endif
constexpr int kFusedWaves = MSTF_FUSED_WAVES;    // token blocks (= wavefronts) per workgroup: 512 tokens per split
constexpr int kKeySubs = kFusedD / kSubTiles;       // sub-chunks of the key phase
constexpr int kValSubs = kFusedD / kSubTiles;       // sub-chunks of the value phase (both halves)

// Wavefronts per SIMD the fused fp16 kernel is built for: its LDS footprint (two stage buffers of kSubTiles tiles) and
// its register budget (MSTF_GATHER_TOP) have to allow it.
#ifndef MSTF_FUSED_OCCUPANCY
#define MSTF_FUSED_OCCUPANCY 4
#endif
constexpr int kFusedResident = 1024 * MSTF_FUSED_OCCUPANCY;  // wavefronts of the fused kernel the 256 CUs hold at once
constexpr int kFusedMaxBpw = 8;

// (The planning helpers below are constexpr, hence usable from device code as well as from the launchers.)
// Token blocks one wavefront of the fp16 kernel walks: 1 while every block can have a resident wavefront of its
// own; beyond that the blocks are spread over one chip-filling set of wavefronts, so that only a wavefront's first
// block waits for memory.
constexpr int fused_blocks_per_wave(int tokens, int Bkv)
{
    const long long blocks = (long long)Bkv * (tokens / 64);
    const long long r = (blocks + kFusedResident - 1) / kFusedResident;
    return r < 1 ? 1 : (r > kFusedMaxBpw ? kFusedMaxBpw : (int)r);
}
// Split slots (= workgroups) per KV head: kFusedWaves * bpw token blocks each.
constexpr int fused_nsplit(int tokens, int bpw = 1)
{
    return (tokens / 64 + kFusedWaves * bpw - 1) / (kFusedWaves * bpw);
}

// Split slots that any token count up to `tokens` can need when the blocks per wavefront follow the count (a launch
// sized once for a cache that grows): far fewer than one block per wavefront would take once the chip is full.
constexpr int fused_nsplit_capacity(int tokens, int Bkv)
{
    int ns = 1;
    for (int n = 64; n <= tokens; n += 64) {
        const int s = fused_nsplit(n, fused_blocks_per_wave(n, Bkv));
        ns = s > ns ? s : ns;
    }
    return ns;
}

// Launches the merge of ns split slots per query row out of a workspace in the layout of the fused kernels
// (defined beside the merge kernel).
int merge_splits(hipStream_t st, const void* workspace, mstf_half* out, float* lse_out, int ns, int head_dim, int Bq);

// Launches the dense-window kernel: the (max, sum, output) triples of the window's 64-token blocks go into split
// slots split0 .. of a workspace with nst slots per query row (defined beside the kernel).
int window_launch(hipStream_t st, const mstf_half* k_win, const mstf_half* v_win, const mstf_half* q, void* workspace,
                  int win_len, const int32_t* win_len_dev, int win_stride, int head_dim, int Bq, int groups, int nst,
                  int split0);
constexpr int window_blocks(int win_len) { return (win_len + 63) / 64; }

// Reductions over the sixteen lanes 4b+j (b = 0..15) that hold column j, without LDS round trips: inside a row of
// sixteen lanes by two rotations (DPP row_ror 4 and 8, folded into the combining instruction), across the four rows by
// v_permlane16_swap / v_permlane32_swap (a and b copies of v: afterwards a holds the even rows / the lower half twice,
// b the odd rows / the upper half twice).  Every lane ends up with the maximum; of the sum, lanes 4b+j of one column may
// differ in the last bit (the rotations add in a different order per lane), and lanes 0..3 are the ones that are used.
typedef uint32_t u32x2v_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float dpp_row_ror(float v, int n4)
{
    const int x = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, n4 == 4 ? __builtin_amdgcn_update_dpp(x, x, 0x124, 0xf, 0xf, false)
                                               : __builtin_amdgcn_update_dpp(x, x, 0x128, 0xf, 0xf, false));
}
__device__ __forceinline__ void rows_swapped(float v, bool halves, float& a, float& b)
{
    const uint32_t x = __builtin_bit_cast(uint32_t, v);
    const u32x2v_t r = halves ? __builtin_amdgcn_permlane32_swap(x, x, false, false)
                              : __builtin_amdgcn_permlane16_swap(x, x, false, false);
    const uint32_t r0 = r[0], r1 = r[1];  // (a bit cast applied to a vector element directly reads element 0)
    a = __builtin_bit_cast(float, r0);
    b = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ float wave_max_same_column(float v)
{
    float a, b;
    v = fmaxf(v, dpp_row_ror(v, 4));
    v = fmaxf(v, dpp_row_ror(v, 8));
    rows_swapped(v, false, a, b);
    v = fmaxf(a, b);
    rows_swapped(v, true, a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float wave_sum_same_column(float v)
{
    float a, b;
    v += dpp_row_ror(v, 4);
    v += dpp_row_ror(v, 8);
    rows_swapped(v, false, a, b);
    v = a + b;
    rows_swapped(v, true, a, b);
    return a + b;
}

// x / c for |x| up to the fp16 range and c = sqrt(head_dim), r = 1 / c rounded: the quotient estimate and one
// correction by the exact remainder - the correctly rounded quotient, as the full division sequence gives it, without
// that sequence's scaling and special cases (a dozen instructions per value), which these operands never need.
__device__ __forceinline__ float div_small(float x, float c, float r)
{
    const float q = x * r;
    return __builtin_fmaf(__builtin_fmaf(-c, q, x), r, q);
}

// Softmax statistics of one 64-token block from its scores; lane 4b+j holds tokens 4b..4b+3 of head 4m+j in acc_k[m].
// Scores are rounded to fp16 and divided by sqrt(d) in fp16 (as the reference's glue does); the un-normalised
// weights exp(w - max) go to LDS as fp16 rows of 64 tokens, kPRow bytes apart, (the B operand of the value phase) and the block's
// (max, sum of the fp16 weights) stay in m_run / l_run.  Tokens >= nt (nt < 64 only in a partial block) get weight 0.
template <int NM, int kPRow = 64 * 2>
__device__ __forceinline__ void block_softmax(const f4_t (&acc_k)[NM], float sqrt_d, int nt, char* pl, int lane,
                                              float (&m_run)[NM], float (&l_run)[NM])
{
    const int j = lane & 3;
    const float rcp_d = 1.0f / sqrt_d;
#pragma unroll
    for (int m = 0; m < NM; m++) {
        float w[4];
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const _Float16 s16 = (_Float16)acc_k[m][r];
            w[r] = ((lane & ~3) + r < nt) ? (float)(_Float16)div_small((float)s16, sqrt_d, rcp_d) : -INFINITY;
            mx = fmaxf(mx, w[r]);
        }
        mx = wave_max_same_column(mx);
        float sum = 0.f;
        h4_t e16;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float e = w[r] == -INFINITY ? 0.f : __expf(w[r] - mx);
            e16[r] = (_Float16)e;
            sum += (float)e16[r];  // the sum matches the fp16 weights that multiply V
        }
        sum = wave_sum_same_column(sum);
        m_run[m] = mx;
        l_run[m] = sum;
        *reinterpret_cast<h4_t*>(pl + (m * 4 + j) * kPRow + (lane & ~3) * 2) = e16;
    }
}

// Workgroup combine of the kFusedWaves blocks of a split: every wavefront parks (output[4*NM][D], max, sum) in its
// own LDS area (`lds_base + wave * wave_stride`, at least NM*4*D*4 + 64 bytes), then one thread per (head, channel)
// folds them and writes either the final fp16 output (write_final, one split only) or the split's partial:
//   part_o[((kv*groups + h)*nsplit + split)*D + d] (un-normalised), part_ml[..][2] = (max, sum).
// An inactive wavefront parks (-inf, 0, 0).
template <int NM>
__device__ __forceinline__ void workgroup_combine(char* lds_base, int wave_stride, int wave, int lane,
                                                  const f4_t (&acc_v)[NM][2], const float (&m_run)[NM],
                                                  const float (&l_run)[NM], int kv, int groups, int split, int nsplit,
                                                  int write_final, _Float16* out, float* part_o, float* part_ml)
{
    constexpr int D = kFusedD;
    const int j = lane & 3;
    {
        // (the wavefront parks its triple in its own LDS region, which only it has used so far: no barrier in front)
        float* po = reinterpret_cast<float*>(lds_base + wave * wave_stride);
#pragma unroll
        for (int m = 0; m < NM; m++) {
            *reinterpret_cast<f4_t*>(po + (m * 4 + j) * D + (lane & ~3)) = acc_v[m][0];
            *reinterpret_cast<f4_t*>(po + (m * 4 + j) * D + 64 + (lane & ~3)) = acc_v[m][1];
            if (lane < 4) {
                po[NM * 4 * D + (m * 4 + j) * 2] = m_run[m];
                po[NM * 4 * D + (m * 4 + j) * 2 + 1] = l_run[m];
            }
        }
    }
    __syncthreads();
    for (int o = (int)threadIdx.x; o < groups * D; o += kFusedWaves * 64) {
        const int h = o / D, c = o - h * D;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < kFusedWaves; w++)
            M = fmaxf(M, reinterpret_cast<const float*>(lds_base + w * wave_stride)[NM * 4 * D + h * 2]);
        float so = 0.f, sl = 0.f;
#pragma unroll
        for (int w = 0; w < kFusedWaves; w++) {
            const float* pw = reinterpret_cast<const float*>(lds_base + w * wave_stride);
            const float mw = pw[NM * 4 * D + h * 2];
            const float f = mw == -INFINITY ? 0.f : __expf(mw - M);
            so += f * pw[h * D + c];
            sl += f * pw[NM * 4 * D + h * 2 + 1];
        }
        const size_t row = (size_t)kv * groups + h;
        if (write_final) {
            out[row * D + c] = (_Float16)(so / sl);
        } else {
            part_o[(row * nsplit + split) * D + c] = so;
            if (c == 0) {
                part_ml[(row * nsplit + split) * 2] = M;
                part_ml[(row * nsplit + split) * 2 + 1] = sl;
            }
        }
    }
}

}  // namespace mstf
