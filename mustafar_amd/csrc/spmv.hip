// Batched key / value SpMV over the bitmap format, and the scale+softmax glue between them.
//
// Both products share one inner loop over runs of consecutive tiles of one KV head:
//   key   : 64 tokens of one token block, tiles = channels       (lane = token)
//   value : 64 channels of one half of head_dim, tiles = tokens   (lane = channel)
// In both cases tile t contributes  D[t][lane] * w[n][t]  to accumulator n of the lane, where
// D[t][lane] is element `lane` of tile t (0 when its bitmap bit is clear) and w is the query row
// (key) or the probability row (value).  A wavefront streams the packed values of 32 tiles at a
// time (contiguous, 16-byte aligned) from HBM straight into its private LDS double buffer
// (global_load_lds, 16 bytes per lane), rebuilds D[t][lane] with a popcount rank (v_mbcnt) per
// tile and feeds groups of four tiles to v_mfma_f32_4x4x4f16, which multiplies them with the weights of
// four accumulators (the GQA query group) at once, so the products cost no vector-ALU issue slots.
// Bitmaps arrive one per lane by a coalesced vector load and are broadcast with v_readlane; tile
// offsets are a running sum of padded popcounts on the scalar ALU; weights are staged in LDS by the
// same LDS-direct loads.
#include "spmv_common.hpp"
#include "spmv_device.hpp"

namespace mstf {

// ------------------------------------------------------------------------------- key
// One wavefront per (KV head, token block): walks the D/32 channel sub-chunks of the block.
// C[(kv*rows + row0 + n)*Lc + token] = sum_d K[token][d] * Bm[(kv*rows + row0 + n)*D + d],  n < NW.
// LDS per wavefront: value double buffer + zero slot + the NW query rows (4*NM rows reserved).
template <int NW>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4))) void key_spmv_kernel(const uint64_t* __restrict__ bmp, const char* __restrict__ nz,
                                                       const uint32_t* __restrict__ idx,
                                                       const uint32_t* __restrict__ nz_off,
                                                       const _Float16* __restrict__ Bm, _Float16* __restrict__ C,
                                                       int Lc, int D, int nblk, int ntasks, int bm_rows_per_kv,
                                                       int row0)
{
    constexpr int NM = (NW + 3) / 4;
    constexpr int kMaxD = 128;
    constexpr int kWaveLds = kNzLds + NM * 4 * kMaxD * 2;
    __shared__ __attribute__((aligned(16))) char lds[4][kWaveLds];
    const int lane = lane_id();
    const int wave = wave_id();
    const int task = (int)blockIdx.x * 4 + wave;
    if (task >= ntasks) return;
    const int kv = task / nblk;
    const int tb = task - kv * nblk;
    const size_t T = (size_t)Lc * D / 64;
    const uint64_t* bmk = bmp + (size_t)kv * T;
    const uint32_t* ixk = idx + (size_t)kv * (T + 1);
    const char* nzk = nz + (size_t)nz_off[kv] * 16u;
    const char* wsrc = reinterpret_cast<const char*>(Bm + ((size_t)kv * bm_rows_per_kv + row0) * D);
    char* my = lds[wave];
    char* wl = my + kNzLds;                       // [4*NM rows][D] fp16; rows >= NW stay unwritten
    const uint32_t wbytes = (uint32_t)NW * D * 2u;  // the NW rows are contiguous in Bm

    f4_t acc[NM];
#pragma unroll
    for (int m = 0; m < NM; m++) acc[m] = f4_t{0.f, 0.f, 0.f, 0.f};
    const size_t tile0 = (size_t)tb * D;
    const uint32_t wrow = lds_addr(wl) + (uint32_t)(lane & 3) * (uint32_t)D * 2u;
    walk_subs<NM>(
        D / kSubTiles, [=](int n) { return tile0 + (size_t)n * kSubTiles; },
        [=](int n) {
            if (n != 0) return;  // the query rows are staged once per task
#pragma unroll
            for (int i = 0; i < (NW * kMaxD * 2 + 1023) / 1024; i++) {
                const uint32_t o = (uint32_t)(i * 64 + lane) * 16u;
                if (o < wbytes) dma16(wsrc + o, wl + i * 1024);
            }
        },
        [=](int n) { return wrow + (uint32_t)n * kSubTiles * 2u; }, (uint32_t)D * 8u, bmk, ixk, nzk, my, lane, acc);
    // lane 4b+j holds tokens 4b..4b+3 of accumulator 4m+j
    const int j = lane & 3;
    _Float16* out = C + ((size_t)kv * bm_rows_per_kv + row0) * Lc + (size_t)tb * 64 + (lane & ~3);
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
// grid = (token splits, D/64 halves, KV heads); WAVES wavefronts per workgroup, each walking
// `nbpw` token blocks of its half and keeping fp32 sums per channel; the workgroup then adds
// its wavefronts' sums through LDS and writes one partial row per accumulator:
//   nsplit == 1 : C[(kv*rows+row0+n)*D + d]                       (fp16, final)
//   nsplit  > 1 : part[((kv*rows+row0+n)*nsplit + split)*D + d]   (fp32, merged by value_merge_kernel)
// LDS per wavefront: value double buffer + zero slot + double-buffered probability rows
// (4*NM rows x kSubTiles tokens per sub-chunk).
template <int NW, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void value_spmv_kernel(
    const uint64_t* __restrict__ bmp, const char* __restrict__ nz, const uint32_t* __restrict__ idx,
    const uint32_t* __restrict__ nz_off, const _Float16* __restrict__ P, _Float16* __restrict__ C,
    float* __restrict__ part, int Lc, int D, int nblk, int nbpw, int nsplit, int p_rows_per_kv, int row0)
{
    constexpr int NM = (NW + 3) / 4;
    constexpr int kWRow = kSubTiles * 2;          // bytes of one probability row per sub-chunk
    constexpr int kWBuf = NM * 4 * kWRow;         // one weight buffer
    constexpr int kNeed = kNzLds + 2 * kWBuf;
    constexpr int kWaveLds = kNeed > NW * 256 ? kNeed : NW * 256;  // the per-wave sums are parked here at the end
    __shared__ __attribute__((aligned(16))) char lds[WAVES][kWaveLds];
    const int lane = lane_id();
    const int wave = wave_id();
    const int split = (int)blockIdx.x;
    const int half = (int)blockIdx.y;
    const int kv = (int)blockIdx.z;
    const size_t T = (size_t)Lc * D / 64;
    const uint64_t* bmk = bmp + (size_t)kv * T;
    const uint32_t* ixk = idx + (size_t)kv * (T + 1);
    const char* nzk = nz + (size_t)nz_off[kv] * 16u;
    const _Float16* wk = P + ((size_t)kv * p_rows_per_kv + row0) * Lc;
    char* my = lds[wave];
    char* wl = my + kNzLds;

    f4_t acc[NM];
#pragma unroll
    for (int m = 0; m < NM; m++) acc[m] = f4_t{0.f, 0.f, 0.f, 0.f};

    const int first = (split * WAVES + wave) * nbpw;
    int last = first + nbpw;
    if (last > nblk) last = nblk;
    constexpr int subs_per_blk = 64 / kSubTiles;
    const uint32_t wrow = lds_addr(wl) + (uint32_t)(lane & 3) * kWRow;
    walk_subs<NM>(
        (last - first) * subs_per_blk,
        [=](int n) {
            return (size_t)(first + n / subs_per_blk) * D + (size_t)half * 64 + (size_t)(n % subs_per_blk) * kSubTiles;
        },
        [=](int n) {
            // the sub-chunk's probabilities, [row][kSubTiles] fp16: one instruction moves 256 bytes = kRowsPer rows
            constexpr int kDwPerRow = kSubTiles / 2, kRowsPer = 64 / kDwPerRow;
            const size_t tok0 = (size_t)(first + n / subs_per_blk) * 64 + (size_t)(n % subs_per_blk) * kSubTiles;
#pragma unroll
            for (int i = 0; i < (NM * 4 + kRowsPer - 1) / kRowsPer; i++) {
                // no lane predicate (a branch here would split the block while the coming scalar batch is live): the
                // lanes of rows >= NW fetch row NW - 1 again, into buffer rows whose products are never stored
                int row = kRowsPer * i + lane / kDwPerRow;
                row = row < NW ? row : NW - 1;
                dma4(wk + (size_t)row * Lc + tok0 + 2 * (lane % kDwPerRow), wl + (n & 1) * kWBuf + i * 256);
            }
        },
        [=](int n) { return wrow + (uint32_t)(n & 1) * kWBuf; }, 4u * kWRow, bmk, ixk, nzk, my, lane, acc);
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
        const size_t row = (size_t)kv * p_rows_per_kv + row0 + n;
        if (nsplit == 1)
            C[row * D + (size_t)half * 64 + ch] = (_Float16)s;
        else
            part[(row * nsplit + split) * D + (size_t)half * 64 + ch] = s;
    }
}

// ------------------------------------------------------------------------------- softmax
__device__ __forceinline__ float block_reduce(float v, bool is_max, float* sh)
{
    for (int o = 32; o > 0; o >>= 1) {
        float t = __shfl_xor(v, o, 64);
        v = is_max ? fmaxf(v, t) : v + t;
    }
    const int wave = (int)(threadIdx.x >> 6);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh[wave] = v;
    __syncthreads();
    float r = sh[0];
    for (int i = 1; i < 4; i++) r = is_max ? fmaxf(r, sh[i]) : r + sh[i];
    return r;
}

// One workgroup per row.  Rows of up to 256 * 8 * kSoftmaxPieces elements stay in registers between the three
// passes (maximum, sum, normalise), so the scores are read from memory once; longer rows fall back to re-reading.
constexpr int kSoftmaxPieces = 4;  // 16-byte pieces per thread: rows of up to 8192 elements
__global__ __launch_bounds__(256) void scale_softmax_kernel(const _Float16* __restrict__ s, _Float16* p, int L,
                                                            int64_t s_stride, int64_t p_stride, float div)
{
    __shared__ float sh[4];
    const _Float16* sr = s + (size_t)blockIdx.x * s_stride;
    _Float16* pr = p + (size_t)blockIdx.x * p_stride;
    const int tid = (int)threadIdx.x;
    const bool vec = (L % 8 == 0) && L <= 256 * 8 * kSoftmaxPieces && ((uintptr_t)sr % 16 == 0) && ((uintptr_t)pr % 16 == 0);
    if (vec) {
        typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
        float w[kSoftmaxPieces][8];
        float mx = -INFINITY;
        // every piece is requested before the first one is used: the loads are unconditional (a piece past the end
        // reads the row's first one instead and is ignored)
        h8_t v[kSoftmaxPieces];
#pragma unroll
        for (int k = 0; k < kSoftmaxPieces; k++) {
            const int i = (k * 256 + tid) * 8;
            v[k] = *reinterpret_cast<const h8_t*>(sr + (i < L ? i : 0));
        }
#pragma unroll
        for (int k = 0; k < kSoftmaxPieces; k++) {
            if ((k * 256 + tid) * 8 < L) {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    w[k][e] = (float)(_Float16)((float)v[k][e] / div);
                    mx = fmaxf(mx, w[k][e]);
                }
            }
        }
        mx = block_reduce(mx, true, sh);
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < kSoftmaxPieces; k++) {
            if ((k * 256 + tid) * 8 < L) {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    w[k][e] = expf(w[k][e] - mx);
                    sum += w[k][e];
                }
            }
        }
        sum = block_reduce(sum, false, sh);
#pragma unroll
        for (int k = 0; k < kSoftmaxPieces; k++) {
            const int i = (k * 256 + tid) * 8;
            if (i < L) {
                h8_t o;
#pragma unroll
                for (int e = 0; e < 8; e++) o[e] = (_Float16)(w[k][e] / sum);
                *reinterpret_cast<h8_t*>(pr + i) = o;
            }
        }
        return;
    }
    float mx = -INFINITY;
    for (int i = tid; i < L; i += 256) {
        const float w = (float)(_Float16)((float)sr[i] / div);
        mx = fmaxf(mx, w);
    }
    mx = block_reduce(mx, true, sh);
    float sum = 0.f;
    for (int i = tid; i < L; i += 256) {
        const float w = (float)(_Float16)((float)sr[i] / div);
        sum += expf(w - mx);
    }
    sum = block_reduce(sum, false, sh);
    for (int i = tid; i < L; i += 256) {
        const float w = (float)(_Float16)((float)sr[i] / div);
        pr[i] = (_Float16)(expf(w - mx) / sum);
    }
}

// ------------------------------------------------------------------------------- host
static int check_spmv_args(const void* bmp, const void* nz, const void* idx, const void* nz_off, const void* Bm,
                           const void* C, int tokens, int head_dim, int Bq, int groups, int n_rows)
{
    if (!bmp || !nz || !idx || !nz_off || !Bm || !C) return MSTF_EINVAL;
    if (tokens <= 0 || head_dim <= 0 || Bq <= 0 || groups <= 0 || n_rows <= 0) return MSTF_EINVAL;
    if (Bq % groups != 0) return MSTF_EINVAL;
    if (tokens % 64 != 0 || head_dim % 64 != 0 || head_dim > 128) return MSTF_EUNSUPPORTED;
    if (!aligned_to(bmp, 8) || !aligned_to(nz, 16) || !aligned_to(idx, 4) || !aligned_to(nz_off, 4) ||
        !aligned_to(Bm, 4) || !aligned_to(C, 2))
        return MSTF_EALIGN;
    return MSTF_OK;
}

template <int NW>
static void launch_key(hipStream_t st, const uint64_t* bmp, const char* nz, const uint32_t* idx,
                       const uint32_t* nz_off, const _Float16* Bm, _Float16* C, int Lc, int D, int Bkv, int rows_per_kv,
                       int row0)
{
    const int nblk = Lc / 64;
    const int ntasks = Bkv * nblk;
    hipLaunchKernelGGL(key_spmv_kernel<NW>, dim3((ntasks + 3) / 4), dim3(256), 0, st, bmp, nz, idx, nz_off, Bm, C, Lc,
                       D, nblk, ntasks, rows_per_kv, row0);
}

template <int NW, int WAVES>
static void launch_value(hipStream_t st, const ValuePlan& pl, const uint64_t* bmp, const char* nz,
                         const uint32_t* idx, const uint32_t* nz_off, const _Float16* P, _Float16* C, float* part,
                         int Lc, int D, int Bkv, int rows_per_kv, int row0)
{
    hipLaunchKernelGGL((value_spmv_kernel<NW, WAVES>), dim3(pl.nsplit, D / 64, Bkv), dim3(WAVES * 64), 0, st, bmp, nz,
                       idx, nz_off, P, C, part, Lc, D, Lc / 64, pl.nbpw, pl.nsplit, rows_per_kv, row0);
}

}  // namespace mstf

using namespace mstf;

extern "C" int mstf_key_spmv_f16(void* stream, const uint64_t* bmp, const mstf_half* nz, const uint32_t* idx,
                                 const uint32_t* nz_off, const mstf_half* Bm, mstf_half* C, int M, int K, int Bq,
                                 int groups, int n_rows)
{
    int rc = check_spmv_args(bmp, nz, idx, nz_off, Bm, C, M, K, Bq, groups, n_rows);
    if (rc != MSTF_OK) return rc;
    hipStream_t st = as_stream(stream);
    const int Bkv = Bq / groups;
    const int rows_per_kv = groups * n_rows;  // rows of Bm / C that share one KV head are contiguous
    const char* nzb = reinterpret_cast<const char*>(nz);
    const _Float16* b = reinterpret_cast<const _Float16*>(Bm);
    _Float16* c = reinterpret_cast<_Float16*>(C);
    for (int row0 = 0; row0 < rows_per_kv;) {
        const int nw = pick_nw(rows_per_kv - row0);
        switch (nw) {
            case 32: launch_key<32>(st, bmp, nzb, idx, nz_off, b, c, M, K, Bkv, rows_per_kv, row0); break;
            case 16: launch_key<16>(st, bmp, nzb, idx, nz_off, b, c, M, K, Bkv, rows_per_kv, row0); break;
            case 8: launch_key<8>(st, bmp, nzb, idx, nz_off, b, c, M, K, Bkv, rows_per_kv, row0); break;
            case 4: launch_key<4>(st, bmp, nzb, idx, nz_off, b, c, M, K, Bkv, rows_per_kv, row0); break;
            case 2: launch_key<2>(st, bmp, nzb, idx, nz_off, b, c, M, K, Bkv, rows_per_kv, row0); break;
            default: launch_key<1>(st, bmp, nzb, idx, nz_off, b, c, M, K, Bkv, rows_per_kv, row0); break;
        }
        rc = check_launch();
        if (rc != MSTF_OK) return rc;
        row0 += nw;
    }
    return MSTF_OK;
}

extern "C" size_t mstf_value_spmv_workspace_bytes(int M, int K, int Bq, int groups, int n_rows)
{
    if (M <= 0 || K <= 0 || Bq <= 0 || groups <= 0 || n_rows <= 0 || K % 64 != 0 || M % 64 != 0 || Bq % groups != 0)
        return 0;
    return value_workspace_bytes(M, K, Bq, groups, n_rows);
}

extern "C" int mstf_value_spmv_f16(void* stream, const uint64_t* bmp, const mstf_half* nz, const uint32_t* idx,
                                   const uint32_t* nz_off, const mstf_half* P, mstf_half* C, int M, int K, int Bq,
                                   int groups, int n_rows, void* workspace, size_t workspace_bytes)
{
    // M = head_dim, K = compressed tokens (the operator's GEMM naming)
    int rc = check_spmv_args(bmp, nz, idx, nz_off, P, C, K, M, Bq, groups, n_rows);
    if (rc != MSTF_OK) return rc;
    const size_t need = mstf_value_spmv_workspace_bytes(M, K, Bq, groups, n_rows);
    if (need > 0 && (!workspace || workspace_bytes < need)) return MSTF_EWORKSPACE;
    if (workspace && !aligned_to(workspace, 16)) return MSTF_EALIGN;
    hipStream_t st = as_stream(stream);
    const int Bkv = Bq / groups;
    const int rows_per_kv = groups * n_rows;
    const char* nzb = reinterpret_cast<const char*>(nz);
    const _Float16* p = reinterpret_cast<const _Float16*>(P);
    _Float16* c = reinterpret_cast<_Float16*>(C);
    float* part = reinterpret_cast<float*>(workspace);
    for (int row0 = 0; row0 < rows_per_kv;) {
        const int nw = pick_nw(rows_per_kv - row0);
        const ValuePlan pl = plan_value(K, M, Bkv, nw);
        switch (nw) {
            case 32: launch_value<32, 4>(st, pl, bmp, nzb, idx, nz_off, p, c, part, K, M, Bkv, rows_per_kv, row0); break;
            case 16: launch_value<16, 4>(st, pl, bmp, nzb, idx, nz_off, p, c, part, K, M, Bkv, rows_per_kv, row0); break;
            case 8: launch_value<8, 8>(st, pl, bmp, nzb, idx, nz_off, p, c, part, K, M, Bkv, rows_per_kv, row0); break;
            case 4: launch_value<4, 8>(st, pl, bmp, nzb, idx, nz_off, p, c, part, K, M, Bkv, rows_per_kv, row0); break;
            case 2: launch_value<2, 8>(st, pl, bmp, nzb, idx, nz_off, p, c, part, K, M, Bkv, rows_per_kv, row0); break;
            default: launch_value<1, 8>(st, pl, bmp, nzb, idx, nz_off, p, c, part, K, M, Bkv, rows_per_kv, row0); break;
        }
        rc = check_launch();
        if (rc != MSTF_OK) return rc;
        if (pl.nsplit > 1) {
            launch_value_merge(st, part, c, pl.nsplit, M, rows_per_kv, row0, nw, Bkv);
            rc = check_launch();
            if (rc != MSTF_OK) return rc;
        }
        row0 += nw;
    }
    return MSTF_OK;
}

extern "C" int mstf_scale_softmax_f16(void* stream, const mstf_half* s, mstf_half* p, int64_t rows, int L,
                                      int64_t s_stride, int64_t p_stride, int head_dim)
{
    if (!s || !p || rows <= 0 || L <= 0 || head_dim <= 0 || s_stride < L || p_stride < L) return MSTF_EINVAL;
    if (rows > 0x7FFFFFFF) return MSTF_EUNSUPPORTED;
    hipLaunchKernelGGL(scale_softmax_kernel, dim3((unsigned)rows), dim3(256), 0, as_stream(stream),
                       reinterpret_cast<const _Float16*>(s), reinterpret_cast<_Float16*>(p), L, s_stride, p_stride,
                       sqrtf((float)head_dim));
    return check_launch();
}
