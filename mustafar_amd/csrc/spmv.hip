// Batched key / value SpMV over the bitmap format, and the scale+softmax glue between them.
//
// Both products share one inner loop.  A "chunk" is 64 consecutive tiles of one KV head:
//   key   chunk = 64 channels x 64 tokens of one token block      (lane = token)
//   value chunk = 64 tokens  x 64 channels of one half of head_dim (lane = channel)
// In both cases tile t of the chunk contributes  D[t][lane] * w[n][t]  to accumulator n of the
// lane, where D[t][lane] is element `lane` of tile t (0 when its bitmap bit is clear) and w is
// the query row (key) or the probability row (value).  A wavefront owns a chunk: it streams the
// chunk's packed values (contiguous, 16-byte aligned) from HBM into its private LDS buffer with
// 16-byte loads, then rebuilds D[t][lane] with a popcount rank (v_mbcnt) per tile and feeds
// pairs of tiles to v_dot2_f32_f16 with the two weights in one scalar register.  Bitmaps, tile
// offsets and weights are wave-uniform and come through scalar loads.
#include "common.hpp"

namespace mstf {

constexpr int kChunkBytes = 64 * 64 * 2;       // worst case: 64 full tiles
constexpr int kWaveLds = kChunkBytes + 16;     // + a 16-byte zero slot read by lanes whose bit is clear

struct ChunkRegs {
    uint4 r[8];
};

// Per-lane 16-byte pieces of a chunk: piece i of lane l is bytes [(i*64+l)*16, +16).
__device__ __forceinline__ void chunk_fetch(ChunkRegs& cr, const char* src, uint32_t bytes, int lane)
{
#pragma unroll
    for (int i = 0; i < 8; i++) {
        if ((uint32_t)(i * 1024) < bytes) {
            uint32_t o = (uint32_t)(i * 64 + lane) * 16u;
            if (o < bytes) cr.r[i] = *reinterpret_cast<const uint4*>(src + o);
        }
    }
}
__device__ __forceinline__ void chunk_stage(const ChunkRegs& cr, char* dst, uint32_t bytes, int lane)
{
#pragma unroll
    for (int i = 0; i < 8; i++) {
        if ((uint32_t)(i * 1024) < bytes) {
            uint32_t o = (uint32_t)(i * 64 + lane) * 16u;
            if (o < bytes) *reinterpret_cast<uint4*>(dst + o) = cr.r[i];
        }
    }
}

// acc[n] += sum_t D[t][lane] * w[n][t] for the 64 tiles of one chunk.
//   bm, ix : the chunk's 64 bitmaps / 64 tile offsets (4-byte units), wave-uniform pointers
//   sbase  : LDS byte address of the staged chunk minus 4*ix[0]
//   zaddr  : LDS byte address of two zero bytes
//   w      : weights of accumulator 0 for tile 0 (fp16), wstride halfs between accumulators
template <int NW>
__device__ __forceinline__ void chunk_accumulate(const uint64_t* bm, const uint32_t* ix, uint32_t sbase,
                                                 uint32_t zaddr, const _Float16* w, size_t wstride, float (&acc)[NW])
{
#pragma unroll 1
    for (int tt = 0; tt < 64; tt += 8) {
        const u32x16_t mv = *reinterpret_cast<const u32x16_a4*>(bm + tt);
        const u32x8_t iv = *reinterpret_cast<const u32x8_a4*>(ix + tt);
        uint32_t v[4];
#pragma unroll
        for (int u = 0; u < 8; u += 2) {
            const uint64_t m0 = lanes_of(u64_of(mv[2 * u], mv[2 * u + 1]));
            const uint64_t m1 = lanes_of(u64_of(mv[2 * u + 2], mv[2 * u + 3]));
            const uint32_t o0 = iv[u] * 4u + sbase;
            const uint32_t o1 = iv[u + 1] * 4u + sbase;
            const uint32_t a0 = lane_bit(m0) ? (o0 + rank_below(m0) * 2u) : zaddr;
            const uint32_t a1 = lane_bit(m1) ? (o1 + rank_below(m1) * 2u) : zaddr;
            h2_t p;
            p.x = lds_load_h(a0);
            p.y = lds_load_h(a1);
            v[u / 2] = as_u32(p);
        }
#pragma unroll
        for (int n = 0; n < NW; n++) {
            const u32x4_t q = *reinterpret_cast<const u32x4_a4*>(w + (size_t)n * wstride + tt);
            const uint32_t q0 = q[0], q1 = q[1], q2 = q[2], q3 = q[3];
            acc[n] = __builtin_amdgcn_fdot2(as_h2(v[0]), as_h2(q0), acc[n], false);
            acc[n] = __builtin_amdgcn_fdot2(as_h2(v[1]), as_h2(q1), acc[n], false);
            acc[n] = __builtin_amdgcn_fdot2(as_h2(v[2]), as_h2(q2), acc[n], false);
            acc[n] = __builtin_amdgcn_fdot2(as_h2(v[3]), as_h2(q3), acc[n], false);
        }
    }
}

__device__ __forceinline__ uint32_t chunk_bytes(const uint32_t* ix)
{
    uint32_t b = (ix[64] - ix[0]) * 4u;
    return b > (uint32_t)kChunkBytes ? (uint32_t)kChunkBytes : b;  // a well-formed chunk never exceeds this
}

// ------------------------------------------------------------------------------- key
// One wavefront per (KV head, token block): loops over the D/64 channel chunks of the block.
// C[(kv*NW + n)*Lc + token] = sum_d K[token][d] * Bm[(kv*NW + n)*D + d].
template <int NW>
__global__ __launch_bounds__(256) void key_spmv_kernel(const uint64_t* __restrict__ bmp, const char* __restrict__ nz,
                                                       const uint32_t* __restrict__ idx,
                                                       const uint32_t* __restrict__ nz_off,
                                                       const _Float16* __restrict__ Bm, _Float16* __restrict__ C,
                                                       int Lc, int D, int nblk, int ntasks, int bm_rows_per_kv,
                                                       int row0)
{
    __shared__ __attribute__((aligned(16))) char lds[4][kWaveLds];
    const int lane = lane_id();
    const int wave = wave_id();
    const int task = (int)blockIdx.x * 4 + wave;
    if (task >= ntasks) return;
    const int kv = task / nblk;
    const int tb = task - kv * nblk;
    const size_t T = (size_t)Lc * D / 64;
    const uint64_t* bmk = bmp + (size_t)kv * T + (size_t)tb * D;
    const uint32_t* ixk = idx + (size_t)kv * (T + 1) + (size_t)tb * D;
    const char* nzk = nz + (size_t)nz_off[kv] * 16u;
    const _Float16* wk = Bm + ((size_t)kv * bm_rows_per_kv + row0) * D;
    char* my = lds[wave];
    const uint32_t lbase = lds_addr(my);
    const uint32_t zaddr = lbase + kChunkBytes;
    if (lane < 4) reinterpret_cast<uint32_t*>(my + kChunkBytes)[lane] = 0u;

    float acc[NW];
#pragma unroll
    for (int n = 0; n < NW; n++) acc[n] = 0.f;

    const int nchunks = D / 64;
    ChunkRegs cr;
    uint32_t bytes = chunk_bytes(ixk);
    chunk_fetch(cr, nzk + (size_t)ixk[0] * 4u, bytes, lane);
    for (int c = 0; c < nchunks; c++) {
        const uint32_t* ixc = ixk + c * 64;
        const uint32_t start = ixc[0];
        chunk_stage(cr, my, bytes, lane);
        if (c + 1 < nchunks) {
            bytes = chunk_bytes(ixc + 64);
            chunk_fetch(cr, nzk + (size_t)ixc[64] * 4u, bytes, lane);
        }
        __builtin_amdgcn_wave_barrier();
        chunk_accumulate<NW>(bmk + c * 64, ixc, lbase - start * 4u, zaddr, wk + c * 64, (size_t)D, acc);
        __builtin_amdgcn_wave_barrier();
    }
    _Float16* out = C + ((size_t)kv * bm_rows_per_kv + row0) * Lc + (size_t)tb * 64 + lane;
#pragma unroll
    for (int n = 0; n < NW; n++) out[(size_t)n * Lc] = (_Float16)acc[n];
}

// ------------------------------------------------------------------------------- value
// grid = (token splits, D/64 halves, KV heads); WAVES wavefronts per workgroup, each walking
// `nbpw` token blocks of its half and keeping fp32 sums per channel; the workgroup then adds
// its wavefronts' sums through LDS and writes one partial row per accumulator:
//   nsplit == 1 : C[(kv*NW+n)*D + d]                       (fp16, final)
//   nsplit  > 1 : part[((kv*NW+n)*nsplit + split)*D + d]   (fp32, merged by value_merge_kernel)
template <int NW, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void value_spmv_kernel(
    const uint64_t* __restrict__ bmp, const char* __restrict__ nz, const uint32_t* __restrict__ idx,
    const uint32_t* __restrict__ nz_off, const _Float16* __restrict__ P, _Float16* __restrict__ C,
    float* __restrict__ part, int Lc, int D, int nblk, int nbpw, int nsplit, int p_rows_per_kv, int row0)
{
    __shared__ __attribute__((aligned(16))) char lds[WAVES][kWaveLds];
    const int lane = lane_id();
    const int wave = wave_id();
    const int split = (int)blockIdx.x;
    const int half = (int)blockIdx.y;
    const int kv = (int)blockIdx.z;
    const size_t T = (size_t)Lc * D / 64;
    const uint64_t* bmk = bmp + (size_t)kv * T + (size_t)half * 64;
    const uint32_t* ixk = idx + (size_t)kv * (T + 1) + (size_t)half * 64;
    const char* nzk = nz + (size_t)nz_off[kv] * 16u;
    const _Float16* wk = P + ((size_t)kv * p_rows_per_kv + row0) * Lc;
    char* my = lds[wave];
    const uint32_t lbase = lds_addr(my);
    const uint32_t zaddr = lbase + kChunkBytes;
    if (lane < 4) reinterpret_cast<uint32_t*>(my + kChunkBytes)[lane] = 0u;

    float acc[NW];
#pragma unroll
    for (int n = 0; n < NW; n++) acc[n] = 0.f;

    const int first = (split * WAVES + wave) * nbpw;
    int last = first + nbpw;
    if (last > nblk) last = nblk;
    if (first < last) {
        ChunkRegs cr;
        uint32_t bytes = chunk_bytes(ixk + (size_t)first * D);
        chunk_fetch(cr, nzk + (size_t)ixk[(size_t)first * D] * 4u, bytes, lane);
        for (int tb = first; tb < last; tb++) {
            const uint32_t* ixc = ixk + (size_t)tb * D;
            const uint32_t start = ixc[0];
            chunk_stage(cr, my, bytes, lane);
            if (tb + 1 < last) {
                bytes = chunk_bytes(ixc + D);
                chunk_fetch(cr, nzk + (size_t)ixc[D] * 4u, bytes, lane);
            }
            __builtin_amdgcn_wave_barrier();
            chunk_accumulate<NW>(bmk + (size_t)tb * D, ixc, lbase - start * 4u, zaddr, wk + (size_t)tb * 64,
                                 (size_t)Lc, acc);
            __builtin_amdgcn_wave_barrier();
        }
    }
    // workgroup reduction: every wavefront parks its sums in its own chunk buffer (NW*256 <= 8192 bytes)
    __syncthreads();
    float* mine = reinterpret_cast<float*>(my);
#pragma unroll
    for (int n = 0; n < NW; n++) mine[n * 64 + lane] = acc[n];
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

// Adds the token-split partials of rows [row0, row0+nw) of every KV head and rounds to fp16.
__global__ __launch_bounds__(256) void value_merge_kernel(const float* __restrict__ part, _Float16* __restrict__ C,
                                                          int nsplit, int D, int rows_per_kv, int row0, int nw,
                                                          size_t total)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const size_t d = i % D;
    const size_t r = i / D;
    const size_t row = (r / nw) * rows_per_kv + row0 + (r % nw);
    float s = 0.f;
    for (int k = 0; k < nsplit; k++) s += part[(row * nsplit + k) * D + d];
    C[row * D + d] = (_Float16)s;
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

__global__ __launch_bounds__(256) void scale_softmax_kernel(const _Float16* __restrict__ s, _Float16* p, int L,
                                                            int64_t s_stride, int64_t p_stride, float div)
{
    __shared__ float sh[4];
    const _Float16* sr = s + (size_t)blockIdx.x * s_stride;
    _Float16* pr = p + (size_t)blockIdx.x * p_stride;
    float mx = -INFINITY;
    for (int i = (int)threadIdx.x; i < L; i += 256) {
        const float w = (float)(_Float16)((float)sr[i] / div);
        mx = fmaxf(mx, w);
    }
    mx = block_reduce(mx, true, sh);
    float sum = 0.f;
    for (int i = (int)threadIdx.x; i < L; i += 256) {
        const float w = (float)(_Float16)((float)sr[i] / div);
        sum += expf(w - mx);
    }
    sum = block_reduce(sum, false, sh);
    for (int i = (int)threadIdx.x; i < L; i += 256) {
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
    if (tokens % 64 != 0 || head_dim % 64 != 0) return MSTF_EUNSUPPORTED;
    if (!aligned_to(bmp, 8) || !aligned_to(nz, 16) || !aligned_to(idx, 4) || !aligned_to(nz_off, 4) ||
        !aligned_to(Bm, 4) || !aligned_to(C, 2))
        return MSTF_EALIGN;
    return MSTF_OK;
}

// Largest accumulator count with an instantiated kernel that fits in `left`.
static int pick_nw(int left)
{
    const int opts[] = {32, 16, 8, 4, 2, 1};
    for (int o : opts)
        if (o <= left) return o;
    return 1;
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

struct ValuePlan {
    int waves;   // wavefronts per workgroup
    int nbpw;    // token blocks per wavefront
    int nsplit;  // workgroups along the token axis
};

static ValuePlan plan_value(int Lc, int D, int Bkv, int nw)
{
    ValuePlan p;
    const int nblk = Lc / 64;
    const long chunks = (long)nblk * (D / 64) * Bkv;
    p.waves = nw > 8 ? 4 : 8;
    // aim at ~4096 resident wavefronts on 256 CUs, at least two token blocks each to pipeline
    long nb = (chunks + 4095) / 4096;
    if (nb < 2) nb = 2;
    if (nb > nblk) nb = nblk;
    p.nbpw = (int)nb;
    p.nsplit = (nblk + p.waves * p.nbpw - 1) / (p.waves * p.nbpw);
    return p;
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
    const int rows_per_kv = groups * n_rows;
    size_t worst = 0;
    for (int row0 = 0; row0 < rows_per_kv;) {
        const int nw = pick_nw(rows_per_kv - row0);
        const ValuePlan pl = plan_value(K, M, Bq / groups, nw);
        const size_t need = pl.nsplit > 1 ? (size_t)Bq * n_rows * pl.nsplit * M * sizeof(float) : 0;
        if (need > worst) worst = need;
        row0 += nw;
    }
    return round_up(worst, 256);
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
            const size_t total = (size_t)Bkv * nw * M;
            hipLaunchKernelGGL(value_merge_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, part, c,
                               pl.nsplit, M, rows_per_kv, row0, nw, total);
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
