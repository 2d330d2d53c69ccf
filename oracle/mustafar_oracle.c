/*
 * CPU oracle for Mustafar's sparse-KV decode-attention path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is a plain-C restatement of the
 * reference algorithm, used only as the checker in tests/, in the smoke test
 * and as the reported CPU baseline of bench.py.  The product (the HIP library)
 * never links, imports or calls anything in here.
 *
 * All fp16 buffers are raw IEEE binary16 bit patterns (uint16_t); conversions
 * are done in software so the file builds with any C99 compiler.
 *
 * Reference files restated (paths relative to the reference checkout):
 *   models/llama_mustafar_kernel.py:194-274      per-token magnitude pruning
 *   kernel/compression.py:8-435                  bitmap format producer (fp16)
 *   kernel/csrc/SpMM_Kernel.cuh:49-211,240-796   bitmap format consumer (index math)
 *   kernel/kernel_wrapper/mustafar_wrapper.cu    operator shapes (C[Bq,8,M])
 *   models/llama_mustafar_Kt_Mag_Vt_Mag.py:836-1026  dense masked attention
 *   kernel_quant/compression_quant.py:7-529      quantised producer
 *   kernel_quant/csrc/SpMM_Kernel_Quant.cuh:35-262   quantised consumer
 *
 * Parity status of each function is listed in oracle/README.md.  Every function is pinned by independent checks;
 * both producers (fp16 and 2-bit) also by arrays that the reference's own Triton programs wrote under Triton's
 * interpreter (tests/golden/ref_fp16.npz, ref_quant.npz).  Parity unpinned: the 4- and 8-bit widths of the quantised
 * producer, which the reference does not have (closed form and error bound only).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef uint16_t h16;

/* ------------------------------------------------------------------ fp16 */

static inline float h2f(h16 h)
{
    uint32_t s = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    uint32_t u;
    if (e == 0) {
        if (m == 0) {
            u = s;
        } else { /* subnormal: normalise */
            int sh = 0;
            while (!(m & 0x400u)) { m <<= 1; sh++; }
            m &= 0x3FFu;
            u = s | ((uint32_t)(113 - sh) << 23) | (m << 13);
        }
    } else if (e == 31) {
        u = s | 0x7F800000u | (m << 13);
    } else {
        u = s | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even, the rounding of torch .to(float16) and of
 * __float2half_rn (kernel/csrc/SpMM_Kernel.cuh:519). */
static inline h16 f2h(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    uint32_t s = (u >> 16) & 0x8000u;
    uint32_t a = u & 0x7FFFFFFFu;
    if (a >= 0x7F800000u) { /* inf / nan */
        return (h16)(s | 0x7C00u | ((a > 0x7F800000u) ? 0x200u : 0u));
    }
    if (a >= 0x477FF000u) { /* rounds to >= 65520 -> inf */
        return (h16)(s | 0x7C00u);
    }
    if (a < 0x33000001u) { /* < 2^-25 (or == 2^-25 tie to even 0) */
        return (h16)s;
    }
    int32_t e = (int32_t)(a >> 23) - 127;
    uint32_t m = (a & 0x7FFFFFu) | 0x800000u;
    int shift;
    uint32_t base;
    if (e < -14) { /* subnormal result */
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        m &= 0x7FFFFFu;
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (h16)(s | (base + q)); /* mantissa carry bumps the exponent correctly */
}

void orc_h2f(const h16* in, float* out, long n)
{
    for (long i = 0; i < n; i++) out[i] = h2f(in[i]);
}
void orc_f2h(const float* in, h16* out, long n)
{
    for (long i = 0; i < n; i++) out[i] = f2h(in[i]);
}

/* ------------------------------------------------- A1: per-token pruning */

static int cmp_u16(const void* a, const void* b)
{
    return (int)*(const uint16_t*)a - (int)*(const uint16_t*)b;
}

/* models/llama_mustafar_kernel.py:215-228.
 *   thr  = kthvalue(abs(row), kth)      (kth-th SMALLEST, 1-based)
 *   mask = abs(row) >= thr              (all ties kept)
 *   out  = row * mask                   (pruned entries become +0 / -0 by sign)
 * fp16 magnitudes of finite values order like their low 15 bits, so the
 * selection is done on integers.  NaN inputs are outside the contract. */
void orc_prune_rows(const h16* x, h16* y, long rows, int D, int kth)
{
    uint16_t* mag = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)D);
    for (long r = 0; r < rows; r++) {
        const h16* xr = x + r * D;
        h16* yr = y + r * D;
        for (int j = 0; j < D; j++) mag[j] = xr[j] & 0x7FFFu;
        qsort(mag, (size_t)D, sizeof(uint16_t), cmp_u16);
        uint16_t thr = mag[kth - 1];
        for (int j = 0; j < D; j++)
            yr[j] = ((xr[j] & 0x7FFFu) >= thr) ? xr[j] : (h16)(xr[j] & 0x8000u);
    }
    free(mag);
}

/* ------------------------------------------- F1/F2 + C1/C2: fp16 producer */

static inline int nonzero_h(h16 v) { return (v & 0x7FFFu) != 0; } /* vals != 0.0 */

/* element of tile t, position i, for an input x[M,N] (one batch entry).
 * key   (kernel/compression.py:32-36): t = tokblk*N + ch,  i = token in block
 * value (kernel/compression.py:87-97): t = tokblk*(N/64*64) + half*64 + tok, i = channel in half */
static inline long key_elem(int M, int N, long t, int i)
{
    (void)M;
    long ch = t % N, tokblk = t / N;
    return (tokblk * 64 + i) * (long)N + ch;
}
static inline long value_elem(int M, int N, long t, int i)
{
    (void)M;
    long tpb = (long)(N / 64) * 64;
    long blk = t / tpb, rem = t % tpb;
    long half = rem / 64, r = rem % 64;
    return (blk * 64 + r) * (long)N + half * 64 + i;
}

/* kernel/compression.py:249-342 (key, is_value=0) and :344-435 (value).
 * x:[B,M,N] fp16 (already pruned; zeros are the holes).
 * bmp:[B,T]  idx:[B,T+1] (uint32 units, exclusive prefix of padded counts)
 * nz: flat fp16, batch b starts at half offset 8*nz_off[b]; capacity nz_cap halfs
 *     (pass nz=NULL to size it); padding halfs are +0.0 (the torch.zeros at :312)
 * nz_off:[B] in 16-byte units (models/llama_mustafar_kernel.py:450-452)
 * returns total halfs. */
uint64_t orc_compress(const h16* x, int B, int M, int N, int is_value, uint64_t* bmp, uint32_t* idx, h16* nz,
                      uint64_t nz_cap, uint32_t* nz_off)
{
    long T = (long)M * N / 64;
    uint64_t base = 0; /* halfs */
    for (int b = 0; b < B; b++) {
        const h16* xb = x + (long)b * M * N;
        uint32_t acc = 0;
        idx[(long)b * (T + 1)] = 0;
        nz_off[b] = (uint32_t)(base / 8);
        for (long t = 0; t < T; t++) {
            uint64_t bits = 0;
            int cnt = 0;
            for (int i = 0; i < 64; i++) {
                h16 v = xb[is_value ? value_elem(M, N, t, i) : key_elem(M, N, t, i)];
                if (nonzero_h(v)) {
                    bits |= 1ull << (63 - i); /* :44 via shifts 2^(63-i) */
                    if (nz && base + 2ull * acc + (uint64_t)cnt < nz_cap) nz[base + 2ull * acc + cnt] = v;
                    cnt++;
                }
            }
            uint32_t padded = (uint32_t)((cnt + 7) & ~7);
            if (nz)
                for (uint32_t p = (uint32_t)cnt; p < padded; p++)
                    if (base + 2ull * acc + p < nz_cap) nz[base + 2ull * acc + p] = 0;
            bmp[(long)b * T + t] = bits;
            acc += padded >> 1; /* :48 */
            idx[(long)b * (T + 1) + t + 1] = acc;
        }
        base += 2ull * acc;
    }
    return base;
}

/* ----------------------------------------- consumer-side decode (fp16) */

/* Rebuilds the dense [M,N] matrix of batch entry b the way the device kernels
 * address it: kernel/csrc/SpMM_Kernel.cuh:262-265 (batch bases),
 * :342-348 / :631-642 (tile index), :174-206 (MSB-first walk, j-th set bit
 * takes the j-th packed value), :100-107 (idx in uint32 units). */
void orc_decode(const uint64_t* bmp, const h16* nz, const uint32_t* idx, const uint32_t* nz_off, int b, int M, int N,
                int is_value, h16* dense)
{
    long T = (long)M * N / 64;
    const h16* nzb = nz + 8ull * nz_off[b];
    const uint32_t* ib = idx + (long)b * (T + 1);
    const uint64_t* bb = bmp + (long)b * T;
    memset(dense, 0, sizeof(h16) * (size_t)M * N);
    for (long t = 0; t < T; t++) {
        uint64_t bits = bb[t];
        const h16* v = nzb + 2ull * ib[t];
        int j = 0;
        while (bits) {
            int pos = __builtin_clzll(bits);
            bits &= ~(0x8000000000000000ull >> pos);
            long e = is_value ? value_elem(M, N, t, pos) : key_elem(M, N, t, pos);
            dense[e] = v[j++];
        }
    }
}

/* --------------------------------------------- K1 / V1: SpMV semantics */

/* mustafar_key_formulation (kernel/kernel_wrapper/mustafar_wrapper.cu:19-133):
 *   C[bq, n, m] = sum_d Ktilde[bq/groups][m, d] * Bm[bq, n, d],  fp32 accumulate, fp16 round.
 * Bm:[Bq,nrows,D]  C:[Bq,nrows,Lc].  Also returns the un-rounded fp32 sums in Cf if non-NULL. */
void orc_key_spmv(const uint64_t* bmp, const h16* nz, const uint32_t* idx, const uint32_t* nz_off, const h16* Bm,
                  h16* C, float* Cf, int Lc, int D, int Bq, int groups, int nrows)
{
    h16* dense = (h16*)malloc(sizeof(h16) * (size_t)Lc * D);
    float* df = (float*)malloc(sizeof(float) * (size_t)Lc * D);
    int cur = -1;
    for (int bq = 0; bq < Bq; bq++) {
        int kv = bq / groups;
        if (kv != cur) {
            orc_decode(bmp, nz, idx, nz_off, kv, Lc, D, 0, dense);
            for (long i = 0; i < (long)Lc * D; i++) df[i] = h2f(dense[i]);
            cur = kv;
        }
        for (int n = 0; n < nrows; n++) {
            const h16* q = Bm + ((long)bq * nrows + n) * D;
            for (int m = 0; m < Lc; m++) {
                float s = 0.f;
                for (int d = 0; d < D; d++) s += df[(long)m * D + d] * h2f(q[d]);
                long o = ((long)bq * nrows + n) * Lc + m;
                C[o] = f2h(s);
                if (Cf) Cf[o] = s;
            }
        }
    }
    free(dense);
    free(df);
}

/* mustafar_value_formulation (mustafar_wrapper.cu:139-263):
 *   C[bq, n, d] = sum_t Vtilde[bq/groups][t, d] * P[bq, n, t].   P:[Bq,nrows,Lc]  C:[Bq,nrows,D] */
void orc_value_spmv(const uint64_t* bmp, const h16* nz, const uint32_t* idx, const uint32_t* nz_off, const h16* P,
                    h16* C, float* Cf, int D, int Lc, int Bq, int groups, int nrows)
{
    h16* dense = (h16*)malloc(sizeof(h16) * (size_t)Lc * D);
    float* df = (float*)malloc(sizeof(float) * (size_t)Lc * D);
    float* acc = (float*)malloc(sizeof(float) * (size_t)D);
    int cur = -1;
    for (int bq = 0; bq < Bq; bq++) {
        int kv = bq / groups;
        if (kv != cur) {
            orc_decode(bmp, nz, idx, nz_off, kv, Lc, D, 1, dense);
            for (long i = 0; i < (long)Lc * D; i++) df[i] = h2f(dense[i]);
            cur = kv;
        }
        for (int n = 0; n < nrows; n++) {
            const h16* p = P + ((long)bq * nrows + n) * Lc;
            for (int d = 0; d < D; d++) acc[d] = 0.f;
            for (int t = 0; t < Lc; t++) {
                float w = h2f(p[t]);
                for (int d = 0; d < D; d++) acc[d] += df[(long)t * D + d] * w;
            }
            for (int d = 0; d < D; d++) {
                long o = ((long)bq * nrows + n) * D + d;
                C[o] = f2h(acc[d]);
                if (Cf) Cf[o] = acc[d];
            }
        }
    }
    free(dense);
    free(df);
    free(acc);
}

/* ------------------------------------------------ S1: scale + softmax */

/* models/llama_mustafar_kernel.py:405,425:
 *   w = s / sqrt(head_dim)   (fp16 tensor / python float -> fp32 math, fp16 round)
 *   p = softmax(w, dtype=float32).to(float16) */
void orc_scale_softmax(const h16* s, h16* p, long rows, int L, float inv_div /* = sqrt(head_dim) as divisor */)
{
    float* w = (float*)malloc(sizeof(float) * (size_t)L);
    for (long r = 0; r < rows; r++) {
        const h16* sr = s + r * L;
        float mx = -INFINITY;
        for (int i = 0; i < L; i++) {
            w[i] = h2f(f2h(h2f(sr[i]) / inv_div));
            if (w[i] > mx) mx = w[i];
        }
        double sum = 0.0;
        for (int i = 0; i < L; i++) {
            w[i] = expf(w[i] - mx);
            sum += w[i];
        }
        float fs = (float)sum;
        for (int i = 0; i < L; i++) p[r * L + i] = f2h(w[i] / fs);
    }
    free(w);
}

/* -------------------------- oracle path: dense masked decode attention */

/* models/llama_mustafar_Kt_Mag_Vt_Mag.py:873-874,963,974 for one new token:
 *   S = q . Kp^T (fp16 out)  ->  /sqrt(D) (fp16)  ->  softmax fp32 -> fp16  ->  O = P . Vp (fp16 out)
 * Kp,Vp: [Bkv, L, D] dense with zeros at pruned positions; q: [Bq, D].
 * scores_out:[Bq,L] (raw, unscaled, fp16)  probs_out:[Bq,L]  out:[Bq,D].
 * Parallel over query heads when built with OpenMP; used as the CPU baseline. */
void orc_dense_masked_attention(const h16* q, const h16* Kp, const h16* Vp, int Bq, int groups, int L, int D,
                                h16* scores_out, h16* probs_out, h16* out)
{
    float div = sqrtf((float)D);
#pragma omp parallel for schedule(static)
    for (int bq = 0; bq < Bq; bq++) {
        int kv = bq / groups;
        const h16* K = Kp + (long)kv * L * D;
        const h16* V = Vp + (long)kv * L * D;
        float* qf = (float*)malloc(sizeof(float) * (size_t)D);
        float* acc = (float*)malloc(sizeof(float) * (size_t)D);
        h16* sc = scores_out + (long)bq * L;
        h16* pr = probs_out + (long)bq * L;
        for (int d = 0; d < D; d++) qf[d] = h2f(q[(long)bq * D + d]);
        for (int t = 0; t < L; t++) {
            float s = 0.f;
            for (int d = 0; d < D; d++) s += h2f(K[(long)t * D + d]) * qf[d];
            sc[t] = f2h(s);
        }
        orc_scale_softmax(sc, pr, 1, L, div);
        for (int d = 0; d < D; d++) acc[d] = 0.f;
        for (int t = 0; t < L; t++) {
            float w = h2f(pr[t]);
            for (int d = 0; d < D; d++) acc[d] += h2f(V[(long)t * D + d]) * w;
        }
        for (int d = 0; d < D; d++) out[(long)bq * D + d] = f2h(acc[d]);
        free(qf);
        free(acc);
    }
}

/* --------------------------------------------------- Q1: quant producer */

/* kernel_quant/compression_quant.py:159-264 (key) / :425-529 (value), with the
 * bit width as a parameter (the reference hard-codes bit=2, capacity=16 at :209-210).
 *   counts[B,T]  raw non-zeros per tile            (:34,:62)
 *   units [B,T]  ceil(count / capacity)             (:221)
 *   tile_off[B,T] GLOBAL uint32 offset into packed  (:226-236)
 *   scale = (max-min)/(2^bit-1), 1 if 0 or empty; zero = floor(-min/scale+0.5)   (:49-57)
 *   code  = clamp(floor(v/scale+0.5)+zero, 0, 2^bit-1)   (:143-145) using the fp16-stored scale/zero (:134-135)
 *   code j of a tile -> bits bit*(j%cap) of word j/cap    (:148-152)
 * scale/zero are computed in fp32 from the fp16 min/max, zero from the unrounded fp32 scale, and each is rounded
 * once to fp16 on the store: tl.min / tl.max widen sub-32-bit floats to fp32 before reducing, so the whole chain of
 * :41-57 is fp32 arithmetic in Triton.  Pinned bit for bit (bit = 2) by arrays the reference's own programs wrote
 * under Triton's interpreter (tests/golden/ref_quant.npz).  bit = 4 / 8 are extensions of this build (the reference
 * producer hard-codes 2): same formulas with 2^bit - 1 steps, pinned by closed form and error bound only.
 * packed may be NULL to size it. returns total uint32 words.
 * group_size 32 (an option of this build, after the harness setting GROUP_SIZE = 32 of
 * benchmark/mem_spd_test_quant.py:33,104, which the reference's producer never reads): scales / zeros are [B,T,2],
 * pair g for the elements 32g .. 32g+31 of the tile, each pair from the minimum and maximum of its own kept elements
 * by the same formulas; codes stay packed in rank order over the whole tile. */
uint64_t orc_compress_quant_grouped(const h16* x, int B, int M, int N, int is_value, int bit, int group_size,
                                    uint64_t* bmp, uint32_t* counts, uint32_t* units, uint32_t* tile_off,
                                    uint32_t* packed, uint64_t packed_cap, h16* scales, h16* zeros)
{
    const int ngrp = 64 / group_size; /* 1 (the reference: one pair per 64-element tile) or 2 (group 32) */
    long T = (long)M * N / 64;
    int cap = 32 / bit;
    float maxq = (float)((1 << bit) - 1);
    uint64_t off = 0;
    for (int b = 0; b < B; b++) {
        const h16* xb = x + (long)b * M * N;
        for (long t = 0; t < T; t++) {
            uint64_t bits = 0;
            int cnt = 0;
            float mn[2] = {INFINITY, INFINITY}, mx[2] = {-INFINITY, -INFINITY};
            int gcnt[2] = {0, 0};
            h16 vals[64];
            int grp[64];
            for (int i = 0; i < 64; i++) {
                h16 v = xb[is_value ? value_elem(M, N, t, i) : key_elem(M, N, t, i)];
                if (nonzero_h(v)) {
                    const int g = i / group_size; /* the group is a matter of the element's position in the tile */
                    bits |= 1ull << (63 - i);
                    float f = h2f(v);
                    if (f < mn[g]) mn[g] = f;
                    if (f > mx[g]) mx[g] = f;
                    gcnt[g]++;
                    grp[cnt] = g;
                    vals[cnt++] = v;
                }
            }
            long ti = (long)b * T + t;
            h16 sh[2], zh[2];
            for (int g = 0; g < ngrp; g++) {
                float scale = 1.f, zero = 0.f;
                if (gcnt[g] > 0) {
                    scale = (mx[g] - mn[g]) / maxq;
                    if (scale == 0.f) scale = 1.f;
                    zero = floorf(-mn[g] / scale + 0.5f);
                }
                sh[g] = f2h(scale);
                zh[g] = f2h(zero);
                scales[ti * ngrp + g] = sh[g];
                zeros[ti * ngrp + g] = zh[g];
            }
            bmp[ti] = bits;
            counts[ti] = (uint32_t)cnt;
            uint32_t u = (uint32_t)((cnt + cap - 1) / cap);
            units[ti] = u;
            tile_off[ti] = (uint32_t)off;
            if (packed) {
                for (uint32_t w = 0; w < u; w++)
                    if (off + w < packed_cap) packed[off + w] = 0;
                for (int j = 0; j < cnt; j++) {
                    float sc = h2f(sh[grp[j]]), zp = h2f(zh[grp[j]]);
                    if (sc == 0.f) sc = 1.f; /* :137-138 */
                    float qf = floorf(h2f(vals[j]) / sc + 0.5f) + zp;
                    if (qf < 0.f) qf = 0.f;
                    if (qf > maxq) qf = maxq;
                    uint32_t qi = (uint32_t)qf;
                    if (off + (uint64_t)(j / cap) < packed_cap) packed[off + j / cap] |= qi << ((j % cap) * bit);
                }
            }
            off += u;
        }
    }
    return off;
}

uint64_t orc_compress_quant(const h16* x, int B, int M, int N, int is_value, int bit, uint64_t* bmp, uint32_t* counts,
                            uint32_t* units, uint32_t* tile_off, uint32_t* packed, uint64_t packed_cap, h16* scales,
                            h16* zeros)
{
    return orc_compress_quant_grouped(x, B, M, N, is_value, bit, 64, bmp, counts, units, tile_off, packed, packed_cap,
                                      scales, zeros);
}

/* Consumer-side dequantised dense rebuild of batch entry b:
 * kernel_quant/csrc/SpMM_Kernel_Quant.cuh:204-242: j-th set bit (MSB first) takes code j;
 * dequant_mode 0: fp32 (q - zero) * scale then round to fp16 (:238-240);
 * dequant_mode 1: fp16 arithmetic hsub then hmul (:190-191). */
void orc_decode_quant_grouped(const uint64_t* bmp, const uint32_t* packed, const uint32_t* tile_off, const h16* scales,
                              const h16* zeros, int b, int M, int N, int is_value, int bit, int dequant_mode,
                              int group_size, h16* dense)
{
    const int ngrp = 64 / group_size;
    long T = (long)M * N / 64;
    int cap = 32 / bit;
    uint32_t mask = (1u << bit) - 1u;
    memset(dense, 0, sizeof(h16) * (size_t)M * N);
    for (long t = 0; t < T; t++) {
        long ti = (long)b * T + t;
        uint64_t bits = bmp[ti];
        const uint32_t* w = packed + tile_off[ti];
        int j = 0;
        while (bits) {
            int pos = __builtin_clzll(bits);
            bits &= ~(0x8000000000000000ull >> pos);
            /* the element's position picks its (scale, zero) pair; codes stay in rank order over the whole tile */
            float sc = h2f(scales[ti * ngrp + pos / group_size]), zp = h2f(zeros[ti * ngrp + pos / group_size]);
            uint32_t qv = (w[j / cap] >> ((j % cap) * bit)) & mask;
            h16 v;
            if (dequant_mode == 1)
                v = f2h(h2f(f2h((float)qv - zp)) * sc);
            else
                v = f2h(((float)qv - zp) * sc);
            dense[is_value ? value_elem(M, N, t, pos) : key_elem(M, N, t, pos)] = v;
            j++;
        }
    }
}

void orc_decode_quant(const uint64_t* bmp, const uint32_t* packed, const uint32_t* tile_off, const h16* scales,
                      const h16* zeros, int b, int M, int N, int is_value, int bit, int dequant_mode, h16* dense)
{
    orc_decode_quant_grouped(bmp, packed, tile_off, scales, zeros, b, M, N, is_value, bit, dequant_mode, 64, dense);
}

/* Q2/Q3 semantics: the K1/V1 products on the dequantised matrix. */
void orc_spmv_quant(const uint64_t* bmp, const uint32_t* packed, const uint32_t* tile_off, const h16* scales,
                    const h16* zeros, const h16* Bm, h16* C, float* Cf, int is_value, int Lc, int D, int Bq, int groups,
                    int nrows, int bit, int dequant_mode)
{
    h16* dense = (h16*)malloc(sizeof(h16) * (size_t)Lc * D);
    float* df = (float*)malloc(sizeof(float) * (size_t)Lc * D);
    float* acc = (float*)malloc(sizeof(float) * (size_t)D);
    int cur = -1;
    for (int bq = 0; bq < Bq; bq++) {
        int kv = bq / groups;
        if (kv != cur) {
            orc_decode_quant(bmp, packed, tile_off, scales, zeros, kv, Lc, D, is_value, bit, dequant_mode, dense);
            for (long i = 0; i < (long)Lc * D; i++) df[i] = h2f(dense[i]);
            cur = kv;
        }
        for (int n = 0; n < nrows; n++) {
            if (!is_value) {
                const h16* q = Bm + ((long)bq * nrows + n) * D;
                for (int m = 0; m < Lc; m++) {
                    float s = 0.f;
                    for (int d = 0; d < D; d++) s += df[(long)m * D + d] * h2f(q[d]);
                    long o = ((long)bq * nrows + n) * Lc + m;
                    C[o] = f2h(s);
                    if (Cf) Cf[o] = s;
                }
            } else {
                const h16* p = Bm + ((long)bq * nrows + n) * Lc;
                for (int d = 0; d < D; d++) acc[d] = 0.f;
                for (int t = 0; t < Lc; t++) {
                    float w = h2f(p[t]);
                    for (int d = 0; d < D; d++) acc[d] += df[(long)t * D + d] * w;
                }
                for (int d = 0; d < D; d++) {
                    long o = ((long)bq * nrows + n) * D + d;
                    C[o] = f2h(acc[d]);
                    if (Cf) Cf[o] = acc[d];
                }
            }
        }
    }
    free(dense);
    free(df);
    free(acc);
}

int orc_num_threads(void)
{
#ifdef _OPENMP
    extern int omp_get_max_threads(void);
    return omp_get_max_threads();
#else
    return 1;
#endif
}
