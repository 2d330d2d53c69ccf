/*
 * libmustafar_hip.so -- C ABI of the MI355X (gfx950) sparse-KV decode-attention kernels.
 *
 * Conventions for every entry point
 *   - all data pointers are DEVICE pointers; `stream` is a hipStream_t passed as void*
 *     (NULL = the default stream); launches are asynchronous, nothing here synchronises;
 *   - fp16 buffers are IEEE binary16 (`mstf_half` = raw 16-bit pattern);
 *   - inputs are borrowed and never modified; outputs are caller-allocated;
 *   - nothing allocates: scratch memory comes in through `workspace` (size from the
 *     matching *_workspace_bytes query, 256-byte aligned);
 *   - the return value is MSTF_OK or a negative MSTF_E* code (never an exception);
 *     mstf_strerror() names it; a failed launch also records the HIP error, readable
 *     with mstf_last_hip_error().
 *
 * Compressed fp16 format ("bitmap format"), per KV head b (D = head_dim, tiles of 64 elements):
 *   key   tile t = tokblk*D + ch            : 64 consecutive tokens of channel ch
 *   value tile t = tokblk*D + half*64 + tok : 64 consecutive channels of one token
 *   bmp[b][t]  bit (63-i) set  <=>  element i of the tile is non-zero
 *   idx[b][t]  start of the tile's packed values, in 4-byte units, relative to the head's base;
 *              idx[b][T] = total; every tile is padded with +0.0 to a multiple of 8 values
 *   nz_off[b]  base of head b inside the flat nz buffer, in 16-byte units
 * This is the layout defined by the reference producer kernel/compression.py:8-435 and
 * consumed by kernel/csrc/SpMM_Kernel.cuh:49-211.
 */
#ifndef MUSTAFAR_HIP_H
#define MUSTAFAR_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t mstf_half;

enum {
    MSTF_OK = 0,
    MSTF_EINVAL = -1,       /* null pointer, non-positive size, inconsistent arguments */
    MSTF_EALIGN = -2,       /* a pointer is not aligned as required */
    MSTF_EUNSUPPORTED = -3, /* shape outside what the kernels cover (e.g. head_dim != 128) */
    MSTF_EWORKSPACE = -4,   /* workspace missing or too small */
    MSTF_ELAUNCH = -5,      /* HIP reported an error at launch; see mstf_last_hip_error() */
    MSTF_ETOOLARGE = -6     /* the problem needs more scratch than the library's fixed buffer holds */
};

const char* mstf_strerror(int code);
int mstf_last_hip_error(void);
/* library version: major*10000 + minor*100 + patch */
int mstf_version(void);
/* Measurement aid (no counterpart in the reference): reads `bytes` of device memory with 16-byte loads per lane from
 * `workgroups` workgroups of 256 threads and does nothing else; sink: at least `workgroups` uint32 (written only in the
 * practically impossible case that the xor of all data read by a workgroup hits a fixed constant).  Timing it gives the
 * plain-read time of a buffer of that size on the box at hand. */
int mstf_probe_read(void* stream, const void* src, size_t bytes, uint32_t* sink, int workgroups);
/* Test aid (no counterpart in the reference): the number of polls a workgroup of the one-pass producers
 * (mstf_compress_*, mstf_append_*, mstf_compress_*_quant*) spends on a wait before it gives up and marks the call.
 * polls < 0 restores the default (2^20).  Process-wide, read at every launch; nothing in the environment changes it.
 * A test sets it to 0 to drive the give-up path from the host while every kernel still runs to its end. */
void mstf_test_set_spin_limit(int64_t polls);

/* ------------------------------------------------------------------ pruning (A1)
 * Replaces dh_prune_key / dh_prune_value (models/llama_mustafar_kernel.py:194-274):
 * per row of D values, thr = kth-th smallest |x|, keep |x| >= thr, pruned entries become
 * +0/-0 by sign (the result of x * mask).  x, y: [rows, D]; y may alias x.  D must be 128. */
int mstf_prune_rows_f16(void* stream, const mstf_half* x, mstf_half* y, int64_t rows, int D, int kth);

/* ------------------------------------------------------------------ compression (C1, C2)
 * Replace convert_key_batched / convert_value_batched (kernel/compression.py:249-342, 344-435)
 * fused with the pruning above.
 *   x [B, M, N] fp16, M % 64 == 0, N == 128.
 *   kth > 0: prune each row first (as mstf_prune_rows_f16) without writing the dense result;
 *   kth == 0: x is already pruned, zeros are the holes (exactly what the reference converts).
 * Phase 1 ("count") writes bmp [B,T], idx [B,T+1], nz_off [B] and *total_halfs (device uint64:
 * number of fp16 values the flat nz buffer must hold).  Phase 2 ("scatter") fills nz.
 * mstf_compress_*_f16 produces everything with one read of x (status words in the workspace order
 * the workgroups; they are cleared by the call itself); with nz == NULL it runs phase 1 only.  Tiles
 * whose values would not fit in nz_capacity_halfs are not written (compare *total_halfs afterwards).
 * A workgroup waits for the totals of the workgroups launched before it; should such a wait of ANY workgroup
 * ever run out of its (bounded) polls, that workgroup writes no values and *total_halfs reads as all ones
 * (the call clears *total_halfs first and raises it with atomic maxima, so the marker survives whichever
 * workgroup finishes last). */
size_t mstf_compress_workspace_bytes(int B, int M, int N);
int mstf_compress_key_f16(void* stream, const mstf_half* x, int B, int M, int N, int kth, uint64_t* bmp,
                          uint32_t* idx, uint32_t* nz_off, uint64_t* total_halfs, mstf_half* nz,
                          uint64_t nz_capacity_halfs, void* workspace, size_t workspace_bytes);
int mstf_compress_value_f16(void* stream, const mstf_half* x, int B, int M, int N, int kth, uint64_t* bmp,
                            uint32_t* idx, uint32_t* nz_off, uint64_t* total_halfs, mstf_half* nz,
                            uint64_t nz_capacity_halfs, void* workspace, size_t workspace_bytes);
/* Phase 2 alone, on the outputs of a finished phase 1 (same x, B, M, N). */
int mstf_scatter_key_f16(void* stream, const mstf_half* x, int B, int M, int N, const uint64_t* bmp,
                         const uint32_t* idx, const uint32_t* nz_off, mstf_half* nz, uint64_t nz_capacity_halfs);
int mstf_scatter_value_f16(void* stream, const mstf_half* x, int B, int M, int N, const uint64_t* bmp,
                           const uint32_t* idx, const uint32_t* nz_off, mstf_half* nz, uint64_t nz_capacity_halfs);
/* Append to a pooled cache: the same pruning and compression of a chunk x[B, M, N] (the reference appends a
 * 256-token chunk per head by re-concatenating every head's values, models/llama_mustafar_kernel.py:461-511),
 * with the destination of the packed values chosen by the caller: head b's values are written at
 * nz + 16 * dst_off[b] and must end at or before nz + 16 * dst_limit[b] (both in 16-byte units).  With one slab
 * per head and dst_off[b] = slab start + idx_so_far[b][T] / 4 the cache grows in place; the format's nz_off[b]
 * is the slab start.  bmp[B, M*N/64] and idx[B, M*N/64 + 1] receive the chunk's bitmaps and its offsets counted
 * from the chunk's first value (add idx_so_far[b][T]).  *overflow is a sticky flag word zeroed by the caller:
 * bit 0 (MSTF_APPEND_OVERFLOW) is set when a unit would pass its head's limit - that unit's values are not
 * written; the chunk's bitmaps and offsets are, and appending the same chunk again with larger slabs repairs it -
 * and bit 1 (MSTF_APPEND_GAVE_UP) when a workgroup's bounded wait for the workgroups in front of it ran out, in
 * which case it wrote no values (the marker *total_halfs carries in the compress contract).  A caller must look
 * at the word before it trusts the appended chunk.  Workspace as for mstf_compress_*_f16. */
#define MSTF_APPEND_OVERFLOW 1u
#define MSTF_APPEND_GAVE_UP 2u
int mstf_append_key_f16(void* stream, const mstf_half* x, int B, int M, int N, int kth, uint64_t* bmp, uint32_t* idx,
                        const uint32_t* dst_off, const uint32_t* dst_limit, mstf_half* nz, uint32_t* overflow,
                        void* workspace, size_t workspace_bytes);
int mstf_append_value_f16(void* stream, const mstf_half* x, int B, int M, int N, int kth, uint64_t* bmp, uint32_t* idx,
                          const uint32_t* dst_off, const uint32_t* dst_limit, mstf_half* nz, uint32_t* overflow,
                          void* workspace, size_t workspace_bytes);

/* Keys and values of the same tokens in one launch instead of two (the reference converts K and V of a context or of a
 * chunk back to back, models/llama_mustafar_kernel.py:540-557 and :461-511): exactly what mstf_compress_key_f16 followed
 * by mstf_compress_value_f16 (both with a value buffer), or mstf_append_key_f16 followed by mstf_append_value_f16,
 * write - the outputs are identical bit for bit - behind one clearing launch, with the workgroups of the two sides in
 * one grid.  A launch with twice the workgroups runs less in lockstep (the loads of the values overlap the arithmetic
 * of the keys): 86 us against 51 + 50 us at 128 heads x 4096 tokens, 159 against 88 + 85 us at 256 heads (51 against
 * 27 + 25 us at 64 heads, where each side is one generation of workgroups).  Both value
 * buffers are required (no sizing-only form); the append form shares one sticky flag word between the sides.
 * Workspace: mstf_compress_kv_workspace_bytes(B, M, N), 256-byte aligned. */
size_t mstf_compress_kv_workspace_bytes(int B, int M, int N);
int mstf_compress_kv_f16(void* stream, const mstf_half* k, const mstf_half* v, int B, int M, int N, int kth_k, int kth_v,
                         uint64_t* k_bmp, uint32_t* k_idx, uint32_t* k_nz_off, uint64_t* k_total_halfs, mstf_half* k_nz,
                         uint64_t k_capacity_halfs, uint64_t* v_bmp, uint32_t* v_idx, uint32_t* v_nz_off,
                         uint64_t* v_total_halfs, mstf_half* v_nz, uint64_t v_capacity_halfs, void* workspace,
                         size_t workspace_bytes);
int mstf_append_kv_f16(void* stream, const mstf_half* k, const mstf_half* v, int B, int M, int N, int kth_k, int kth_v,
                       uint64_t* k_bmp, uint32_t* k_idx, const uint32_t* k_dst_off, const uint32_t* k_dst_limit,
                       mstf_half* k_nz, uint64_t* v_bmp, uint32_t* v_idx, const uint32_t* v_dst_off,
                       const uint32_t* v_dst_limit, mstf_half* v_nz, uint32_t* overflow, void* workspace,
                       size_t workspace_bytes);

/* ------------------------------------------------------------------ compression from the projection output
 * The prefill of the reference turns the projection outputs [batch, tokens, heads * 128] into [batch, heads,
 * tokens, 128] views, rotates the keys (apply_rotary_pos_emb of transformers 4.43.1, called at
 * models/llama_mustafar_kernel.py:373-374), prunes the first M tokens in place and copies them into a contiguous
 * [batch * heads, M, 128] matrix for the compressor (:540-560).  These entry points read the rows where the
 * projection left them and fuse the rotation:
 *   source element (batch entry bt, token t, KV head h, channel c) = x[bt*stride_batch + t*stride_token +
 *   h*stride_head + c], strides in elements and multiples of 8, `rows` tokens per head; heads are numbered
 *   b = bt*heads + h in every output, as the reference's reshape numbers them;
 *   cos, sin (both or neither; keys only): fp16 [batch entry][token][128] with strides rope_stride_batch (0 when all
 *   batch entries share the positions) and rope_stride_token.  Every one of the `rows` tokens becomes
 *   (x * cos) + (rotate_half(x) * sin), each product and the sum rounded to fp16 as the half-precision tensor
 *   expression rounds them, and is written to rot (strides like x; rot may be x itself with the same strides -
 *   the one case in which an input is modified - but must not overlap it otherwise);
 *   the first M tokens (M % 64 == 0, M <= rows; M may be 0 with cos / sin: rotation only) are then pruned and
 *   compressed exactly as mstf_compress_*_f16 / mstf_append_*_f16 would compress the contiguous copy, with
 *   B = batch * heads.  nz must be given (there is no sizing-only mode).  Workspace:
 *   mstf_compress_workspace_bytes(batch * heads, M, 128). */
typedef struct mstf_proj_source {
    const mstf_half* x;
    int64_t stride_batch, stride_token, stride_head;
    int batch, heads, rows;
    const mstf_half* cos;
    const mstf_half* sin;
    int64_t rope_stride_batch, rope_stride_token;
    mstf_half* rot;
    int64_t rot_stride_batch, rot_stride_token, rot_stride_head;
} mstf_proj_source;
int mstf_compress_proj_f16(void* stream, const mstf_proj_source* src, int is_value, int M, int N, int kth,
                           uint64_t* bmp, uint32_t* idx, uint32_t* nz_off, uint64_t* total_halfs, mstf_half* nz,
                           uint64_t nz_capacity_halfs, void* workspace, size_t workspace_bytes);
int mstf_append_proj_f16(void* stream, const mstf_proj_source* src, int is_value, int M, int N, int kth,
                         uint64_t* bmp, uint32_t* idx, const uint32_t* dst_off, const uint32_t* dst_limit,
                         mstf_half* nz, uint32_t* overflow, void* workspace, size_t workspace_bytes);

/* ------------------------------------------------------------------ key SpMV (K1)
 * Replaces mustafar_key_formulation (kernel/kernel_wrapper/mustafar_wrapper.cu:19-133 ->
 * Key_SplitK_API, kernel/csrc/SpMM_API.cu:179 -> Key_Kernel, kernel/csrc/SpMM_Kernel.cuh:240-520):
 *   C[bq, n, m] = sum_d Ktilde[bq / groups][m, d] * Bm[bq, n, d]      (fp32 accumulate, fp16 result)
 * Bm [Bq, n_rows, K] fp16, C [Bq, n_rows, M] fp16.  M = compressed tokens (M % 64 == 0),
 * K = head_dim (128), Bq = query heads x batch, groups = query heads per KV head.
 * n_rows = 8 reproduces the reference operator (its N is hard-wired to 8, mustafar_wrapper.cu:125);
 * n_rows = 1 is the decode fast path without the 7 padding rows.
 * Every compressed byte is read once per KV head, not once per query head. */
int mstf_key_spmv_f16(void* stream, const uint64_t* bmp, const mstf_half* nz, const uint32_t* idx,
                      const uint32_t* nz_off, const mstf_half* Bm, mstf_half* C, int M, int K, int Bq, int groups,
                      int n_rows);

/* ------------------------------------------------------------------ value SpMV (V1)
 * Replaces mustafar_value_formulation (mustafar_wrapper.cu:139-263 -> Value_SplitK_API,
 * SpMM_API.cu:331 -> Value_Kernel, SpMM_Kernel.cuh:535-796 + SplitK_Reduction, Reduction_Kernel.cuh:26-48):
 *   C[bq, n, d] = sum_t Vtilde[bq / groups][t, d] * P[bq, n, t]
 * P [Bq, n_rows, K] fp16, C [Bq, n_rows, M] fp16.  M = head_dim (128), K = compressed tokens.
 * Tokens are split over workgroups; fp32 partial sums go through `workspace`. */
size_t mstf_value_spmv_workspace_bytes(int M, int K, int Bq, int groups, int n_rows);
int mstf_value_spmv_f16(void* stream, const uint64_t* bmp, const mstf_half* nz, const uint32_t* idx,
                        const uint32_t* nz_off, const mstf_half* P, mstf_half* C, int M, int K, int Bq, int groups,
                        int n_rows, void* workspace, size_t workspace_bytes);

/* ------------------------------------------------------------------ scale + softmax (S1)
 * The glue between the two products (models/llama_mustafar_kernel.py:405,425):
 *   w = fp16(s / sqrt(head_dim));  p = fp16(softmax_fp32(w))   over each row of length L.
 * s, p: [rows, L] fp16 with row strides (in elements) s_stride / p_stride; p may alias s. */
int mstf_scale_softmax_f16(void* stream, const mstf_half* s, mstf_half* p, int64_t rows, int L, int64_t s_stride,
                           int64_t p_stride, int head_dim);

/* ------------------------------------------------------------------ fused decode attention
 * One launch for the whole compressed part of a decode step, i.e. the sequence
 * mustafar_key_formulation -> / sqrt(head_dim) -> softmax(fp32) -> mustafar_value_formulation of the
 * caller (models/llama_mustafar_kernel.py:394-396,405,425,434-436) for one query row per head:
 *   out[bq, :] = softmax_t( fp16(q[bq].Ktilde[t]) / sqrt(d) ) . Vtilde[t, :]     over the `tokens` cached tokens
 * q, out: [Bq, head_dim] fp16 (head_dim 128, groups <= 8).  Scores and probabilities stay on chip.
 * lse_out (nullable) [Bq, 2] fp32 receives (max, sum of exp(w - max)) per row, so a caller that keeps a
 * dense local window can combine that window's attention with this result under one softmax. */
size_t mstf_decode_attention_workspace_bytes(int tokens, int head_dim, int Bq, int groups);
int mstf_decode_attention_f16(void* stream, const uint64_t* k_bmp, const mstf_half* k_nz, const uint32_t* k_idx,
                              const uint32_t* k_nz_off, const uint64_t* v_bmp, const mstf_half* v_nz,
                              const uint32_t* v_idx, const uint32_t* v_nz_off, const mstf_half* q, mstf_half* out,
                              float* lse_out, int tokens, int head_dim, int Bq, int groups, void* workspace,
                              size_t workspace_bytes);
/* mstf_decode_attention_f16 for callers that cannot allocate or hand over a workspace (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The split partials live
 * in a device array of MSTF_STATIC_SCRATCH_BYTES that is part of the library image: each GPU the library runs on holds
 * one copy until the process ends, and every call on a GPU uses that GPU's copy.  Same arguments, results and checks
 * as mstf_decode_attention_f16 without the workspace pair; a problem whose partials
 * (mstf_decode_attention_workspace_bytes) exceed the buffer is refused with MSTF_ETOOLARGE before anything is
 * launched (4096 tokens fit up to Bq = 1008 query rows; at the headline shape - 256 rows - up to 15872 tokens).  Calls
 * no hipMalloc / hipFree or other allocating routine; the first call on a device looks the array's address up
 * (hipGetSymbolAddress, with that device current - make that first call outside a graph capture).  Nothing has to be
 * cleared between calls: the kernels write every partial they later read.  Calls that overlap on one GPU (two streams,
 * two threads) share the buffer and race: serialise them, or use the workspace form. */
#define MSTF_STATIC_SCRATCH_BYTES ((size_t)4 << 20)
int mstf_decode_attention_static_f16(void* stream, const uint64_t* k_bmp, const mstf_half* k_nz, const uint32_t* k_idx,
                                     const uint32_t* k_nz_off, const uint64_t* v_bmp, const mstf_half* v_nz,
                                     const uint32_t* v_idx, const uint32_t* v_nz_off, const mstf_half* q,
                                     mstf_half* out, float* lse_out, int tokens, int head_dim, int Bq, int groups);
/* The two phases of mstf_decode_attention_f16 as separate calls, for a caller that shards the cached
 * tokens (each shard runs `partial` on its tokens, the (max, sum, output) triples are then combined).
 * partial: per token split s and query row: workspace = float part_o[Bq][ns][head_dim] followed by
 *   float part_ml[Bq][ns][2] = (max, sum of exp(w - max)), part_o un-normalised;
 *   ns = mstf_decode_attention_splits(tokens, head_dim, Bq, groups) <= ceil(tokens / 512): a split covers 512
 *   tokens while every 64-token block can have a resident wavefront of its own, a multiple of that beyond.
 * merge: log-sum-exp combine of the ns splits into out (fp16) and, if given, lse_out. */
int mstf_decode_attention_splits(int tokens, int head_dim, int Bq, int groups);
int mstf_decode_attention_partial_f16(void* stream, const uint64_t* k_bmp, const mstf_half* k_nz, const uint32_t* k_idx,
                                      const uint32_t* k_nz_off, const uint64_t* v_bmp, const mstf_half* v_nz,
                                      const uint32_t* v_idx, const uint32_t* v_nz_off, const mstf_half* q, int tokens,
                                      int head_dim, int Bq, int groups, void* workspace, size_t workspace_bytes);
int mstf_decode_attention_merge_f16(void* stream, const void* workspace, size_t workspace_bytes, mstf_half* out,
                                    float* lse_out, int tokens, int head_dim, int Bq, int groups);
/* The whole attention of a decode step, compressed tokens and dense local window under one softmax
 * (models/llama_mustafar_kernel.py:391-441: key SpMV | q.K_win^T, / sqrt(d), softmax, value SpMV + P_win.V_win):
 * the fused kernel over the `tokens` compressed tokens, a dense kernel over the window, one merge.
 * k_win, v_win: [Bq / groups][win_stride][head_dim] fp16, the first win_len tokens of every KV head valid (the new
 * token included).  tokens may be 0 (nothing compressed yet; the compressed-side pointers are then ignored).
 * win_len_dev (nullable): the valid length is read from device memory instead - min(*win_len_dev, win_len), at
 * least 1 - and win_len only sizes the launch and the workspace; a call recorded into a HIP graph then replays
 * with a window that grows between replays.
 * Workspace: mstf_decode_attention_window_workspace_bytes(tokens, largest win_len, head_dim, Bq, groups). */
size_t mstf_decode_attention_window_workspace_bytes(int tokens, int max_window, int head_dim, int Bq, int groups);
int mstf_decode_attention_window_f16(void* stream, const uint64_t* k_bmp, const mstf_half* k_nz, const uint32_t* k_idx,
                                     const uint32_t* k_nz_off, const uint64_t* v_bmp, const mstf_half* v_nz,
                                     const uint32_t* v_idx, const uint32_t* v_nz_off, const mstf_half* q,
                                     const mstf_half* k_win, const mstf_half* v_win, int win_len,
                                     const int32_t* win_len_dev, int win_stride, mstf_half* out, float* lse_out,
                                     int tokens, int head_dim, int Bq, int groups, void* workspace,
                                     size_t workspace_bytes);

/* mstf_decode_attention_window_f16 over a cache that is pre-allocated for more tokens than it holds and grows in
 * place (mstf_append_*_f16 into per-head slabs): the bitmap rows of two heads lie tile_capacity tiles apart
 * (tile_capacity >= max_tokens * head_dim / 64), the offset rows tile_capacity + 1, and the number of cached tokens
 * is read from device memory - min(*tokens_dev, max_tokens), a multiple of 64, may be 0 - while max_tokens sizes the
 * launch and the workspace (mstf_decode_attention_window_workspace_bytes(max_tokens, ...)).  A call recorded into a
 * HIP graph therefore stays valid while chunks are appended between replays: no array moves and no argument
 * changes (the reference re-concatenates every per-tile array per chunk, models/llama_mustafar_kernel.py:461-511). */
int mstf_decode_attention_window_pool_f16(void* stream, const uint64_t* k_bmp, const mstf_half* k_nz, const uint32_t* k_idx,
                                          const uint32_t* k_nz_off, const uint64_t* v_bmp, const mstf_half* v_nz,
                                          const uint32_t* v_idx, const uint32_t* v_nz_off, const mstf_half* q,
                                          const mstf_half* k_win, const mstf_half* v_win, int win_len,
                                          const int32_t* win_len_dev, int win_stride, mstf_half* out, float* lse_out,
                                          int max_tokens, const int32_t* tokens_dev, int64_t tile_capacity, int head_dim,
                                          int Bq, int groups, void* workspace, size_t workspace_bytes);

/* The whole cache side of a decode step of one layer in two launches (models/llama_mustafar_kernel.py:363-374: views
 * of the projection outputs and apply_rotary_pos_emb; :391, :430: torch.cat of the new key / value row onto the local
 * windows; :391-441: key SpMV | q.K_win^T, / sqrt(d), softmax, value SpMV + P_win.V_win): what
 * mstf_window_append_f16 followed by mstf_decode_attention_window_pool_f16 compute, bit for bit, with the rotation of
 * the query heads, the rotation and append of the new key / value row and the attention over the dense window inside
 * the launch of the compressed tokens (wavefronts take a 64-token block of the window behind their compressed blocks;
 * the one whose block holds the new row rotates and stores it), then the merge.  A launch costs about 5 us on this GPU whatever it does,
 * so a step of 32 layers is 0.3 ms shorter than with the four launches of the two calls.
 * Arguments as for those two calls: q_in / k_in / v_in [bs][n_q * 128] / [bs][n_kv * 128] fp16 with their batch
 * strides (not rotated), cos / sin [bs][128] (rope_stride; both NULL: no rotation), the window buffers
 * [bs * n_kv][win_stride][128]; win_len bounds the count of valid window rows AFTER the step (it sizes the launch and
 * the workspace) and, without win_len_dev, is that count; with win_len_dev the count is read on the device.  The new
 * row goes to row count - 1; a count outside 1 .. win_stride appends nothing and sets *overflow (nullable, sticky).
 * The compressed side is a pooled cache (tokens_dev, tile_capacity, max_tokens as for
 * mstf_decode_attention_window_pool_f16).  out [bs * n_q][128].  Workspace:
 * mstf_decode_attention_window_workspace_bytes(max_tokens, win_len, 128, bs * n_q, n_q / n_kv). */
int mstf_decode_step_pool_f16(void* stream, const uint64_t* k_bmp, const mstf_half* k_nz, const uint32_t* k_idx,
                              const uint32_t* k_nz_off, const uint64_t* v_bmp, const mstf_half* v_nz, const uint32_t* v_idx,
                              const uint32_t* v_nz_off, const mstf_half* q_in, int64_t q_stride, const mstf_half* k_in,
                              int64_t k_stride, const mstf_half* v_in, int64_t v_stride, int bs, int n_q, int n_kv,
                              const mstf_half* cos, const mstf_half* sin, int64_t rope_stride, mstf_half* k_win,
                              mstf_half* v_win, int win_stride, int win_len, const int32_t* win_len_dev,
                              uint32_t* overflow, mstf_half* out, float* lse_out, int max_tokens,
                              const int32_t* tokens_dev, int64_t tile_capacity, int head_dim, void* workspace,
                              size_t workspace_bytes);

/* The caller's per-token work in front of the attention call, in one launch (models/llama_mustafar_kernel.py:363-374:
 * the views of the projection outputs and apply_rotary_pos_emb; :391, :430: torch.cat of the new key / value row onto
 * the local windows):
 *   q_out[b * n_q + h, :]                    = rope(q_in[b, h, :])        (what the attention entry points take as q)
 *   k_win[b * n_kv + h, row, :]              = rope(k_in[b, h, :])
 *   v_win[b * n_kv + h, row, :]              = v_in[b, h, :]
 * with rope(x) = x * cos + rotate_half(x) * sin in fp16, every product and the sum rounded on its own (the arithmetic
 * of the half-precision expression), rotate_half(x) = [-x[64:], x[:64]].
 * q_in [bs][n_q * 128], k_in / v_in [bs][n_kv * 128] fp16: the projection outputs of the new token, *_stride halfs
 * between two batch entries (three slices of one fused projection are fine); cos, sin [bs][128] fp16 for the token's
 * position, rope_stride halfs between batch entries (0: one position for all), both NULL: no rotation.  q_in and
 * q_out both NULL: keys and values only.
 * k_win, v_win [bs * n_kv][win_stride][128] as for mstf_decode_attention_window_f16.  win_len counts the valid rows of
 * the window AFTER this call, the new token included - the same number the attention call takes - and row =
 * win_len - 1; with win_len_dev the count is read from device memory instead (a call recorded into a HIP graph
 * replays with the counter the caller advances between or inside the replays).  A count outside 1 .. win_stride
 * writes no key / value row and sets *overflow (nullable, sticky) to 1. */
int mstf_window_append_f16(void* stream, const mstf_half* q_in, int64_t q_stride, const mstf_half* k_in,
                           int64_t k_stride, const mstf_half* v_in, int64_t v_stride, int bs, int n_q, int n_kv,
                           int head_dim, const mstf_half* cos, const mstf_half* sin, int64_t rope_stride,
                           mstf_half* q_out, mstf_half* k_win, mstf_half* v_win, int win_stride, int win_len,
                           const int32_t* win_len_dev, uint32_t* overflow);

/* ------------------------------------------------------------------ quantised format (Q1-Q4)
 * Producer: convert_{key,value}_batched_quant (kernel_quant/compression_quant.py:159-264, 425-529),
 * with the bit width a parameter (the reference hard-codes 2).  Same tiles and bitmaps as above;
 *   counts[B,T] raw non-zeros; units[B,T] = ceil(count / capacity), capacity = 32 / bit;
 *   tile_off[B,T] GLOBAL 4-byte-word offset of the tile inside `packed`;
 *   scales/zeros[B,T] fp16: scale = (max - min) / (2^bit - 1) (1 when 0 or empty),
 *   zero = floor(-min / scale + 0.5); code = clamp(floor(v / scale + 0.5) + zero, 0, 2^bit - 1);
 *   code j of a tile sits at bits bit*(j % capacity) of word j / capacity.
 * kth as in mstf_compress_*_f16.  packed == NULL runs the sizing phase only; with packed the input is read once and
 * the workgroups are ordered as in mstf_compress_*_f16 (*total_words reads as all ones should a bounded wait of any
 * workgroup run out). */
size_t mstf_compress_quant_workspace_bytes(int B, int M, int N);
int mstf_compress_key_quant(void* stream, const mstf_half* x, int B, int M, int N, int kth, int bit, uint64_t* bmp,
                            uint32_t* tile_off, uint32_t* counts, uint32_t* units, mstf_half* scales,
                            mstf_half* zeros, uint64_t* total_words, uint32_t* packed, uint64_t packed_capacity_words,
                            void* workspace, size_t workspace_bytes);
int mstf_compress_value_quant(void* stream, const mstf_half* x, int B, int M, int N, int kth, int bit, uint64_t* bmp,
                              uint32_t* tile_off, uint32_t* counts, uint32_t* units, mstf_half* scales,
                              mstf_half* zeros, uint64_t* total_words, uint32_t* packed,
                              uint64_t packed_capacity_words, void* workspace, size_t workspace_bytes);

/* Consumers: mustafar_key_formulation_quant[_meta] (kernel_quant/kernel_wrapper/mustafar_wrapper_quant.cu:14-214
 * -> Key_Kernel_Quant, kernel_quant/csrc/SpMM_Kernel_Quant.cuh:273-503) and
 * mustafar_value_formulation_quant[_decode_n1] (mustafar_wrapper_quant.cu:216-457 -> Value_Kernel_Quant,
 * SpMM_Kernel_Quant.cuh:510-735).  Same products as the fp16 entry points on the dequantised
 * matrix (q - zero) * scale; dequant_mode 0 = fp32 arithmetic rounded once to fp16, 1 = fp16
 * arithmetic (SpMM_Kernel_Quant.cuh:190-191,238-240).  counts/units may be NULL (derived from the
 * bitmaps, as the non-_meta key entry point does).  bit in {2, 4, 8}; capacity must equal 32 / bit.
 * The words of the 128 tiles of one side of a 64-token block must be contiguous in `packed`, in tile order (what
 * the producer writes); blocks may lie anywhere, so a cache grown the reference's way - a chunk's words appended
 * behind the old ones, its offsets shifted (models/llama_mustafar_quant_kernel.py:322-345) - is read as it is.
 * scales and zeros 4-byte aligned, head_dim 64 or 128. */
int mstf_key_spmv_quant(void* stream, const uint64_t* bmp, const uint32_t* packed, const uint32_t* tile_off,
                        const uint32_t* counts, const uint32_t* units, const mstf_half* scales,
                        const mstf_half* zeros, const mstf_half* Bm, mstf_half* C, int M, int K, int Bq, int groups,
                        int n_rows, int bit, int capacity, int dequant_mode);
size_t mstf_value_spmv_quant_workspace_bytes(int M, int K, int Bq, int groups, int n_rows);
int mstf_value_spmv_quant(void* stream, const uint64_t* bmp, const uint32_t* packed, const uint32_t* tile_off,
                          const uint32_t* counts, const uint32_t* units, const mstf_half* scales,
                          const mstf_half* zeros, const mstf_half* P, mstf_half* C, int M, int K, int Bq, int groups,
                          int n_rows, int bit, int capacity, int dequant_mode, void* workspace,
                          size_t workspace_bytes);
/* The fused decode step of mstf_decode_attention_f16 over a quantised cache: key side and value side as produced by
 * mstf_compress_{key,value}_quant (counts / units are not needed).  Workspace as for mstf_decode_attention_f16. */
int mstf_decode_attention_quant(void* stream, const uint64_t* k_bmp, const uint32_t* k_packed, const uint32_t* k_tile_off,
                                const mstf_half* k_scales, const mstf_half* k_zeros, const uint64_t* v_bmp,
                                const uint32_t* v_packed, const uint32_t* v_tile_off, const mstf_half* v_scales,
                                const mstf_half* v_zeros, const mstf_half* q, mstf_half* out, float* lse_out, int tokens,
                                int head_dim, int Bq, int groups, int bit, int capacity, int dequant_mode,
                                void* workspace, size_t workspace_bytes);
/* mstf_decode_attention_window_f16 over a quantised cache: the whole attention of a decode step of the quantised
 * caller (models/llama_mustafar_quant_kernel.py:437-575: key formulation | q.K_win^T, / sqrt(d), softmax, value
 * formulation + P_win.V_win) as the quantised fused kernel, the dense-window kernel and one merge.  Window
 * arguments, win_len_dev and the workspace size as for mstf_decode_attention_window_f16. */
int mstf_decode_attention_window_quant(void* stream, const uint64_t* k_bmp, const uint32_t* k_packed,
                                       const uint32_t* k_tile_off, const mstf_half* k_scales, const mstf_half* k_zeros,
                                       const uint64_t* v_bmp, const uint32_t* v_packed, const uint32_t* v_tile_off,
                                       const mstf_half* v_scales, const mstf_half* v_zeros, const mstf_half* q,
                                       const mstf_half* k_win, const mstf_half* v_win, int win_len,
                                       const int32_t* win_len_dev, int win_stride, mstf_half* out, float* lse_out,
                                       int tokens, int head_dim, int Bq, int groups, int bit, int capacity,
                                       int dequant_mode, void* workspace, size_t workspace_bytes);

/* mstf_decode_attention_window_quant over a quantised cache whose per-tile arrays are pre-allocated for max_tokens
 * tokens and filled in place: bitmaps, word offsets, scales and zero-points of two heads lie tile_capacity entries
 * apart (tile_capacity >= max_tokens * head_dim / 64, even), tile_off holds offsets into `packed` wherever the words
 * of a 64-token block were put (the consumers only need the words of one block to be contiguous), and the number of
 * cached tokens is read from device memory - min(*tokens_dev, max_tokens), a multiple of 64, may be 0 - while
 * max_tokens sizes the launch and the workspace.  A call recorded into a HIP graph stays valid while chunks are
 * appended between replays (the reference concatenates every array per chunk,
 * models/llama_mustafar_quant_kernel.py:322-345). */
int mstf_decode_attention_window_quant_pool(void* stream, const uint64_t* k_bmp, const uint32_t* k_packed,
                                            const uint32_t* k_tile_off, const mstf_half* k_scales,
                                            const mstf_half* k_zeros, const uint64_t* v_bmp, const uint32_t* v_packed,
                                            const uint32_t* v_tile_off, const mstf_half* v_scales,
                                            const mstf_half* v_zeros, const mstf_half* q, const mstf_half* k_win,
                                            const mstf_half* v_win, int win_len, const int32_t* win_len_dev,
                                            int win_stride, mstf_half* out, float* lse_out, int max_tokens,
                                            const int32_t* tokens_dev, int64_t tile_capacity, int head_dim, int Bq,
                                            int groups, int bit, int capacity, int dequant_mode, void* workspace,
                                            size_t workspace_bytes);

/* mstf_decode_step_pool_f16 for the quantised pooled cache: the cache side of a decode step of one layer in two
 * launches (models/llama_mustafar_quant_kernel.py:445-567: rotation of the new query / key heads, torch.cat of the new
 * key / value row onto the local windows, key formulation | q.K_win^T, / sqrt(d), softmax, value formulation +
 * P_win.V_win) - what mstf_window_append_f16 followed by mstf_decode_attention_window_quant_pool compute, bit for bit.
 * Step arguments as for mstf_decode_step_pool_f16, cache arguments as for mstf_decode_attention_window_quant_pool
 * (one scale / zero pair per tile). */
int mstf_decode_step_quant_pool(void* stream, const uint64_t* k_bmp, const uint32_t* k_packed, const uint32_t* k_tile_off,
                                const mstf_half* k_scales, const mstf_half* k_zeros, const uint64_t* v_bmp,
                                const uint32_t* v_packed, const uint32_t* v_tile_off, const mstf_half* v_scales,
                                const mstf_half* v_zeros, const mstf_half* q_in, int64_t q_stride, const mstf_half* k_in,
                                int64_t k_stride, const mstf_half* v_in, int64_t v_stride, int bs, int n_q, int n_kv,
                                const mstf_half* cos, const mstf_half* sin, int64_t rope_stride, mstf_half* k_win,
                                mstf_half* v_win, int win_stride, int win_len, const int32_t* win_len_dev,
                                uint32_t* overflow, mstf_half* out, float* lse_out, int max_tokens,
                                const int32_t* tokens_dev, int64_t tile_capacity, int head_dim, int bit, int capacity,
                                int dequant_mode, void* workspace, size_t workspace_bytes);

/* ------------------------------------------------------------------ group-32 scale / zero option
 * No counterpart in the reference's kernels: its harness carries GROUP_SIZE = 32 (benchmark/mem_spd_test_quant.py:33,
 * 104) but the producer quantises per 64-element tile (kernel_quant/compression_quant.py:47-57, 209-210).  With
 * group_size 32 every tile has two (scale, zero) pairs, scales / zeros are fp16 [B][T][2] (4-byte aligned), pair g
 * serves the elements 32g .. 32g+31 of the tile and is computed from the minimum and maximum of that half's kept
 * elements by the formulas above; bitmaps, counts, units, tile_off and the rank-ordered packing of the codes are
 * unchanged (the first popcount(upper bitmap half) codes of a tile belong to pair 0).  group_size 64 is the layout of
 * the entry points above.  Otherwise the arguments are those of mstf_compress_{key,value}_quant (is_value picks the
 * tile orientation), mstf_key_spmv_quant, mstf_value_spmv_quant and mstf_decode_attention_quant, without the unused
 * counts / units of the consumers. */
int mstf_compress_quant_grouped(void* stream, const mstf_half* x, int is_value, int B, int M, int N, int kth, int bit,
                                int group_size, uint64_t* bmp, uint32_t* tile_off, uint32_t* counts, uint32_t* units,
                                mstf_half* scales, mstf_half* zeros, uint64_t* total_words, uint32_t* packed,
                                uint64_t packed_capacity_words, void* workspace, size_t workspace_bytes);
int mstf_key_spmv_quant_grouped(void* stream, const uint64_t* bmp, const uint32_t* packed, const uint32_t* tile_off,
                                const mstf_half* scales, const mstf_half* zeros, const mstf_half* Bm, mstf_half* C, int M,
                                int K, int Bq, int groups, int n_rows, int bit, int capacity, int dequant_mode,
                                int group_size);
int mstf_value_spmv_quant_grouped(void* stream, const uint64_t* bmp, const uint32_t* packed, const uint32_t* tile_off,
                                  const mstf_half* scales, const mstf_half* zeros, const mstf_half* P, mstf_half* C, int M,
                                  int K, int Bq, int groups, int n_rows, int bit, int capacity, int dequant_mode,
                                  int group_size, void* workspace, size_t workspace_bytes);
int mstf_decode_attention_quant_grouped(void* stream, const uint64_t* k_bmp, const uint32_t* k_packed,
                                        const uint32_t* k_tile_off, const mstf_half* k_scales, const mstf_half* k_zeros,
                                        const uint64_t* v_bmp, const uint32_t* v_packed, const uint32_t* v_tile_off,
                                        const mstf_half* v_scales, const mstf_half* v_zeros, const mstf_half* q,
                                        mstf_half* out, float* lse_out, int tokens, int head_dim, int Bq, int groups,
                                        int bit, int capacity, int dequant_mode, int group_size, void* workspace,
                                        size_t workspace_bytes);


#ifdef __cplusplus
}
#endif
#endif /* MUSTAFAR_HIP_H */
