// The caller's per-token device work in front of the decode attention (models/llama_mustafar_kernel.py:363-374,
// 391, 430): rotary embedding of the new token's query and key heads, the query rows laid out as the attention
// kernels read them, key and value rows appended to the dense local window.  One launch instead of the caller's
// view / transpose / rotate / concatenate sequence; the window lives in a pre-allocated buffer and the row comes
// from a device-side counter, so the call can be recorded into a HIP graph.
#include "compress_common.hpp"

namespace mstf {

struct StepRows {
    const _Float16* x;
    int64_t stride;  // halfs between two batch entries
    int heads;
};

// grid = ceil(bs * (n_q + 2 n_kv) / 8), 64 threads: eight lanes per head, a lane holds channels c .. c+7 < 64 of the
// head and their partners 64 channels on (the two halves the rotation mixes).
__global__ __launch_bounds__(64) void window_append_kernel(StepRows qs, StepRows ks, StepRows vs,
                                                           const _Float16* __restrict__ cos,
                                                           const _Float16* __restrict__ sin, int64_t rope_stride,
                                                           _Float16* __restrict__ q_out, _Float16* __restrict__ k_win,
                                                           _Float16* __restrict__ v_win, int win_stride, int win_len,
                                                           const int32_t* __restrict__ win_len_dev,
                                                           uint32_t* __restrict__ overflow, int bs)
{
    const int H = qs.heads + ks.heads + vs.heads;
    const int head = (int)blockIdx.x * 8 + (int)(threadIdx.x >> 3);
    if (head >= bs * H) return;
    const int b = head / H, h = head - b * H;
    const int c = (int)(threadIdx.x & 7) * 8;
    // the count of valid rows includes the new token: it goes to row count - 1
    const int len = win_len_dev ? *win_len_dev : win_len;
    const bool fits = len >= 1 && len <= win_stride;
    const bool is_q = h < qs.heads, is_k = !is_q && h < qs.heads + ks.heads;
    const StepRows& s = is_q ? qs : (is_k ? ks : vs);
    const int hs = is_q ? h : (is_k ? h - qs.heads : h - qs.heads - ks.heads);
    if (!is_q && !fits) {
        if (overflow && c == 0) *overflow = 1u;  // every writer stores the same value
        return;
    }
    const _Float16* xp = s.x + b * s.stride + (int64_t)hs * kD + c;
    uint4 o0 = *reinterpret_cast<const uint4*>(xp);
    uint4 o1 = *reinterpret_cast<const uint4*>(xp + 64);
    if (cos && (is_q || is_k)) {
        const _Float16* cp = cos + b * rope_stride + c;
        const _Float16* sp = sin + b * rope_stride + c;
        const uint4 c0 = *reinterpret_cast<const uint4*>(cp), c1 = *reinterpret_cast<const uint4*>(cp + 64);
        const uint4 s0 = *reinterpret_cast<const uint4*>(sp), s1 = *reinterpret_cast<const uint4*>(sp + 64);
        const uint4 x0 = o0, x1 = o1;
        rope_piece(x0, x1, c0, c1, s0, s1, o0, o1);
    }
    _Float16* dst;
    if (is_q) {
        if (!q_out) return;
        dst = q_out + ((int64_t)b * qs.heads + hs) * kD + c;
    } else {
        _Float16* win = is_k ? k_win : v_win;
        const int heads = is_k ? ks.heads : vs.heads;
        dst = win + (((int64_t)b * heads + hs) * win_stride + (len - 1)) * kD + c;
    }
    *reinterpret_cast<uint4*>(dst) = o0;
    *reinterpret_cast<uint4*>(dst + 64) = o1;
}

}  // namespace mstf

using namespace mstf;

extern "C" int mstf_window_append_f16(void* stream, const mstf_half* q_in, int64_t q_stride, const mstf_half* k_in,
                                      int64_t k_stride, const mstf_half* v_in, int64_t v_stride, int bs, int n_q,
                                      int n_kv, int head_dim, const mstf_half* cos, const mstf_half* sin,
                                      int64_t rope_stride, mstf_half* q_out, mstf_half* k_win, mstf_half* v_win,
                                      int win_stride, int win_len, const int32_t* win_len_dev, uint32_t* overflow)
{
    if (!k_in || !v_in || !k_win || !v_win) return MSTF_EINVAL;
    if ((q_in == nullptr) != (q_out == nullptr)) return MSTF_EINVAL;
    if ((cos == nullptr) != (sin == nullptr)) return MSTF_EINVAL;
    if (bs <= 0 || n_q < 0 || n_kv <= 0 || win_stride <= 0) return MSTF_EINVAL;
    if (!win_len_dev && (win_len < 1 || win_len > win_stride)) return MSTF_EINVAL;
    if (head_dim != kD) return MSTF_EUNSUPPORTED;
    if ((int64_t)bs * ((int64_t)n_q + 2 * (int64_t)n_kv) > 0x7FFFFFF0) return MSTF_EUNSUPPORTED;
    if (q_stride % 8 != 0 || k_stride % 8 != 0 || v_stride % 8 != 0 || rope_stride % 8 != 0) return MSTF_EALIGN;
    if (!aligned_to(q_in, 16) || !aligned_to(k_in, 16) || !aligned_to(v_in, 16) || !aligned_to(cos, 16) ||
        !aligned_to(sin, 16) || !aligned_to(q_out, 16) || !aligned_to(k_win, 16) || !aligned_to(v_win, 16) ||
        !aligned_to(win_len_dev, 4) || !aligned_to(overflow, 4))
        return MSTF_EALIGN;
    const int nq = q_in ? n_q : 0;
    const StepRows qs = {reinterpret_cast<const _Float16*>(q_in), q_stride, nq};
    const StepRows ks = {reinterpret_cast<const _Float16*>(k_in), k_stride, n_kv};
    const StepRows vs = {reinterpret_cast<const _Float16*>(v_in), v_stride, n_kv};
    const int heads_all = bs * (nq + 2 * n_kv);
    hipLaunchKernelGGL(window_append_kernel, dim3((unsigned)((heads_all + 7) / 8)), dim3(64), 0, as_stream(stream), qs, ks,
                       vs, reinterpret_cast<const _Float16*>(cos), reinterpret_cast<const _Float16*>(sin), rope_stride,
                       reinterpret_cast<_Float16*>(q_out), reinterpret_cast<_Float16*>(k_win),
                       reinterpret_cast<_Float16*>(v_win), win_stride, win_len, win_len_dev, overflow, bs);
    return check_launch();
}
