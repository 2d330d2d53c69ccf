"""numpy/ctypes front-end of the CPU oracle (oracle/mustafar_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke test and by the
`cpu_baseline` leg of bench.py.  The product package never imports this module.

Every function takes/returns numpy arrays; fp16 data are ``np.float16``.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libmustafar_oracle.so")


def build(force=False):
    """Compile the C restatement with gcc (no GPU involved)."""
    src = os.path.join(_HERE, "mustafar_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "all"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.orc_compress.restype = ctypes.c_uint64
        _lib.orc_compress_quant.restype = ctypes.c_uint64
        _lib.orc_compress_quant_grouped.restype = ctypes.c_uint64
        _lib.orc_num_threads.restype = ctypes.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _c(a, dt):
    a = np.ascontiguousarray(a)
    assert a.dtype == dt, (a.dtype, dt)
    return a


def num_threads():
    return int(lib().orc_num_threads())


# ---------------------------------------------------------------- pruning
def kth_from_sparsity(sparsity, D):
    """models/llama_mustafar_kernel.py:215 -- max(1, int(target_sparsity * D))."""
    return max(1, int(sparsity * D))


def prune_rows(x, kth):
    """dh_prune_key / dh_prune_value on the last axis (models/llama_mustafar_kernel.py:194-274)."""
    x = _c(x, np.float16)
    D = x.shape[-1]
    y = np.empty_like(x)
    lib().orc_prune_rows(_p(x), _p(y), ctypes.c_long(x.size // D), ctypes.c_int(D), ctypes.c_int(kth))
    return y


# ------------------------------------------------------------ fp16 format
def compress(x, is_value):
    """convert_key_batched / convert_value_batched (kernel/compression.py:249-435).

    x: [B, M, N] fp16, already pruned.  Returns (bmp int64 [B,T], idx int32 [B,T+1],
    nz_flat fp16, nz_off int32 [B] in 16-byte units)."""
    x = _c(x, np.float16)
    B, M, N = x.shape
    T = M * N // 64
    bmp = np.empty((B, T), np.uint64)
    idx = np.empty((B, T + 1), np.uint32)
    off = np.empty((B,), np.uint32)
    args = (ctypes.c_int(B), ctypes.c_int(M), ctypes.c_int(N), ctypes.c_int(int(is_value)))
    total = lib().orc_compress(_p(x), *args, _p(bmp), _p(idx), None, ctypes.c_uint64(0), _p(off))
    nz = np.full((int(total),), np.float16(np.nan))
    lib().orc_compress(_p(x), *args, _p(bmp), _p(idx), _p(nz), ctypes.c_uint64(int(total)), _p(off))
    return bmp.view(np.int64), idx.view(np.int32), nz, off.view(np.int32)


def split_nz(nz_flat, idx):
    """The per-batch list the reference returns (kernel/compression.py:330-338)."""
    out, start = [], 0
    for b in range(idx.shape[0]):
        n = 2 * int(idx[b, -1])
        out.append(nz_flat[start:start + n].copy())
        start += n
    return out


def decode(bmp, nz, idx, nz_off, b, M, N, is_value):
    """Dense [M,N] of batch entry b, addressed like kernel/csrc/SpMM_Kernel.cuh does."""
    dense = np.empty((M, N), np.float16)
    lib().orc_decode(_p(_c(bmp, np.int64)), _p(_c(nz, np.float16)), _p(_c(idx, np.int32)), _p(_c(nz_off, np.int32)),
                     ctypes.c_int(b), ctypes.c_int(M), ctypes.c_int(N), ctypes.c_int(int(is_value)), _p(dense))
    return dense


def key_spmv(bmp, nz, idx, nz_off, Bm, Lc, D, groups):
    """mustafar_key_formulation semantics.  Bm: [Bq, nrows, D] -> (C fp16, C fp32) [Bq, nrows, Lc]."""
    Bm = _c(Bm, np.float16)
    Bq, nrows, _ = Bm.shape
    C = np.empty((Bq, nrows, Lc), np.float16)
    Cf = np.empty((Bq, nrows, Lc), np.float32)
    lib().orc_key_spmv(_p(_c(bmp, np.int64)), _p(_c(nz, np.float16)), _p(_c(idx, np.int32)), _p(_c(nz_off, np.int32)),
                       _p(Bm), _p(C), _p(Cf), ctypes.c_int(Lc), ctypes.c_int(D), ctypes.c_int(Bq),
                       ctypes.c_int(groups), ctypes.c_int(nrows))
    return C, Cf


def value_spmv(bmp, nz, idx, nz_off, P, D, Lc, groups):
    """mustafar_value_formulation semantics.  P: [Bq, nrows, Lc] -> (C fp16, C fp32) [Bq, nrows, D]."""
    P = _c(P, np.float16)
    Bq, nrows, _ = P.shape
    C = np.empty((Bq, nrows, D), np.float16)
    Cf = np.empty((Bq, nrows, D), np.float32)
    lib().orc_value_spmv(_p(_c(bmp, np.int64)), _p(_c(nz, np.float16)), _p(_c(idx, np.int32)),
                         _p(_c(nz_off, np.int32)), _p(P), _p(C), _p(Cf), ctypes.c_int(D), ctypes.c_int(Lc),
                         ctypes.c_int(Bq), ctypes.c_int(groups), ctypes.c_int(nrows))
    return C, Cf


def scale_softmax(s, head_dim):
    """w = s / sqrt(head_dim) in fp16, softmax in fp32, back to fp16 (llama_mustafar_kernel.py:405,425)."""
    s = _c(s, np.float16)
    L = s.shape[-1]
    p = np.empty_like(s)
    lib().orc_scale_softmax(_p(s), _p(p), ctypes.c_long(s.size // L), ctypes.c_int(L),
                            ctypes.c_float(np.sqrt(np.float32(head_dim))))
    return p


def dense_masked_attention(q, Kp, Vp, groups):
    """Decode branch of the dense masked model (llama_mustafar_Kt_Mag_Vt_Mag.py:873-874,963,974).

    q: [Bq, D]; Kp, Vp: [Bkv, L, D] pruned dense.  Returns (scores, probs, out)."""
    q, Kp, Vp = _c(q, np.float16), _c(Kp, np.float16), _c(Vp, np.float16)
    Bq, D = q.shape
    L = Kp.shape[1]
    scores = np.empty((Bq, L), np.float16)
    probs = np.empty((Bq, L), np.float16)
    out = np.empty((Bq, D), np.float16)
    lib().orc_dense_masked_attention(_p(q), _p(Kp), _p(Vp), ctypes.c_int(Bq), ctypes.c_int(groups), ctypes.c_int(L),
                                     ctypes.c_int(D), _p(scores), _p(probs), _p(out))
    return scores, probs, out


# ----------------------------------------------------------- quant format
def compress_quant(x, is_value, bit=2, group_size=64):
    """convert_{key,value}_batched_quant (kernel_quant/compression_quant.py:159-264, 425-529).

    Returns (bmp int64 [B,T], tile_off int32 [B,T], packed int32 flat, counts int32, units int32,
    scales fp16, zeros fp16); scales / zeros are [B,T] for group_size 64 (the reference) and [B,T,2] for 32."""
    x = _c(x, np.float16)
    B, M, N = x.shape
    T = M * N // 64
    assert group_size in (32, 64)
    bmp = np.empty((B, T), np.uint64)
    counts = np.empty((B, T), np.uint32)
    units = np.empty((B, T), np.uint32)
    toff = np.empty((B, T), np.uint32)
    shape = (B, T) if group_size == 64 else (B, T, 2)
    scales = np.empty(shape, np.float16)
    zeros = np.empty(shape, np.float16)
    a = (ctypes.c_int(B), ctypes.c_int(M), ctypes.c_int(N), ctypes.c_int(int(is_value)), ctypes.c_int(bit),
         ctypes.c_int(group_size))
    fn = lib().orc_compress_quant_grouped
    total = fn(_p(x), *a, _p(bmp), _p(counts), _p(units), _p(toff), None, ctypes.c_uint64(0), _p(scales), _p(zeros))
    packed = np.zeros((int(total),), np.uint32)
    fn(_p(x), *a, _p(bmp), _p(counts), _p(units), _p(toff), _p(packed), ctypes.c_uint64(int(total)), _p(scales),
       _p(zeros))
    return (bmp.view(np.int64), toff.view(np.int32), packed.view(np.int32), counts.view(np.int32),
            units.view(np.int32), scales, zeros)


def decode_quant(bmp, packed, tile_off, scales, zeros, b, M, N, is_value, bit=2, dequant_mode=0):
    """Dense dequantised [M, N] of batch entry b; the group size follows from the shape of scales ([B,T] or [B,T,2])."""
    dense = np.empty((M, N), np.float16)
    group_size = 32 if np.ndim(scales) == 3 and np.shape(scales)[2] == 2 else 64
    lib().orc_decode_quant_grouped(_p(_c(bmp, np.int64)), _p(_c(packed, np.int32)), _p(_c(tile_off, np.int32)),
                                   _p(_c(scales, np.float16)), _p(_c(zeros, np.float16)), ctypes.c_int(b),
                                   ctypes.c_int(M), ctypes.c_int(N), ctypes.c_int(int(is_value)), ctypes.c_int(bit),
                                   ctypes.c_int(dequant_mode), ctypes.c_int(group_size), _p(dense))
    return dense


def spmv_quant(bmp, packed, tile_off, scales, zeros, Bm, is_value, Lc, D, groups, bit=2, dequant_mode=0):
    """Key (is_value=0, Bm [Bq,nrows,D] -> [Bq,nrows,Lc]) or value (Bm [Bq,nrows,Lc] -> [Bq,nrows,D])."""
    Bm = _c(Bm, np.float16)
    Bq, nrows, _ = Bm.shape
    out_w = D if is_value else Lc
    C = np.empty((Bq, nrows, out_w), np.float16)
    Cf = np.empty((Bq, nrows, out_w), np.float32)
    lib().orc_spmv_quant(_p(_c(bmp, np.int64)), _p(_c(packed, np.int32)), _p(_c(tile_off, np.int32)),
                         _p(_c(scales, np.float16)), _p(_c(zeros, np.float16)), _p(Bm), _p(C), _p(Cf),
                         ctypes.c_int(int(is_value)), ctypes.c_int(Lc), ctypes.c_int(D), ctypes.c_int(Bq),
                         ctypes.c_int(groups), ctypes.c_int(nrows), ctypes.c_int(bit), ctypes.c_int(dequant_mode))
    return C, Cf


# ------------------------------------------------------- rotary embedding in front of the compressor
def rope_tables(positions, D=128, theta=500000.0):
    """cos, sin [len(positions), D] fp16 as LlamaRotaryEmbedding of transformers 4.43.1 builds them (the reference
    calls it at models/llama_mustafar_kernel.py:373): inv_freq = theta^(-2i/D), emb = [freqs, freqs], cos and sin in
    fp32, cast to the activations' dtype."""
    inv = (1.0 / (np.float32(theta) ** (np.arange(0, D, 2, dtype=np.float32) / np.float32(D)))).astype(np.float32)
    f = np.asarray(positions, np.float32)[:, None] * inv[None, :]
    emb = np.concatenate([f, f], axis=-1)
    return np.cos(emb).astype(np.float16), np.sin(emb).astype(np.float16)


def rope_rows(x, cos, sin):
    """apply_rotary_pos_emb of transformers 4.43.1 (called at models/llama_mustafar_kernel.py:374) on fp16 rows
    x [..., tokens, D] with cos, sin [tokens, D]: (x * cos) + (rotate_half(x) * sin), every product and the sum
    rounded to fp16 (numpy's float16 arithmetic rounds each operation once, like the half-precision tensor ops)."""
    x = np.asarray(x, np.float16)
    h = x.shape[-1] // 2
    rot = np.concatenate([-x[..., h:], x[..., :h]], axis=-1)
    return ((x * cos).astype(np.float16) + (rot * sin).astype(np.float16)).astype(np.float16)


# ------------------------------------------------------- synthetic inputs
def make_kv(seed, Bkv, L, D=128, outlier_channels=4, outlier_scale=10.0):
    """Seeded K and V: fp16 N(0,1); K gets `outlier_channels` channels per head scaled by `outlier_scale`."""
    rng = np.random.default_rng(seed)
    K = rng.standard_normal((Bkv, L, D), dtype=np.float32)
    V = rng.standard_normal((Bkv, L, D), dtype=np.float32)
    for b in range(Bkv):
        ch = rng.choice(D, size=outlier_channels, replace=False)
        K[b][:, ch] *= outlier_scale
    return K.astype(np.float16), V.astype(np.float16)
