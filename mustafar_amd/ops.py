"""Zero-copy device path: fused prune+compress into a flat cache, SpMVs with one row per head.

Everything stays on the device; the only host synchronisation is the optional read-back of the
packed size when the caller did not provide a capacity.
"""
import math

import torch

from ._lib import check, lib

class Workspace:
    """Scratch memory for the entry points that need it (split partials, compressor scans), owned by one caller.

    A cache, a decode loop or a benchmark that records its calls into a HIP graph creates one sized for its largest
    call BEFORE capturing and passes it as `ws=`: the buffer then never moves, and calls on different streams with
    different workspaces are independent.  `get` hands out the buffer if it is large enough; growing replaces it but
    keeps the old buffers alive (a captured graph may still point at them), and growing while the current stream is
    being captured is an error."""

    def __init__(self, device, nbytes=1 << 20):
        self.device = torch.device(device)
        self._bufs = [torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=self.device)]

    @property
    def tensor(self):
        return self._bufs[-1]

    def reserve(self, nbytes):
        """Makes room for nbytes; to be called outside any graph capture."""
        if self.tensor.numel() < nbytes:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("workspace of %d bytes is too small for a call that needs %d and cannot grow while "
                                   "the stream is being captured: reserve() it before the capture"
                                   % (self.tensor.numel(), nbytes))
            self._bufs.append(torch.empty(int(nbytes), dtype=torch.uint8, device=self.device))
        return self.tensor

    def get(self, nbytes):
        return self.reserve(nbytes)


_WS = {}


def _stream():
    return torch.cuda.current_stream().cuda_stream


def workspace(device, nbytes, ws=None):
    """The scratch tensor for a call that needs nbytes: the caller's Workspace (`ws`) or, for the mirrors of the
    reference's operators, which have no such argument, a default one per (device, stream) - so two streams never
    share a buffer unless the caller passes the same Workspace to both."""
    if ws is not None:
        return ws.get(nbytes) if isinstance(ws, Workspace) else ws
    device = torch.device(device)
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device(), _stream())
    w = _WS.get(key)
    if w is None:
        w = _WS[key] = Workspace(device)
    return w.get(nbytes)


def kth_from_sparsity(sparsity, head_dim):
    """Rank of the pruning threshold: max(1, int(target_sparsity * D)) as in dh_prune_key."""
    return max(1, int(sparsity * head_dim))


class CompressedKV:
    """One side (K or V) of the compressed cache, flat on the device.

    bmp int64 [B, T], idx int32 [B, T+1], nz fp16 flat, nz_off int32 [B] (16-byte units)."""

    def __init__(self, bmp, idx, nz, nz_off, tokens, head_dim, is_value, total_halfs=None):
        self.bmp, self.idx, self.nz, self.nz_off = bmp, idx, nz, nz_off
        self.tokens, self.head_dim, self.is_value = tokens, head_dim, is_value
        self.total_halfs = total_halfs

    @property
    def heads(self):
        return self.bmp.shape[0]

    def used_halfs(self):
        """Number of fp16 values in use (reads the device-side total once).  The one-pass compressor reports a wait that
        ran out - which the dispatch order rules out - as a total of all ones: that raises here."""
        n = int(self.total_halfs)
        if n < 0 or n > (1 << 62):
            raise RuntimeError("the compressor gave up waiting for an earlier workgroup; the packed values are incomplete")
        return n

    def packed(self):
        """The used part of the flat value buffer (needs the host-side size)."""
        return self.nz[:self.used_halfs()]

    def nbytes(self):
        """Algorithmic size: bitmaps + offsets + packed values actually used."""
        used = self.nz.numel() if self.total_halfs is None else self.used_halfs()
        return self.bmp.numel() * 8 + self.idx.numel() * 4 + used * 2


def prune_rows(x, kth, out=None):
    """dh_prune_key / dh_prune_value on the last axis (D = 128)."""
    assert x.is_cuda and x.dtype == torch.float16 and x.is_contiguous()
    D = x.shape[-1]
    y = torch.empty_like(x) if out is None else out
    check(lib().mstf_prune_rows_f16(_stream(), x.data_ptr(), y.data_ptr(), x.numel() // D, D, int(kth)),
          "mstf_prune_rows_f16")
    return y


def compress(x, is_value, kth=0, capacity_halfs=None, ws=None):
    """Prune (kth > 0) and compress x [B, M, N] into the bitmap format.

    With capacity_halfs=None the packed size is read back once (like the reference's .item());
    with a capacity the call is fully asynchronous and `total_halfs` stays on the device."""
    assert x.is_cuda and x.dtype == torch.float16 and x.dim() == 3
    x = x.contiguous()
    B, M, N = x.shape
    T = M * N // 64
    dev = x.device
    L = lib()
    bmp = torch.empty((B, T), dtype=torch.int64, device=dev)
    idx = torch.empty((B, T + 1), dtype=torch.int32, device=dev)
    nz_off = torch.empty((B,), dtype=torch.int32, device=dev)
    total = torch.empty((1,), dtype=torch.int64, device=dev)
    wsb = L.mstf_compress_workspace_bytes(B, M, N)
    ws = workspace(dev, wsb, ws)
    fn = L.mstf_compress_value_f16 if is_value else L.mstf_compress_key_f16
    name = "mstf_compress_value_f16" if is_value else "mstf_compress_key_f16"
    if capacity_halfs is None:
        check(fn(_stream(), x.data_ptr(), B, M, N, int(kth), bmp.data_ptr(), idx.data_ptr(), nz_off.data_ptr(),
                 total.data_ptr(), None, 0, ws.data_ptr(), ws.numel()), name)
        n = int(total.item())
        nz = torch.empty((max(n, 8),), dtype=torch.float16, device=dev)
        sc = L.mstf_scatter_value_f16 if is_value else L.mstf_scatter_key_f16
        check(sc(_stream(), x.data_ptr(), B, M, N, bmp.data_ptr(), idx.data_ptr(), nz_off.data_ptr(), nz.data_ptr(),
                 n), name.replace("compress", "scatter"))
        if n == 0:
            nz.zero_()
        return CompressedKV(bmp, idx, nz if n == 0 else nz[:n], nz_off, M, N, is_value, n)
    nz = torch.empty((int(capacity_halfs),), dtype=torch.float16, device=dev)
    check(fn(_stream(), x.data_ptr(), B, M, N, int(kth), bmp.data_ptr(), idx.data_ptr(), nz_off.data_ptr(),
             total.data_ptr(), nz.data_ptr(), int(capacity_halfs), ws.data_ptr(), ws.numel()), name)
    return CompressedKV(bmp, idx, nz, nz_off, M, N, is_value, total)


def compress_kv(k, v, kth_k=0, kth_v=0, capacity_halfs=None, ws=None):
    """compress(k, False, kth_k) and compress(v, True, kth_v) of the same tokens in one launch (mstf_compress_kv_f16):
    identical outputs, less time - a launch of both sides runs less in lockstep than two launches of one side each.
    k, v: [B, M, N]; capacity_halfs (default: room for the dense rows) sizes both value buffers, the totals stay on
    the device.  Returns (CompressedKV of the keys, CompressedKV of the values)."""
    assert k.is_cuda and v.is_cuda and k.dtype == v.dtype == torch.float16 and k.dim() == 3 and k.shape == v.shape
    k, v = k.contiguous(), v.contiguous()
    B, M, N = k.shape
    T = M * N // 64
    dev = k.device
    L = lib()
    cap = B * M * N if capacity_halfs is None else int(capacity_halfs)
    out = []
    for _ in range(2):
        out.append((torch.empty((B, T), dtype=torch.int64, device=dev), torch.empty((B, T + 1), dtype=torch.int32, device=dev),
                    torch.empty((B,), dtype=torch.int32, device=dev), torch.empty((1,), dtype=torch.int64, device=dev),
                    torch.empty((cap,), dtype=torch.float16, device=dev)))
    ws = workspace(dev, L.mstf_compress_kv_workspace_bytes(B, M, N), ws)
    (kb, ki, ko, kt, kn), (vb, vi, vo, vt, vn) = out
    check(L.mstf_compress_kv_f16(_stream(), k.data_ptr(), v.data_ptr(), B, M, N, int(kth_k), int(kth_v), kb.data_ptr(),
                                 ki.data_ptr(), ko.data_ptr(), kt.data_ptr(), kn.data_ptr(), cap, vb.data_ptr(),
                                 vi.data_ptr(), vo.data_ptr(), vt.data_ptr(), vn.data_ptr(), cap, ws.data_ptr(),
                                 ws.numel()), "mstf_compress_kv_f16")
    return CompressedKV(kb, ki, kn, ko, M, N, False, kt), CompressedKV(vb, vi, vn, vo, M, N, True, vt)


def proj_source(x, cos=None, sin=None, rot=None):
    """The mstf_proj_source of x [batch, rows, heads, 128] fp16 (any strides with contiguous channels, e.g. a view of
    a projection output [batch, rows, heads * 128]).  cos, sin: [rows, 128] or [batch, rows, 128] fp16 (keys only);
    rot: where the rotated rows go, shaped like x (default: x itself, in place).  Returns (struct, rot)."""
    from ._lib import ProjSource
    assert x.is_cuda and x.dtype == torch.float16 and x.dim() == 4 and x.stride(3) == 1
    src = ProjSource()
    src.x = x.data_ptr()
    src.stride_batch, src.stride_token, src.stride_head = x.stride(0), x.stride(1), x.stride(2)
    src.batch, src.rows, src.heads = x.shape[0], x.shape[1], x.shape[2]
    if cos is not None:
        assert sin is not None and cos.dtype == sin.dtype == torch.float16 and cos.shape == sin.shape
        assert cos.stride(-1) == 1 and sin.stride() == cos.stride() and cos.shape[-2] >= x.shape[1]
        rot = x if rot is None else rot
        assert rot.shape == x.shape and rot.dtype == torch.float16 and rot.stride(3) == 1
        src.cos, src.sin = cos.data_ptr(), sin.data_ptr()
        src.rope_stride_batch = cos.stride(0) if cos.dim() == 3 and cos.shape[0] > 1 else 0
        src.rope_stride_token = cos.stride(-2)
        src.rot = rot.data_ptr()
        src.rot_stride_batch, src.rot_stride_token, src.rot_stride_head = rot.stride(0), rot.stride(1), rot.stride(2)
    return src, rot


def compress_proj(x, is_value, kth, M, cos=None, sin=None, rot=None, capacity_halfs=None, ws=None):
    """Prune and compress the first M tokens of x [batch, rows, heads, 128] where the projection left them, the keys
    rotated first when cos / sin are given (all rows are rotated and written to rot).  Heads are numbered
    batch * heads + head.  Returns (CompressedKV, rot)."""
    import ctypes
    src, rot = proj_source(x, cos, sin, rot)
    B, N, dev = x.shape[0] * x.shape[2], x.shape[3], x.device
    T = M * N // 64
    L = lib()
    cap = B * M * N if capacity_halfs is None else int(capacity_halfs)
    bmp = torch.empty((B, T), dtype=torch.int64, device=dev)
    idx = torch.empty((B, T + 1), dtype=torch.int32, device=dev)
    nz_off = torch.empty((B,), dtype=torch.int32, device=dev)
    total = torch.empty((1,), dtype=torch.int64, device=dev)
    nz = torch.empty((max(cap, 8),), dtype=torch.float16, device=dev)
    ws = workspace(dev, L.mstf_compress_workspace_bytes(B, max(M, 64), N), ws)
    check(L.mstf_compress_proj_f16(_stream(), ctypes.byref(src), int(is_value), M, N, int(kth), bmp.data_ptr(),
                                   idx.data_ptr(), nz_off.data_ptr(), total.data_ptr(), nz.data_ptr(), cap,
                                   ws.data_ptr(), ws.numel()), "mstf_compress_proj_f16")
    if M == 0:
        return None, rot
    if capacity_halfs is None:
        n = int(total.item())
        return CompressedKV(bmp, idx, nz[:n], nz_off, M, N, is_value, n), rot
    return CompressedKV(bmp, idx, nz, nz_off, M, N, is_value, total), rot


def key_spmv(ck, q, groups, n_rows=1, out=None):
    """scores[bq, n, t] = sum_d K[bq // groups][t, d] * q[bq, n, d]   (unscaled).  q: [Bq, n_rows, D]."""
    assert q.dtype == torch.float16 and q.is_contiguous()
    Bq = q.numel() // (n_rows * ck.head_dim)
    C = torch.empty((Bq, n_rows, ck.tokens), dtype=torch.float16, device=q.device) if out is None else out
    check(lib().mstf_key_spmv_f16(_stream(), ck.bmp.data_ptr(), ck.nz.data_ptr(), ck.idx.data_ptr(),
                                  ck.nz_off.data_ptr(), q.data_ptr(), C.data_ptr(), ck.tokens, ck.head_dim, Bq,
                                  groups, n_rows), "mstf_key_spmv_f16")
    return C


def value_spmv(cv, p, groups, n_rows=1, out=None, ws=None):
    """out[bq, n, d] = sum_t V[bq // groups][t, d] * p[bq, n, t].  p: [Bq, n_rows, Lc]."""
    assert p.dtype == torch.float16 and p.is_contiguous()
    Bq = p.numel() // (n_rows * cv.tokens)
    L = lib()
    C = torch.empty((Bq, n_rows, cv.head_dim), dtype=torch.float16, device=p.device) if out is None else out
    wsb = L.mstf_value_spmv_workspace_bytes(cv.head_dim, cv.tokens, Bq, groups, n_rows)
    ws = workspace(p.device, wsb, ws)
    check(L.mstf_value_spmv_f16(_stream(), cv.bmp.data_ptr(), cv.nz.data_ptr(), cv.idx.data_ptr(),
                                cv.nz_off.data_ptr(), p.data_ptr(), C.data_ptr(), cv.head_dim, cv.tokens, Bq, groups,
                                n_rows, ws.data_ptr(), ws.numel()), "mstf_value_spmv_f16")
    return C


def decode_attention(ck, cv, q, groups, out=None, lse=None, ws=None):
    """Fused key SpMV -> scale+softmax -> value SpMV over the compressed tokens, one query row per head.

    q: [Bq, D] fp16 -> out [Bq, D] fp16.  lse (optional fp32 [Bq, 2]) receives (max, sum) of every row."""
    assert q.dtype == torch.float16 and q.is_contiguous()
    D = ck.head_dim
    Bq = q.numel() // D
    L = lib()
    o = torch.empty((Bq, D), dtype=torch.float16, device=q.device) if out is None else out
    ws = workspace(q.device, L.mstf_decode_attention_workspace_bytes(ck.tokens, D, Bq, groups), ws)
    check(L.mstf_decode_attention_f16(_stream(), ck.bmp.data_ptr(), ck.nz.data_ptr(), ck.idx.data_ptr(),
                                      ck.nz_off.data_ptr(), cv.bmp.data_ptr(), cv.nz.data_ptr(), cv.idx.data_ptr(),
                                      cv.nz_off.data_ptr(), q.data_ptr(), o.data_ptr(),
                                      lse.data_ptr() if lse is not None else None, ck.tokens, D, Bq, groups,
                                      ws.data_ptr(), ws.numel()), "mstf_decode_attention_f16")
    return o


def decode_attention_static(ck, cv, q, groups, out=None, lse=None):
    """decode_attention through the entry point that uses the library's own fixed scratch buffer: no workspace is
    passed and nothing is allocated by the library (calls on one GPU must not overlap)."""
    assert q.dtype == torch.float16 and q.is_contiguous()
    D = ck.head_dim
    Bq = q.numel() // D
    o = torch.empty((Bq, D), dtype=torch.float16, device=q.device) if out is None else out
    check(lib().mstf_decode_attention_static_f16(_stream(), ck.bmp.data_ptr(), ck.nz.data_ptr(), ck.idx.data_ptr(),
                                                 ck.nz_off.data_ptr(), cv.bmp.data_ptr(), cv.nz.data_ptr(),
                                                 cv.idx.data_ptr(), cv.nz_off.data_ptr(), q.data_ptr(), o.data_ptr(),
                                                 lse.data_ptr() if lse is not None else None, ck.tokens, D, Bq, groups),
          "mstf_decode_attention_static_f16")
    return o


def decode_attention_window(ck, cv, q, k_win, v_win, win_len, groups, out=None, lse=None, win_len_dev=None, ws=None):
    """Attention of one decode step over [compressed tokens | dense window] under one softmax, three launches.

    ck, cv: CompressedKV or None (nothing compressed yet); q: [Bq, D]; k_win, v_win: [Bkv, win_stride, D] fp16 with
    the first win_len tokens valid.  win_len_dev (int32 tensor of one element): the valid length is read on the
    device and win_len is only its upper bound, so that the call can be captured in a HIP graph."""
    assert q.dtype == torch.float16 and q.is_contiguous()
    assert k_win.dtype == torch.float16 and k_win.is_contiguous() and v_win.is_contiguous() and k_win.shape == v_win.shape
    D = k_win.shape[-1]
    Bq = q.numel() // D
    tokens = ck.tokens if ck is not None else 0
    L = lib()
    o = torch.empty((Bq, D), dtype=torch.float16, device=q.device) if out is None else out
    ws = workspace(q.device, L.mstf_decode_attention_window_workspace_bytes(tokens, int(win_len), D, Bq, groups), ws)
    cp = [t.data_ptr() for t in (ck.bmp, ck.nz, ck.idx, ck.nz_off, cv.bmp, cv.nz, cv.idx, cv.nz_off)] if tokens else [None] * 8
    check(L.mstf_decode_attention_window_f16(_stream(), *cp, q.data_ptr(), k_win.data_ptr(), v_win.data_ptr(), int(win_len),
                                             win_len_dev.data_ptr() if win_len_dev is not None else None,
                                             k_win.shape[1], o.data_ptr(), lse.data_ptr() if lse is not None else None,
                                             tokens, D, Bq, groups, ws.data_ptr(), ws.numel()),
          "mstf_decode_attention_window_f16")
    return o


def decode_attention_window_pool(k_pool, v_pool, q, k_win, v_win, win_len, groups, win_len_dev, out=None, lse=None,
                                 ws=None):
    """decode_attention_window over two cache.CompressedPool sides that grow in place: the pools' pre-allocated
    per-tile arrays are read with their row stride and the number of compressed tokens comes from the pool's device
    counter, so nothing about the call changes when a chunk is appended (a HIP graph holding it stays valid)."""
    assert q.dtype == torch.float16 and q.is_contiguous()
    assert k_win.dtype == torch.float16 and k_win.is_contiguous() and v_win.is_contiguous() and k_win.shape == v_win.shape
    assert k_pool.max_tokens == v_pool.max_tokens
    D = k_win.shape[-1]
    Bq = q.numel() // D
    L = lib()
    o = torch.empty((Bq, D), dtype=torch.float16, device=q.device) if out is None else out
    ws = workspace(q.device, L.mstf_decode_attention_window_workspace_bytes(k_pool.max_tokens, int(win_len), D, Bq,
                                                                           groups), ws)
    cp = [t.data_ptr() for t in (k_pool.bmp_store, k_pool.nz, k_pool.idx_store, k_pool.nz_off, v_pool.bmp_store, v_pool.nz,
                                 v_pool.idx_store, v_pool.nz_off)]
    check(L.mstf_decode_attention_window_pool_f16(_stream(), *cp, q.data_ptr(), k_win.data_ptr(), v_win.data_ptr(),
                                                  int(win_len), win_len_dev.data_ptr() if win_len_dev is not None else None,
                                                  k_win.shape[1], o.data_ptr(), lse.data_ptr() if lse is not None else None,
                                                  k_pool.max_tokens, k_pool.tokens_dev.data_ptr(), k_pool.tile_capacity, D,
                                                  Bq, groups, ws.data_ptr(), ws.numel()),
          "mstf_decode_attention_window_pool_f16")
    return o


def decode_step_pool(k_pool, v_pool, q_in, k_in, v_in, k_win, v_win, win_len, cos=None, sin=None, win_len_dev=None,
                     overflow=None, out=None, lse=None, ws=None):
    """The cache side of a decode step in two launches (mstf_decode_step_pool_f16): window_append followed by
    decode_attention_window_pool, bit for bit, with rotation, append and the attention over the window inside the
    launch of the compressed tokens.  q_in [bs, n_q * D], k_in / v_in [bs, n_kv * D]: the projection outputs of the
    new token (views with a batch stride are fine); cos, sin [D] or [bs, D] or None; k_win, v_win
    [bs * n_kv, win_stride, D]; win_len bounds the count of valid rows after the step, win_len_dev holds it."""
    D = k_win.shape[-1]
    bs = k_in.shape[0]
    n_kv, n_q = k_in.shape[-1] // D, q_in.shape[-1] // D
    for t in (q_in, k_in, v_in):
        assert t.dtype == torch.float16 and t.dim() == 2 and t.stride(1) == 1 and t.shape[0] == bs
    assert k_win.dtype == torch.float16 and k_win.is_contiguous() and v_win.is_contiguous() and k_win.shape == v_win.shape
    assert k_win.shape[0] == bs * n_kv and v_in.shape[-1] == n_kv * D and n_q % n_kv == 0
    assert k_pool.max_tokens == v_pool.max_tokens
    rope_stride = 0
    if cos is not None:
        assert cos.dtype == torch.float16 and sin.dtype == torch.float16 and cos.shape == sin.shape
        assert cos.shape[-1] == D and cos.stride(-1) == 1 and sin.stride(-1) == 1
        if cos.dim() == 2 and cos.shape[0] > 1:
            assert cos.shape[0] == bs and cos.stride(0) == sin.stride(0)
            rope_stride = cos.stride(0)
    L = lib()
    Bq = bs * n_q
    o = torch.empty((Bq, D), dtype=torch.float16, device=q_in.device) if out is None else out
    ws = workspace(q_in.device, L.mstf_decode_attention_window_workspace_bytes(k_pool.max_tokens, int(win_len), D, Bq,
                                                                              n_q // n_kv), ws)
    cp = [t.data_ptr() for t in (k_pool.bmp_store, k_pool.nz, k_pool.idx_store, k_pool.nz_off, v_pool.bmp_store, v_pool.nz,
                                 v_pool.idx_store, v_pool.nz_off)]
    check(L.mstf_decode_step_pool_f16(
        _stream(), *cp, q_in.data_ptr(), q_in.stride(0), k_in.data_ptr(), k_in.stride(0), v_in.data_ptr(), v_in.stride(0),
        bs, n_q, n_kv, cos.data_ptr() if cos is not None else None, sin.data_ptr() if sin is not None else None,
        rope_stride, k_win.data_ptr(), v_win.data_ptr(), k_win.shape[1], int(win_len),
        win_len_dev.data_ptr() if win_len_dev is not None else None, overflow.data_ptr() if overflow is not None else None,
        o.data_ptr(), lse.data_ptr() if lse is not None else None, k_pool.max_tokens, k_pool.tokens_dev.data_ptr(),
        k_pool.tile_capacity, D, ws.data_ptr(), ws.numel()), "mstf_decode_step_pool_f16")
    return o


def window_append(k_in, v_in, k_win, v_win, win_len, q_in=None, cos=None, sin=None, q_out=None, win_len_dev=None,
                  overflow=None):
    """The per-token work in front of the attention call in one launch (models/llama_mustafar_kernel.py:363-374, 391,
    430): q_in [bs, n_q * D], k_in / v_in [bs, n_kv * D] fp16 are the projection outputs of the new token (views with
    a batch stride are fine); query and key heads are rotated with cos, sin [D] or [bs, D] (None: no rotation), the
    query rows returned as [bs * n_q, D], key and value rows written to row win_len - 1 of the window buffers
    k_win, v_win [bs * n_kv, win_stride, D].  win_len counts the valid rows after the call, the new token included;
    with win_len_dev (int32 tensor) the count is read on the device.  Returns q_out (None without q_in)."""
    D = k_win.shape[-1]
    bs = k_in.shape[0]
    n_kv = k_in.shape[-1] // D
    for t in (k_in, v_in) + ((q_in,) if q_in is not None else ()):
        assert t.dtype == torch.float16 and t.dim() == 2 and t.stride(1) == 1 and t.shape[0] == bs
    assert k_win.dtype == torch.float16 and k_win.is_contiguous() and v_win.is_contiguous() and k_win.shape == v_win.shape
    assert k_win.shape[0] == bs * n_kv and v_in.shape[-1] == n_kv * D
    n_q = 0
    if q_in is not None:
        n_q = q_in.shape[-1] // D
        if q_out is None:
            q_out = torch.empty((bs * n_q, D), dtype=torch.float16, device=q_in.device)
        assert q_out.dtype == torch.float16 and q_out.is_contiguous() and q_out.numel() == bs * n_q * D
    rope_stride = 0
    if cos is not None:
        assert cos.dtype == torch.float16 and sin.dtype == torch.float16 and cos.shape == sin.shape
        assert cos.shape[-1] == D and cos.stride(-1) == 1 and sin.stride(-1) == 1
        if cos.dim() == 2 and cos.shape[0] > 1:
            assert cos.shape[0] == bs and cos.stride(0) == sin.stride(0)
            rope_stride = cos.stride(0)
    check(lib().mstf_window_append_f16(
        _stream(), q_in.data_ptr() if q_in is not None else None, q_in.stride(0) if q_in is not None else 0,
        k_in.data_ptr(), k_in.stride(0), v_in.data_ptr(), v_in.stride(0), bs, n_q, n_kv, D,
        cos.data_ptr() if cos is not None else None, sin.data_ptr() if sin is not None else None, rope_stride,
        q_out.data_ptr() if q_out is not None else None, k_win.data_ptr(), v_win.data_ptr(), k_win.shape[1], int(win_len),
        win_len_dev.data_ptr() if win_len_dev is not None else None, overflow.data_ptr() if overflow is not None else None),
        "mstf_window_append_f16")
    return q_out


def decode_attention_partial(ck, cv, q, groups, ws=None):
    """First phase of decode_attention: un-normalised outputs and (max, sum) per 512-token split, left in `ws`."""
    assert q.dtype == torch.float16 and q.is_contiguous()
    D = ck.head_dim
    Bq = q.numel() // D
    L = lib()
    ws = workspace(q.device, L.mstf_decode_attention_workspace_bytes(ck.tokens, D, Bq, groups), ws)
    check(L.mstf_decode_attention_partial_f16(_stream(), ck.bmp.data_ptr(), ck.nz.data_ptr(), ck.idx.data_ptr(),
                                              ck.nz_off.data_ptr(), cv.bmp.data_ptr(), cv.nz.data_ptr(),
                                              cv.idx.data_ptr(), cv.nz_off.data_ptr(), q.data_ptr(), ck.tokens, D, Bq,
                                              groups, ws.data_ptr(), ws.numel()), "mstf_decode_attention_partial_f16")
    return ws


def decode_attention_merge(ws, tokens, head_dim, Bq, groups, out=None, lse=None):
    """Second phase of decode_attention: combines the splits left in `ws` by decode_attention_partial."""
    o = torch.empty((Bq, head_dim), dtype=torch.float16, device=ws.device) if out is None else out
    check(lib().mstf_decode_attention_merge_f16(_stream(), ws.data_ptr(), ws.numel(), o.data_ptr(),
                                                lse.data_ptr() if lse is not None else None, tokens, head_dim, Bq,
                                                groups), "mstf_decode_attention_merge_f16")
    return o


def scale_softmax(s, head_dim, out=None):
    """softmax(s / sqrt(head_dim), dtype=float32).to(float16) over the last axis."""
    assert s.dtype == torch.float16 and s.stride(-1) == 1
    L = s.shape[-1]
    s2 = s.reshape(-1, L)
    p = torch.empty_like(s2) if out is None else out.reshape(-1, L)
    check(lib().mstf_scale_softmax_f16(_stream(), s2.data_ptr(), p.data_ptr(), s2.shape[0], L, s2.stride(0),
                                       p.stride(0), int(head_dim)), "mstf_scale_softmax_f16")
    return p.reshape(s.shape)


def sqrt_head_dim(head_dim):
    return math.sqrt(head_dim)
