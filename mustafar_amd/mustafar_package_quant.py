"""Drop-in for the reference's `mustafar_package_quant` extension
(kernel_quant/kernel_wrapper/pybind_quant.cpp:10-177, mustafar_wrapper_quant.cu): the four operators
and their four aliases, same keyword names, checks and output shapes.

Differences that do not change results: `split_k` and `value_tile_config` only steer how the
reference splits its launch (its tile64 / fused configurations address the wrong tiles); here the
split is chosen by the library and both arguments are accepted and ignored.  `tile_counts` /
`tile_units` are validated but not read: they follow from the bitmaps.

An addition of this build: when `scales` / `zeros` are [B, T, 2] (as `convert_*_batched_quant(group_size=32)` return
them) every operator here reads two (scale, zero) pairs per tile, pair g for the elements 32g .. 32g+31.
"""
import torch

from . import ops
from ._lib import check, lib


def _group_size(bmp, scales, zeros):
    """64 for [B, T] scales (the reference), 32 for [B, T, 2]."""
    if scales.shape != zeros.shape:
        raise RuntimeError("scales and zeros must have the same shape.")
    if scales.numel() == bmp.numel():
        return 64
    if scales.numel() == 2 * bmp.numel() and scales.shape[-1] == 2:
        return 32
    raise RuntimeError("scales must hold one or two entries per tile.")


def _common_checks(B, tensors, int_names, half_names):
    dev = B.device
    for name, t in tensors.items():
        if t.device != dev:
            raise RuntimeError("All input tensors must be on the same device.")
    if B.dtype != torch.float16:
        raise RuntimeError("Tensor B must be of type float16.")
    if tensors["bmp"].dtype != torch.int64:
        raise RuntimeError("Tensor bmp must be of type int64.")
    for name in int_names:
        if tensors[name].dtype != torch.int32:
            raise RuntimeError("Tensor %s must be of type int32." % name)
    for name in half_names:
        if tensors[name].dtype != torch.float16:
            raise RuntimeError("Tensor %s must be of type float16." % name)
    if not all(t.is_contiguous() for t in tensors.values()):
        raise RuntimeError("All tensors must be contiguous.")
    if not (B.is_cuda and all(t.is_cuda for t in tensors.values())):
        raise RuntimeError("All tensors must be on CUDA device.")
    if tensors["NZ_quant"].numel() == 0:
        raise RuntimeError("NZ_quant is empty.")


def _key(bmp, NZ_quant, tile_offsets, tile_counts, tile_units, scales, zeros, B, M_Global, K_Global, Batch_Size,
         num_key_value_groups, bit, capacity, dequant_mode):
    tensors = {"bmp": bmp, "NZ_quant": NZ_quant, "tile_offsets": tile_offsets, "scales": scales, "zeros": zeros}
    ints = ["NZ_quant", "tile_offsets"]
    if tile_counts is not None:
        tensors["tile_counts"], tensors["tile_units"] = tile_counts, tile_units
        ints += ["tile_counts", "tile_units"]
    _common_checks(B, tensors, ints, ["scales", "zeros"])
    if not B.is_contiguous():
        raise RuntimeError("All tensors must be contiguous.")
    if B.numel() != Batch_Size * 8 * K_Global:
        raise RuntimeError("Tensor B must hold Batch_Size x 8 x K_Global elements.")
    C = torch.empty((Batch_Size, 8, M_Global), dtype=torch.float16, device=B.device)
    check(lib().mstf_key_spmv_quant_grouped(torch.cuda.current_stream().cuda_stream, bmp.data_ptr(), NZ_quant.data_ptr(),
                                            tile_offsets.data_ptr(), scales.data_ptr(), zeros.data_ptr(), B.data_ptr(),
                                            C.data_ptr(), int(M_Global), int(K_Global), int(Batch_Size),
                                            int(num_key_value_groups), 8, int(bit), int(capacity), int(dequant_mode),
                                            _group_size(bmp, scales, zeros)), "mustafar_key_formulation_quant")
    return C


def mustafar_key_formulation_quant(bmp, NZ_quant, tile_offsets, scales, zeros, B, M_Global, K_Global, Batch_Size,
                                   num_key_value_groups, bit, capacity, dequant_mode=0):
    return _key(bmp, NZ_quant, tile_offsets, None, None, scales, zeros, B, M_Global, K_Global, Batch_Size,
                num_key_value_groups, bit, capacity, dequant_mode)


def mustafar_key_formulation_quant_meta(bmp, NZ_quant, tile_offsets, tile_counts, tile_units, scales, zeros, B, M_Global,
                                        K_Global, Batch_Size, num_key_value_groups, bit, capacity, dequant_mode=0):
    return _key(bmp, NZ_quant, tile_offsets, tile_counts, tile_units, scales, zeros, B, M_Global, K_Global, Batch_Size,
                num_key_value_groups, bit, capacity, dequant_mode)


def _value(bmp, NZ_quant, tile_offsets, tile_counts, tile_units, scales, zeros, P, n_rows, M_Global, K_Global,
           Batch_Size, num_key_value_groups, bit, capacity, dequant_mode, what):
    tensors = {"bmp": bmp, "NZ_quant": NZ_quant, "tile_offsets": tile_offsets, "tile_counts": tile_counts,
               "tile_units": tile_units, "scales": scales, "zeros": zeros}
    _common_checks(P, tensors, ["NZ_quant", "tile_offsets", "tile_counts", "tile_units"], ["scales", "zeros"])
    if P.numel() != Batch_Size * n_rows * K_Global:
        raise RuntimeError("score tensor has the wrong number of elements.")
    P = P.contiguous()
    L = lib()
    shape = (Batch_Size, 8, M_Global) if n_rows == 8 else (Batch_Size, M_Global)
    C = torch.empty(shape, dtype=torch.float16, device=P.device)
    wsb = L.mstf_value_spmv_quant_workspace_bytes(int(M_Global), int(K_Global), int(Batch_Size),
                                                  int(num_key_value_groups), n_rows)
    ws = ops.workspace(P.device, wsb)
    check(L.mstf_value_spmv_quant_grouped(torch.cuda.current_stream().cuda_stream, bmp.data_ptr(), NZ_quant.data_ptr(),
                                          tile_offsets.data_ptr(), scales.data_ptr(), zeros.data_ptr(), P.data_ptr(),
                                          C.data_ptr(), int(M_Global), int(K_Global), int(Batch_Size),
                                          int(num_key_value_groups), n_rows, int(bit), int(capacity), int(dequant_mode),
                                          _group_size(bmp, scales, zeros), ws.data_ptr(), ws.numel()), what)
    return C


def mustafar_value_formulation_quant(bmp, NZ_quant, tile_offsets, tile_counts, tile_units, scales, zeros, B,
                                     Reduction_Workspace, M_Global, K_Global, Batch_Size, num_key_value_groups, bit,
                                     capacity, dequant_mode=0, split_k=1, value_tile_config=0):
    return _value(bmp, NZ_quant, tile_offsets, tile_counts, tile_units, scales, zeros, B, 8, M_Global, K_Global,
                  Batch_Size, num_key_value_groups, bit, capacity, dequant_mode, "mustafar_value_formulation_quant")


def mustafar_value_formulation_quant_decode_n1(bmp, NZ_quant, tile_offsets, tile_counts, tile_units, scales, zeros,
                                               score, Reduction_Workspace, M_Global, K_Global, Batch_Size,
                                               num_key_value_groups, bit, capacity, dequant_mode=0, split_k=1):
    """score: [Batch_Size, K_Global] -> [Batch_Size, M_Global]."""
    return _value(bmp, NZ_quant, tile_offsets, tile_counts, tile_units, scales, zeros, score, 1, M_Global, K_Global,
                  Batch_Size, num_key_value_groups, bit, capacity, dequant_mode,
                  "mustafar_value_formulation_quant_decode_n1")


def decode_attention_quant(key_side, value_side, q, num_key_value_groups, bit, dequant_mode=0, out=None, lse=None,
                           ws=None):
    """One launch for key SpMV -> / sqrt(d) -> softmax -> value SpMV over a quantised cache (no counterpart in the
    reference, which runs the three steps separately).

    key_side, value_side: (bitmaps, tile_offsets, packed, scales, zeros) as convert_*_batched_quant return them
    (7-tuples with counts and units are accepted); q: [Bq, 128] fp16 -> [Bq, 128] fp16.  lse (optional fp32 [Bq, 2])
    receives (max, sum) of every row."""
    def five(side):
        return side if len(side) == 5 else (side[0], side[1], side[2], side[5], side[6])
    kb, ko, kp, ks, kz = five(key_side)
    vb, vo, vp, vs, vz = five(value_side)
    D = q.shape[-1]
    Bq = q.numel() // D
    tokens = kb.shape[1] * 64 // D
    L = lib()
    o = torch.empty((Bq, D), dtype=torch.float16, device=q.device) if out is None else out
    ws = ops.workspace(q.device, L.mstf_decode_attention_workspace_bytes(tokens, D, Bq, num_key_value_groups), ws)
    group_size = _group_size(kb, ks, kz)
    if _group_size(vb, vs, vz) != group_size:
        raise RuntimeError("key side and value side must use the same group size.")
    check(L.mstf_decode_attention_quant_grouped(torch.cuda.current_stream().cuda_stream, kb.data_ptr(), kp.data_ptr(),
                                                ko.data_ptr(), ks.data_ptr(), kz.data_ptr(), vb.data_ptr(), vp.data_ptr(),
                                                vo.data_ptr(), vs.data_ptr(), vz.data_ptr(), q.contiguous().data_ptr(),
                                                o.data_ptr(), lse.data_ptr() if lse is not None else None, tokens, D, Bq,
                                                int(num_key_value_groups), int(bit), 32 // int(bit), int(dequant_mode),
                                                group_size, ws.data_ptr(), ws.numel()), "mstf_decode_attention_quant")
    return o


def decode_attention_window_quant(key_side, value_side, q, k_win, v_win, win_len, num_key_value_groups, bit,
                                  dequant_mode=0, out=None, lse=None, win_len_dev=None, ws=None):
    """The whole attention of a decode step over [quantised compressed tokens | dense window] in three launches
    (ops.decode_attention_window for the quantised format).  key_side / value_side may be None while nothing is
    compressed yet.  k_win, v_win: [Bkv, stride, 128] fp16, the first win_len tokens valid; win_len_dev: optional
    int32 device scalar with the valid length (for replay from a captured graph)."""
    def five(side):
        return side if len(side) == 5 else (side[0], side[1], side[2], side[5], side[6])
    D = q.shape[-1]
    Bq = q.numel() // D
    L = lib()
    o = torch.empty((Bq, D), dtype=torch.float16, device=q.device) if out is None else out
    if key_side is not None:
        kb, ko, kp, ks, kz = five(key_side)
        vb, vo, vp, vs, vz = five(value_side)
        tokens = kb.shape[1] * 64 // D
        if _group_size(kb, ks, kz) != 64 or _group_size(vb, vs, vz) != 64:
            raise RuntimeError("the window entry point reads one scale / zero pair per tile (group_size 64).")
        ptrs = [kb.data_ptr(), kp.data_ptr(), ko.data_ptr(), ks.data_ptr(), kz.data_ptr(), vb.data_ptr(), vp.data_ptr(),
                vo.data_ptr(), vs.data_ptr(), vz.data_ptr()]
    else:
        tokens, ptrs = 0, [None] * 10
    ws = ops.workspace(q.device, L.mstf_decode_attention_window_workspace_bytes(tokens, int(win_len), D, Bq,
                                                                                int(num_key_value_groups)), ws)
    check(L.mstf_decode_attention_window_quant(
        torch.cuda.current_stream().cuda_stream, *ptrs, q.contiguous().data_ptr(), k_win.data_ptr(), v_win.data_ptr(),
        int(win_len), win_len_dev.data_ptr() if win_len_dev is not None else None, int(k_win.shape[1]), o.data_ptr(),
        lse.data_ptr() if lse is not None else None, tokens, D, Bq, int(num_key_value_groups), int(bit), 32 // int(bit),
        int(dequant_mode), ws.data_ptr(), ws.numel()), "mstf_decode_attention_window_quant")
    return o


def decode_attention_window_quant_pool(k_pool, v_pool, q, k_win, v_win, win_len, num_key_value_groups, dequant_mode=0,
                                       out=None, lse=None, win_len_dev=None, ws=None):
    """decode_attention_window_quant over two cache.QuantPool sides that grow in place: the pools' pre-allocated
    per-tile arrays are read with their row stride and the number of compressed tokens comes from the pool's device
    counter, so nothing about the call changes when a chunk is appended (a HIP graph holding it stays valid)."""
    assert q.dtype == torch.float16 and q.is_contiguous()
    assert k_win.dtype == torch.float16 and k_win.is_contiguous() and v_win.is_contiguous() and k_win.shape == v_win.shape
    assert k_pool.max_tokens == v_pool.max_tokens and k_pool.bit == v_pool.bit
    D = q.shape[-1]
    Bq = q.numel() // D
    L = lib()
    o = torch.empty((Bq, D), dtype=torch.float16, device=q.device) if out is None else out
    ws = ops.workspace(q.device, L.mstf_decode_attention_window_workspace_bytes(k_pool.max_tokens, int(win_len), D, Bq,
                                                                                int(num_key_value_groups)), ws)
    ptrs = []
    for p in (k_pool, v_pool):
        ptrs += [p.bmp_store.data_ptr(), p.packed.data_ptr(), p.off_store.data_ptr(), p.scales_store.data_ptr(),
                 p.zeros_store.data_ptr()]
    bit = int(k_pool.bit)
    check(L.mstf_decode_attention_window_quant_pool(
        torch.cuda.current_stream().cuda_stream, *ptrs, q.data_ptr(), k_win.data_ptr(), v_win.data_ptr(), int(win_len),
        win_len_dev.data_ptr() if win_len_dev is not None else None, int(k_win.shape[1]), o.data_ptr(),
        lse.data_ptr() if lse is not None else None, k_pool.max_tokens, k_pool.tokens_dev.data_ptr(),
        k_pool.tile_capacity, D, Bq, int(num_key_value_groups), bit, 32 // bit, int(dequant_mode), ws.data_ptr(),
        ws.numel()), "mstf_decode_attention_window_quant_pool")
    return o


def decode_step_quant_pool(k_pool, v_pool, q_in, k_in, v_in, k_win, v_win, win_len, cos=None, sin=None, dequant_mode=0,
                           win_len_dev=None, overflow=None, out=None, lse=None, ws=None):
    """ops.decode_step_pool over two cache.QuantPool sides (mstf_decode_step_quant_pool): ops.window_append followed
    by decode_attention_window_quant_pool, bit for bit, in two launches - rotation of the new query / key heads,
    append of the new rows to the window and the attention over the window run inside the launch of the compressed
    tokens.  Arguments as for ops.decode_step_pool."""
    D = k_win.shape[-1]
    bs = k_in.shape[0]
    n_kv, n_q = k_in.shape[-1] // D, q_in.shape[-1] // D
    for t in (q_in, k_in, v_in):
        assert t.dtype == torch.float16 and t.dim() == 2 and t.stride(1) == 1 and t.shape[0] == bs
    assert k_win.dtype == torch.float16 and k_win.is_contiguous() and v_win.is_contiguous() and k_win.shape == v_win.shape
    assert k_win.shape[0] == bs * n_kv and v_in.shape[-1] == n_kv * D and n_q % n_kv == 0
    assert k_pool.max_tokens == v_pool.max_tokens and k_pool.bit == v_pool.bit
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
    ws = ops.workspace(q_in.device, L.mstf_decode_attention_window_workspace_bytes(k_pool.max_tokens, int(win_len), D, Bq,
                                                                                   n_q // n_kv), ws)
    ptrs = []
    for p in (k_pool, v_pool):
        ptrs += [p.bmp_store.data_ptr(), p.packed.data_ptr(), p.off_store.data_ptr(), p.scales_store.data_ptr(),
                 p.zeros_store.data_ptr()]
    bit = int(k_pool.bit)
    check(L.mstf_decode_step_quant_pool(
        torch.cuda.current_stream().cuda_stream, *ptrs, q_in.data_ptr(), q_in.stride(0), k_in.data_ptr(), k_in.stride(0),
        v_in.data_ptr(), v_in.stride(0), bs, n_q, n_kv, cos.data_ptr() if cos is not None else None,
        sin.data_ptr() if sin is not None else None, rope_stride, k_win.data_ptr(), v_win.data_ptr(), k_win.shape[1],
        int(win_len), win_len_dev.data_ptr() if win_len_dev is not None else None,
        overflow.data_ptr() if overflow is not None else None, o.data_ptr(), lse.data_ptr() if lse is not None else None,
        k_pool.max_tokens, k_pool.tokens_dev.data_ptr(), k_pool.tile_capacity, D, bit, 32 // bit, int(dequant_mode),
        ws.data_ptr(), ws.numel()), "mstf_decode_step_quant_pool")
    return o


# aliases the reference exports for its model code (pybind_quant.cpp:96-176)
mustafar_quant_sparse_forward = mustafar_key_formulation_quant
mustafar_quant_sparse_forward_meta = mustafar_key_formulation_quant_meta
mustafar_quant_sparse_value_forward = mustafar_value_formulation_quant
mustafar_quant_sparse_value_forward_decode_n1 = mustafar_value_formulation_quant_decode_n1
