"""GPU parity of the quantised path (2- and 4-bit) against the CPU oracle, through the C ABI.

Bit-exact against the oracle: bitmaps, raw counts, units, global tile offsets, fp16 scales / zeros
and the packed codes (the oracle evaluates the reference's closed forms in fp32 and rounds once;
parity with the Triton original's intermediate precision is not pinned by any reference fixture).
Within 1e-2 (relative to the row maximum): quantised key / value products against the dense masked
attention on the dequantised cache, and against the fp32 sums of the oracle.
"""
import numpy as np
import pytest
import torch

from oracle import oracle as orc

from _metrics import check_chain, rel_err   # row metric and element-wise allclose(rtol, atol = rtol * rms) in one number

pytestmark = pytest.mark.gpu

QTOL = 1e-2  # tolerance of the north-star metric for 4-bit and 2-bit non-zeros


def dev():
    return torch.device("cuda:0")


def to_gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev())


def pruned(seed, B, M, kth=89):
    K, V = orc.make_kv(seed, B, M)
    K[0, :64, 7] = 0          # an empty key tile
    V[0, 3, :] = 0            # empty value tiles
    K[0, 64:128, 11] = np.float16(1.25)   # a constant tile: scale falls back to 1
    return orc.prune_rows(K, kth), orc.prune_rows(V, kth)


@pytest.mark.parametrize("group_size", [64, 32])
@pytest.mark.parametrize("bit", [2, 4])
@pytest.mark.parametrize("is_value", [0, 1])
def test_quant_compress_bit_exact(bit, is_value, group_size):
    from mustafar_amd import compression_quant as cq
    Kp, Vp = pruned(31 + bit, 3, 256)
    x = Vp if is_value else Kp
    if group_size == 32:
        x[1, 70, 64:96] = 0                       # a value tile whose first group is empty
        x[2, 64:96, 20] = 0                       # a key tile whose first group is empty
        x[2, 128:160, 21] = np.float16(-3.5)      # a group of equal survivors
    ref = orc.compress_quant(x, is_value, bit, group_size)
    if is_value:
        got = cq.convert_value_batched_quant(to_gpu(x), bit=bit, group_size=group_size)
    else:
        got = cq.convert_key_batched_quant(to_gpu(x), return_metadata=True, bit=bit, group_size=group_size)
        short = cq.convert_key_batched_quant(to_gpu(x), bit=bit, group_size=group_size)
        assert len(short) == 5
    assert tuple(got[5].shape) == ((3, 512) if group_size == 64 else (3, 512, 2))
    names = ["bitmaps", "tile_offsets", "packed", "counts", "units", "scales", "zeros"]
    dtypes = [torch.int64, torch.int32, torch.int32, torch.int32, torch.int32, torch.float16, torch.float16]
    for name, g, r, dt in zip(names, got, ref, dtypes):
        assert g.dtype == dt, name
        g = g.cpu().numpy()
        if g.dtype == np.float16:
            assert np.array_equal(g.view(np.uint16), r.view(np.uint16)), name
        else:
            assert np.array_equal(g, r), name


@pytest.mark.parametrize("bit", [2, 4])
@pytest.mark.parametrize("dequant_mode", [0, 1])
def test_quant_formulations_reference_api(bit, dequant_mode):
    """The drop-in operators with the reference's argument lists (models/llama_mustafar_quant_kernel.py:445-567)."""
    from mustafar_amd import compression_quant as cq, mustafar_package_quant as mq
    groups, Bkv, Lc, D = 4, 2, 256, 128
    Bq = Bkv * groups
    cap = 32 // bit
    Kp, Vp = pruned(41, Bkv, Lc)
    kb, ko, kp, kc, ku, ks, kz = cq.convert_key_batched_quant(to_gpu(Kp), return_metadata=True, bit=bit)
    vb, vo, vp, vc, vu, vs, vz = cq.convert_value_batched_quant(to_gpu(Vp), bit=bit)
    rk = orc.compress_quant(Kp, 0, bit)
    rv = orc.compress_quant(Vp, 1, bit)
    rng = np.random.default_rng(3)
    q = rng.standard_normal((Bq, 1, D)).astype(np.float16)
    padded_query = torch.nn.functional.pad(to_gpu(q), (0, 0, 0, 7)).contiguous()
    att = mq.mustafar_key_formulation_quant(kb, kp, ko, ks, kz, padded_query, Lc, D, Bq, groups, bit, cap,
                                            dequant_mode=dequant_mode)
    att_meta = mq.mustafar_quant_sparse_forward_meta(kb, kp, ko, kc, ku, ks, kz, padded_query, Lc, D, Bq, groups, bit,
                                                     cap, dequant_mode)
    assert tuple(att.shape) == (Bq, 8, Lc) and att.dtype == torch.float16
    assert torch.equal(att, att_meta)
    C, Cf = orc.spmv_quant(rk[0], rk[2], rk[1], rk[5], rk[6], padded_query.cpu().numpy(), 0, Lc, D, groups, bit,
                           dequant_mode)
    assert rel_err(att.cpu().numpy()[:, 0], Cf[:, 0]) < 2e-3
    assert not att[:, 1:].any()

    P = orc.scale_softmax(C[:, 0], D)
    padded_score = torch.nn.functional.pad(to_gpu(P).view(Bq, 1, Lc), (0, 0, 0, 7)).contiguous()
    ws = torch.zeros(1, dtype=torch.float16, device=dev())
    out = mq.mustafar_value_formulation_quant(vb, vp, vo, vc, vu, vs, vz, padded_score, ws, D, Lc, Bq, groups, bit, cap,
                                              dequant_mode=dequant_mode, split_k=4, value_tile_config=1)
    assert tuple(out.shape) == (Bq, 8, D)
    O, Of = orc.spmv_quant(rv[0], rv[2], rv[1], rv[5], rv[6], padded_score.cpu().numpy(), 1, Lc, D, groups, bit,
                           dequant_mode)
    assert rel_err(out.cpu().numpy()[:, 0], Of[:, 0]) < 2e-3
    n1 = mq.mustafar_value_formulation_quant_decode_n1(vb, vp, vo, vc, vu, vs, vz, to_gpu(P), ws, D, Lc, Bq, groups,
                                                       bit, cap, dequant_mode)
    assert tuple(n1.shape) == (Bq, D)
    assert rel_err(n1.cpu().numpy(), Of[:, 0]) < 2e-3
    with pytest.raises(RuntimeError):
        mq.mustafar_key_formulation_quant(kb, kp, ko, ks.float(), kz, padded_query, Lc, D, Bq, groups, bit, cap)
    with pytest.raises(RuntimeError):   # capacity must be 32 // bit
        mq.mustafar_key_formulation_quant(kb, kp, ko, ks, kz, padded_query, Lc, D, Bq, groups, bit, cap + 1)


@pytest.mark.parametrize("group_size", [64, 32])
@pytest.mark.parametrize("bit", [2, 4])
@pytest.mark.parametrize("groups,Bkv,Lc", [(4, 2, 1024), (1, 3, 256), (8, 1, 512)])
def test_quant_decode_attention_against_dense_masked_oracle(bit, groups, Bkv, Lc, group_size):
    """Quantised compress -> key SpMV -> softmax -> value SpMV against the oracle's dense masked attention run
    on the dequantised cache (the reference semantics of the quantised path), one query token per head."""
    from mustafar_amd import compression_quant as cq, mustafar_package_quant as mq, ops
    D = 128
    Bq = Bkv * groups
    cap = 32 // bit
    K, V = orc.make_kv(500 + Lc + bit, Bkv, Lc, D)
    Kp, Vp = orc.prune_rows(K, 89), orc.prune_rows(V, 89)
    rk = orc.compress_quant(Kp, 0, bit, group_size)
    rv = orc.compress_quant(Vp, 1, bit, group_size)
    Kd = np.stack([orc.decode_quant(rk[0], rk[2], rk[1], rk[5], rk[6], b, Lc, D, 0, bit, 0) for b in range(Bkv)])
    Vd = np.stack([orc.decode_quant(rv[0], rv[2], rv[1], rv[5], rv[6], b, Lc, D, 1, bit, 0) for b in range(Bkv)])
    q = np.random.default_rng(Lc).standard_normal((Bq, D)).astype(np.float16)
    sc_ref, pr_ref, out_ref = orc.dense_masked_attention(q, Kd, Vd, groups)

    kb, ko, kp, kc, ku, ks, kz = cq.convert_key_batched_quant(to_gpu(Kp), return_metadata=True, bit=bit,
                                                              group_size=group_size)
    vb, vo, vp, vc, vu, vs, vz = cq.convert_value_batched_quant(to_gpu(Vp), bit=bit, group_size=group_size)
    L = __import__("mustafar_amd._lib", fromlist=["lib"]).lib()
    st = torch.cuda.current_stream().cuda_stream
    s = torch.empty((Bq, 1, Lc), dtype=torch.float16, device=dev())
    qg = to_gpu(q).view(Bq, 1, D)
    if group_size == 64:
        assert L.mstf_key_spmv_quant(st, kb.data_ptr(), kp.data_ptr(), ko.data_ptr(), None, None, ks.data_ptr(),
                                     kz.data_ptr(), qg.data_ptr(), s.data_ptr(), Lc, D, Bq, groups, 1, bit, cap, 0) == 0
    else:
        assert L.mstf_key_spmv_quant_grouped(st, kb.data_ptr(), kp.data_ptr(), ko.data_ptr(), ks.data_ptr(), kz.data_ptr(),
                                             qg.data_ptr(), s.data_ptr(), Lc, D, Bq, groups, 1, bit, cap, 0, 32) == 0
    p = ops.scale_softmax(s, D)
    o = mq.mustafar_value_formulation_quant_decode_n1(vb, vp, vo, vc, vu, vs, vz, p.view(Bq, Lc), None, D, Lc, Bq,
                                                      groups, bit, cap)
    check_chain(QTOL, sc_ref, pr_ref, out_ref, Vd, groups, s=s[:, 0], p=p[:, 0], o=o)
    # the quantisation itself stays within half a step of the fp16 cache
    err = np.abs(Kd.astype(np.float32) - np.where(Kp != 0, Kp, 0).astype(np.float32))
    if group_size == 64:
        step = np.repeat(rk[5].astype(np.float32).reshape(Bkv, Lc // 64, D), 64, axis=1)   # key tile = 64 tokens x 1 channel
    else:    # pair g of tile (block, channel) serves tokens 32g .. 32g+31 of the block
        step = np.repeat(rk[5].astype(np.float32).reshape(Bkv, Lc // 64, D, 2).transpose(0, 1, 3, 2).reshape(Bkv, Lc // 32, D),
                         32, axis=1)
    assert (err <= 0.5 * step * 1.01 + 2e-3 * np.abs(Kp.astype(np.float32)) + 1e-6).all()


@pytest.mark.parametrize("group_size", [64, 32])
@pytest.mark.parametrize("bit", [2, 4, 8])
@pytest.mark.parametrize("dequant_mode", [0, 1])
@pytest.mark.parametrize("kth", [89, 38])
def test_quant_dequantised_values_bit_exact(bit, dequant_mode, group_size, kth):
    """One-hot query rows / probability rows turn the SpMVs into a read-out of the dequantised cache: every
    output is a single product value * 1, so it must equal the oracle's decode bit for bit.  Some tiles sit far
    from zero (zero-point beyond +-1024), which takes the kernels' literal per-mode arithmetic.  kth 89: a stage
    holds a few tiles with more than 32 survivors (outlier channels, the full tiles set below), finished one by one;
    kth 38: most tiles have more than 32 and the stage takes the second half of the dequantisation."""
    from mustafar_amd import compression_quant as cq
    from mustafar_amd import mustafar_package_quant as mpq
    B, M, D, groups = 2, 128, 128, 4
    Kp, Vp = pruned(57 + bit, B, M, kth)
    k = np.arange(64)
    steps = {2: 3, 4: 10, 8: 64}[bit]          # spread chosen so that |zero| lands between 1024 and 8192
    Kp[1, :64, 5] = (300.0 + (k % steps) * (0.25 if bit < 8 else 0.5)).astype(np.float16)     # zero << -1024
    Kp[1, 64:, 9] = (-90.0 - (k % {2: 4, 4: 16, 8: 64}[bit]) * 0.0625).astype(np.float16)     # zero >> 1024
    Vp[1, 7, :64] = (512.0 + (k % steps) * 0.5).astype(np.float16)
    Bq = B * groups
    for is_value, x in ((0, Kp), (1, Vp)):
        ref = orc.compress_quant(x, is_value, bit, group_size)
        assert np.abs(ref[6].astype(np.float32)).max() > 1024      # the slow path is exercised
        dense = np.stack([orc.decode_quant(ref[0], ref[2], ref[1], ref[5], ref[6], b, M, D, is_value, bit, dequant_mode)
                          for b in range(B)])                      # [B, M, D]
        g = [to_gpu(a) for a in ref]
        if not is_value:
            # query row n of head h selects channel 8*h + n (+ 32 per pass): four passes cover 128 channels
            for base in range(0, D, 32):
                q = np.zeros((Bq, 8, D), np.float16)
                for h in range(groups):
                    for n in range(8):
                        q[h::groups, n, base + 8 * h + n] = 1
                out = mpq.mustafar_key_formulation_quant_meta(g[0], g[2], g[1], g[3], g[4], g[5], g[6], to_gpu(q), M, D,
                                                              Bq, groups, bit, 32 // bit, dequant_mode).cpu().numpy()
                for h in range(groups):
                    for n in range(8):
                        for b in range(B):
                            got = out[b * groups + h, n].view(np.uint16)
                            want = dense[b, :, base + 8 * h + n].view(np.uint16)
                            # +0 and -0 are the same value: an absent element is +0 here, -0 after decode of a pruned -x
                            assert np.array_equal(got & ((got != 0x8000) * 0xFFFF), want & ((want != 0x8000) * 0xFFFF))
        else:
            for base in range(0, M, 32):
                pr = np.zeros((Bq, 8, M), np.float16)
                for h in range(groups):
                    for n in range(8):
                        pr[h::groups, n, base + 8 * h + n] = 1
                out = mpq.mustafar_value_formulation_quant(g[0], g[2], g[1], g[3], g[4], g[5], g[6], to_gpu(pr), None, D, M,
                                                           Bq, groups, bit, 32 // bit, dequant_mode).cpu().numpy()
                for h in range(groups):
                    for n in range(8):
                        for b in range(B):
                            got = out[b * groups + h, n].view(np.uint16)
                            want = dense[b, base + 8 * h + n, :].view(np.uint16)
                            assert np.array_equal(got & ((got != 0x8000) * 0xFFFF), want & ((want != 0x8000) * 0xFFFF))


@pytest.mark.parametrize("group_size", [64, 32])
@pytest.mark.parametrize("bit", [2, 4, 8])
@pytest.mark.parametrize("groups,Bkv,Lc", [(4, 2, 1024), (8, 1, 576), (1, 3, 64)])
def test_fused_quant_decode_attention(bit, groups, Bkv, Lc, group_size):
    """The one-launch path against dense masked attention on the dequantised cache (1e-2) and against the
    three-launch quantised path (same dequantised values, so only the softmax rounding differs)."""
    from mustafar_amd import compression_quant as cq
    from mustafar_amd import mustafar_package_quant as mpq
    from mustafar_amd import ops
    D = 128
    Bq = Bkv * groups
    Kp, Vp = pruned(90 + bit + Lc, Bkv, Lc)
    kq = cq.convert_key_batched_quant(to_gpu(Kp), return_metadata=True, bit=bit, group_size=group_size)
    vq = cq.convert_value_batched_quant(to_gpu(Vp), bit=bit, group_size=group_size)
    kr = [t.cpu().numpy() for t in kq]
    vr = [t.cpu().numpy() for t in vq]
    Kd = np.stack([orc.decode_quant(kr[0], kr[2], kr[1], kr[5], kr[6], b, Lc, D, 0, bit) for b in range(Bkv)])
    Vd = np.stack([orc.decode_quant(vr[0], vr[2], vr[1], vr[5], vr[6], b, Lc, D, 1, bit) for b in range(Bkv)])
    q = np.random.default_rng(bit + Lc).standard_normal((Bq, D)).astype(np.float16)
    sc_ref, pr_ref, out_ref = orc.dense_masked_attention(q, Kd, Vd, groups)
    lse = torch.empty((Bq, 2), dtype=torch.float32, device=dev())
    o = mpq.decode_attention_quant(kq, vq, to_gpu(q), groups, bit, lse=lse)
    o2 = mpq.decode_attention_quant(kq, vq, to_gpu(q), groups, bit)
    assert torch.equal(o, o2) or rel_err(o2.cpu().numpy(), o.cpu().numpy()) < 1e-3
    # three-launch path
    qp = np.zeros((Bq, 8, D), np.float16)
    qp[:, 0] = q
    s = mpq.mustafar_key_formulation_quant_meta(kq[0], kq[2], kq[1], kq[3], kq[4], kq[5], kq[6], to_gpu(qp), Lc, D, Bq,
                                                groups, bit, 32 // bit)[:, 0].contiguous()
    # the cache is the same dequantised one on both sides: fp16 accuracy, well inside the 1e-2 of the quantised path
    check_chain(2e-3, sc_ref, pr_ref, out_ref, Vd, groups, s=s, fused=o)
    p = ops.scale_softmax(s, D)
    o3 = mpq.mustafar_value_formulation_quant_decode_n1(vq[0], vq[2], vq[1], vq[3], vq[4], vq[5], vq[6], p, None, D, Lc,
                                                        Bq, groups, bit, 32 // bit)
    assert rel_err(o.cpu().numpy(), o3.cpu().numpy()) < 2e-3


def test_quant_c_abi_rejects_bad_arguments():
    from mustafar_amd._lib import lib
    L = lib()
    z = torch.zeros(256, dtype=torch.int64, device=dev())
    a = z.data_ptr()
    assert L.mstf_key_spmv_quant(None, a, a, a, None, None, a, a, a, a, 64, 128, 1, 1, 1, 3, 10, 0) == -3   # bit
    assert L.mstf_key_spmv_quant(None, a, a, a, None, None, a, a, a, a, 64, 128, 1, 1, 1, 2, 8, 0) == -1    # capacity
    assert L.mstf_key_spmv_quant(None, a, a, a, None, None, a, a, a, a, 64, 128, 1, 1, 1, 2, 16, 2) == -1   # mode
    assert L.mstf_key_spmv_quant(None, a, None, a, None, None, a, a, a, a, 64, 128, 1, 1, 1, 2, 16, 0) == -1
    assert L.mstf_compress_key_quant(None, a, 1, 64, 128, 0, 2, a, a, a, a, a, a, a, None, 0, None, 0) == -4


@pytest.mark.parametrize("bit,groups,Bkv,Lc,Lw", [(2, 4, 2, 512, 300), (4, 8, 1, 256, 64), (2, 1, 3, 0, 257),
                                                  (8, 2, 2, 1024, 511)])
def test_quant_decode_attention_with_dense_window(bit, groups, Bkv, Lc, Lw):
    """Quantised compressed tokens and dense window under one softmax (mstf_decode_attention_window_quant) against the
    oracle's dense masked attention over [dequantised compressed part | window]; Lc = 0 is the window alone."""
    from mustafar_amd import compression_quant as cq
    from mustafar_amd import mustafar_package_quant as mpq
    D = 128
    Bq = Bkv * groups
    K, V = orc.make_kv(700 + Lc + Lw + bit, Bkv, Lc + Lw, D)
    q = np.random.default_rng(Lw + bit).standard_normal((Bq, D)).astype(np.float16)
    Kf, Vf = K.copy(), V.copy()
    kq = vq = None
    if Lc > 0:
        Kp = orc.prune_rows(np.ascontiguousarray(K[:, :Lc]), 89)
        Vp = orc.prune_rows(np.ascontiguousarray(V[:, :Lc]), 89)
        kq = cq.convert_key_batched_quant(to_gpu(Kp), return_metadata=True, bit=bit)
        vq = cq.convert_value_batched_quant(to_gpu(Vp), bit=bit)
        kr = [t.cpu().numpy() for t in kq]
        vr = [t.cpu().numpy() for t in vq]
        Kf[:, :Lc] = np.stack([orc.decode_quant(kr[0], kr[2], kr[1], kr[5], kr[6], b, Lc, D, 0, bit) for b in range(Bkv)])
        Vf[:, :Lc] = np.stack([orc.decode_quant(vr[0], vr[2], vr[1], vr[5], vr[6], b, Lc, D, 1, bit) for b in range(Bkv)])
    _, _, out_ref = orc.dense_masked_attention(q, Kf, Vf, groups)
    cap = Lw + 21
    kw = torch.full((Bkv, cap, D), float("nan"), dtype=torch.float16, device=dev())
    vw = torch.full((Bkv, cap, D), float("nan"), dtype=torch.float16, device=dev())
    kw[:, :Lw] = to_gpu(K[:, Lc:])
    vw[:, :Lw] = to_gpu(V[:, Lc:])
    o = mpq.decode_attention_window_quant(kq, vq, to_gpu(q), kw, vw, Lw, groups, bit)
    assert rel_err(o.cpu().numpy(), out_ref) < QTOL
    wl = torch.tensor([Lw], dtype=torch.int32, device=dev())
    o_dev = mpq.decode_attention_window_quant(kq, vq, to_gpu(q), kw, vw, cap, groups, bit, win_len_dev=wl)
    assert torch.equal(o_dev, o)


@pytest.mark.parametrize("B,M,is_value", [(301, 128, 0), (77, 192, 1)])
def test_quant_compress_many_heads_and_sizing_only(B, M, is_value):
    """Hundreds of heads (the scan sums the unit totals of all earlier heads with vector loads and a tail) against
    the oracle, and the sizing-only call (packed == NULL), which must leave the same final tile offsets and total."""
    from mustafar_amd import compression_quant as cq, ops
    from mustafar_amd._lib import lib
    K, V = orc.make_kv(B + M, B, M)
    x = orc.prune_rows(V if is_value else K, 89)
    ref = orc.compress_quant(x, is_value, 2)
    fn = cq.convert_value_batched_quant if is_value else cq.convert_key_batched_quant
    got = fn(to_gpu(x), bit=2) if is_value else fn(to_gpu(x), return_metadata=True, bit=2)
    assert np.array_equal(got[0].cpu().numpy(), ref[0])
    assert np.array_equal(got[1].cpu().numpy(), ref[1].astype(np.int32))
    assert np.array_equal(got[2].cpu().numpy(), ref[2])
    # sizing only
    L = lib()
    xg = to_gpu(x)
    T = M * 128 // 64
    d = dev()
    bmp = torch.empty((B, T), dtype=torch.int64, device=d)
    toff = torch.empty((B, T), dtype=torch.int32, device=d)
    cnt, uni = torch.empty_like(toff), torch.empty_like(toff)
    sc = torch.empty((B, T), dtype=torch.float16, device=d)
    zp = torch.empty_like(sc)
    total = torch.zeros(1, dtype=torch.int64, device=d)
    ws = ops.workspace(d, L.mstf_compress_quant_workspace_bytes(B, M, 128))
    f = L.mstf_compress_value_quant if is_value else L.mstf_compress_key_quant
    rc = f(torch.cuda.current_stream().cuda_stream, xg.data_ptr(), B, M, 128, 0, 2, bmp.data_ptr(), toff.data_ptr(),
           cnt.data_ptr(), uni.data_ptr(), sc.data_ptr(), zp.data_ptr(), total.data_ptr(), None, 0, ws.data_ptr(), ws.numel())
    assert rc == 0
    assert int(total.item()) == ref[2].size
    assert np.array_equal(toff.cpu().numpy(), ref[1].astype(np.int32))
