"""Fused decode attention (one launch) against the oracle's dense masked attention and against the
three-launch path, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc

from _metrics import check_chain, rel_err   # row metric and element-wise allclose(rtol, atol = rtol * rms) in one number

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("groups,Bkv,Lc,sparsity", [(4, 2, 1024, 0.7), (4, 3, 64, 0.7), (1, 4, 576, 0.5),
                                                    (8, 1, 1536, 0.7), (2, 2, 512, 0.9), (4, 1, 4096, 0.7)])
def test_fused_decode_attention(groups, Bkv, Lc, sparsity):
    from mustafar_amd import ops
    dev = torch.device("cuda:0")
    D = 128
    Bq = Bkv * groups
    kth = orc.kth_from_sparsity(sparsity, D)
    K, V = orc.make_kv(900 + Lc + groups, Bkv, Lc, D)
    q = np.random.default_rng(Lc + groups).standard_normal((Bq, D)).astype(np.float16)
    Kp, Vp = orc.prune_rows(K, kth), orc.prune_rows(V, kth)
    sc_ref, pr_ref, out_ref = orc.dense_masked_attention(q, Kp, Vp, groups)
    ck = ops.compress(torch.from_numpy(K).to(dev), False, kth=kth)
    cv = ops.compress(torch.from_numpy(V).to(dev), True, kth=kth)
    qg = torch.from_numpy(q).to(dev)
    lse = torch.empty((Bq, 2), dtype=torch.float32, device=dev)
    o = ops.decode_attention(ck, cv, qg, groups, lse=lse)
    s = ops.key_spmv(ck, qg.view(Bq, 1, D), groups)
    check_chain(2e-3, sc_ref, pr_ref, out_ref, Vp, groups, s=s[:, 0], fused=o)
    o2 = ops.decode_attention(ck, cv, qg, groups)            # route without (max, sum) output
    check_chain(2e-3, sc_ref, pr_ref, out_ref, Vp, groups, s=s[:, 0], fused=o2)
    # (max, sum) against the oracle's scaled scores
    w = (sc_ref.astype(np.float32) / np.float32(np.sqrt(128.0))).astype(np.float16).astype(np.float32)
    m_ref = w.max(-1)
    l_ref = np.exp(w - m_ref[:, None]).sum(-1)
    got = lse.cpu().numpy()
    assert np.abs(got[:, 0] - m_ref).max() <= 2e-2 * np.maximum(np.abs(m_ref).max(), 1)
    assert np.abs(got[:, 1] * np.exp(got[:, 0] - m_ref) - l_ref).max() <= 5e-3 * l_ref.max()
    # and against the three-launch path
    p = ops.scale_softmax(s, D)
    o3 = ops.value_spmv(cv, p, groups)
    assert rel_err(o.cpu().numpy(), o3.cpu().numpy()[:, 0]) < 2e-3


def test_partial_then_merge_equals_fused():
    from mustafar_amd import ops
    dev = torch.device("cuda:0")
    D, groups, Bkv, Lc = 128, 4, 2, 1600
    Bq = Bkv * groups
    kth = orc.kth_from_sparsity(0.7, D)
    K, V = orc.make_kv(77, Bkv, Lc, D)
    ck = ops.compress(torch.from_numpy(K).to(dev), False, kth=kth)
    cv = ops.compress(torch.from_numpy(V).to(dev), True, kth=kth)
    qg = torch.from_numpy(np.random.default_rng(3).standard_normal((Bq, D)).astype(np.float16)).to(dev)
    lse = torch.empty((Bq, 2), dtype=torch.float32, device=dev)
    lse2 = torch.empty_like(lse)
    o = ops.decode_attention(ck, cv, qg, groups, lse=lse)
    ws = ops.decode_attention_partial(ck, cv, qg, groups)
    o2 = ops.decode_attention_merge(ws, Lc, D, Bq, groups, lse=lse2)
    assert torch.equal(o, o2) and torch.equal(lse, lse2)
    # the splits themselves: (max, sum, un-normalised output) of every 512-token range, combined on the host
    from mustafar_amd._lib import lib
    ns = lib().mstf_decode_attention_splits(Lc, D, Bq, groups)
    assert ns == (Lc // 64 + 7) // 8   # few blocks: 512 tokens per split
    raw = ws[: Bq * ns * (D + 2) * 4].view(torch.float32).cpu().numpy()
    po = raw[: Bq * ns * D].reshape(Bq, ns, D).astype(np.float64)
    ml = raw[Bq * ns * D:].reshape(Bq, ns, 2).astype(np.float64)
    M = ml[:, :, 0].max(1, keepdims=True)
    f = np.exp(ml[:, :, 0] - M)
    host = (f[:, :, None] * po).sum(1) / (f * ml[:, :, 1]).sum(1, keepdims=True)
    assert rel_err(o.cpu().numpy(), host) < 1e-3


@pytest.mark.parametrize("groups,Bkv,Lc,Lw", [(4, 2, 512, 300), (8, 1, 256, 64), (1, 3, 0, 257), (4, 2, 0, 1), (2, 2, 1024, 511)])
def test_decode_attention_with_dense_window(groups, Bkv, Lc, Lw):
    """Compressed tokens and dense window under one softmax against the oracle's dense masked attention over
    [pruned compressed part | window]; Lc = 0 is the window alone."""
    from mustafar_amd import ops
    dev = torch.device("cuda:0")
    D = 128
    Bq = Bkv * groups
    kth = orc.kth_from_sparsity(0.7, D)
    K, V = orc.make_kv(300 + Lc + Lw + groups, Bkv, Lc + Lw, D)
    q = np.random.default_rng(Lw).standard_normal((Bq, D)).astype(np.float16)
    Kf, Vf = K.copy(), V.copy()
    ck = cv = None
    if Lc > 0:
        Kf[:, :Lc] = orc.prune_rows(np.ascontiguousarray(K[:, :Lc]), kth)
        Vf[:, :Lc] = orc.prune_rows(np.ascontiguousarray(V[:, :Lc]), kth)
        ck = ops.compress(torch.from_numpy(np.ascontiguousarray(K[:, :Lc])).to(dev), False, kth=kth)
        cv = ops.compress(torch.from_numpy(np.ascontiguousarray(V[:, :Lc])).to(dev), True, kth=kth)
    sc_ref, _, out_ref = orc.dense_masked_attention(q, Kf, Vf, groups)
    cap = Lw + 37                                   # a buffer longer than the window, rows beyond it poisoned
    kw = torch.full((Bkv, cap, D), float("nan"), dtype=torch.float16, device=dev)
    vw = torch.full((Bkv, cap, D), float("nan"), dtype=torch.float16, device=dev)
    kw[:, :Lw] = torch.from_numpy(np.ascontiguousarray(K[:, Lc:])).to(dev)
    vw[:, :Lw] = torch.from_numpy(np.ascontiguousarray(V[:, Lc:])).to(dev)
    lse = torch.empty((Bq, 2), dtype=torch.float32, device=dev)
    o = ops.decode_attention_window(ck, cv, torch.from_numpy(q).to(dev), kw, vw, Lw, groups, lse=lse)
    assert rel_err(o.cpu().numpy(), out_ref) < 2e-3
    # the same with the length read on the device and the launch sized for the whole buffer
    wl = torch.tensor([Lw], dtype=torch.int32, device=dev)
    o_dev = ops.decode_attention_window(ck, cv, torch.from_numpy(q).to(dev), kw, vw, cap, groups, win_len_dev=wl)
    assert torch.equal(o_dev, o)
    w = (sc_ref.astype(np.float32) / np.float32(np.sqrt(128.0))).astype(np.float16).astype(np.float32)
    m_ref = w.max(-1)
    got = lse.cpu().numpy()
    assert np.abs(got[:, 0] - m_ref).max() <= 2e-2 * np.maximum(np.abs(m_ref).max(), 1)
    l_ref = np.exp(w - m_ref[:, None]).sum(-1)
    assert np.abs(got[:, 1] * np.exp(got[:, 0] - m_ref) - l_ref).max() <= 5e-3 * l_ref.max()


def test_fused_rejects_bad_arguments():
    from mustafar_amd._lib import lib
    L = lib()
    z = torch.zeros(1024, dtype=torch.int64, device="cuda:0")
    a = z.data_ptr()
    args = (a, a, a, a, a, a, a, a, a, a, None)
    assert L.mstf_decode_attention_f16(None, *args, 64, 128, 4, 4, None, 0) == -4
    assert L.mstf_decode_attention_f16(None, *args, 64, 64, 4, 4, a, 1 << 13) == -3
    assert L.mstf_decode_attention_f16(None, *args, 100, 128, 4, 4, a, 1 << 13) == -3
    assert L.mstf_decode_attention_f16(None, *args, 64, 128, 5, 4, a, 1 << 13) == -1
    assert L.mstf_decode_attention_workspace_bytes(4096, 128, 256, 4) == 256 * 8 * 130 * 4
    assert L.mstf_decode_attention_partial_f16(None, *args[:9], 64, 128, 4, 4, None, 0) == -4
    assert L.mstf_decode_attention_window_f16(None, *args[:9], a, a, 0, None, 8, a, None, 64, 128, 4, 4, a, 1 << 20) == -1
    assert L.mstf_decode_attention_window_f16(None, *args[:9], a, a, 9, None, 8, a, None, 64, 128, 4, 4, a, 1 << 20) == -1
    assert L.mstf_decode_attention_window_f16(None, *args[:9], a, a, 8, None, 8, a, None, 64, 128, 4, 4, a, 16) == -4
    assert L.mstf_decode_attention_window_workspace_bytes(4096, 512, 128, 256, 4) == 256 * 16 * 130 * 4
    assert L.mstf_decode_attention_merge_f16(None, a, 1 << 13, None, None, 64, 128, 4, 4) == -1
    assert L.mstf_decode_attention_merge_f16(None, a, 16, a, None, 64, 128, 4, 4) == -4


@pytest.mark.parametrize("groups,Bkv,held,capacity,Lw", [(4, 2, 512, 1024, 300), (2, 3, 0, 512, 70), (8, 1, 1024, 1024, 1)])
def test_pooled_entry_point_reads_a_cache_that_is_allocated_for_more(groups, Bkv, held, capacity, Lw):
    """mstf_decode_attention_window_pool_f16 (row stride of the per-tile arrays = capacity, token count read from device
    memory) against mstf_decode_attention_window_f16 on contiguous copies of the same cache: identical bit for bit,
    with the cache partly filled, empty and full."""
    from mustafar_amd import ops
    from mustafar_amd.cache import CompressedPool
    dev = torch.device("cuda:0")
    D = 128
    Bq = Bkv * groups
    K, V = orc.make_kv(400 + held + Lw, Bkv, max(held, 64) + Lw, D)
    kp, vp = CompressedPool(Bkv, D, capacity, False, dev), CompressedPool(Bkv, D, capacity, True, dev)
    Kt, Vt = torch.from_numpy(K).to(dev), torch.from_numpy(V).to(dev)
    for s in range(0, held, 256):                          # grown chunk by chunk, in place
        kp.append(Kt[:, s:s + 256], 89)
        vp.append(Vt[:, s:s + 256], 89)
    assert kp.tokens == held and int(kp.tokens_dev) == held
    q = torch.from_numpy(np.random.default_rng(Lw).standard_normal((Bq, D)).astype(np.float16)).to(dev)
    cap = Lw + 5
    kw = torch.full((Bkv, cap, D), float("nan"), dtype=torch.float16, device=dev)
    vw = torch.full((Bkv, cap, D), float("nan"), dtype=torch.float16, device=dev)
    kw[:, :Lw] = Kt[:, max(held, 64):max(held, 64) + Lw]
    vw[:, :Lw] = Vt[:, max(held, 64):max(held, 64) + Lw]
    wl = torch.tensor([Lw], dtype=torch.int32, device=dev)
    got = ops.decode_attention_window_pool(kp, vp, q, kw, vw, cap, groups, wl)
    want = ops.decode_attention_window(kp.view() if held else None, vp.view() if held else None, q, kw, vw, cap, groups,
                                       win_len_dev=wl)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
