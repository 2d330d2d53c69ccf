"""GPU parity of the fp16 path against the CPU oracle, through the C ABI.

Bit-exact: pruning, bitmaps, tile offsets, nz_off, packed values (incl. +0.0 padding).
Within 2e-3 (relative to the row maximum): key scores, probabilities, value outputs.
"""
import numpy as np
import pytest
import torch

from oracle import oracle as orc

from _metrics import check_chain, rel_err   # row metric and element-wise allclose(rtol, atol = rtol * rms) in one number

pytestmark = pytest.mark.gpu

RTOL = 2e-3  # fp16 tolerance of the north-star metric


def dev():
    return torch.device("cuda:0")


def to_gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev())


def special_inputs(seed, B, M, D=128):
    """Seeded K/V plus the edge cases the format has: exact ties at the threshold, an all-equal
    row, rows with many zeros, a full key tile (outlier channel) and an empty key tile."""
    K, V = orc.make_kv(seed, B, M, D)
    K[0, 1, :] = np.float16(0.75)                    # all-equal row: everything kept
    K[0, 2, :64] = np.float16(1.0)
    K[0, 2, 64:] = np.float16(-1.0)                  # |x| ties everywhere
    K[0, 3, 5:120] = 0                               # more zeros than the pruning rank
    V[0, 4, :] = 0                                   # an all-zero token
    V[0, 5, 40:90] = np.float16(-0.0)
    if B > 1:
        K[1, :, 9] = 0                               # empty key tiles (channel never survives)
        V[1, 7, :] = np.float16(3.0)
    return K, V


@pytest.mark.parametrize("kth", [64, 89, 115, 1, 128])
def test_prune_rows_bit_exact(kth):
    from mustafar_amd import ops
    K, V = special_inputs(5, 2, 192)
    x = np.concatenate([K.reshape(-1, 128), V.reshape(-1, 128)])[:700]   # not a multiple of 64 rows
    y = ops.prune_rows(to_gpu(x), kth).cpu().numpy()
    ref = orc.prune_rows(x, kth)
    assert np.array_equal(y.view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("is_value", [0, 1])
@pytest.mark.parametrize("kth", [0, 64, 89, 115])
def test_compress_bit_exact(is_value, kth):
    from mustafar_amd import ops
    K, V = special_inputs(7 + kth, 3, 256)
    x = V if is_value else K
    if kth == 0:
        x = orc.prune_rows(x, 89)
        xp = x
    else:
        xp = orc.prune_rows(x, kth)
    rb, ri, rnz, roff = orc.compress(xp, is_value)
    ck = ops.compress(to_gpu(x), bool(is_value), kth=kth)
    assert np.array_equal(ck.bmp.cpu().numpy(), rb)
    assert np.array_equal(ck.idx.cpu().numpy(), ri)
    assert np.array_equal(ck.nz_off.cpu().numpy(), roff)
    assert int(ck.total_halfs) == rnz.size
    assert np.array_equal(ck.packed().cpu().numpy().view(np.uint16), rnz.view(np.uint16))


@pytest.mark.parametrize("is_value", [0, 1])
def test_compress_with_capacity_is_async_and_guarded(is_value):
    from mustafar_amd import ops
    K, V = special_inputs(3, 2, 128)
    x = V if is_value else K
    rb, ri, rnz, roff = orc.compress(orc.prune_rows(x, 89), is_value)
    # ample capacity: identical prefix
    ck = ops.compress(to_gpu(x), bool(is_value), kth=89, capacity_halfs=rnz.size + 4096)
    assert int(ck.total_halfs.item()) == rnz.size
    assert np.array_equal(ck.nz.cpu().numpy()[:rnz.size].view(np.uint16), rnz.view(np.uint16))
    # too small: the reported total still says what is needed and nothing is written past the end
    cap = rnz.size // 2 // 8 * 8
    ck2 = ops.compress(to_gpu(x), bool(is_value), kth=89, capacity_halfs=cap)
    assert int(ck2.total_halfs.item()) == rnz.size
    assert ck2.nz.numel() == cap


def test_reference_api_convert_and_formulation():
    """The drop-in modules: same signatures, shapes, dtypes and the caller's glue (torch.cat of the
    per-batch lists, nz_offset rule) as models/llama_mustafar_kernel.py:394-396,434-436,545-557."""
    from mustafar_amd import compression, mustafar_package
    groups, Bkv, Lc, D = 4, 2, 256, 128
    Bq = Bkv * groups
    K, V = special_inputs(11, Bkv, Lc)
    Kp, Vp = orc.prune_rows(K, 89), orc.prune_rows(V, 89)
    k_bmps, k_idxs, k_nzs = compression.convert_key_batched(to_gpu(Kp))
    v_bmps, v_idxs, v_nzs = compression.convert_value_batched(to_gpu(Vp))
    rb, ri, rnz, roff = orc.compress(Kp, 0)
    assert k_bmps.dtype == torch.int64 and tuple(k_bmps.shape) == (Bkv, Lc * D // 64)
    assert k_idxs.dtype == torch.int32 and tuple(k_idxs.shape) == (Bkv, Lc * D // 64 + 1)
    assert isinstance(k_nzs, list) and len(k_nzs) == Bkv
    assert [t.numel() for t in k_nzs] == [2 * int(ri[b, -1]) for b in range(Bkv)]
    assert np.array_equal(torch.cat(k_nzs).cpu().numpy().view(np.uint16), rnz.view(np.uint16))
    k_off = torch.zeros(Bkv, dtype=torch.int32, device=dev())
    v_off = torch.zeros(Bkv, dtype=torch.int32, device=dev())
    for i in range(1, Bkv):
        k_off[i] = k_off[i - 1] + k_idxs[i - 1][-1] // 4
        v_off[i] = v_off[i - 1] + v_idxs[i - 1][-1] // 4
    assert np.array_equal(k_off.cpu().numpy(), roff)
    assert np.array_equal(compression.nz_offsets(k_idxs).cpu().numpy(), roff)

    rng = np.random.default_rng(0)
    q = rng.standard_normal((Bq, 1, D)).astype(np.float16)
    padded_query = torch.nn.functional.pad(to_gpu(q), (0, 0, 0, 7))
    padded_query[:, 5] = to_gpu(rng.standard_normal((Bq, D)).astype(np.float16))   # a live padded row
    att = mustafar_package.mustafar_key_formulation(k_bmps, torch.cat(k_nzs), k_idxs, k_off, padded_query, Lc, D, Bq,
                                                    groups)
    assert tuple(att.shape) == (Bq, 8, Lc) and att.dtype == torch.float16
    C, Cf = orc.key_spmv(rb, rnz, ri, roff, padded_query.cpu().numpy(), Lc, D, groups)
    assert rel_err(att.cpu().numpy(), Cf) < RTOL
    assert not att[:, 1].any()          # zero query rows give zero scores

    P = orc.scale_softmax(C[:, 0], D)
    padded_score = torch.nn.functional.pad(to_gpu(P).view(Bq, 1, Lc), (0, 0, 0, 7)).contiguous()
    ws = torch.zeros(1, dtype=torch.float16, device=dev())
    out = mustafar_package.mustafar_value_formulation(v_bmps, torch.cat(v_nzs), v_idxs, v_off, padded_score, ws, D, Lc,
                                                      Bq, groups)
    assert tuple(out.shape) == (Bq, 8, D)
    vb, vi, vnz, voff = orc.compress(Vp, 1)
    O, Of = orc.value_spmv(vb, vnz, vi, voff, padded_score.cpu().numpy(), D, Lc, groups)
    assert rel_err(out.cpu().numpy()[:, 0], Of[:, 0]) < RTOL
    assert not out[:, 1:].any()

    with pytest.raises(RuntimeError):
        mustafar_package.mustafar_key_formulation(k_bmps.to(torch.int32), torch.cat(k_nzs), k_idxs, k_off,
                                                  padded_query, Lc, D, Bq, groups)
    with pytest.raises(RuntimeError):
        mustafar_package.mustafar_key_formulation(k_bmps, torch.cat(k_nzs).float(), k_idxs, k_off, padded_query, Lc,
                                                  D, Bq, groups)
    with pytest.raises(RuntimeError):
        mustafar_package.mustafar_key_formulation(k_bmps.cpu(), torch.cat(k_nzs), k_idxs, k_off, padded_query, Lc, D,
                                                  Bq, groups)


@pytest.mark.parametrize("groups,Bkv,Lc,sparsity", [(1, 4, 512, 0.7), (4, 2, 1024, 0.7), (4, 2, 512, 0.5),
                                                    (8, 1, 256, 0.9), (2, 3, 64, 0.7)])
def test_decode_attention_against_dense_masked_oracle(groups, Bkv, Lc, sparsity):
    """compress -> key SpMV -> scale+softmax -> value SpMV on the GPU against the dense masked
    attention of the oracle on the same seeded inputs (one new query token per head)."""
    from mustafar_amd import ops
    D = 128
    Bq = Bkv * groups
    kth = orc.kth_from_sparsity(sparsity, D)
    K, V = orc.make_kv(100 + Lc + groups, Bkv, Lc, D)
    rng = np.random.default_rng(Lc)
    q = rng.standard_normal((Bq, D)).astype(np.float16)
    Kp, Vp = orc.prune_rows(K, kth), orc.prune_rows(V, kth)
    sc_ref, pr_ref, out_ref = orc.dense_masked_attention(q, Kp, Vp, groups)

    ck = ops.compress(to_gpu(K), False, kth=kth)
    cv = ops.compress(to_gpu(V), True, kth=kth)
    s = ops.key_spmv(ck, to_gpu(q).view(Bq, 1, D), groups)
    p = ops.scale_softmax(s, D)
    o = ops.value_spmv(cv, p, groups)
    check_chain(RTOL, sc_ref, pr_ref, out_ref, Vp, groups, s=s[:, 0], p=p[:, 0], o=o[:, 0])
    # and each product separately against the fp32 sums of the oracle fed the same inputs
    kb = orc.compress(Kp, 0)
    _, Cf = orc.key_spmv(kb[0], kb[2], kb[1], kb[3], q.reshape(Bq, 1, D), Lc, D, groups)
    assert rel_err(s.cpu().numpy(), Cf) < 1e-3
    vb = orc.compress(Vp, 1)
    _, Of = orc.value_spmv(vb[0], vb[2], vb[1], vb[3], pr_ref.reshape(Bq, 1, Lc), D, Lc, groups)
    o2 = ops.value_spmv(cv, to_gpu(pr_ref).view(Bq, 1, Lc), groups)
    assert rel_err(o2.cpu().numpy(), Of) < 1e-3


def test_softmax_strided_and_inplace():
    from mustafar_amd import ops
    rng = np.random.default_rng(1)
    s = (rng.standard_normal((6, 1000)) * 20).astype(np.float16)
    ref = orc.scale_softmax(s, 128)
    g = to_gpu(s)
    p = ops.scale_softmax(g, 128)
    assert rel_err(p.cpu().numpy(), ref) < 1e-3
    big = torch.zeros((6, 1200), dtype=torch.float16, device=dev())
    big[:, :1000] = g
    view = big[:, :1000]
    ops.scale_softmax(view, 128, out=view)      # strided rows, in place
    assert rel_err(view.cpu().numpy(), ref) < 1e-3


def test_special_bitmaps():
    """All-zero cache -> zero scores/outputs; a single non-zero; an identity query picks a channel."""
    from mustafar_amd import ops
    D, Lc, groups = 128, 128, 2
    z = torch.zeros((1, Lc, D), dtype=torch.float16, device=dev())
    ck = ops.compress(z, False, kth=0)
    cv = ops.compress(z, True, kth=0)
    assert int(ck.total_halfs) == 0 and not ck.bmp.any() and not ck.idx.any()
    q = torch.ones((groups, 1, D), dtype=torch.float16, device=dev())
    assert not ops.key_spmv(ck, q, groups).any()
    p = torch.ones((groups, 1, Lc), dtype=torch.float16, device=dev())
    assert not ops.value_spmv(cv, p, groups).any()
    one = z.clone()
    one[0, 77, 33] = 2.5
    ck1 = ops.compress(one, False, kth=0)
    s = ops.key_spmv(ck1, q, groups)
    assert s[0, 0, 77] == 2.5 and s.sum() == 2.5 * groups
    K, _ = orc.make_kv(2, 1, Lc)
    Kp = orc.prune_rows(K, 89)
    ck2 = ops.compress(to_gpu(Kp), False, kth=0)
    e = torch.zeros((groups, 1, D), dtype=torch.float16, device=dev())
    e[:, 0, 17] = 1
    s2 = ops.key_spmv(ck2, e, groups).cpu().numpy()
    want = np.where(Kp[0, :, 17] != 0, Kp[0, :, 17], np.float16(0))
    assert np.array_equal(s2[0, 0], want) and np.array_equal(s2[1, 0], want)


def test_c_abi_rejects_bad_arguments():
    """Host-forcible failure paths: error code, no launch."""
    from mustafar_amd._lib import lib
    L = lib()
    x = torch.zeros((1, 64, 128), dtype=torch.float16, device=dev())
    bmp = torch.zeros(128, dtype=torch.int64, device=dev())
    idx = torch.zeros(129, dtype=torch.int32, device=dev())
    off = torch.zeros(1, dtype=torch.int32, device=dev())
    q = torch.zeros((1, 1, 128), dtype=torch.float16, device=dev())
    C = torch.zeros((1, 1, 64), dtype=torch.float16, device=dev())
    nz = torch.zeros(64, dtype=torch.float16, device=dev())
    a = (bmp.data_ptr(), nz.data_ptr(), idx.data_ptr(), off.data_ptr(), q.data_ptr(), C.data_ptr())
    assert L.mstf_key_spmv_f16(None, *a, 64, 128, 1, 1, 1) == 0
    assert L.mstf_key_spmv_f16(None, None, *a[1:], 64, 128, 1, 1, 1) == -1          # null pointer
    assert L.mstf_key_spmv_f16(None, *a, 100, 128, 1, 1, 1) == -3                    # tokens % 64
    assert L.mstf_key_spmv_f16(None, *a, 64, 128, 3, 2, 1) == -1                     # Bq % groups
    assert L.mstf_key_spmv_f16(None, a[0], a[1] + 2, *a[2:], 64, 128, 1, 1, 1) == -2  # nz not 16-byte aligned
    assert L.mstf_value_spmv_f16(None, *a, 128, 4096, 8, 4, 1, None, 0) == -4        # workspace missing
    assert L.mstf_prune_rows_f16(None, x.data_ptr(), x.data_ptr(), 64, 96, 10) == -3  # head_dim
    assert L.mstf_prune_rows_f16(None, x.data_ptr(), x.data_ptr(), 64, 128, 0) == -1  # kth
    tot = torch.zeros(1, dtype=torch.int64, device=dev())
    assert L.mstf_compress_key_f16(None, x.data_ptr(), 1, 64, 128, 0, bmp.data_ptr(), idx.data_ptr(), off.data_ptr(),
                                   tot.data_ptr(), None, 0, None, 0) == -4
    assert b"workspace" in L.mstf_strerror(-4)
    torch.cuda.synchronize()


def test_config0_shape_against_oracle():
    """The reference's CPU-runnable case: batch 1, 32 heads (MHA), head_dim 128, 4096 tokens, K with 4 outlier
    channels per head, 70 % pruning on K and V, one query token.  Formats bit-exact against the oracle at the full
    size; raw scores, probabilities and attention output against its dense masked attention."""
    from mustafar_amd import ops
    heads, L, D, groups = 32, 4096, 128, 1
    kth = orc.kth_from_sparsity(0.7, D)
    K, V = orc.make_kv(0, heads, L, D)
    q = np.random.default_rng(1).standard_normal((heads, D)).astype(np.float16)
    Kp, Vp = orc.prune_rows(K, kth), orc.prune_rows(V, kth)
    s_ref, p_ref, o_ref = orc.dense_masked_attention(q, Kp, Vp, groups)
    ck = ops.compress(to_gpu(K), False, kth=kth)
    cv = ops.compress(to_gpu(V), True, kth=kth)
    for c, xp, is_value in ((ck, Kp, 0), (cv, Vp, 1)):
        rb, ri, rnz, roff = orc.compress(xp, is_value)
        assert np.array_equal(c.bmp.cpu().numpy(), rb) and np.array_equal(c.idx.cpu().numpy(), ri)
        assert np.array_equal(c.nz_off.cpu().numpy(), roff)
        assert np.array_equal(c.packed().cpu().numpy().view(np.uint16), rnz.view(np.uint16))
    qg = to_gpu(q)
    s = ops.key_spmv(ck, qg.view(heads, 1, D), groups)
    p = ops.scale_softmax(s, D)
    o = ops.value_spmv(cv, p, groups)
    check_chain(RTOL, s_ref, p_ref, o_ref, Vp, groups, s=s[:, 0], p=p[:, 0], o=o[:, 0],
                fused=ops.decode_attention(ck, cv, qg, groups))


@pytest.fixture
def no_polls():
    """Forces the one-pass producers' bounded waits to zero polls from the host (every kernel still runs to its end);
    the default comes back afterwards."""
    from mustafar_amd._lib import lib
    lib().mstf_test_set_spin_limit(0)
    yield
    lib().mstf_test_set_spin_limit(-1)


def test_one_pass_compressor_flags_a_wait_that_ran_out(no_polls):
    """The one-pass compressor orders its workgroups through status words and bounds every wait.  With the bound forced
    to zero polls from the host, a workgroup whose predecessors have not published yet gives up: then the total must
    read as all ones whichever workgroup it was (and the host layer must raise), otherwise everything must be exactly
    right - never a silently wrong result."""
    from mustafar_amd import ops
    from mustafar_amd._lib import lib
    dev = torch.device("cuda:0")
    K, _ = orc.make_kv(31, 16, 1024, 128)
    Kt = torch.from_numpy(K).to(dev)
    rb, ri, rnz, roff = orc.compress(orc.prune_rows(K, 89), 0)
    for _ in range(4):
        ck = ops.compress(Kt, False, kth=89, capacity_halfs=Kt.numel())
        torch.cuda.synchronize()
        if int(ck.total_halfs) == -1:
            with pytest.raises(RuntimeError, match="gave up"):
                ck.packed()
        else:
            assert int(ck.total_halfs) == rnz.size
            assert np.array_equal(ck.bmp.cpu().numpy(), rb) and np.array_equal(ck.idx.cpu().numpy(), ri)
            assert np.array_equal(ck.packed().cpu().numpy().view(np.uint16), rnz.view(np.uint16))
    lib().mstf_test_set_spin_limit(-1)
    ck = ops.compress(Kt, False, kth=89, capacity_halfs=Kt.numel())
    assert int(ck.total_halfs) == rnz.size
    assert np.array_equal(ck.packed().cpu().numpy().view(np.uint16), rnz.view(np.uint16))


def test_append_flags_a_wait_that_ran_out(no_polls):
    """The pooled append has no total to carry the marker: a workgroup that gives up sets bit 1 of the flag word and
    the pool raises; an append that is not flagged is exact."""
    from mustafar_amd.cache import CompressedPool
    dev = torch.device("cuda:0")
    heads, M, D = 16, 1024, 128
    K, _ = orc.make_kv(32, heads, M, D)
    Kt = torch.from_numpy(K).to(dev)
    rb, ri, rnz, roff = orc.compress(orc.prune_rows(K, 89), 0)
    for _ in range(4):
        pool = CompressedPool(heads, D, M, False, dev)
        try:
            pool.append(Kt, 89)
        except RuntimeError as e:
            assert "gave up" in str(e) and int(pool.overflow) & 2
            continue
        assert int(pool.overflow) == 0
        assert np.array_equal(pool.bmp.cpu().numpy(), rb) and np.array_equal(pool.idx.cpu().numpy(), ri)
        for b in range(heads):
            want = rnz[8 * int(roff[b]):8 * int(roff[b]) + 2 * int(ri[b, -1])]
            assert np.array_equal(pool.head_values(b).cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_quantised_producer_flags_a_wait_that_ran_out(no_polls):
    from mustafar_amd import compression_quant as cq
    dev = torch.device("cuda:0")
    _, V = orc.make_kv(33, 16, 1024, 128)
    Vp = orc.prune_rows(V, 89)
    ref = orc.compress_quant(Vp, 1, 2)
    Vt = torch.from_numpy(Vp).to(dev)
    for gs in (64, 32):
        for _ in range(3):
            out = cq._produce(Vt, True, 2, 0, gs)
            total = out[-1]
            torch.cuda.synchronize()
            if int(total) == -1:
                with pytest.raises(RuntimeError, match="gave up"):
                    cq.words_written(total)
            elif gs == 64:
                n = cq.words_written(total)
                assert np.array_equal(out[2][:n].cpu().numpy().view(np.uint32), ref[2].view(np.uint32))


@pytest.mark.parametrize("B,M,kth_k,kth_v", [(3, 256, 89, 89), (2, 128, 38, 115), (5, 64, 0, 64), (1, 1024, 128, 1),
                                              (16, 512, 89, 89)])
def test_keys_and_values_in_one_launch_equal_the_two_calls(B, M, kth_k, kth_v):
    """mstf_compress_kv_f16 against mstf_compress_key_f16 + mstf_compress_value_f16 (one-pass form): bitmaps, offsets,
    nz_off, totals and packed values bit for bit, for 4, 2 and 1 units per workgroup, kth = 0 (input already pruned),
    1 and 128."""
    from mustafar_amd import ops
    D = 128
    K, V = orc.make_kv(77 + B * M, B, M, D)
    if kth_k == 0:
        K = orc.prune_rows(K, 89)
    Kt, Vt = torch.from_numpy(K).to("cuda:0"), torch.from_numpy(V).to("cuda:0")
    ck, cv = ops.compress_kv(Kt, Vt, kth_k, kth_v)
    for got, x, is_value, kth in ((ck, Kt, False, kth_k), (cv, Vt, True, kth_v)):
        ref = ops.compress(x, is_value, kth=kth, capacity_halfs=x.numel())
        n = int(ref.total_halfs)
        assert int(got.total_halfs) == n
        assert torch.equal(got.bmp, ref.bmp) and torch.equal(got.idx, ref.idx) and torch.equal(got.nz_off, ref.nz_off)
        assert torch.equal(got.nz[:n].view(torch.int16), ref.nz[:n].view(torch.int16))
