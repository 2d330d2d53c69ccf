"""Seeded random shapes and contents through the C ABI against the CPU oracle: heads, token counts, pruning ranks,
query groups and input styles (dense normal, many exact zeros, few distinct magnitudes, constant rows) drawn from a
fixed seed per case.  Formats bit-exact, attention within 2e-3."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc

from _metrics import rel_err   # row metric and element-wise allclose(rtol, atol = rtol * rms) in one number

pytestmark = pytest.mark.gpu
D = 128


def to_gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


def draw(rng, B, M, style):
    x = rng.standard_normal((B, M, D)).astype(np.float32)
    if style == 1:      # many exact zeros (more than the pruning rank in many rows)
        x[rng.random((B, M, D)) < 0.8] = 0.0
    elif style == 2:    # few distinct magnitudes: ties at the threshold everywhere
        x = np.sign(x) * rng.integers(0, 4, (B, M, D)).astype(np.float32) * 0.5
    elif style == 3:    # constant rows mixed with normal ones, negative zeros
        x[:, ::3, :] = 0.25
        x[:, 1::7, :] = -0.0
    elif style == 4:    # wide dynamic range including fp16 subnormals
        x = x * np.exp2(rng.integers(-20, 8, (B, M, 1))).astype(np.float32)
    return x.astype(np.float16)


@pytest.mark.parametrize("seed", range(16))
def test_random_case(seed):
    from mustafar_amd import ops
    rng = np.random.default_rng(9000 + seed)
    groups = int(rng.choice([1, 2, 3, 4, 5, 8]))
    Bkv = int(rng.integers(1, 5))
    M = 64 * int(rng.integers(1, 13))
    kth_k = int(rng.choice([1, 38, 64, 89, 115, 127, 128]))
    kth_v = int(rng.choice([1, 64, 89, 115, 128]))
    K, V = draw(rng, Bkv, M, seed % 5), draw(rng, Bkv, M, (seed // 5) % 5)
    Kp, Vp = orc.prune_rows(K, kth_k), orc.prune_rows(V, kth_v)
    assert np.array_equal(ops.prune_rows(to_gpu(K).view(-1, D), kth_k).cpu().numpy().view(np.uint16).reshape(K.shape),
                          Kp.view(np.uint16))
    ck = ops.compress(to_gpu(K), False, kth=kth_k)
    cv = ops.compress(to_gpu(V), True, kth=kth_v)
    for c, xp, is_value in ((ck, Kp, 0), (cv, Vp, 1)):
        rb, ri, rnz, roff = orc.compress(xp, is_value)
        assert np.array_equal(c.bmp.cpu().numpy(), rb) and np.array_equal(c.idx.cpu().numpy(), ri)
        assert np.array_equal(c.nz_off.cpu().numpy(), roff) and int(c.total_halfs) == rnz.size
        assert np.array_equal(c.packed().cpu().numpy().view(np.uint16), rnz.view(np.uint16))
    # the same through the one-pass form (a value buffer given up front; 1, 2 or 4 units per workgroup by M / 64)
    for x, xp, is_value, kth in ((K, Kp, 0, kth_k), (V, Vp, 1, kth_v)):
        c1 = ops.compress(to_gpu(x), bool(is_value), kth=kth, capacity_halfs=x.size)
        rb, ri, rnz, roff = orc.compress(xp, is_value)
        assert np.array_equal(c1.bmp.cpu().numpy(), rb) and np.array_equal(c1.idx.cpu().numpy(), ri)
        assert np.array_equal(c1.nz_off.cpu().numpy(), roff) and int(c1.total_halfs) == rnz.size
        assert np.array_equal(c1.packed().cpu().numpy().view(np.uint16), rnz.view(np.uint16))
        c0 = ops.compress(to_gpu(xp), bool(is_value), kth=0, capacity_halfs=x.size)     # already pruned input
        assert np.array_equal(c0.bmp.cpu().numpy(), rb) and np.array_equal(c0.idx.cpu().numpy(), ri)
        assert np.array_equal(c0.packed().cpu().numpy().view(np.uint16), rnz.view(np.uint16))
    Bq = Bkv * groups
    q = rng.standard_normal((Bq, D)).astype(np.float16)
    s_ref, p_ref, o_ref = orc.dense_masked_attention(q, Kp, Vp, groups)
    qg = to_gpu(q)
    s = ops.key_spmv(ck, qg.view(Bq, 1, D), groups)
    assert rel_err(s.cpu().numpy()[:, 0], s_ref) < 2e-3 or np.abs(s_ref).max() == 0
    o = ops.decode_attention(ck, cv, qg, groups)
    o3 = ops.value_spmv(cv, ops.scale_softmax(s, D), groups)
    scale = max(np.abs(o_ref.astype(np.float64)).max(), 1e-30)
    assert np.abs(o.cpu().numpy().astype(np.float64) - o_ref).max() < 2e-3 * scale
    assert np.abs(o3.cpu().numpy()[:, 0].astype(np.float64) - o_ref).max() < 2e-3 * scale


@pytest.mark.parametrize("seed", range(8))
def test_random_case_quantised(seed):
    """The quantised producer bit-exact against the oracle, and the one-launch quantised attention against dense
    masked attention on the oracle's dequantised cache (1e-2), on the same kind of drawn inputs."""
    from mustafar_amd import compression_quant as cq
    from mustafar_amd import mustafar_package_quant as mpq
    rng = np.random.default_rng(9500 + seed)
    bit = int(rng.choice([2, 4, 8]))
    mode = int(rng.integers(0, 2))
    groups = int(rng.choice([1, 2, 4, 7, 8]))
    Bkv = int(rng.integers(1, 4))
    M = 64 * int(rng.integers(1, 9))
    kth = int(rng.choice([38, 64, 89, 115]))
    Kp = orc.prune_rows(draw(rng, Bkv, M, seed % 5), kth)
    Vp = orc.prune_rows(draw(rng, Bkv, M, (seed + 2) % 5), kth)
    kq = cq.convert_key_batched_quant(to_gpu(Kp), return_metadata=True, bit=bit)
    vq = cq.convert_value_batched_quant(to_gpu(Vp), bit=bit)
    for got, xp, is_value in ((kq, Kp, 0), (vq, Vp, 1)):
        for g, r in zip(got, orc.compress_quant(xp, is_value, bit)):
            g = g.cpu().numpy()
            if g.dtype == np.float16:
                assert np.array_equal(g.view(np.uint16), r.view(np.uint16))
            else:
                assert np.array_equal(g, r)
    kr = [t.cpu().numpy() for t in kq]
    vr = [t.cpu().numpy() for t in vq]
    Kd = np.stack([orc.decode_quant(kr[0], kr[2], kr[1], kr[5], kr[6], b, M, D, 0, bit, mode) for b in range(Bkv)])
    Vd = np.stack([orc.decode_quant(vr[0], vr[2], vr[1], vr[5], vr[6], b, M, D, 1, bit, mode) for b in range(Bkv)])
    q = rng.standard_normal((Bkv * groups, D)).astype(np.float16)
    _, _, o_ref = orc.dense_masked_attention(q, Kd, Vd, groups)
    o = mpq.decode_attention_quant(kq, vq, to_gpu(q), groups, bit, dequant_mode=mode)
    scale = max(np.abs(o_ref.astype(np.float64)).max(), 1e-30)
    assert np.abs(o.cpu().numpy().astype(np.float64) - o_ref).max() < 1e-2 * scale
