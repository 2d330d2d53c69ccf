"""The HIP path, through the C ABI, against the committed known-answer fixtures (tests/golden/*.npz): bit-exact for
pruned rows, bitmaps, offsets and packed values (fp16 and quantised), 2e-3 / 1e-2 for the attention results."""
import os

import numpy as np
import pytest
import torch

from _metrics import check_chain, rel_err   # row metric and element-wise allclose(rtol, atol = rtol * rms) in one number

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def gpu_f16(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.float16)).to("cuda:0")


def bits(t):
    return t.cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("fused_prune", [True, False])
def test_compress_reproduces_the_fixture(fused_prune):
    from mustafar_amd import ops
    g = load("kat_fp16.npz")
    kth = int(g["kth"])
    for src, pruned, pre, is_value in (("K", "Kp", "k", False), ("V", "Vp", "v", True)):
        x = gpu_f16(g[src])
        xp = ops.prune_rows(x.view(-1, 128), kth).view(x.shape)
        assert np.array_equal(bits(xp), g[pruned])
        c = ops.compress(x, is_value, kth=kth) if fused_prune else ops.compress(gpu_f16(g[pruned]), is_value, kth=0)
        assert np.array_equal(c.bmp.cpu().numpy(), g[pre + "_bmp"])
        assert np.array_equal(c.idx.cpu().numpy(), g[pre + "_idx"])
        assert np.array_equal(c.nz_off.cpu().numpy(), g[pre + "_nz_off"])
        assert np.array_equal(bits(c.packed()), g[pre + "_nz"])


def test_attention_reproduces_the_fixture():
    from mustafar_amd import ops
    g = load("kat_attention.npz")
    kth, groups = int(g["kth"]), int(g["groups"])
    q = gpu_f16(g["q"])
    Bq, D = q.shape
    want_s, want_p, want_o = (g[n].view(np.float16) for n in ("scores", "probs", "out"))
    ck = ops.compress(gpu_f16(g["K"]), False, kth=kth)
    cv = ops.compress(gpu_f16(g["V"]), True, kth=kth)
    s = ops.key_spmv(ck, q.view(Bq, 1, D), groups)
    p = ops.scale_softmax(s, D)
    o = ops.value_spmv(cv, p, groups)
    Vp = ops.prune_rows(gpu_f16(g["V"]).view(-1, 128), kth).view(-1, want_s.shape[1], 128).cpu().numpy()
    check_chain(2e-3, want_s, want_p, want_o, Vp, groups, s=s[:, 0], p=p[:, 0], o=o[:, 0],
                fused=ops.decode_attention(ck, cv, q, groups))


@pytest.mark.parametrize("bit", [2, 4])
def test_quant_producer_reproduces_the_fixture(bit):
    from mustafar_amd import compression_quant as cq
    g, want = load("kat_fp16.npz"), load("kat_quant.npz")
    names = ["bmp", "tile_off", "packed", "counts", "units", "scales", "zeros"]
    for pruned, pre, is_value in (("Kp", "k", False), ("Vp", "v", True)):
        x = gpu_f16(g[pruned])
        got = cq.convert_value_batched_quant(x, bit=bit) if is_value else \
            cq.convert_key_batched_quant(x, return_metadata=True, bit=bit)
        for name, t in zip(names, got):
            a = t.cpu().numpy()
            a = a.view(np.uint16) if a.dtype == np.float16 else a
            assert np.array_equal(a, want["%s%d_%s" % (pre, bit, name)]), name


# Fixtures written by the reference's own Triton producers (tests/golden/make_ref_fixtures.py, Triton interpreter on
# CPU tensors): the HIP producers must reproduce every array bit for bit.
REF_CASES = [("kat_k", "Kp", False), ("kat_v", "Vp", True), ("rnd_k", None, False), ("rnd_v", None, True)]


def _ref_input(r, pruned):
    return gpu_f16(load("kat_fp16.npz")[pruned]) if pruned else gpu_f16(r["rnd_x"])


@pytest.mark.parametrize("case,pruned,is_value", REF_CASES)
def test_quant_producer_matches_reference_triton_programs(case, pruned, is_value):
    from mustafar_amd import compression_quant as cq
    rq = load("ref_quant.npz")
    x = _ref_input(rq, pruned)
    got = cq.convert_value_batched_quant(x) if is_value else cq.convert_key_batched_quant(x, return_metadata=True)
    for name, t in zip(["bmp", "tile_off", "packed", "counts", "units", "scales", "zeros"], got):
        a = t.cpu().numpy()
        a = a.view(np.uint16) if a.dtype == np.float16 else a
        assert np.array_equal(a, rq["%s_%s" % (case, name)]), name


@pytest.mark.parametrize("case,pruned,is_value", REF_CASES)
def test_fp16_producer_matches_reference_triton_programs(case, pruned, is_value):
    from mustafar_amd import compression as cf
    rf = load("ref_fp16.npz")
    x = _ref_input(rf, pruned)
    bmp, idx, nzs = cf.convert_value_batched(x) if is_value else cf.convert_key_batched(x)
    assert np.array_equal(bmp.cpu().numpy(), rf[case + "_bmp"])
    assert np.array_equal(idx.cpu().numpy(), rf[case + "_idx"])
    assert np.array_equal(np.concatenate([bits(t) for t in nzs]), rf[case + "_nz"])
