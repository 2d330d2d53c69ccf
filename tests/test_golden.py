"""The CPU oracle against the committed known-answer fixtures (tests/golden/*.npz, written by
tests/golden/make_fixtures.py, which cross-checks every array against a plain-numpy restatement of the format)."""
import os

import numpy as np
import pytest

from oracle import oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def f16(a):
    return np.ascontiguousarray(a).view(np.float16)


def u16(a):
    return np.ascontiguousarray(a).view(np.uint16)


def test_prune_and_compress_reproduce_the_fixture():
    g = load("kat_fp16.npz")
    kth = int(g["kth"])
    for src, pruned, pre, is_value in (("K", "Kp", "k", 0), ("V", "Vp", "v", 1)):
        xp = orc.prune_rows(f16(g[src]), kth)
        assert np.array_equal(u16(xp), g[pruned])
        bmp, idx, nz, off = orc.compress(xp, is_value)
        assert np.array_equal(bmp, g[pre + "_bmp"]) and np.array_equal(idx, g[pre + "_idx"])
        assert np.array_equal(off, g[pre + "_nz_off"]) and np.array_equal(u16(nz), g[pre + "_nz"])


def test_fixture_holds_the_edge_cases():
    g = load("kat_fp16.npz")
    for pre in ("k", "v"):
        pops = np.array([bin(int(w)).count("1") for w in g[pre + "_bmp"].view(np.uint64).ravel()])
        assert {0, 1, 64} <= set(pops.tolist())
        idx = g[pre + "_idx"].astype(np.int64)
        assert np.array_equal((idx[:, 1:] - idx[:, :-1]).ravel(), ((pops + 7) // 8) * 4)
    # ties at the threshold keep more than N - kth + 1 elements (row 2 of head 0 is all |1.0|)
    assert int((g["Kp"][0, 2] & 0x7FFF != 0).sum()) == 128


def test_attention_reproduces_the_fixture():
    g = load("kat_attention.npz")
    kth, groups = int(g["kth"]), int(g["groups"])
    Kp, Vp = orc.prune_rows(f16(g["K"]), kth), orc.prune_rows(f16(g["V"]), kth)
    s, p, o = orc.dense_masked_attention(f16(g["q"]), Kp, Vp, groups)
    for got, want in ((s, g["scores"]), (p, g["probs"]), (o, g["out"])):
        a, b = got.astype(np.float64), f16(want).astype(np.float64)
        assert (np.abs(a - b).max(-1) / np.abs(b).max(-1)).max() < 1e-3   # same arithmetic, another build of the oracle
    # the sparse operators of the oracle on the compressed form give the same scores and output
    kb, ki, knz, koff = orc.compress(Kp, 0)
    vb, vi, vnz, voff = orc.compress(Vp, 1)
    Bq, L, D = f16(g["q"]).shape[0], Kp.shape[1], Kp.shape[2]
    C, _ = orc.key_spmv(kb, knz, ki, koff, f16(g["q"]).reshape(Bq, 1, D), L, D, groups)
    assert np.array_equal(u16(C[:, 0]), u16(s))


@pytest.mark.parametrize("bit", [2, 4])
def test_quant_producer_reproduces_the_fixture(bit):
    g, q = load("kat_fp16.npz"), load("kat_quant.npz")
    for pruned, pre, is_value in (("Kp", "k", 0), ("Vp", "v", 1)):
        got = orc.compress_quant(f16(g[pruned]), is_value, bit)
        names = ["bmp", "tile_off", "packed", "counts", "units", "scales", "zeros"]
        for name, a in zip(names, got):
            want = q["%s%d_%s" % (pre, bit, name)]
            a = u16(a) if a.dtype == np.float16 else a
            assert np.array_equal(a, want), name


# ------------------------------------------------------------------ fixtures written by the reference's own programs
# ref_quant.npz / ref_fp16.npz come from tests/golden/make_ref_fixtures.py: the reference's @triton.jit producers
# (kernel_quant/compression_quant.py:7-157, 267-422; kernel/compression.py:8-247) executed by Triton's interpreter
# on CPU tensors.  They pin the intermediate precision of scale / zero (tl.min / tl.max widen fp16 to fp32, so the
# whole chain runs in fp32 and is rounded once on the store) and the packed codes, bit for bit.
REF_CASES = [("kat_k", "Kp", 0), ("kat_v", "Vp", 1), ("rnd_k", None, 0), ("rnd_v", None, 1)]


def _ref_input(rq, pruned):
    return f16(load("kat_fp16.npz")[pruned]) if pruned else f16(rq["rnd_x"])


@pytest.mark.parametrize("case,pruned,is_value", REF_CASES)
def test_quant_producer_matches_reference_triton_programs(case, pruned, is_value):
    rq = load("ref_quant.npz")
    x = _ref_input(rq, pruned)
    got = orc.compress_quant(x, is_value, 2)
    for name, a in zip(["bmp", "tile_off", "packed", "counts", "units", "scales", "zeros"], got):
        a = u16(a) if a.dtype == np.float16 else a
        assert np.array_equal(a, rq["%s_%s" % (case, name)]), name


@pytest.mark.parametrize("case,pruned,is_value", REF_CASES)
def test_fp16_producer_matches_reference_triton_programs(case, pruned, is_value):
    rf = load("ref_fp16.npz")
    x = _ref_input(rf, pruned)
    bmp, idx, nz, off = orc.compress(x, is_value)
    assert np.array_equal(bmp, rf[case + "_bmp"]) and np.array_equal(idx, rf[case + "_idx"])
    assert np.array_equal(u16(nz), rf[case + "_nz"])
    # nz_off is the caller's running total in 16-byte units (models/llama_mustafar_kernel.py:450-452)
    assert np.array_equal(off, np.concatenate([[0], np.cumsum(idx[:-1, -1] // 4)]))


def test_reference_fixture_separates_the_candidate_precisions():
    """The fixture must be able to tell an fp16 chain from the fp32 one: a fair share of its tiles round differently."""
    rq = load("ref_quant.npz")
    x = f16(rq["rnd_x"])
    n_diff = n = 0
    for b in range(x.shape[0]):
        for t in range(x.shape[1]):
            for h in range(2):
                v = x[b, t, h * 64:(h + 1) * 64]
                v = v[v != 0]
                if v.size < 2 or not np.isfinite(np.float16(v.max() - v.min())):
                    continue
                chain16 = np.float16(np.float16(v.max() - v.min()) / np.float16(3))
                once32 = np.float16((np.float32(v.max()) - np.float32(v.min())) / np.float32(3))
                n += 1
                n_diff += chain16 != once32
    assert n > 300 and n_diff > 0.1 * n
