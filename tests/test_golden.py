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
