"""The oracle's rotary embedding (oracle.rope_rows) pinned on the CPU: against transformers' own
apply_rotary_pos_emb where that package is importable, against the same expression written with torch's
half-precision tensor operators, and against what the mathematics fixes."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc


def bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


def inputs(seed, shape, first_pos):
    x = np.random.default_rng(seed).standard_normal(shape).astype(np.float16)
    cos, sin = orc.rope_tables(np.arange(shape[-2]) + first_pos)
    return x, cos, sin


def test_rope_rows_equals_transformers_bit_for_bit():
    m = pytest.importorskip("transformers.models.llama.modeling_llama")
    x, cos, sin = inputs(1, (2, 3, 100, 128), 4000)
    ref = m.apply_rotary_pos_emb(torch.from_numpy(x), torch.from_numpy(x), torch.from_numpy(cos)[None],
                                 torch.from_numpy(sin)[None])[1].numpy()
    assert np.array_equal(bits(orc.rope_rows(x, cos, sin)), bits(ref))


def test_rope_rows_equals_the_half_precision_tensor_expression():
    x, cos, sin = inputs(2, (4, 77, 128), 0)
    xt, c, s = torch.from_numpy(x), torch.from_numpy(cos), torch.from_numpy(sin)
    rot = torch.cat((-xt[..., 64:], xt[..., :64]), dim=-1)
    ref = (xt * c) + (rot * s)
    assert ref.dtype == torch.float16
    assert np.array_equal(bits(orc.rope_rows(x, cos, sin)), bits(ref.numpy()))
    # a fused multiply-add would round differently somewhere in a sample of this size
    fused = (xt.double() * c.double() + rot.double() * s.double()).to(torch.float16)
    assert not np.array_equal(bits(fused.numpy()), bits(ref.numpy()))


def test_rope_rows_fixed_points_and_rotation():
    x, cos, sin = inputs(3, (5, 64, 128), 0)
    out = orc.rope_rows(x, cos, sin)
    assert np.array_equal(bits(out[:, 0]), bits(x[:, 0]))                       # position 0: cos 1, sin 0
    # a rotation of every (c, c + 64) pair: lengths are kept and the angle is position * inv_freq[c]
    a, b = x[..., :64].astype(np.float64), x[..., 64:].astype(np.float64)
    oa, ob = out[..., :64].astype(np.float64), out[..., 64:].astype(np.float64)
    assert np.allclose(np.hypot(oa, ob), np.hypot(a, b), rtol=0, atol=8e-3)
    inv = 1.0 / (500000.0 ** (np.arange(0, 128, 2) / 128.0))
    ang = np.arange(64)[:, None] * inv[None, :]
    assert np.allclose(oa, a * np.cos(ang) - b * np.sin(ang), atol=8e-3)
    assert np.allclose(ob, b * np.cos(ang) + a * np.sin(ang), atol=8e-3)
    # swapping the sign of the rotated half (a plausible slip) fails the check above
    wrong = a * np.cos(ang) + b * np.sin(ang)
    assert not np.allclose(oa, wrong, atol=8e-3)


def test_rope_tables_follow_the_llama_definition():
    cos, sin = orc.rope_tables(np.arange(300) + 17, 128, 500000.0)
    assert cos.dtype == np.float16 and cos.shape == (300, 128)
    assert np.array_equal(bits(cos[:, :64]), bits(cos[:, 64:])) and np.array_equal(bits(sin[:, :64]), bits(sin[:, 64:]))
    inv = 1.0 / (500000.0 ** (np.arange(0, 128, 2) / 128.0))
    ang = (np.arange(300) + 17)[:, None] * inv[None, :]
    assert np.abs(cos[:, :64].astype(np.float64) - np.cos(ang)).max() < 1.5e-3
    assert np.abs(sin[:, :64].astype(np.float64) - np.sin(ang)).max() < 1.5e-3
