"""The two error metrics every floating-point parity test holds the HIP path to, folded into one number.

    row metric     : max|a - b| / max|b|                      per row (last axis)
    element metric : |a - b| / (rms(b) + |b|)                 per element, rms over the row

`rel_err(a, b) < tol` holds exactly when the row metric is below tol for every row AND
numpy.allclose(a, b, rtol=tol, atol=tol * rms(b)) holds element by element - the relative error of an element is
ill-defined near zero, hence the absolute term scaled by the row's own magnitude.  tol is 2e-3 for the fp16 path and
1e-2 for the quantised one.
"""
import numpy as np


def _np(x):
    if hasattr(x, "detach"):
        x = x.detach().float().cpu().numpy()
    return np.asarray(x, dtype=np.float64)


def row_err(a, b):
    a, b = _np(a), _np(b)
    return float((np.abs(a - b).max(-1) / np.maximum(np.abs(b).max(-1), 1e-30)).max())


def elem_err(a, b):
    a, b = _np(a), _np(b)
    rms = np.sqrt((b * b).mean(-1, keepdims=True))
    return float((np.abs(a - b) / np.maximum(rms + np.abs(b), 1e-30)).max())


def rel_err(a, b):
    return max(row_err(a, b), elem_err(a, b))


# ------------------------------------------------------------------ composed results
# The reference rounds the raw scores q.K^T to fp16 before the softmax.  Two correct implementations that add the
# products in different orders round a few scores (about one in a thousand) to neighbouring fp16 values; one ulp of a
# score of a few hundred (outlier channels) is 0.25, i.e. 2 % of that token's probability.  Such a flip is within the
# score tolerance but moves individual probabilities and output elements by more than 2e-3.  The composed results are
# therefore held to two things: the row metric against the end-to-end oracle, and BOTH metrics against the oracle
# continued from the scores the GPU produced (which are themselves held to both metrics against the oracle's scores).
def continue_from_scores(s16, Vp, groups, head_dim=128):
    """Oracle softmax and value product on given fp16 scores [Bq, L]; Vp [Bkv, L, D] pruned (or dequantised) values.
    Returns (probabilities fp16 [Bq, L], output fp16 [Bq, D])."""
    from oracle import oracle as orc
    s16 = np.ascontiguousarray(s16, dtype=np.float16)
    p = orc.scale_softmax(s16, head_dim)
    return p, value_product(p, Vp, groups)


def value_product(p16, Vp, groups):
    """fp32-accumulated P.V rounded to fp16, query row bq reading KV head bq // groups."""
    p = np.asarray(p16, dtype=np.float32)
    Bq, L = p.shape
    V = np.asarray(Vp, dtype=np.float32)
    o = np.einsum("bgl,bld->bgd", p.reshape(V.shape[0], groups, L), V, dtype=np.float32)
    return o.reshape(Bq, -1).astype(np.float16)


def check_chain(tol, s_ref, p_ref, o_ref, Vp, groups, s=None, p=None, o=None, fused=None, head_dim=128):
    """s, p, o: the three-launch results [Bq, L] / [Bq, L] / [Bq, D]; fused: the one-launch output; any may be None
    (fused needs s).  *_ref: the oracle's dense masked attention end to end."""
    if s is not None:
        assert rel_err(s, s_ref) < tol, ("scores", row_err(s, s_ref), elem_err(s, s_ref))
    p_cont = o_cont = None
    if s is not None:
        p_cont, o_cont = continue_from_scores(_np(s).astype(np.float16), Vp, groups, head_dim)
    if p is not None:
        assert row_err(p, p_ref) < tol, ("probabilities, end to end", row_err(p, p_ref))
        assert rel_err(p, p_cont) < tol, ("probabilities from the same scores", row_err(p, p_cont), elem_err(p, p_cont))
    if o is not None:
        assert row_err(o, o_ref) < tol, ("output, end to end", row_err(o, o_ref))
        want = value_product(_np(p).astype(np.float16), Vp, groups) if p is not None else o_cont
        assert rel_err(o, want) < tol, ("output from the same probabilities", row_err(o, want), elem_err(o, want))
    if fused is not None:
        assert row_err(fused, o_ref) < tol, ("fused output, end to end", row_err(fused, o_ref))
        assert rel_err(fused, o_cont) < tol, ("fused output from the same scores", row_err(fused, o_cont),
                                              elem_err(fused, o_cont))
