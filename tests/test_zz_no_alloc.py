"""The entry point that allocates nothing (mstf_decode_attention_static_f16) against mstf_decode_attention_f16,
through the C ABI: same kernels on the library's own scratch buffer, so the results must be identical bit for bit.
Two calls in a row, the second on a smaller problem (the buffer keeps the first call's partials)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(seed, Bkv, groups, tokens):
    from mustafar_amd import ops
    from oracle import oracle as orc
    dev = torch.device("cuda:0")
    K, V = orc.make_kv(seed, Bkv, tokens, 128)
    q = torch.from_numpy(np.random.default_rng(seed).standard_normal((Bkv * groups, 128)).astype(np.float16)).to(dev)
    kth = orc.kth_from_sparsity(0.7, 128)
    ck = ops.compress(torch.from_numpy(K).to(dev), False, kth=kth)
    cv = ops.compress(torch.from_numpy(V).to(dev), True, kth=kth)
    return ck, cv, q


def test_static_entry_point_matches_the_workspace_form_twice():
    from mustafar_amd import ops
    big = _case(11, 4, 4, 2048)      # 4 splits per row
    small = _case(12, 2, 4, 576)     # 2 splits, the second one partly filled; fewer rows than the call before
    one = _case(13, 1, 2, 256)       # a single split: the kernel writes the final output itself
    for ck, cv, q in (big, small, one, big):
        Bq = q.shape[0]
        for with_lse in (False, True):
            lse_a = torch.zeros((Bq, 2), dtype=torch.float32, device=q.device) if with_lse else None
            lse_b = torch.zeros((Bq, 2), dtype=torch.float32, device=q.device) if with_lse else None
            want = ops.decode_attention(ck, cv, q, q.shape[0] // ck.heads, lse=lse_a)
            got = ops.decode_attention_static(ck, cv, q, q.shape[0] // ck.heads, lse=lse_b)
            torch.cuda.synchronize()
            assert torch.equal(got.view(torch.int16), want.view(torch.int16))
            if with_lse:
                assert torch.equal(lse_a, lse_b)


def test_static_entry_point_refuses_what_does_not_fit():
    from mustafar_amd import _lib
    L = _lib.lib()
    one = 256   # any non-null, aligned value: the size check comes before the pointers are used
    args = [None] + [one] * 10 + [None]
    assert L.mstf_decode_attention_static_f16(*args, 4096, 128, 1012, 4) == -6         # partials beyond 4 MiB
    assert L.mstf_decode_attention_static_f16(*args, 16384, 128, 256, 4) == -6
    assert b"scratch" in L.mstf_strerror(-6)
    assert L.mstf_decode_attention_static_f16(*args, 4096, 64, 256, 4) == -3           # head_dim
    assert L.mstf_decode_attention_static_f16(None, *([None] * 11), 4096, 128, 256, 4) == -1
