"""Size-independent properties at the headline size (batch 8 x 8 KV heads, 4096 tokens, 70 %), where the CPU
oracle would take minutes: the checker here is plain torch on the device - kthvalue pruning, fp32 matmuls - which
shares no code with the kernels under test.

  * format invariants of the compressed cache (padding rule, offsets, popcounts) and checksums of its content
    against the torch-pruned dense tensor;
  * fused and three-launch sparse decode attention against dense masked attention on the torch-pruned tensors,
    2e-3 relative to the row maximum (the north-star tolerance).
"""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

BKV, L, D, GROUPS, KTH = 64, 4096, 128, 4, 89


def popcount64(x):
    x = x.clone()
    c = torch.zeros_like(x)
    for _ in range(64):
        c += x & 1
        x = (x >> 1) & 0x7FFFFFFFFFFFFFFF
    return c


def torch_prune(x, kth):
    """x * (|x| >= kth-th smallest |x| of the row), models/llama_mustafar_kernel.py:194-232 restated with torch ops."""
    a = x.abs().float()
    thr = torch.kthvalue(a, kth, dim=-1, keepdim=True).values
    return torch.where(a >= thr, x, torch.zeros_like(x))


@pytest.fixture(scope="module")
def data():
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(4096)
    K = torch.randn((BKV, L, D), generator=g, device=dev).half()
    V = torch.randn((BKV, L, D), generator=g, device=dev).half()
    K[:, :, 5] *= 10
    K[:, :, 77] *= 10
    q = torch.randn((BKV * GROUPS, D), generator=g, device=dev).half()
    return K, V, q, torch_prune(K, KTH), torch_prune(V, KTH)


@pytest.mark.parametrize("is_value", [0, 1])
def test_format_invariants_and_checksums(data, is_value):
    from mustafar_amd import ops
    K, V, _, Kp, Vp = data
    x, xp = (V, Vp) if is_value else (K, Kp)
    c = ops.compress(x, bool(is_value), kth=KTH)
    T = L * D // 64
    assert c.bmp.shape == (BKV, T) and c.idx.shape == (BKV, T + 1)
    pop = popcount64(c.bmp)
    idx = c.idx.to(torch.int64)
    # every tile padded to a multiple of 8 values, offsets in 4-byte units, exclusive prefix
    assert torch.equal(idx[:, 1:] - idx[:, :-1], ((pop + 7) // 8) * 4)
    assert int(idx[:, 0].abs().sum()) == 0 and int((idx % 4).abs().sum()) == 0
    # head offsets in 16-byte units, heads back to back
    per_head = idx[:, -1] // 4
    assert torch.equal(c.nz_off.to(torch.int64)[1:], torch.cumsum(per_head, 0)[:-1]) and int(c.nz_off[0]) == 0
    assert int(c.total_halfs) == int(2 * idx[:, -1].sum())
    # the kept elements are exactly the torch-pruned ones: per-tile counts ...
    if is_value:
        tiles = xp.view(BKV, L // 64, 64, 2, 64).permute(0, 1, 3, 2, 4)      # [b, blk, half, tok, ch]
    else:
        tiles = xp.view(BKV, L // 64, 64, D).permute(0, 1, 3, 2)             # [b, blk, ch, tok]
    tiles = tiles.reshape(BKV, T, 64)
    assert torch.equal((tiles != 0).sum(-1), pop)
    # ... bit positions (element i <-> bit 63 - i) ...
    w = (1 << torch.arange(62, -1, -1, device=x.device, dtype=torch.int64))
    low63 = ((tiles[:, :, 1:] != 0).to(torch.int64) * w).sum(-1)
    assert torch.equal(c.bmp & 0x7FFFFFFFFFFFFFFF, low63)
    assert torch.equal(c.bmp < 0, tiles[:, :, 0] != 0)
    # ... and values: checksums of the packed stream (sum, sum of magnitudes, non-zero count) against the dense tensor
    nz = c.packed().double()
    assert nz.numel() == int(c.total_halfs)
    assert abs(float(nz.sum()) - float(xp.double().sum())) < 1e-6 * float(xp.double().abs().sum())
    assert float(nz.abs().sum()) == pytest.approx(float(xp.double().abs().sum()), rel=1e-12)
    assert int((nz != 0).sum()) == int(pop.sum())


def dense_masked_attention(q, Kp, Vp, groups=GROUPS):
    """The reference's dense path on pruned tensors (models/llama_mustafar_Kt_Mag_Vt_Mag.py:836-1026): fp16 scores with
    fp32 accumulation, / sqrt(d) in fp16, fp32 softmax rounded to fp16, fp32-accumulated P.V rounded to fp16."""
    bkv, length = Kp.shape[0], Kp.shape[1]
    qh = q.view(bkv, groups, D).float()
    s = torch.einsum("bgd,bld->bgl", qh, Kp.float()).half()
    w = (s / math.sqrt(D)).float()
    p = torch.softmax(w, -1).half()
    o = torch.einsum("bgl,bld->bgd", p.float(), Vp.float()).half()
    return s.view(-1, length), p.view(-1, length), o.view(-1, D)


def rel_rowmax(a, b):
    a, b = a.double(), b.double()
    return float(((a - b).abs().amax(-1) / b.abs().amax(-1).clamp_min(1e-30)).max())


def test_decode_attention_full_size(data):
    from mustafar_amd import ops
    K, V, q, Kp, Vp = data
    s_ref, p_ref, o_ref = dense_masked_attention(q, Kp, Vp)
    ck = ops.compress(K, False, kth=KTH)
    cv = ops.compress(V, True, kth=KTH)
    Bq = BKV * GROUPS
    s = ops.key_spmv(ck, q.view(Bq, 1, D), GROUPS)
    assert rel_rowmax(s[:, 0], s_ref) < 2e-3
    p = ops.scale_softmax(s, D)
    assert rel_rowmax(p[:, 0], p_ref) < 2e-3
    o = ops.value_spmv(cv, p, GROUPS)
    assert rel_rowmax(o[:, 0], o_ref) < 2e-3
    lse = torch.empty((Bq, 2), dtype=torch.float32, device=q.device)
    of = ops.decode_attention(ck, cv, q, GROUPS, lse=lse)
    assert rel_rowmax(of, o_ref) < 2e-3
    # (max, sum) of the scaled scores
    w = (s_ref / math.sqrt(D)).float()
    m_ref = w.amax(-1)
    assert float((lse[:, 0] - m_ref).abs().max()) <= 2e-2 * max(float(m_ref.abs().max()), 1.0)
    l_ref = torch.exp(w - m_ref[:, None]).sum(-1)
    assert float((lse[:, 1] * torch.exp(lse[:, 0] - m_ref) - l_ref).abs().max()) <= 5e-3 * float(l_ref.max())
    # linearity of the value product in the probabilities: P -> 0.5 P halves the output exactly (power of two)
    o_half = ops.value_spmv(cv, (p * 0.5).contiguous(), GROUPS)
    assert torch.equal(o_half.float() * 2, o.float()) or rel_rowmax(o_half[:, 0] * 2, o[:, 0]) < 1e-3


@pytest.mark.parametrize("bkv,blocks,groups", [(140, 31, 4), (150, 56, 2), (40, 112, 8), (600, 64, 1), (8, 2048, 4)])
def test_decode_attention_many_blocks(bkv, blocks, groups):
    """More 64-token blocks than resident wavefronts: every wavefront of the fused kernel walks several blocks
    (2, 3, 2, 8 and 4 here, with a ragged last wavefront in the first two; the last case is one long context of
    131072 tokens per head, which also takes the softmax kernel beyond the rows it keeps in registers) and folds them before the workgroup combine."""
    from mustafar_amd import ops
    from mustafar_amd._lib import lib
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(bkv * 1000 + blocks)
    length = blocks * 64
    K = torch.randn((bkv, length, D), generator=g, device=dev).half()
    V = torch.randn((bkv, length, D), generator=g, device=dev).half()
    K[:, :, 9] *= 8
    q = torch.randn((bkv * groups, D), generator=g, device=dev).half()
    Bq = bkv * groups
    ns = lib().mstf_decode_attention_splits(length, D, Bq, groups)
    assert 0 < ns < (blocks + 7) // 8 or blocks <= 8
    s_ref, _, o_ref = dense_masked_attention(q, torch_prune(K, KTH), torch_prune(V, KTH), groups)
    ck = ops.compress(K, False, kth=KTH)
    cv = ops.compress(V, True, kth=KTH)
    lse = torch.empty((Bq, 2), dtype=torch.float32, device=dev)
    o = ops.decode_attention(ck, cv, q, groups, lse=lse)
    # Beyond ~32K tokens the reference formula rounds its probabilities into the fp16 subnormals and loses accuracy
    # of its own; the fused kernel keeps un-normalised weights (<= 1) in fp16 and normalises in fp32.  So the fused
    # output is held to 2e-3 against the same attention with fp32 probabilities, and to a looser bound against the
    # reference formula for the long case; the three-launch path, which rounds as the reference does, is held to it.
    w = (s_ref / math.sqrt(D)).float()
    Vp = torch_prune(V, KTH)
    o_exact = torch.einsum("bgl,bld->bgd", torch.softmax(w, -1).view(bkv, groups, length), Vp.float()).half().view(-1, D)
    assert rel_rowmax(o, o_exact) < 2e-3
    tol_ref = 2e-3 if length <= 32768 else 4e-3
    assert rel_rowmax(o, o_ref) < tol_ref
    m_ref = w.amax(-1)
    assert float((lse[:, 0] - m_ref).abs().max()) <= 2e-2 * max(float(m_ref.abs().max()), 1.0)
    l_ref = torch.exp(w - m_ref[:, None]).sum(-1)
    assert float((lse[:, 1] * torch.exp(lse[:, 0] - m_ref) - l_ref).abs().max()) <= 5e-3 * float(l_ref.max())
    o2 = ops.decode_attention(ck, cv, q, groups)            # route without (max, sum) output
    assert rel_rowmax(o2, o_exact) < 2e-3
    # the three-launch path on the same cache
    p = ops.scale_softmax(ops.key_spmv(ck, q.view(Bq, 1, D), groups), D)
    o3 = ops.value_spmv(cv, p, groups)
    assert rel_rowmax(o3[:, 0], o_ref) < 2e-3
    assert rel_rowmax(o, o3[:, 0]) < tol_ref


def test_compress_twice_is_idempotent(data):
    """Compressing the already pruned tensor with kth = 0 gives the same cache as pruning inside the compressor."""
    from mustafar_amd import ops
    K, _, _, Kp, _ = data
    a = ops.compress(K, False, kth=KTH)
    b = ops.compress(Kp, False, kth=0)
    assert torch.equal(a.bmp, b.bmp) and torch.equal(a.idx, b.idx) and torch.equal(a.nz_off, b.nz_off)
    assert torch.equal(a.packed().view(torch.int16), b.packed().view(torch.int16))
    pr = ops.prune_rows(K.view(-1, D), KTH).view(BKV, L, D)
    assert torch.equal(pr.view(torch.int16) & 0x7FFF, Kp.view(torch.int16) & 0x7FFF)   # magnitudes; pruned keep +-0


def test_compress_from_projection_layout_full_size():
    """Batch 8 x 4096 tokens x 8 KV heads straight from a projection-shaped buffer [8, 4096, 48 heads, 128] (keys
    rotated in the kernel): the rotated rows equal the half-precision tensor expression evaluated by torch on the
    device, and both sides' compressed arrays equal those of the contiguous route, bit for bit."""
    from mustafar_amd import ops
    dev = torch.device("cuda:0")
    bs, n_q, n_kv = 8, 32, 8
    g = torch.Generator(device=dev)
    g.manual_seed(31)
    qkv = torch.randn((bs, L, n_q + 2 * n_kv, D), generator=g, device=dev, dtype=torch.float32).half()
    qkv[:, :, n_q + 3, 17] *= 12                        # an outlier channel in one key head
    kx, vx = qkv[:, :, n_q:n_q + n_kv], qkv[:, :, n_q + n_kv:]
    pos = torch.arange(L, device=dev, dtype=torch.float32)
    inv = 1.0 / (500000.0 ** (torch.arange(0, D, 2, device=dev, dtype=torch.float32) / D))
    ang = pos[:, None] * inv[None, :]
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1).half(), torch.cat([ang.sin(), ang.sin()], -1).half()
    kt = kx.transpose(1, 2)                             # [bs, n_kv, L, D]
    k_ref = (kt * cos) + (torch.cat((-kt[..., D // 2:], kt[..., :D // 2]), dim=-1) * sin)
    v_ref = vx.transpose(1, 2).contiguous()
    Lc = L - 256
    ck_ref = ops.compress(k_ref[:, :, :Lc].reshape(bs * n_kv, Lc, D), False, kth=KTH)
    cv_ref = ops.compress(v_ref[:, :, :Lc].reshape(bs * n_kv, Lc, D), True, kth=KTH)
    q_before = qkv[:, :, :n_q].clone()
    ck, rot = ops.compress_proj(kx, False, KTH, Lc, cos, sin)          # rotates qkv's key heads in place
    cv, _ = ops.compress_proj(vx, True, KTH, Lc)
    assert rot.data_ptr() == kx.data_ptr()
    assert torch.equal(kx.transpose(1, 2).contiguous().view(torch.int16), k_ref.contiguous().view(torch.int16))
    assert torch.equal(qkv[:, :, :n_q], q_before) and torch.equal(vx.transpose(1, 2), v_ref)   # neighbours untouched
    for a, b in ((ck, ck_ref), (cv, cv_ref)):
        assert torch.equal(a.bmp, b.bmp) and torch.equal(a.idx, b.idx) and torch.equal(a.nz_off, b.nz_off)
        assert int(a.total_halfs) == int(b.total_halfs)
        assert torch.equal(a.nz.view(torch.int16), b.nz.view(torch.int16))
