"""Compression straight from the projection output (rows [batch, tokens, heads, 128], keys rotated in the kernel),
through the C ABI: the rotated rows and every output array must equal, bit for bit, what the oracle gets on the
transposed, rotated, contiguous copy the reference builds first."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import oracle as orc

pytestmark = pytest.mark.gpu

D = 128


def bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


def oracle_side(x, M, kth, is_value, cos=None, sin=None):
    """x [batch, rows, heads, D] -> (rotated rows in x's layout, oracle compress of the [batch*heads, M, D] copy)."""
    xt = np.ascontiguousarray(x.transpose(0, 2, 1, 3))                 # [batch, heads, rows, D]
    if cos is not None:
        c = cos if cos.ndim == 3 else cos[None]
        xt = orc.rope_rows(xt, c[:, None], (sin if sin.ndim == 3 else sin[None])[:, None])
    flat = np.ascontiguousarray(xt.reshape(-1, xt.shape[2], D)[:, :M])
    comp = orc.compress(orc.prune_rows(flat, kth) if kth > 0 else flat, is_value) if M > 0 else None
    return np.ascontiguousarray(xt.transpose(0, 2, 1, 3)), comp


def check_compressed(c, comp):
    bmp, idx, nz, off = comp
    assert np.array_equal(c.bmp.cpu().numpy(), bmp)
    assert np.array_equal(c.idx.cpu().numpy(), idx)
    assert np.array_equal(c.nz_off.cpu().numpy(), off)
    assert int(c.total_halfs) == nz.size
    assert np.array_equal(bits(c.nz.cpu().numpy()), bits(nz))


@pytest.mark.parametrize("batch,heads,rows,M,layout", [
    (2, 2, 200, 128, "packed"),        # projection output as it is, tail of 72 rows (a partial last unit)
    (1, 8, 320, 256, "packed"),
    (2, 3, 64, 64, "padded"),          # rows == M, strides with gaps between tokens and batch entries
    (1, 2, 129, 0, "packed"),          # nothing compressed yet: rotation only
    (3, 1, 256, 192, "separate"),      # rotated rows to a second buffer with other strides, x untouched
    (1, 2, 192, 128, "batched_rope"),  # positions differ per batch entry
])
def test_rotate_prune_compress_keys(batch, heads, rows, M, layout):
    from mustafar_amd import ops
    dev = torch.device("cuda:0")
    if layout == "batched_rope":
        batch = 2
    kth = orc.kth_from_sparsity(0.7, D)
    rng = np.random.default_rng(batch * 1000 + heads * 100 + rows)
    K, _ = orc.make_kv(5 + rows, batch * heads, rows, D)
    x = np.ascontiguousarray(K.reshape(batch, heads, rows, D).transpose(0, 2, 1, 3))   # [batch, rows, heads, D]
    if layout == "batched_rope":
        pos = np.stack([np.arange(rows) + 3, np.arange(rows) + 4000])
        cs = [orc.rope_tables(p) for p in pos]
        cos, sin = np.stack([c for c, _ in cs]), np.stack([s for _, s in cs])
    else:
        cos, sin = orc.rope_tables(np.arange(rows) + int(rng.integers(0, 5000)))
    rot_ref, comp = oracle_side(x, M, kth, False, cos, sin)
    if layout == "padded":
        buf = torch.full((batch, rows + 3, heads * D + 64), float("nan"), dtype=torch.float16, device=dev)
        xg = buf[:, :rows, :heads * D].unflatten(2, (heads, D))
        xg.copy_(torch.from_numpy(x))
    else:
        xg = torch.from_numpy(x).to(dev).view(batch, rows, heads * D).view(batch, rows, heads, D)
    cg, sg = torch.from_numpy(cos).to(dev), torch.from_numpy(sin).to(dev)
    rot = None
    if layout == "separate":
        rot = torch.zeros((batch, heads, rows, D), dtype=torch.float16, device=dev).transpose(1, 2)   # head-major
    c, r = ops.compress_proj(xg, False, kth, M, cg, sg, rot)
    assert np.array_equal(bits(r.cpu().numpy()), bits(rot_ref))
    if layout == "separate":
        assert np.array_equal(bits(xg.cpu().numpy()), bits(x))
    if layout == "padded":
        assert torch.isnan(buf[:, rows:]).all() and torch.isnan(buf[:, :, heads * D:]).all()
    if M == 0:
        assert c is None
    else:
        check_compressed(c, comp)


@pytest.mark.parametrize("batch,heads,rows,M,kth", [(2, 2, 200, 128, 89), (1, 8, 256, 256, 64), (2, 4, 512, 256, 0)])
def test_prune_compress_values_in_place_of_the_projection(batch, heads, rows, M, kth):
    from mustafar_amd import ops
    dev = torch.device("cuda:0")
    _, V = orc.make_kv(9 + rows, batch * heads, rows, D)
    if kth == 0:
        V = orc.prune_rows(V, 100)                                      # already pruned: zeros are the holes
    x = np.ascontiguousarray(V.reshape(batch, heads, rows, D).transpose(0, 2, 1, 3))
    _, comp = oracle_side(x, M, kth, True)
    xg = torch.from_numpy(x).to(dev)
    c, _ = ops.compress_proj(xg, True, kth, M)
    check_compressed(c, comp)
    assert np.array_equal(bits(xg.cpu().numpy()), bits(x))
    # keys without rotation take the same route
    _, compk = oracle_side(x, M, kth, False)
    ck, _ = ops.compress_proj(xg, False, kth, M)
    check_compressed(ck, compk)


@pytest.mark.parametrize("pooled,window_kernel", [(False, False), (True, True)])
def test_prefill_from_projection_equals_prefill_from_copies(pooled, window_kernel):
    """SparseKVCache.prefill_proj on the projection outputs against prefill on the rotated, transposed tensors the
    reference builds: identical compressed part, identical window, identical decode output."""
    from mustafar_amd.cache import SparseKVCache
    dev = torch.device("cuda:0")
    bs, n_kv, g, L = 2, 2, 4, 700
    K, V = orc.make_kv(123, bs * n_kv, L, D)
    kx = np.ascontiguousarray(K.reshape(bs, n_kv, L, D).transpose(0, 2, 1, 3))
    vx = np.ascontiguousarray(V.reshape(bs, n_kv, L, D).transpose(0, 2, 1, 3))
    cos, sin = orc.rope_tables(np.arange(L))
    k_rot, _ = oracle_side(kx, 0, 0, False, cos, sin)
    mk = dict(fused=True, max_tokens=1024 if pooled else 0, window_kernel=window_kernel)
    a = SparseKVCache(g, D, 0.7, 0.7, 256, **mk)
    a.prefill(torch.from_numpy(k_rot).to(dev).transpose(1, 2), torch.from_numpy(vx).to(dev).transpose(1, 2))
    b = SparseKVCache(g, D, 0.7, 0.7, 256, **mk)
    kg = torch.from_numpy(kx).to(dev).view(bs, L, n_kv * D).view(bs, L, n_kv, D)
    vg = torch.from_numpy(vx).to(dev).view(bs, L, n_kv * D).view(bs, L, n_kv, D)
    Kr, Vr = b.prefill_proj(kg, vg, torch.from_numpy(cos).to(dev), torch.from_numpy(sin).to(dev))
    assert np.array_equal(bits(Kr.transpose(1, 2).cpu().numpy()), bits(k_rot)) and Vr.shape == (bs, n_kv, L, D)
    assert a.compressed_length == b.compressed_length == 256
    for sa, sb in ((a.k, b.k), (a.v, b.v)):
        assert torch.equal(sa.bmp, sb.bmp) and torch.equal(sa.idx, sb.idx)
        for h in range(bs * n_kv):
            n = 2 * int(sa.idx[h, -1])
            va = sa.nz[8 * int(sa.nz_off[h]):8 * int(sa.nz_off[h]) + n]
            vb = sb.nz[8 * int(sb.nz_off[h]):8 * int(sb.nz_off[h]) + n]
            assert torch.equal(va.view(torch.int16), vb.view(torch.int16))
    assert torch.equal(a.k_win.view(torch.int16), b.k_win.view(torch.int16))
    assert torch.equal(a.v_win.view(torch.int16), b.v_win.view(torch.int16))
    rng = np.random.default_rng(4)
    q = torch.from_numpy(rng.standard_normal((bs, n_kv * g, 1, D)).astype(np.float16)).to(dev)
    kn = torch.from_numpy(rng.standard_normal((bs, n_kv, 1, D)).astype(np.float16)).to(dev)
    vn = torch.from_numpy(rng.standard_normal((bs, n_kv, 1, D)).astype(np.float16)).to(dev)
    assert torch.equal(a.decode(q, kn, vn), b.decode(q, kn, vn))


def test_proj_rejects_bad_arguments():
    from mustafar_amd._lib import ProjSource, lib
    L = lib()
    z = torch.zeros(1 << 16, dtype=torch.float16, device="cuda:0")
    a = z.data_ptr()

    def src(**kw):
        s = ProjSource()
        s.x, s.stride_batch, s.stride_token, s.stride_head = a, 64 * 256, 256, 128
        s.batch, s.heads, s.rows = 1, 2, 64
        for k, v in kw.items():
            setattr(s, k, v)
        return ctypes.byref(s)
    out = (a, a, a, a, a, 1 << 14, a, 1 << 16)
    call = L.mstf_compress_proj_f16
    assert call(None, None, 0, 64, 128, 89, *out) == -1              # every call below is refused before a launch
    assert call(None, src(), 0, 128, 128, 89, *out) == -1            # M beyond the rows
    assert call(None, src(), 0, 0, 128, 89, *out) == -1              # nothing to do without rotation
    assert call(None, src(), 0, 32, 128, 89, *out) == -3
    assert call(None, src(), 0, 64, 64, 32, *out) == -3
    assert call(None, src(stride_token=252), 0, 64, 128, 89, *out) == -1
    assert call(None, src(x=a + 2), 0, 64, 128, 89, *out) == -2
    assert call(None, src(cos=a), 0, 64, 128, 89, *out) == -1        # cos without sin / rot
    assert call(None, src(cos=a, sin=a, rot=a, rot_stride_token=256, rot_stride_head=128, rope_stride_token=128),
                1, 64, 128, 89, *out) == -1                          # values are not rotated
    assert call(None, src(), 0, 64, 128, 89, a, a, a, a, None, 0, a, 1 << 16) == -1   # no sizing-only mode
    assert call(None, src(), 0, 64, 128, 89, a, a, a, a, a, 1 << 14, a, 16) == -4
    app = L.mstf_append_proj_f16
    assert app(None, src(), 0, 64, 128, 89, a, a, None, a, a, a, a, 1 << 16) == -1
    torch.cuda.synchronize()


@pytest.mark.parametrize("seed", range(8))
def test_random_layouts_against_oracle(seed):
    """Seeded random batch / heads / rows / M / strides (gaps between tokens, heads and batch entries, a non-zero
    storage offset), keys with rotation and values without, all arrays bit-exact against the oracle."""
    from mustafar_amd import ops
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(9000 + seed)
    batch, heads = int(rng.integers(1, 4)), int(rng.integers(1, 6))
    nblk = int(rng.integers(1, 5))
    M = 64 * nblk
    rows = M + int(rng.integers(0, 130))
    is_value = bool(seed & 1)
    kth = int(rng.choice([0, 1, 64, 89, 115, 128])) if is_value else int(rng.choice([1, 64, 89, 115]))
    K, V = orc.make_kv(400 + seed, batch * heads, rows, D)
    src = V if is_value else K
    if kth == 0:
        src = orc.prune_rows(src, 96)
    x = np.ascontiguousarray(src.reshape(batch, heads, rows, D).transpose(0, 2, 1, 3))
    pad_h, pad_t, pad_b, lead = (8 * int(rng.integers(0, 5)) for _ in range(4))
    row_len = heads * (D + pad_h) + pad_t
    buf = torch.full((lead + batch * ((rows + 2) * row_len + pad_b),), float("nan"), dtype=torch.float16, device=dev)
    xg = buf[lead:].as_strided((batch, rows, heads, D), ((rows + 2) * row_len + pad_b, row_len, D + pad_h, 1))
    xg.copy_(torch.from_numpy(x))
    before = buf.clone()
    if is_value:
        _, comp = oracle_side(x, M, kth, True)
        c, _ = ops.compress_proj(xg, True, kth, M)
        assert torch.equal(buf.view(torch.int16), before.view(torch.int16))          # the source is only read
    else:
        cos, sin = orc.rope_tables(np.arange(rows) + int(rng.integers(0, 8000)))
        rot_ref, comp = oracle_side(x, M, kth, False, cos, sin)
        c, r = ops.compress_proj(xg, False, kth, M, torch.from_numpy(cos).to(dev), torch.from_numpy(sin).to(dev))
        assert np.array_equal(bits(r.cpu().numpy()), bits(rot_ref))
        xg.copy_(torch.from_numpy(x))                                                 # undo the in-place rotation:
        assert torch.equal(buf.view(torch.int16), before.view(torch.int16))          # nothing else was written
    check_compressed(c, comp)


def test_append_proj_overflow_grows_and_does_not_rotate_twice():
    """A chunk from the projection layout that does not fit: the pool grows and appends it again; the keys, rotated
    in place by the first attempt, are not rotated a second time."""
    from mustafar_amd.cache import CompressedPool
    dev = torch.device("cuda:0")
    batch, heads, rows = 1, 3, 256
    K, _ = orc.make_kv(9, batch * heads, rows, D)
    kx = np.ascontiguousarray(K.reshape(batch, heads, rows, D).transpose(0, 2, 1, 3))
    cos, sin = orc.rope_tables(np.arange(rows))
    rot_ref, comp = oracle_side(kx, rows, 89, False, cos, sin)
    x = torch.from_numpy(kx).to(dev)
    pool = CompressedPool(heads, D, 256, False, dev, slab_fraction=0.2)    # 64 tokens fit, 256 do not
    r = pool.append_proj(x, 89, rows, torch.from_numpy(cos).to(dev), torch.from_numpy(sin).to(dev))
    assert pool.generation == 1 and int(pool.overflow) == 0 and pool.tokens == rows
    assert np.array_equal(bits(r.cpu().numpy()), bits(rot_ref))
    rb, ri, rnz, roff = comp
    assert np.array_equal(pool.bmp.cpu().numpy(), rb) and np.array_equal(pool.idx.cpu().numpy(), ri)
    for b in range(heads):
        want = rnz[8 * int(roff[b]):8 * int(roff[b]) + 2 * int(ri[b, -1])]
        assert np.array_equal(pool.head_values(b).cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_short_prompt_through_prefill_proj_is_only_rotated():
    from mustafar_amd.cache import SparseKVCache
    dev = torch.device("cuda:0")
    bs, n_kv, L = 2, 2, 200                                # shorter than the residual length: nothing is compressed
    K, V = orc.make_kv(77, bs * n_kv, L, D)
    kx = np.ascontiguousarray(K.reshape(bs, n_kv, L, D).transpose(0, 2, 1, 3))
    vx = np.ascontiguousarray(V.reshape(bs, n_kv, L, D).transpose(0, 2, 1, 3))
    cos, sin = orc.rope_tables(np.arange(L))
    k_rot, _ = oracle_side(kx, 0, 0, False, cos, sin)
    for pooled in (False, True):
        c = SparseKVCache(4, D, 0.7, 0.7, 256, fused=True, max_tokens=512 if pooled else 0, window_kernel=pooled)
        Kr, Vr = c.prefill_proj(torch.from_numpy(kx).to(dev), torch.from_numpy(vx).to(dev), torch.from_numpy(cos).to(dev),
                                torch.from_numpy(sin).to(dev))
        assert c.compressed_length == 0 and c.kv_len == L and c.k is None
        assert np.array_equal(bits(c.k_win.cpu().numpy()), bits(k_rot.transpose(0, 2, 1, 3)))
        assert np.array_equal(bits(c.v_win.cpu().numpy()), bits(vx.transpose(0, 2, 1, 3)))


def test_quantised_cache_prefill_from_projection():
    """QuantSparseKVCache.prefill_proj (rotation by the kernel, quantised producer on the transposed views) against
    prefill on the rotated tensors: identical lists, identical window."""
    from mustafar_amd.cache import QuantSparseKVCache
    dev = torch.device("cuda:0")
    bs, n_kv, L = 2, 2, 600
    K, V = orc.make_kv(321, bs * n_kv, L, D)
    kx = np.ascontiguousarray(K.reshape(bs, n_kv, L, D).transpose(0, 2, 1, 3))
    vx = np.ascontiguousarray(V.reshape(bs, n_kv, L, D).transpose(0, 2, 1, 3))
    cos, sin = orc.rope_tables(np.arange(L))
    k_rot, _ = oracle_side(kx, 0, 0, False, cos, sin)
    a = QuantSparseKVCache(4, D, 0.7, 0.7, 256, bit=2, fused=True, window_kernel=True)
    a.prefill(torch.from_numpy(k_rot).to(dev).transpose(1, 2), torch.from_numpy(vx).to(dev).transpose(1, 2))
    b = QuantSparseKVCache(4, D, 0.7, 0.7, 256, bit=2, fused=True, window_kernel=True)
    b.prefill_proj(torch.from_numpy(kx).to(dev), torch.from_numpy(vx).to(dev), torch.from_numpy(cos).to(dev),
                   torch.from_numpy(sin).to(dev))
    assert a.compressed_length == b.compressed_length == 256
    for sa, sb in ((a.k, b.k), (a.v, b.v)):
        assert len(sa) == len(sb)
        for ta, tb in zip(sa, sb):
            assert torch.equal(ta.view(torch.uint8), tb.view(torch.uint8))
    assert torch.equal(a.k_win.view(torch.int16), b.k_win.view(torch.int16))
    assert torch.equal(a.v_win.view(torch.int16), b.v_win.view(torch.int16))
