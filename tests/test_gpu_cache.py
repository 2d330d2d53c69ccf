"""The caller's cache state machine (prefill split, 256-token chunk appends) on the GPU: the appended
cache must be byte-identical to a one-shot compression of the same tokens, and every decode step must
match the oracle's dense masked attention over [pruned compressed part | dense window]."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc

from _metrics import rel_err   # row metric and element-wise allclose(rtol, atol = rtol * rms) in one number

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fused,pooled,window_kernel", [(False, False, False), (True, False, False), (True, True, False),
                                                        (True, True, True)])
def test_prefill_decode_append_matches_one_shot_and_oracle(fused, pooled, window_kernel):
    from mustafar_amd import ops
    from mustafar_amd.cache import SparseKVCache
    dev = torch.device("cuda:0")
    bs, n_kv, g, D, res = 2, 2, 4, 128, 256
    L0, steps = 700, 330                       # prefill: Lc = 256, window 444; appends at kv_len 768 and 1024
    total = L0 + steps
    K, V = orc.make_kv(77, bs * n_kv, total, D)
    rng = np.random.default_rng(1)
    Q = rng.standard_normal((steps, bs * n_kv * g, D)).astype(np.float16)
    Kt = torch.from_numpy(K).to(dev).view(bs, n_kv, total, D)
    Vt = torch.from_numpy(V).to(dev).view(bs, n_kv, total, D)
    cache = SparseKVCache(g, D, 0.7, 0.7, res, fused=fused, max_tokens=1024 if pooled else 0,
                          window_kernel=window_kernel)
    cache.prefill(Kt[:, :, :L0], Vt[:, :, :L0])
    assert cache.compressed_length == ((L0 - res) // 256) * 256 == 256
    checked = 0
    for t in range(steps):
        pos = L0 + t
        Lc_before = cache.compressed_length
        q = torch.from_numpy(Q[t]).to(dev).view(bs, n_kv * g, 1, D)
        out = cache.decode(q, Kt[:, :, pos:pos + 1], Vt[:, :, pos:pos + 1])
        if t % 37 == 0 or cache.compressed_length != Lc_before or t == steps - 1:
            Kf, Vf = K[:, :pos + 1].copy(), V[:, :pos + 1].copy()
            Kf[:, :Lc_before] = orc.prune_rows(np.ascontiguousarray(Kf[:, :Lc_before]), 89)
            Vf[:, :Lc_before] = orc.prune_rows(np.ascontiguousarray(Vf[:, :Lc_before]), 89)
            _, _, ref = orc.dense_masked_attention(Q[t], Kf, Vf, g)
            assert rel_err(out.cpu().numpy().reshape(-1, D), ref) < 2e-3, (t, pos)
            checked += 1
    assert cache.kv_len == total and cache.compressed_length == 768      # two appends happened
    assert cache.k_win.shape[2] == total - 768
    assert checked >= 10
    # incremental == one-shot, byte for byte (in a pooled cache every head's values sit in its own slab)
    Lc = cache.compressed_length
    for side, pool, is_value in ((cache.k, cache.k_pool, 0), (cache.v, cache.v_pool, 1)):
        src = V if is_value else K
        rb, ri, rnz, roff = orc.compress(orc.prune_rows(np.ascontiguousarray(src[:, :Lc]), 89), is_value)
        assert np.array_equal(side.bmp.cpu().numpy(), rb)
        assert np.array_equal(side.idx.cpu().numpy(), ri)
        if pooled:
            assert int(pool.overflow) == 0
            for b in range(bs * n_kv):
                want = rnz[8 * int(roff[b]):8 * int(roff[b]) + 2 * int(ri[b, -1])]
                assert np.array_equal(pool.head_values(b).cpu().numpy().view(np.uint16), want.view(np.uint16))
        else:
            assert np.array_equal(side.nz_off.cpu().numpy(), roff)
            assert np.array_equal(side.packed().cpu().numpy().view(np.uint16), rnz.view(np.uint16))
    if not pooled:
        one = ops.compress(Kt[:, :, :Lc].reshape(bs * n_kv, Lc, D).contiguous(), False, kth=89)
        assert torch.equal(one.bmp, cache.k.bmp) and torch.equal(one.idx, cache.k.idx)
        assert torch.equal(one.packed(), cache.k.packed())


def test_pool_that_overflows_grows_and_ends_up_like_one_that_never_did():
    """A chunk that does not fit a head's slab sets bit 0 of the flag word and writes none of the unit's values; what
    was there stays.  The pool then grows - larger slabs, old values copied, the chunk appended again - and holds
    exactly what a pool with dense-size slabs holds (and what the oracle packs)."""
    from mustafar_amd.cache import CompressedPool
    dev = torch.device("cuda:0")
    heads, D = 3, 128
    K, _ = orc.make_kv(9, heads, 256, D)
    Kt = torch.from_numpy(K).to(dev)
    pool = CompressedPool(heads, D, 256, False, dev, slab_fraction=0.2)    # 30 % survive: 64 tokens fit, 256 do not
    pool.append(Kt[:, :64], 89)
    assert int(pool.overflow) == 0 and pool.generation == 0
    before, off_before, seen = pool.nz.clone(), pool.nz_off.clone(), []
    grow = pool._grow_slabs

    def watched_grow():
        # at this point the failed append has run: flag read by the pool, old values untouched
        for b in range(heads):
            n = 2 * int(pool.idx_store[b, 128])
            s0 = 8 * int(off_before[b])
            assert torch.equal(pool.nz[s0:s0 + n], before[s0:s0 + n])
        seen.append(pool.slab16)
        grow()
    pool._grow_slabs = watched_grow
    pool.append(Kt[:, 64:256], 89)
    assert seen and pool.generation == 1 and pool.slab16 > seen[0] and int(pool.overflow) == 0 and pool.tokens == 256
    ref = CompressedPool(heads, D, 256, False, dev, slab_fraction=1.0)
    ref.append(Kt[:, :64], 89)
    ref.append(Kt[:, 64:256], 89)
    assert ref.generation == 0
    assert torch.equal(pool.bmp, ref.bmp) and torch.equal(pool.idx, ref.idx)
    rb, ri, rnz, roff = orc.compress(orc.prune_rows(K, 89), 0)
    assert np.array_equal(pool.bmp.cpu().numpy(), rb) and np.array_equal(pool.idx.cpu().numpy(), ri)
    for b in range(heads):
        assert torch.equal(pool.head_values(b).view(torch.int16), ref.head_values(b).view(torch.int16))
        want = rnz[8 * int(roff[b]):8 * int(roff[b]) + 2 * int(ri[b, -1])]
        assert np.array_equal(pool.head_values(b).cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_pair_append_equals_two_appends_and_survives_an_overflow():
    """cache.append_pair (keys and values of a chunk in one launch, one shared flag word) against one append per side:
    same bitmaps, offsets and values; with slabs too small for the second chunk - of one side only, and of both - the
    chunk is taken back, appended side by side and each pool grows its own slabs."""
    from mustafar_amd.cache import CompressedPool, append_pair
    dev = torch.device("cuda:0")
    heads, D = 3, 128
    K, V = orc.make_kv(19, heads, 256, D)
    Kt, Vt = torch.from_numpy(K).to(dev), torch.from_numpy(V).to(dev)
    refs = []
    for x, is_value in ((Kt, False), (Vt, True)):
        r = CompressedPool(heads, D, 256, is_value, dev, slab_fraction=1.0)
        r.append(x[:, :64], 89)
        r.append(x[:, 64:256], 89)
        refs.append(r)
    for fk, fv, grown in ((1.0, 1.0, (0, 0)), (0.2, 1.0, (1, 0)), (0.2, 0.2, (1, 1))):
        kp = CompressedPool(heads, D, 256, False, dev, slab_fraction=fk)
        vp = CompressedPool(heads, D, 256, True, dev, slab_fraction=fv)
        append_pair(kp, vp, Kt[:, :64], Vt[:, :64], 89, 89)
        append_pair(kp, vp, Kt[:, 64:256], Vt[:, 64:256], 89, 89)
        assert (kp.generation, vp.generation) == grown and int(kp.overflow) == 0 and int(vp.overflow) == 0
        for p, r in ((kp, refs[0]), (vp, refs[1])):
            assert p.tokens == 256 and int(p.tokens_dev) == 256
            assert torch.equal(p.bmp, r.bmp) and torch.equal(p.idx, r.idx)
            for b in range(heads):
                assert torch.equal(p.head_values(b).view(torch.int16), r.head_values(b).view(torch.int16))


def test_quantised_pool_that_overflows_grows_and_ends_up_like_one_that_never_did():
    from mustafar_amd.cache import QuantPool
    dev = torch.device("cuda:0")
    heads, D = 3, 128
    _, V = orc.make_kv(19, heads, 256, D)
    Vt = torch.from_numpy(V).to(dev)
    pool = QuantPool(heads, D, 256, True, 2, dev, packed_fraction=0.2)     # 64 tokens fit, 256 do not
    ref = QuantPool(heads, D, 256, True, 2, dev)
    for p in (pool, ref):
        p.append(Vt[:, :64], 89)
    assert pool.generation == 0
    for p in (pool, ref):
        p.append(Vt[:, 64:256], 89)
    assert pool.generation == 1 and ref.generation == 0 and pool.reserved == ref.reserved and pool.tokens == 256
    for a, b in zip(pool.view(), ref.view()):
        if a.dim() == 1:
            assert torch.equal(a[:pool.reserved], b[:ref.reserved])
        else:
            assert torch.equal(a, b)


def test_default_pool_sizes_hold_the_seeded_cache_without_growing():
    """slab_fraction_for / packed_fraction_for: 70 % sparsity, K with outlier channels - no growth, and the bytes held
    are the fractions of the dense bytes the docstrings state."""
    from mustafar_amd.cache import QuantSparseKVCache, SparseKVCache
    dev = torch.device("cuda:0")
    bs, n_kv, g, D, L = 2, 2, 4, 128, 1024 + 256
    K, V = orc.make_kv(23, bs * n_kv, L, D)
    Kt = torch.from_numpy(K).to(dev).view(bs, n_kv, L, D)
    Vt = torch.from_numpy(V).to(dev).view(bs, n_kv, L, D)
    dense = 2 * bs * n_kv * 1024 * D * 2
    for cache, bound in ((SparseKVCache(g, D, 0.7, 0.7, 256, fused=True, window_kernel=True, max_tokens=1024), 0.55),
                         (QuantSparseKVCache(g, D, 0.7, 0.7, 256, bit=2, fused=True, window_kernel=True, max_tokens=1024),
                          0.30)):
        cache.prefill(Kt, Vt)
        assert cache.compressed_length == 1024
        assert cache.k_pool.generation == 0 and cache.v_pool.generation == 0
        pool_bytes, _ = cache.kv_bytes()
        assert pool_bytes <= bound * dense, (pool_bytes / dense, bound)


@pytest.mark.parametrize("window_kernel", [False, True])
def test_short_prompt_stays_dense_until_first_chunk(window_kernel):
    from mustafar_amd.cache import SparseKVCache
    dev = torch.device("cuda:0")
    bs, n_kv, g, D = 1, 2, 2, 128
    K, V = orc.make_kv(5, bs * n_kv, 300, D)
    Kt = torch.from_numpy(K).to(dev).view(bs, n_kv, 300, D)
    Vt = torch.from_numpy(V).to(dev).view(bs, n_kv, 300, D)
    cache = SparseKVCache(g, D, 0.5, 0.5, 32, window_kernel=window_kernel)
    cache.prefill(Kt[:, :, :200], Vt[:, :, :200])       # (200 - 32) // 256 == 0 -> nothing compressed
    assert cache.compressed_length == 0 and cache.k is None
    q = torch.randn((bs, n_kv * g, 1, D), device=dev, dtype=torch.float16)
    for pos in range(200, 300):
        out = cache.decode(q, Kt[:, :, pos:pos + 1], Vt[:, :, pos:pos + 1])
    assert cache.compressed_length == 256 and cache.kv_len == 300   # 288 - 32 - 0 == 256 triggers the first chunk
    assert torch.isfinite(out).all()


def test_short_prompt_on_the_pooled_quantised_cache_matches_the_concatenating_one():
    """Nothing compressed after the prefill: the pooled quantised cache attends with empty pools (token count 0 on the
    device), then quantises its first chunk in place; every step equals the cache that appends by concatenation."""
    from mustafar_amd.cache import QuantSparseKVCache
    dev = torch.device("cuda:0")
    bs, n_kv, g, D = 1, 2, 2, 128
    K, V = orc.make_kv(8, bs * n_kv, 320, D)
    Kt = torch.from_numpy(K).to(dev).view(bs, n_kv, 320, D)
    Vt = torch.from_numpy(V).to(dev).view(bs, n_kv, 320, D)
    a = QuantSparseKVCache(g, D, 0.7, 0.7, 32, bit=2, fused=True, window_kernel=True)
    b = QuantSparseKVCache(g, D, 0.7, 0.7, 32, bit=2, fused=True, window_kernel=True, max_tokens=512)
    for c in (a, b):
        c.prefill(Kt[:, :, :200], Vt[:, :, :200])
        assert c.compressed_length == 0
    gen = torch.Generator(device=dev)
    gen.manual_seed(4)
    for pos in range(200, 320):
        q = torch.randn((bs, n_kv * g, 1, D), generator=gen, device=dev, dtype=torch.float16)
        oa = a.decode(q, Kt[:, :, pos:pos + 1], Vt[:, :, pos:pos + 1])
        ob = b.decode(q, Kt[:, :, pos:pos + 1], Vt[:, :, pos:pos + 1])
        assert torch.equal(oa.view(torch.int16), ob.view(torch.int16)), pos
    assert a.compressed_length == b.compressed_length == 256


@pytest.mark.parametrize("fused,bit,window_kernel,pooled", [(False, 2, False, False), (True, 2, False, False),
                                                            (True, 4, False, False), (True, 2, True, False),
                                                            (True, 8, True, False), (False, 2, False, True),
                                                            (True, 2, True, True), (True, 4, True, True)])
def test_quantised_cache_prefill_decode_append(fused, bit, window_kernel, pooled):
    """The quantised caller's state machine: after the prefill and two chunk appends (the reference's append: words
    behind the old ones, offsets shifted) every checked decode step matches dense masked attention over
    [oracle-dequantised compressed part | dense window] within 1e-2, and the per-tile arrays equal a one-shot
    quantisation of the same tokens."""
    from mustafar_amd.cache import QuantSparseKVCache
    dev = torch.device("cuda:0")
    bs, n_kv, g, D, res = 1, 2, 4, 128, 64
    L0, steps = 400, 300                       # prefill: Lc = 256, window 144; appends at kv_len 576 and 832?
    total = L0 + steps
    K, V = orc.make_kv(123, bs * n_kv, total, D)
    rng = np.random.default_rng(2)
    Q = rng.standard_normal((steps, bs * n_kv * g, D)).astype(np.float16)
    Kt = torch.from_numpy(K).to(dev).view(bs, n_kv, total, D)
    Vt = torch.from_numpy(V).to(dev).view(bs, n_kv, total, D)
    # pooled: pre-allocated per-tile arrays and word buffer filled in place, pruning fused into the producer
    cache = QuantSparseKVCache(g, D, 0.7, 0.7, res, bit=bit, fused=fused, window_kernel=window_kernel,
                               max_tokens=768 if pooled else 0)
    cache.prefill(Kt[:, :, :L0], Vt[:, :, :L0])
    assert cache.compressed_length == 256

    def dequantised(src, Lc, is_value):
        xp = orc.prune_rows(np.ascontiguousarray(src[:, :Lc]), 89)
        b, off, packed, _, _, sc, zp = orc.compress_quant(xp, is_value, bit)
        return np.stack([orc.decode_quant(b, packed, off, sc, zp, h, Lc, D, is_value, bit, 0) for h in range(bs * n_kv)])

    checked = 0
    for t in range(steps):
        pos = L0 + t
        Lc_before = cache.compressed_length
        q = torch.from_numpy(Q[t]).to(dev).view(bs, n_kv * g, 1, D)
        out = cache.decode(q, Kt[:, :, pos:pos + 1], Vt[:, :, pos:pos + 1])
        if t % 53 == 0 or cache.compressed_length != Lc_before or t == steps - 1:
            Kf, Vf = K[:, :pos + 1].copy(), V[:, :pos + 1].copy()
            Kf[:, :Lc_before] = dequantised(K, Lc_before, 0)
            Vf[:, :Lc_before] = dequantised(V, Lc_before, 1)
            _, _, ref = orc.dense_masked_attention(Q[t], Kf, Vf, g)
            assert rel_err(out.cpu().numpy().reshape(-1, D), ref) < 1e-2, (t, pos)
            checked += 1
    assert cache.compressed_length == 512 and cache.kv_len == total and checked >= 6
    # per-tile arrays equal a one-shot quantisation; the packed words are the same words, chunk by chunk
    Lc = cache.compressed_length
    sides = (cache.k_pool.view(), cache.v_pool.view()) if pooled else (cache.k, cache.v)
    for side, src, is_value in ((sides[0], K, 0), (sides[1], V, 1)):
        ref = orc.compress_quant(orc.prune_rows(np.ascontiguousarray(src[:, :Lc]), 89), is_value, bit)
        for i in (0, 3, 4):
            assert np.array_equal(side[i].cpu().numpy(), ref[i])
        for i in (5, 6):
            assert np.array_equal(side[i].cpu().numpy().view(np.uint16), ref[i].view(np.uint16))
        got_off, got_words = side[1].cpu().numpy(), side[2].cpu().numpy()
        units = ref[4]
        for h in range(bs * n_kv):
            for t in (0, 17, units.shape[1] // 2 + 3, units.shape[1] - 1):
                n = int(units[h, t])
                assert np.array_equal(got_words[got_off[h, t]:got_off[h, t] + n], ref[2][ref[1][h, t]:ref[1][h, t] + n])


def test_workspaces_are_owned_and_do_not_move_under_capture():
    """Every cache has its own scratch buffer; the default one is per (device, stream); a buffer that was handed out
    stays alive when a larger one replaces it; growing while the stream is being captured is refused."""
    from mustafar_amd import ops
    from mustafar_amd.cache import SparseKVCache
    dev = torch.device("cuda:0")
    a, b = ops.Workspace(dev, 1024), ops.Workspace(dev, 1024)
    assert a.tensor.data_ptr() != b.tensor.data_ptr()
    first = a.get(512)
    ptr = first.data_ptr()
    big = a.get(1 << 16)                                   # grows: a new buffer, the old one kept alive
    assert big.numel() >= 1 << 16 and first.data_ptr() == ptr and a._bufs[0] is first
    assert a.get(100).data_ptr() == big.data_ptr()          # no shrink, no further move
    # default workspaces: one per stream
    s1 = torch.cuda.Stream()
    d0 = ops.workspace(dev, 256)
    with torch.cuda.stream(s1):
        d1 = ops.workspace(dev, 256)
    assert d0.data_ptr() != d1.data_ptr()
    # a capture must not make a workspace grow
    small = ops.Workspace(dev, 256)
    g = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="reserve"):
        with torch.cuda.graph(g):
            small.get(1 << 20)
    small.reserve(1 << 20)                                  # outside the capture it is fine
    cache_a = SparseKVCache(4, max_tokens=512, window_kernel=True)
    cache_b = SparseKVCache(4, max_tokens=512, window_kernel=True)
    assert cache_a._workspace(dev) is not cache_b._workspace(dev)


@pytest.mark.parametrize("per_entry_positions,counter_on_device", [(False, True), (True, False)])
def test_window_append_rotates_and_appends_the_new_token(per_entry_positions, counter_on_device):
    """mstf_window_append_f16 against the oracle's apply_rotary_pos_emb restatement and a plain row write: rotated
    query rows in the attention's layout, rotated key row and value row at row win_len - 1 of the window buffers,
    every other row untouched - bit for bit; inputs are the three slices of one fused projection output."""
    from mustafar_amd import ops
    dev = torch.device("cuda:0")
    bs, n_q, n_kv, D, stride, wlen = 3, 8, 2, 128, 40, 17
    rng = np.random.default_rng(11)
    H = n_q + 2 * n_kv
    proj = rng.standard_normal((bs, H * D)).astype(np.float16)
    pos = rng.integers(0, 9000, size=bs) if per_entry_positions else np.full(bs, 4242)
    cos, sin = orc.rope_tables(pos)                                   # [bs, D]
    kwin0 = rng.standard_normal((bs * n_kv, stride, D)).astype(np.float16)
    vwin0 = rng.standard_normal((bs * n_kv, stride, D)).astype(np.float16)
    pt = torch.from_numpy(proj).to(dev)
    kw, vw = torch.from_numpy(kwin0).to(dev), torch.from_numpy(vwin0).to(dev)
    ct = torch.from_numpy(cos if per_entry_positions else cos[0]).to(dev)
    st = torch.from_numpy(sin if per_entry_positions else sin[0]).to(dev)
    counter = torch.full((1,), wlen, dtype=torch.int32, device=dev) if counter_on_device else None
    ovf = torch.zeros((1,), dtype=torch.int32, device=dev)
    q2 = ops.window_append(pt[:, n_q * D: (n_q + n_kv) * D], pt[:, (n_q + n_kv) * D:], kw, vw,
                           stride if counter_on_device else wlen, q_in=pt[:, : n_q * D], cos=ct, sin=st,
                           win_len_dev=counter, overflow=ovf)
    x = proj.reshape(bs, H, 1, D)
    rot = orc.rope_rows(x[:, : n_q + n_kv], cos[:, None, None, :], sin[:, None, None, :])
    assert np.array_equal(q2.cpu().numpy().view(np.int16), rot[:, :n_q].reshape(bs * n_q, D).view(np.int16))
    kexp, vexp = kwin0.copy(), vwin0.copy()
    kexp[:, wlen - 1] = rot[:, n_q:].reshape(bs * n_kv, D)
    vexp[:, wlen - 1] = x[:, n_q + n_kv:].reshape(bs * n_kv, D)
    assert np.array_equal(kw.cpu().numpy().view(np.int16), kexp.view(np.int16))
    assert np.array_equal(vw.cpu().numpy().view(np.int16), vexp.view(np.int16))
    assert int(ovf.item()) == 0
    # keys and values only, no rotation; then a count past the buffer: nothing written, flag set
    ops.window_append(pt[:, :n_kv * D], pt[:, n_kv * D: 2 * n_kv * D], kw, vw, wlen + 1)
    kexp[:, wlen] = proj[:, :n_kv * D].reshape(bs * n_kv, D)
    vexp[:, wlen] = proj[:, n_kv * D: 2 * n_kv * D].reshape(bs * n_kv, D)
    assert np.array_equal(kw.cpu().numpy().view(np.int16), kexp.view(np.int16))
    assert np.array_equal(vw.cpu().numpy().view(np.int16), vexp.view(np.int16))
    big = torch.full((1,), stride + 1, dtype=torch.int32, device=dev)
    ops.window_append(pt[:, :n_kv * D], pt[:, n_kv * D: 2 * n_kv * D], kw, vw, stride, win_len_dev=big, overflow=ovf)
    assert int(ovf.item()) == 1
    assert np.array_equal(kw.cpu().numpy().view(np.int16), kexp.view(np.int16))
    assert np.array_equal(vw.cpu().numpy().view(np.int16), vexp.view(np.int16))
    with pytest.raises(RuntimeError):
        ops.window_append(pt[:, :n_kv * D], pt[:, n_kv * D: 2 * n_kv * D], kw, vw, stride + 1)   # host count past the buffer


def test_caches_sharing_a_window_counter_advance_together():
    """Two layers' caches on one device counter (share_clock): decode_device_proj on both, then advance on both, gives
    what two independent caches give from decode() on rotated inputs; decode() on a sharing cache is refused."""
    from mustafar_amd.cache import SparseKVCache
    dev = torch.device("cuda:0")
    bs, n_kv, g, D, res = 2, 2, 4, 128, 256
    L0, steps = 600, 180                                   # a chunk leaves the window at kv_len 768
    rng = np.random.default_rng(3)
    n_q = n_kv * g
    H = n_q + 2 * n_kv

    def make(seed):
        K, V = orc.make_kv(seed, bs * n_kv, L0, D)
        Kt = torch.from_numpy(K).to(dev).view(bs, n_kv, L0, D)
        Vt = torch.from_numpy(V).to(dev).view(bs, n_kv, L0, D)
        a = SparseKVCache(g, D, 0.7, 0.7, res, fused=True, max_tokens=1024, window_kernel=True)
        b = SparseKVCache(g, D, 0.7, 0.7, res, fused=True, max_tokens=1024, window_kernel=True)
        a.prefill(Kt, Vt)
        b.prefill(Kt, Vt)
        return a, b

    lone = [make(5)[0], make(6)[0]]
    shared = [make(5)[1], make(6)[1]]
    shared[1].share_clock(shared[0])
    with pytest.raises(RuntimeError):
        shared[1].decode(torch.zeros((bs, n_q, 1, D), dtype=torch.float16, device=dev),
                         torch.zeros((bs, n_kv, 1, D), dtype=torch.float16, device=dev),
                         torch.zeros((bs, n_kv, 1, D), dtype=torch.float16, device=dev))
    for t in range(steps):
        cos, sin = orc.rope_tables(np.array([L0 + t]))
        ct, st = torch.from_numpy(cos[0]).to(dev), torch.from_numpy(sin[0]).to(dev)
        outs = []
        for layer in range(2):
            proj = rng.standard_normal((bs, H * D)).astype(np.float16)
            pt = torch.from_numpy(proj).to(dev)
            outs.append(shared[layer].decode_device_proj(pt[:, : n_q * D], pt[:, n_q * D: (n_q + n_kv) * D],
                                                         pt[:, (n_q + n_kv) * D:], ct, st))
            x = proj.reshape(bs, H, 1, D)
            rot = orc.rope_rows(x[:, : n_q + n_kv], cos[:, None, None, :], sin[:, None, None, :])
            want = lone[layer].decode(torch.from_numpy(np.ascontiguousarray(rot[:, :n_q])).to(dev),
                                      torch.from_numpy(np.ascontiguousarray(rot[:, n_q:])).to(dev),
                                      torch.from_numpy(np.ascontiguousarray(x[:, n_q + n_kv:])).to(dev))
            assert torch.equal(outs[layer].view(torch.int16), want.view(torch.int16)), (t, layer)
        for c in shared:
            c.advance()
    assert shared[0].compressed_length == lone[0].compressed_length == 512


@pytest.mark.parametrize("bs,n_kv,g,L0,steps,per_entry", [(2, 2, 4, 600, 200, False), (1, 1, 8, 300, 70, True),
                                                           (3, 2, 2, 1100, 40, False)])
@pytest.mark.parametrize("bit", [0, 2, 4])
def test_two_launch_step_equals_the_append_and_attention_calls(bs, n_kv, g, L0, steps, per_entry, bit):
    """mstf_decode_step_pool_f16 / mstf_decode_step_quant_pool (bit > 0) (rotation, append and window attention inside
    the launch of the compressed tokens, then the merge) against mstf_window_append_f16 +
    mstf_decode_attention_window_pool_f16 / mstf_decode_attention_window_quant_pool on a twin cache: the
    attention output of every step and the window buffers are identical bit for bit, across a chunk append, with an
    empty compressed part at the start (second case), partial and full window blocks, and the count overrunning the
    window buffer flagged the same way."""
    from mustafar_amd.cache import QuantSparseKVCache, SparseKVCache
    dev = torch.device("cuda:0")
    D, res = 128, 256
    n_q = n_kv * g
    H = n_q + 2 * n_kv
    K, V = orc.make_kv(40 + L0, bs * n_kv, L0, D)
    Kt = torch.from_numpy(K).to(dev).view(bs, n_kv, L0, D)
    Vt = torch.from_numpy(V).to(dev).view(bs, n_kv, L0, D)
    caches = []
    for step_launch in (True, False):
        if bit:
            c = QuantSparseKVCache(g, D, 0.7, 0.7, res, bit=bit, fused=True, window_kernel=True, max_tokens=1536)
        else:
            c = SparseKVCache(g, D, 0.7, 0.7, res, fused=True, window_kernel=True, max_tokens=1536)
        c.step_launch = step_launch
        c.prefill(Kt, Vt)
        caches.append(c)
    a, b = caches
    gen = torch.Generator(device=dev)
    gen.manual_seed(L0)
    for t in range(steps):
        proj = torch.randn((bs, H * D), generator=gen, device=dev, dtype=torch.float32).half()
        pos = np.arange(bs) * 7 + L0 + t if per_entry else np.full(bs, L0 + t)
        cos, sin = orc.rope_tables(pos)
        ct = torch.from_numpy(cos if per_entry else cos[0]).to(dev)
        st = torch.from_numpy(sin if per_entry else sin[0]).to(dev)
        outs = [c.decode_device_proj(proj[:, : n_q * D], proj[:, n_q * D: (n_q + n_kv) * D], proj[:, (n_q + n_kv) * D:], ct, st)
                for c in (a, b)]
        assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16)), t
        w = a._wlen + 1
        assert torch.equal(a._kbuf[:, :w].view(torch.int16), b._kbuf[:, :w].view(torch.int16)), t
        assert torch.equal(a._vbuf[:, :w].view(torch.int16), b._vbuf[:, :w].view(torch.int16)), t
        for c in (a, b):
            c.advance()
    assert a.compressed_length == b.compressed_length and int(a._wovf) == 0 and int(b._wovf) == 0


def test_two_launch_step_flags_a_count_past_the_window_buffer():
    from mustafar_amd import ops
    from mustafar_amd.cache import SparseKVCache
    dev = torch.device("cuda:0")
    bs, n_kv, g, D = 1, 2, 4, 128
    n_q = n_kv * g
    K, V = orc.make_kv(3, bs * n_kv, 600, D)
    c = SparseKVCache(g, D, 0.7, 0.7, 256, fused=True, window_kernel=True, max_tokens=1024)
    c.prefill(torch.from_numpy(K).to(dev).view(bs, n_kv, 600, D), torch.from_numpy(V).to(dev).view(bs, n_kv, 600, D))
    # (the attention of such a step covers the whole buffer, rows never written included: give them values)
    torch.nan_to_num_(c._kbuf, nan=0.0, posinf=0.0, neginf=0.0).clamp_(-4, 4)
    torch.nan_to_num_(c._vbuf, nan=0.0, posinf=0.0, neginf=0.0).clamp_(-4, 4)
    kb, vb = c._kbuf.clone(), c._vbuf.clone()
    proj = torch.randn((bs, (n_q + 2 * n_kv) * D), device=dev).half()
    big = torch.full((1,), c._kbuf.shape[1] + 1, dtype=torch.int32, device=dev)
    ovf = torch.zeros((1,), dtype=torch.int32, device=dev)
    out = ops.decode_step_pool(c.k_pool, c.v_pool, proj[:, : n_q * D], proj[:, n_q * D: (n_q + n_kv) * D],
                               proj[:, (n_q + n_kv) * D:], c._kbuf, c._vbuf, c._kbuf.shape[1], win_len_dev=big, overflow=ovf)
    torch.cuda.synchronize()
    assert int(ovf) == 1 and torch.isfinite(out).all()
    assert torch.equal(c._kbuf.view(torch.int16), kb.view(torch.int16)) and torch.equal(c._vbuf.view(torch.int16), vb.view(torch.int16))


@pytest.mark.parametrize("seed", range(6))
def test_two_launch_step_against_the_oracle_on_random_shapes(seed):
    """The two-launch decode step on drawn shapes (batch, KV heads, query heads per KV head, prompt length, 2-bit or
    fp16 cache, per-entry or shared positions) against the CPU oracle: rotation of the new query / key heads by
    oracle.rope_rows, dense masked attention over [pruned compressed tokens | dense window with the new row], 2e-3
    (1e-2 for the quantised cache: the oracle attends over the dequantised codes there)."""
    from mustafar_amd.cache import QuantSparseKVCache, SparseKVCache
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(7700 + seed)
    D, res = 128, 256
    bs = int(rng.integers(1, 4))
    n_kv = int(rng.integers(1, 3))
    g = int(rng.choice([1, 2, 4, 5, 8]))
    L0 = int(rng.integers(260, 900))
    quant = seed % 3 == 2
    per_entry = bool(seed % 2)
    n_q, Bkv = n_kv * g, bs * n_kv
    K, V = orc.make_kv(500 + seed, Bkv, L0, D)
    if quant:
        c = QuantSparseKVCache(g, D, 0.7, 0.7, res, bit=2, fused=True, window_kernel=True, max_tokens=1280)
    else:
        c = SparseKVCache(g, D, 0.7, 0.7, res, fused=True, window_kernel=True, max_tokens=1280)
    assert c.step_launch
    c.prefill(torch.from_numpy(K).to(dev).view(bs, n_kv, L0, D), torch.from_numpy(V).to(dev).view(bs, n_kv, L0, D))
    K_all, V_all = K.copy(), V.copy()                      # [Bkv, tokens, D]; the prompt's keys count as rotated
    steps = 3 if L0 % 256 < 250 else 8
    for t in range(steps):
        proj = rng.standard_normal((bs, (n_q + 2 * n_kv) * D)).astype(np.float16)
        pos = np.arange(bs) * 5 + L0 + t if per_entry else np.full(bs, L0 + t)
        cos, sin = orc.rope_tables(pos)                    # [bs, D]
        pt = torch.from_numpy(proj).to(dev)
        ct = torch.from_numpy(cos if per_entry else cos[0]).to(dev)
        st = torch.from_numpy(sin if per_entry else sin[0]).to(dev)
        out = c.decode_device_proj(pt[:, : n_q * D], pt[:, n_q * D: (n_q + n_kv) * D], pt[:, (n_q + n_kv) * D:], ct, st)
        q = proj[:, : n_q * D].reshape(bs, n_q, D)
        k = proj[:, n_q * D: (n_q + n_kv) * D].reshape(bs, n_kv, D)
        v = proj[:, (n_q + n_kv) * D:].reshape(bs, n_kv, D)
        qr = orc.rope_rows(q, cos[:, None, :], sin[:, None, :]).reshape(bs * n_q, D)
        kr = orc.rope_rows(k, cos[:, None, :], sin[:, None, :]).reshape(Bkv, 1, D)
        K_all = np.concatenate([K_all, kr], 1)
        V_all = np.concatenate([V_all, v.reshape(Bkv, 1, D)], 1)
        Lc = c.compressed_length
        Kp, Vp = K_all.copy(), V_all.copy()
        if Lc:
            Kp[:, :Lc] = orc.prune_rows(K_all[:, :Lc], c.kth_k)
            Vp[:, :Lc] = orc.prune_rows(V_all[:, :Lc], c.kth_v)
            if quant:
                for x, is_value in ((Kp, 0), (Vp, 1)):
                    r = orc.compress_quant(np.ascontiguousarray(x[:, :Lc]), is_value, 2)
                    x[:, :Lc] = np.stack([orc.decode_quant(r[0], r[2], r[1], r[5], r[6], b, Lc, D, is_value, 2, 0)
                                          for b in range(Bkv)])
        s_ref, _, o_ref = orc.dense_masked_attention(qr, Kp, Vp, g)
        got = out.reshape(bs * n_q, D).float().cpu().numpy().astype(np.float64)
        scale = max(np.abs(o_ref.astype(np.float64)).max(), 1e-30)
        # per row: the stated tolerance plus one fp16 ulp of the row's largest score / sqrt(d) - with the outlier
        # channels of these keys the scores reach +-100, where two correct summation orders round a score to
        # neighbouring fp16 values and a token's probability moves by that much (tests/test_gpu_config4.py)
        smax = np.abs(s_ref.astype(np.float64)).reshape(bs * n_q, -1).max(axis=1)
        ulp = np.exp2(np.floor(np.log2(np.maximum(smax, 2.0 ** -14))) - 10)
        tol = (1e-2 if quant else 2e-3) + ulp / np.sqrt(D)
        err = np.abs(got - o_ref).max(axis=1) / scale
        assert (err < tol).all() and np.median(err) < (1e-2 if quant else 2e-3), (seed, t, float(err.max()))
        c.advance()
    assert int(c._wovf) == 0
