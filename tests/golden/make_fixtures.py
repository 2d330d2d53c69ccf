"""Writes the known-answer fixtures of tests/golden/ (run from the repository root: python tests/golden/make_fixtures.py).

The reference holds no golden vectors for this path, so the fixtures are produced by the CPU oracle on small seeded
inputs that contain the edge cases of the format, and each array is cross-checked here, before it is written,
against an independent restatement in plain numpy that follows the reference's producer/consumer definitions
directly (kernel/compression.py:32-54, 87-97, 164-174; kernel/csrc/SpMM_Kernel.cuh:262-265, 342-348, 631-642):

  kat_fp16.npz       K, V [2, 128, 128] fp16 (ties at the threshold, an all-equal row, an all-zero token, -0.0 runs, an
                     outlier channel = full key tiles, an empty key tile, tiles with 1 and with 8 non-zeros), kth = 89;
                     pruned rows, and per side bmp / idx / nz_off / packed values
  kat_attention.npz  Bkv 2 x 4 query heads x 256 tokens: q, raw scores q.K~^T (fp16), probabilities, attention output
  kat_quant.npz      the 2- and 4-bit producer outputs for the pruned K, V of kat_fp16

Stored as unsigned 16-bit patterns where the dtype is fp16, so that the comparison is on bits.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as orc  # noqa: E402

D, KTH = 128, 89


def inputs():
    K, V = orc.make_kv(20261125, 2, 128, D)
    K[0, 1, :] = np.float16(0.75)                    # all-equal row: everything kept
    K[0, 2, :64] = np.float16(1.0)
    K[0, 2, 64:] = np.float16(-1.0)                  # |x| ties everywhere
    K[0, 3, 5:120] = 0                               # more zeros than the pruning rank
    K[0, :64, 33] = np.float16(50.0)                 # a full key tile (the channel survives in all 64 tokens)
    K[1, :, 9] = 0                                   # empty key tiles (the channel never survives)
    K[1, :64, 17] = 0
    K[1, 5, 17] = np.float16(900.0)                  # a key tile with a single non-zero
    K[1, 64:72, 21] = np.float16(700.0)              # a key tile with at least 8 survivors in a row of tokens
    V[0, 4, :] = 0                                   # an all-zero token: two empty value tiles
    V[0, 5, 40:90] = np.float16(-0.0)
    V[1, 7, :] = np.float16(3.0)                     # full value tiles
    V[1, 8, :] = 0
    V[1, 8, 3] = np.float16(-2.5)                    # a value tile with a single non-zero
    return K, V


def numpy_prune(x, kth):
    """models/llama_mustafar_kernel.py:215-228 with numpy: threshold = kth-th smallest |x| of the row, keep >=."""
    a = np.abs(x.astype(np.float32))
    thr = np.partition(a, kth - 1, axis=-1)[..., kth - 1:kth]
    return np.where(a >= thr, x, np.float16(0.0)).astype(np.float16)


def numpy_compress(xp, is_value):
    """Tile walk written from the format definition, one tile at a time (no code shared with the oracle)."""
    B, M, N = xp.shape
    bmps, idxs, nzs = [], [], []
    for b in range(B):
        bm, ix, nz = [], [0], []
        for blk in range(M // 64):
            rows = xp[b, blk * 64:(blk + 1) * 64]            # [64 tokens, N]
            if is_value:
                tiles = [rows[t, h * 64:(h + 1) * 64] for h in range(N // 64) for t in range(64)]
            else:
                tiles = [rows[:, c] for c in range(N)]
            for tile in tiles:
                keep = tile.view(np.uint16) & 0x7FFF != 0    # != 0.0 (both zeros are dropped)
                word = 0
                for i in range(64):
                    if keep[i]:
                        word |= 1 << (63 - i)
                vals = list(tile[keep].view(np.uint16))
                vals += [0] * ((-len(vals)) % 8)             # +0.0 padding to a multiple of 8 halfs
                bm.append(word)
                nz += vals
                ix.append(ix[-1] + len(vals) // 2)           # 4-byte units
        bmps.append(np.array(bm, dtype=np.uint64).view(np.int64))
        idxs.append(np.array(ix, dtype=np.int32))
        nzs.append(np.array(nz, dtype=np.uint16))
    off = np.cumsum([0] + [n.size // 8 for n in nzs[:-1]]).astype(np.int32)   # 16-byte units
    return np.stack(bmps), np.stack(idxs), np.concatenate(nzs), off


def numpy_attention(q, Kp, Vp, groups):
    """models/llama_mustafar_Kt_Mag_Vt_Mag.py:836-1026 in float64, rounded where the reference rounds to fp16."""
    Bkv, L, _ = Kp.shape
    qh = q.reshape(Bkv, groups, D).astype(np.float64)
    s = np.einsum("bgd,bld->bgl", qh, Kp.astype(np.float64)).astype(np.float16)
    w = (s.astype(np.float32) / np.float32(np.sqrt(D))).astype(np.float16).astype(np.float64)
    e = np.exp(w - w.max(-1, keepdims=True))
    p = (e / e.sum(-1, keepdims=True)).astype(np.float16)
    o = np.einsum("bgl,bld->bgd", p.astype(np.float64), Vp.astype(np.float64)).astype(np.float16)
    return s.reshape(-1, L), p.reshape(-1, L), o.reshape(-1, D)


def u16(a):
    return np.ascontiguousarray(a).view(np.uint16)


def main():
    K, V = inputs()
    Kp, Vp = orc.prune_rows(K, KTH), orc.prune_rows(V, KTH)
    assert np.array_equal(u16(Kp) & 0x7FFF, u16(numpy_prune(K, KTH)) & 0x7FFF)   # pruned entries keep their sign bit
    assert np.array_equal(u16(Vp) & 0x7FFF, u16(numpy_prune(V, KTH)) & 0x7FFF)
    out = {"K": u16(K), "V": u16(V), "kth": np.int32(KTH), "Kp": u16(Kp), "Vp": u16(Vp)}
    for name, xp, is_value in (("k", Kp, 0), ("v", Vp, 1)):
        bmp, idx, nz, off = orc.compress(xp, is_value)
        nb, ni, nnz, noff = numpy_compress(xp, is_value)
        assert np.array_equal(bmp, nb) and np.array_equal(idx, ni) and np.array_equal(off, noff)
        assert np.array_equal(u16(nz), nnz)
        for b in range(xp.shape[0]):
            assert np.array_equal(u16(orc.decode(bmp, nz, idx, off, b, xp.shape[1], D, is_value)) & 0x7FFF,
                                  u16(xp[b]) & 0x7FFF)
        pops = np.array([bin(int(w) & (2 ** 64 - 1)).count("1") for w in bmp.view(np.uint64).ravel()])
        assert {0, 1, 64} <= set(pops.tolist()) and (pops[pops > 0] % 8 == 0).any()   # the edge cases are present
        out.update({name + "_bmp": bmp, name + "_idx": idx, name + "_nz": u16(nz), name + "_nz_off": off})
    np.savez_compressed(os.path.join(HERE, "kat_fp16.npz"), **out)

    groups, Bkv, L = 4, 2, 256
    Ka, Va = orc.make_kv(77001, Bkv, L, D)
    Kap, Vap = orc.prune_rows(Ka, KTH), orc.prune_rows(Va, KTH)
    q = np.random.default_rng(77002).standard_normal((Bkv * groups, D)).astype(np.float16)
    s, p, o = orc.dense_masked_attention(q, Kap, Vap, groups)
    ns, npr, no = numpy_attention(q, Kap, Vap, groups)

    def close(a, b, tol):
        a, b = a.astype(np.float64), b.astype(np.float64)
        return (np.abs(a - b).max(-1) / np.abs(b).max(-1)).max() < tol
    assert close(s, ns, 1e-3) and close(p, npr, 2e-3) and close(o, no, 2e-3)
    np.savez_compressed(os.path.join(HERE, "kat_attention.npz"), K=u16(Ka), V=u16(Va), q=u16(q), kth=np.int32(KTH),
                        groups=np.int32(groups), scores=u16(s), probs=u16(p), out=u16(o))

    qout = {}
    for bit in (2, 4):
        for name, xp, is_value in (("k", Kp, 0), ("v", Vp, 1)):
            bmp, toff, packed, counts, units, scales, zeros = orc.compress_quant(xp, is_value, bit)
            nb = numpy_compress(xp, is_value)[0]
            assert np.array_equal(bmp, nb)
            pops = np.array([bin(int(w) & (2 ** 64 - 1)).count("1") for w in bmp.view(np.uint64).ravel()])
            cap = 32 // bit
            assert np.array_equal(counts.ravel(), pops) and np.array_equal(units.ravel(), (pops + cap - 1) // cap)
            assert np.array_equal(toff.ravel(), np.cumsum(np.concatenate([[0], units.ravel()[:-1]])))
            # dequantised values stay within half a step of the original (closed form of the quantiser)
            for b in range(xp.shape[0]):
                deq = orc.decode_quant(bmp, packed, toff, scales, zeros, b, xp.shape[1], D, is_value, bit, 0)
                keep = u16(xp[b]) & 0x7FFF != 0
                assert np.array_equal(deq != 0, keep) or (np.abs(deq[~keep]) == 0).all()
            pre = "%s%d_" % (name, bit)
            qout.update({pre + "bmp": bmp, pre + "tile_off": toff, pre + "packed": packed, pre + "counts": counts,
                         pre + "units": units, pre + "scales": u16(scales), pre + "zeros": u16(zeros)})
    np.savez_compressed(os.path.join(HERE, "kat_quant.npz"), **qout)
    for f in ("kat_fp16.npz", "kat_attention.npz", "kat_quant.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
