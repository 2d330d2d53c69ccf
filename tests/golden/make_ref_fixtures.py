"""Writes tests/golden/ref_quant.npz and ref_fp16.npz with the REFERENCE's own Triton programs.

Runs in the build container only (the reference tree is not shipped anywhere else):
    python tests/golden/make_ref_fixtures.py [/root/reference]

The reference's producers are `@triton.jit` programs.  Triton's interpreter (TRITON_INTERPRET=1) executes them on
CPU tensors with Triton's own type-promotion rules, so the fp16 chain of the quantisation parameters
(kernel_quant/compression_quant.py:41-57: fp16 min/max, fp16 subtraction, fp16 division by 3, zero-point from the
rounded scale) comes out as the programs define it.  The host wrappers around them
(compression_quant.py:159-264, 425-529; kernel/compression.py:249-435) insist on CUDA tensors, so the few lines of
host glue (prefix sums of the counts) are redone here with numpy; every array that is written comes out of a
reference program except the offsets, which are the wrappers' cumsum formulas.

Inputs: the pruned K / V of kat_fp16.npz (format edge cases) and seeded random tiles, among them tiles with one
survivor, equal survivors (scale 0 -> 1), large magnitudes and small ranges.  Arrays are stored as bit patterns.
"""
import importlib.util
import os
import sys

os.environ["TRITON_INTERPRET"] = "1"

import numpy as np  # noqa: E402
import torch  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"


def load(path, name):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def shifts():
    return torch.from_numpy(np.left_shift(np.int64(1), np.arange(63, -1, -1, dtype=np.int64)))


def ref_quant(cq, x, is_value):
    """x [B, M, 128] fp16 (already pruned) through the reference's two quantising programs."""
    B, M, N = x.shape
    xt = torch.from_numpy(x.copy())
    flat = (xt.contiguous() if is_value else xt.transpose(1, 2).contiguous()).view(-1)
    T = M * N // 64
    bmp = torch.empty((B, T), dtype=torch.int64)
    cnt = torch.empty((B, T), dtype=torch.int32)
    sc = torch.empty((B, T), dtype=torch.float16)
    zp = torch.empty((B, T), dtype=torch.float16)
    calc = cq.calculate_bitmap_and_scale_value_batched if is_value else cq.calculate_bitmap_and_scale_key_batched
    comp = cq.compress_value_batched if is_value else cq.compress_key_batched
    grid = (T, B)
    calc[grid](flat, bmp.view(-1), cnt.view(-1), sc.view(-1), zp.view(-1), total_elems=B * M * N,
               shifts_ptr=shifts(), stride_batch=T * 64, M=M, N=N)
    bit, cap = 2, 16
    units = (cnt.numpy().astype(np.int64) + cap - 1) // cap
    per_b = units.sum(1)
    base = np.concatenate([[0], np.cumsum(per_b)[:-1]])
    intra = np.concatenate([np.zeros((B, 1), np.int64), np.cumsum(units, 1)[:, :-1]], 1)
    toff = torch.from_numpy((base[:, None] + intra).astype(np.int32))
    packed = torch.zeros((int(per_b.sum()),), dtype=torch.int32)
    if packed.numel():
        comp[grid](flat, bmp.view(-1), cnt.view(-1), toff.contiguous().view(-1), packed, sc.view(-1), zp.view(-1),
                   bit, cap, total_elems=B * M * N, stride_batch=T * 64, M=M, N=N)
    return {"bmp": bmp.numpy(), "tile_off": toff.numpy(), "packed": packed.numpy(), "counts": cnt.numpy(),
            "units": units.astype(np.int32), "scales": sc.numpy().view(np.uint16), "zeros": zp.numpy().view(np.uint16)}


def ref_fp16(cf, x, is_value):
    """x [B, M, 128] fp16 (already pruned) through the reference's two fp16 programs."""
    B, M, N = x.shape
    xt = torch.from_numpy(x.copy())
    flat = (xt.contiguous() if is_value else xt.transpose(1, 2).contiguous()).view(-1)
    T = M * N // 64
    bmp = torch.empty((B, T), dtype=torch.int64)
    cnt = torch.empty((B, T), dtype=torch.int32)
    calc = cf.calculate_bitmap_value_batched if is_value else cf.calculate_bitmap_key_batched
    comp = cf.compress_value_batched if is_value else cf.compress_key_batched
    grid = (T, B)
    calc[grid](flat, bmp.view(-1), cnt.view(-1), total_elems=B * M * N, shifts_ptr=shifts(), stride_batch=T * 64,
               M=M, N=N)
    acc = np.concatenate([np.zeros((B, 1), np.int32), np.cumsum(cnt.numpy(), 1).astype(np.int32)], 1)
    total = 2 * acc[:, -1].astype(np.int64)
    offs = np.cumsum(total)
    boff = torch.from_numpy(np.concatenate([[0], offs[:-1]]).astype(np.int32))
    packed = torch.zeros((int(offs[-1]),), dtype=torch.float16)
    comp[grid](flat, bmp.view(-1), torch.from_numpy(acc).contiguous().view(-1), packed, boff, total_elems=B * M * N,
               stride_batch=T * 64, M=M, N=N)
    return {"bmp": bmp.numpy(), "idx": acc, "nz": packed.numpy().view(np.uint16), "counts": cnt.numpy()}


def random_tiles(seed, n_tokens):
    """[2, n_tokens, 128] fp16 with ~70 % holes and the quantiser's awkward cases planted."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((2, n_tokens, 128)).astype(np.float32)
    x[0] *= rng.choice([0.01, 0.1, 1.0, 8.0, 300.0], size=(n_tokens, 1))     # ranges from tiny to large
    x[1, :, :32] += rng.choice([-40.0, 0.0, 40.0], size=(n_tokens, 1))       # far-off-centre tiles: |zero| large
    x[1, :, 64:96] = np.abs(x[1, :, 64:96]) + 2000.0                         # zero-points beyond -1024
    keep = rng.random(x.shape) < 0.3
    x = np.where(keep, x, 0.0).astype(np.float16)
    x[0, 3, :64] = 0
    x[0, 3, 11] = np.float16(-7.25)                                          # single survivor: scale 0 -> 1
    x[0, 5, :64] = 0
    x[0, 5, 1:9] = np.float16(0.3333)                                        # equal survivors
    x[0, 6, :] = 0                                                           # empty value tiles
    x[0, 7, :64] = np.float16(65504.0) * np.where(np.arange(64) % 2, 1, -1)  # max - min overflows fp16
    x[0, 8, :64] = np.float16(6e-8) * (np.arange(64) % 4)                    # subnormal range
    return x


def main():
    cq = load(os.path.join(REF, "kernel_quant", "compression_quant.py"), "ref_compression_quant")
    cf = load(os.path.join(REF, "kernel", "compression.py"), "ref_compression")
    kat = np.load(os.path.join(HERE, "kat_fp16.npz"))
    Kp, Vp = kat["Kp"].view(np.float16), kat["Vp"].view(np.float16)
    R = random_tiles(20261125, 128)
    cases = {"kat_k": (Kp, 0), "kat_v": (Vp, 1), "rnd_k": (R, 0), "rnd_v": (R, 1)}
    out_q, out_f = {"rnd_x": R.view(np.uint16)}, {"rnd_x": R.view(np.uint16)}
    for name, (x, is_value) in cases.items():
        for k, v in ref_quant(cq, x, is_value).items():
            out_q["%s_%s" % (name, k)] = v
        for k, v in ref_fp16(cf, x, is_value).items():
            out_f["%s_%s" % (name, k)] = v
        print(name, "done", flush=True)
    np.savez_compressed(os.path.join(HERE, "ref_quant.npz"), **out_q)
    np.savez_compressed(os.path.join(HERE, "ref_fp16.npz"), **out_f)
    for f in ("ref_quant.npz", "ref_fp16.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
