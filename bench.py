#!/usr/bin/env python3
"""Headline benchmark: sparse decode attention of one Llama-3-8B layer on one MI355X.

Workload (BASELINE.json configs[1]): batch 8, 32 query / 8 KV heads, head_dim 128, 4096 cached
tokens, per-token magnitude pruning at 70 % on K and V, fp16.  A step is one decode-attention
pass for one new token over the compressed cache: key SpMV -> scale+softmax -> value SpMV, run as
the fused kernel plus its split merge (or, with --unfused, as the three separate operator launches
of the reference's call sequence).  Several distinct caches are rotated between steps so that
reads come from HBM, not from the 256 MB Infinity Cache.  Prints exactly one JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--sparsity 0.7] [--no-cpu] [--unfused]
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "decode_attention_bs8_ctx4096_s70_traffic.txt")


def measured_traffic(args):
    """HBM bytes per launch of the fused kernel from the committed counter summary (FETCH_SIZE + WRITE_SIZE,
    calibrated on a copy of known size); only valid for the default workload, None otherwise."""
    if (args.batch, args.ctx, args.sparsity, args.unfused) != (8, 4096, 0.7, False) or not os.path.exists(TRAFFIC_FILE):
        return None
    for line in open(TRAFFIC_FILE):
        if line.startswith("traffic_bytes_per_launch:"):
            return int(float(line.split(":", 1)[1]))
    return None


def make_kv(torch, dev, Bkv, L, D, gen):
    """fp16 N(0,1) K and V; K gets 4 outlier channels per head scaled x10."""
    K = torch.randn((Bkv, L, D), generator=gen, device=dev, dtype=torch.float32)
    V = torch.randn((Bkv, L, D), generator=gen, device=dev, dtype=torch.float32)
    ch = torch.stack([torch.randperm(D, generator=gen, device=dev)[:4] for _ in range(Bkv)])
    scale = torch.ones((Bkv, 1, D), device=dev)
    scale.scatter_(2, ch.view(Bkv, 1, 4), 10.0)
    return (K * scale).half(), V.half()


def event_time_us(torch, fn, iters):
    """Average duration of fn() over `iters` back-to-back launches, HIP events on the launch stream."""
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / iters


def cpu_baseline(args, bs, nkv, groups, L, D, kth):
    """The oracle's dense masked attention (prune -> q.K^T -> /sqrt(d) -> fp32 softmax -> P.V) on the
    host cores, on a bounded sample: the layer shape at up to --cpu-batch batch entries, repeated for about 10 s."""
    import numpy as np
    from oracle import oracle as orc
    sample_bs = max(1, min(bs, args.cpu_batch))
    Bkv = sample_bs * nkv
    K, V = orc.make_kv(1234, Bkv, L, D)
    q = np.random.default_rng(5).standard_normal((Bkv * groups, D)).astype(np.float16)
    t0 = time.perf_counter()
    Kp, Vp = orc.prune_rows(K, kth), orc.prune_rows(V, kth)
    t_prune = time.perf_counter() - t0
    orc.dense_masked_attention(q, Kp, Vp, groups)  # warm-up
    reps, t_att = 0, 0.0
    while reps < 3 or (t_att < 10.0 and reps < 1000):
        t0 = time.perf_counter()
        orc.dense_masked_attention(q, Kp, Vp, groups)
        t_att += time.perf_counter() - t0
        reps += 1
    per_layer_us = t_att / reps * 1e6 * (bs / sample_bs)
    return {
        "value": round(per_layer_us, 1),
        "unit": "us/layer",
        "cores": orc.num_threads(),
        "kind": "port",
        "sample": "oracle dense masked decode attention, batch %d of %d (x%d heads, ctx %d), %d timed runs, "
                  "scaled to the full batch; pruning of that sample took %.2f s once (single thread)"
                  % (sample_bs, bs, nkv * groups, L, reps, t_prune),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--sparsity", type=float, default=0.7)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--ctx", type=int, default=4096)
    ap.add_argument("--caches", type=int, default=6, help="distinct compressed caches rotated between steps")
    ap.add_argument("--cpu-batch", type=int, default=8, help="batch entries in the CPU-baseline sample")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-graph", action="store_true", help="launch every step from Python instead of replaying HIP graphs")
    ap.add_argument("--unfused", action="store_true", help="step = the three separate operator launches")
    ap.add_argument("--no-quant", action="store_true", help="skip the stage timings of the quantised format")
    ap.add_argument("--no-dense", action="store_true", help="skip the dense fp16 attention timed beside the sparse path")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no cross-GPU exchange and every box here has one GPU "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    from mustafar_amd import ops

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    bs, nq, nkv, D, L = args.batch, 32, 8, 128, args.ctx
    groups = nq // nkv
    Bkv, Bq = bs * nkv, bs * nq
    kth = ops.kth_from_sparsity(args.sparsity, D)
    gen = torch.Generator(device=dev)
    gen.manual_seed(20260312)

    # ---- build the rotating compressed caches (also times the fused prune+compress kernels)
    caches = []
    dense = []   # the same tokens uncompressed, for the dense fp16 attention timed beside the sparse path
    t_ck = t_cv = 0.0
    for i in range(args.caches):
        K, V = make_kv(torch, dev, Bkv, L, D, gen)
        cap = K.numel()
        if i == 0:
            ops.compress(K, False, kth=kth, capacity_halfs=cap)  # warm-up (module load)
        t_ck += event_time_us(torch, lambda: caches.append([ops.compress(K, False, kth=kth, capacity_halfs=cap)]), 1)
        t_cv += event_time_us(torch, lambda: caches[-1].append(ops.compress(V, True, kth=kth, capacity_halfs=cap)), 1)
        if i == args.caches - 1:
            # GPU time of the compressors without the launch gaps of the Python calls: one capture, replayed
            try:
                def graphed_us(x, is_value):
                    g = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(g):
                        keep = ops.compress(x, is_value, kth=kth, capacity_halfs=cap)
                    g.replay()
                    t = event_time_us(torch, g.replay, 5)
                    del keep
                    return t
                tg_ck, tg_cv = graphed_us(K, False), graphed_us(V, True)
            except Exception as e:  # pragma: no cover - reported as null in the JSON line
                print("compress graph capture failed (%s)" % e, file=sys.stderr)
                tg_ck = tg_cv = None
        if not args.no_dense:
            dense.append((K.view(bs, nkv, L, D), V.view(bs, nkv, L, D)))
        del K, V
    t_ck /= args.caches
    t_cv /= args.caches
    kbytes = caches[0][0].bmp.numel() * 8 + caches[0][0].idx.numel() * 4 + int(caches[0][0].total_halfs.item()) * 2
    vbytes = caches[0][1].bmp.numel() * 8 + caches[0][1].idx.numel() * 4 + int(caches[0][1].total_halfs.item()) * 2

    q = torch.randn((Bq, 1, D), generator=gen, device=dev, dtype=torch.float32).half()
    q2 = q.view(Bq, D)
    s = torch.empty((Bq, 1, L), dtype=torch.float16, device=dev)
    p = torch.empty((Bq, 1, L), dtype=torch.float16, device=dev)
    o = torch.empty((Bq, 1, D), dtype=torch.float16, device=dev)
    o2 = o.view(Bq, D)
    it = [0]

    def launch(i):
        ck, cv = caches[i % args.caches]
        if args.unfused:
            ops.key_spmv(ck, q, groups, out=s)
            ops.scale_softmax(s, D, out=p)
            ops.value_spmv(cv, p, groups, out=o)
        else:
            ops.decode_attention(ck, cv, q2, groups, out=o2)

    # The launches are captured once and replayed, so that the timed region measures the GPU work of a step
    # rather than the Python call overhead of its launches: one graph holds one step on each of the rotating
    # caches back to back (as a decode iteration holds the attention of consecutive layers in one graph), and
    # one single-step graph per cache serves the remainder when K is not a multiple of the cache count.
    graphs = ring = None
    if not args.no_graph:
        try:
            for i in range(args.caches):
                launch(i)  # warm-up outside capture (module load, workspace growth)
            torch.cuda.synchronize()
            graphs = []
            for i in range(args.caches):
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    launch(i)
                graphs.append(g)
            ring = torch.cuda.CUDAGraph()
            with torch.cuda.graph(ring):
                for i in range(args.caches):
                    launch(i)
        except Exception as e:  # pragma: no cover - reported in the JSON line
            print("graph capture failed (%s); launching from Python" % e, file=sys.stderr)
            graphs = ring = None

    def run_steps(k):
        """Exactly k steps, continuing the rotation over the caches."""
        if graphs is None:
            for _ in range(k):
                launch(it[0] % args.caches)
                it[0] += 1
            return
        while k > 0:
            i = it[0] % args.caches
            if i == 0 and k >= args.caches:
                ring.replay()
                it[0] += args.caches
                k -= args.caches
            else:
                graphs[i].replay()
                it[0] += 1
                k -= 1

    run_steps(args.warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run_steps(args.steps)
    torch.cuda.synchronize()
    wall_us = (time.perf_counter() - t0) * 1e6 / args.steps

    # the same step on ONE cache over and over: its compressed bytes stay in the last-level cache between steps.
    # Reported beside `value` (which rotates the caches so that every step reads from HBM), never instead of it.
    warm_us = None
    if graphs is not None:
        warm_ring = torch.cuda.CUDAGraph()
        with torch.cuda.graph(warm_ring):
            for _ in range(args.caches):
                launch(0)
        reps = max(1, args.steps // args.caches)
        for _ in range(3):
            warm_ring.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            warm_ring.replay()
        torch.cuda.synchronize()
        warm_us = (time.perf_counter() - t0) * 1e6 / (reps * args.caches)

    # ---- per-kernel averages over back-to-back launches on rotating caches (HIP events on the launch stream)
    def rot(j):
        c = caches[it[0] % args.caches][j]
        it[0] += 1
        return c

    def fused_only():
        i = it[0] % args.caches
        it[0] += 1
        ops.decode_attention_partial(caches[i][0], caches[i][1], q2, groups)

    n = max(args.steps, 50)
    launch(0)
    fused_us = event_time_us(torch, fused_only, n)
    ws = ops.decode_attention_partial(caches[0][0], caches[0][1], q2, groups)
    merge_us = event_time_us(torch, lambda: ops.decode_attention_merge(ws, L, D, Bq, groups, out=o2), n)
    key_us = event_time_us(torch, lambda: ops.key_spmv(rot(0), q, groups, out=s), n)
    val_us = event_time_us(torch, lambda: ops.value_spmv(rot(1), p, groups, out=o), n)
    sm_us = event_time_us(torch, lambda: ops.scale_softmax(s, D, out=p), n)

    # dense fp16 decode attention over the same (unpruned) tokens with library operators, cold caches rotated alike:
    # what the sparse path has to beat.  "matmul" batches the query heads of a KV head into one product, so K and V
    # are read once per KV head as in the sparse kernels; "sdpa" is torch's fused attention operator.
    dense_us = None
    if dense:
        import torch.nn.functional as F
        q5 = q.view(bs, nkv, groups, D)
        q4 = q.view(bs, nq, 1, D)

        def dense_matmul(i):
            Kd, Vd = dense[i]
            w = torch.matmul(q5, Kd.transpose(2, 3)) / math.sqrt(D)
            return torch.matmul(torch.softmax(w, -1, dtype=torch.float32).half(), Vd)

        def dense_sdpa(i):
            Kd, Vd = dense[i]
            return F.scaled_dot_product_attention(q4, Kd, Vd, enable_gqa=True)

        def ring_time_us(fn):
            """One step on each rotating cache captured into one HIP graph (as the sparse step is), replayed."""
            for i in range(args.caches):
                fn(i)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for i in range(args.caches):
                    fn(i)
            g.replay()
            reps = max(n // args.caches, 5)
            return event_time_us(torch, g.replay, reps) / args.caches

        dense_us = {"matmul_softmax_matmul": round(ring_time_us(dense_matmul), 2),
                    "sdpa": round(ring_time_us(dense_sdpa), 2), "bytes": int(2 * Bkv * L * D * 2)}

    # quantised format (2- and 4-bit codes) on the same shape: producer once, then the key / value SpMVs with one
    # row per query head through the C ABI
    quant_us = {}
    if not args.no_quant:
        from mustafar_amd import compression_quant as cq
        from mustafar_amd._lib import lib, check
        Lh = lib()
        Kd, Vd = make_kv(torch, dev, Bkv, L, D, gen)
        Kd, Vd = ops.prune_rows(Kd.view(-1, D), kth).view(Bkv, L, D), ops.prune_rows(Vd.view(-1, D), kth).view(Bkv, L, D)
        p1 = torch.softmax(torch.randn((Bq, L), generator=gen, device=dev), -1).half()
        s1 = torch.empty((Bq, L), dtype=torch.float16, device=dev)
        for bit in (2, 4):
            kq = cq.convert_key_batched_quant(Kd, return_metadata=True, bit=bit)
            vq = cq.convert_value_batched_quant(Vd, bit=bit)
            st = torch.cuda.current_stream().cuda_stream
            wsq = ops.workspace(dev, Lh.mstf_value_spmv_quant_workspace_bytes(D, L, Bq, groups, 1))

            def qkey():
                check(Lh.mstf_key_spmv_quant(st, kq[0].data_ptr(), kq[2].data_ptr(), kq[1].data_ptr(), None, None,
                                             kq[5].data_ptr(), kq[6].data_ptr(), q2.data_ptr(), s1.data_ptr(), L, D, Bq,
                                             groups, 1, bit, 32 // bit, 0), "mstf_key_spmv_quant")

            def qval():
                check(Lh.mstf_value_spmv_quant(st, vq[0].data_ptr(), vq[2].data_ptr(), vq[1].data_ptr(), None, None,
                                               vq[5].data_ptr(), vq[6].data_ptr(), p1.data_ptr(), o2.data_ptr(), D, L, Bq,
                                               groups, 1, bit, 32 // bit, 0, wsq.data_ptr(), wsq.numel()),
                      "mstf_value_spmv_quant")

            from mustafar_amd import mustafar_package_quant as mpq

            def qfused():
                mpq.decode_attention_quant(kq, vq, q2, groups, bit, out=o2)

            qkey(), qval(), qfused()
            nbytes = lambda t: sum(x.numel() * x.element_size() for x in (t[0], t[1], t[2], t[5], t[6]))
            quant_us["%dbit" % bit] = {"key_spmv": round(event_time_us(torch, qkey, 30), 2),
                                       "value_spmv": round(event_time_us(torch, qval, 30), 2),
                                       "fused_decode_attention_incl_merge": round(event_time_us(torch, qfused, 30), 2),
                                       "bytes_per_token_per_kv_head": {"key": round(nbytes(kq) / Bkv / L, 2),
                                                                       "value": round(nbytes(vq) / Bkv / L, 2)}}
            del kq, vq
        del Kd, Vd

    # a copy of known size, so that a counter run of this same command can be calibrated (outside every timed region)
    cal_src = torch.zeros(64 << 20, dtype=torch.int32, device=dev)
    cal_dst = torch.empty_like(cal_src)
    for _ in range(5):
        torch.add(cal_src, 1, out=cal_dst)
    torch.cuda.synchronize()
    del cal_src, cal_dst

    # algorithmic bytes per launch: compressed side read once per KV head + weights in + result out (one row per head)
    key_alg = kbytes + Bq * D * 2 + Bq * L * 2
    val_alg = vbytes + Bq * L * 2 + Bq * D * 2
    fused_alg = kbytes + vbytes + Bq * D * 2 + Bq * D * 2
    if not args.unfused:
        dom, dom_us, dom_bytes = "decode_attention_kernel", fused_us, fused_alg
    elif val_us >= key_us:
        dom, dom_us, dom_bytes = "value_spmv_kernel", val_us, val_alg
    else:
        dom, dom_us, dom_bytes = "key_spmv_kernel", key_us, key_alg
    achieved = dom_bytes / dom_us / 1e3  # GB/s
    step_desc = ("step = the three operator launches (key SpMV, scale/softmax, value SpMV)" if args.unfused
                 else "step = fused decode-attention kernel + split merge")

    out = {
        "metric": "sparse decode-attn us/layer (Llama-3-8B shape, bs=%d, ctx=%d, %d%% K/V sparsity)"
                  % (bs, L, round(args.sparsity * 100)),
        "value": round(wall_us, 2),
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_us / 1e3, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE configs[1]: Llama-3-8B GQA decode-attention layer, batch %d, 32 query / 8 KV heads, "
                        "head_dim 128, %d cached tokens, per-token magnitude pruning %.0f%% on K and V, one new token; "
                        "%s; %d caches rotated (cold HBM reads); %s"
                        % (bs, L, args.sparsity * 100, step_desc, args.caches,
                           "steps replayed from HIP graphs (%d consecutive steps per graph)" % args.caches if graphs is not None else "steps launched from Python"),
            "compressed_bytes_per_token_per_kv_head": {"key": round(kbytes / Bkv / L, 2),
                                                       "value": round(vbytes / Bkv / L, 2)},
        },
        "tokens_per_s": round(bs / (wall_us * 1e-6), 1),
        "warm_cache_us_per_layer": None if warm_us is None else round(warm_us, 2),
        "stages_us": {"fused_decode_attention": round(fused_us, 2), "fused_merge": round(merge_us, 2),
                      "key_spmv": round(key_us, 2), "scale_softmax": round(sm_us, 2), "value_spmv": round(val_us, 2),
                      "prune_compress_key_ctx": round(t_ck, 1), "prune_compress_value_ctx": round(t_cv, 1)},
        # the compressors alone (configs[2] reports them): GPU time from a replayed capture, bytes read (dense fp16
        # context) and written (bitmaps + offsets + packed values), and the resulting rate
        "compress": {
            "key": {"us": None if tg_ck is None else round(tg_ck, 1), "read_bytes": int(Bkv * L * D * 2),
                    "written_bytes": int(kbytes),
                    "gbs": None if tg_ck is None else round((Bkv * L * D * 2 + kbytes) / tg_ck / 1e3, 1)},
            "value": {"us": None if tg_cv is None else round(tg_cv, 1), "read_bytes": int(Bkv * L * D * 2),
                      "written_bytes": int(vbytes),
                      "gbs": None if tg_cv is None else round((Bkv * L * D * 2 + vbytes) / tg_cv / 1e3, 1)}},
        "quant_stages_us": quant_us,
        "dense_fp16_attention_us": dense_us,
        "hbm_gbs_on_compressed_bytes": {"fused_decode_attention": round(fused_alg / fused_us / 1e3, 1),
                                        "key_spmv": round(key_alg / key_us / 1e3, 1),
                                        "value_spmv": round(val_alg / val_us / 1e3, 1),
                                        "whole_step": round(fused_alg / wall_us / 1e3, 1)},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": measured_traffic(args),
                     "algorithmic_bytes": int(dom_bytes), "avg_launch_us": round(dom_us, 2)},
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args, bs, nkv, groups, L, D, kth)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
