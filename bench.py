#!/usr/bin/env python3
"""Headline benchmark: sparse decode attention of one Llama-3-8B layer on one MI355X.

Workload (BASELINE.json configs[1]): batch 8, 32 query / 8 KV heads, head_dim 128, 4096 cached
tokens, per-token magnitude pruning at 70 % on K and V, fp16.  A step is one decode-attention
pass for one new token over the compressed cache: key SpMV -> scale+softmax -> value SpMV, run as
the fused kernel plus its split merge (or, with --unfused, as the three separate operator launches
of the reference's call sequence).  Several distinct caches are rotated between steps so that
reads come from HBM, not from the 256 MB Infinity Cache.  Prints exactly one JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--sparsity 0.7] [--no-cpu] [--unfused] [--no-configs]

Beside the headline the line carries `configs`: the other benchmark configurations measured in the same run
(configs[1] at 50 %, configs[2] compressors at batch 16, configs[3] quantised decode at batch 32, the configs[4]
decode loop over its 256 new tokens); every kernel time in the line is the GPU time of launches replayed from HIP graphs on rotating caches.
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
KSTATS_FILE = os.path.join(ROOT, "profiles", "decode_attention_bs8_ctx4096_s70_kernel_stats.md")


def measured_traffic(args):
    """HBM bytes per launch of the fused kernel from the committed counter summary (FETCH_SIZE + WRITE_SIZE,
    calibrated on a copy of known size); only valid for the default workload, None otherwise."""
    if (args.batch, args.ctx, args.sparsity, args.unfused) != (8, 4096, 0.7, False) or not os.path.exists(TRAFFIC_FILE):
        return None
    for line in open(TRAFFIC_FILE):
        if line.startswith("traffic_bytes_per_launch:"):
            return int(float(line.split(":", 1)[1]))
    return None


def profiled_launch_us(args):
    """Average duration of the fused kernel in the committed rocprofv3 --kernel-trace --stats summary of this command
    (default workload only): carried in the line beside the live HIP-event average."""
    if (args.batch, args.ctx, args.sparsity, args.unfused) != (8, 4096, 0.7, False) or not os.path.exists(KSTATS_FILE):
        return None
    for line in open(KSTATS_FILE):
        if line.startswith("rocprof_avg_launch_us:"):
            return float(line.split(":", 1)[1])
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


RING_ROUNDS = 4   # passes over the rotating caches captured into one graph


def settle(torch, fn, seconds):
    """Runs fn() untimed for `seconds`: after an idle period (set-up on the host, a graph capture) the GPU needs some
    tens of milliseconds of load before its clocks are where a decode loop keeps them - launches timed right after
    such a pause read 5 - 8 % longer than the same launches a moment later."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        fn()
        torch.cuda.synchronize()


def ring_time_us(torch, fn, n_slots, reps):
    """GPU time of one fn(i): RING_ROUNDS passes of fn(0) .. fn(n_slots - 1) are captured back to back into one HIP
    graph (slot i works on rotating cache i, so its reads are cold), the graph is replayed `reps` times between two HIP
    events.  A replay starts with a bubble of a few microseconds on the GPU; with a few dozen launches per graph - as
    a decode iteration of a model holds the launches of all its layers - it no longer weighs on the per-launch figure."""
    for i in range(n_slots):
        fn(i)   # warm-up outside the capture (module load, workspace growth)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(RING_ROUNDS):
            for i in range(n_slots):
                fn(i)
    settle(torch, g.replay, 0.02)
    return event_time_us(torch, g.replay, max(1, -(-reps // RING_ROUNDS))) / (n_slots * RING_ROUNDS)


def read_calibration(torch):
    """Plain reads (mstf_probe_read: 16 bytes per lane, nothing else) of cold buffers: per size the average launch time
    over rotating copies (at least 1 GiB apart in total, so that nothing is served from the last-level cache)."""
    from mustafar_amd._lib import lib, check
    L = lib()
    dev = torch.device("cuda:0")
    sink = torch.zeros(1 << 16, dtype=torch.int32, device=dev)
    out = {"what": "plain read of a cold buffer, 16 bytes per lane, 256 threads per workgroup; HIP-graph replays of one "
                   "launch per rotating copy", "sizes": []}
    for mb, wgs in ((31, 4096), (62, 4096), (62, 2048), (134, 4096), (249, 4096), (512, 8192), (1024, 8192)):
        nbytes = mb << 20
        copies = max(2, min(8, (1536 << 20) // nbytes))
        bufs = [torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(copies)]

        def run(i):
            check(L.mstf_probe_read(torch.cuda.current_stream().cuda_stream, bufs[i].data_ptr(), nbytes, sink.data_ptr(), wgs),
                  "mstf_probe_read")
        us = ring_time_us(torch, run, copies, 20)
        out["sizes"].append({"MiB": mb, "workgroups": wgs, "copies": copies, "us": round(us, 2),
                             "gbs": round(nbytes / us / 1e3, 1), "frac_of_8TBs": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 3)})
        del bufs
        torch.cuda.empty_cache()
    return out


def compressed_bytes(c):
    return c.bmp.numel() * 8 + c.idx.numel() * 4 + int(c.total_halfs.item()) * 2


def build_caches(torch, ops, dev, gen, Bkv, L, D, kth, n, keep_dense=False):
    caches, dense = [], []
    for _ in range(n):
        K, V = make_kv(torch, dev, Bkv, L, D, gen)
        caches.append((ops.compress(K, False, kth=kth, capacity_halfs=K.numel()),
                       ops.compress(V, True, kth=kth, capacity_halfs=V.numel())))
        if keep_dense:
            dense.append((K, V))
        del K, V
    return caches, dense


def fp16_decode_record(torch, ops, dev, gen, bs, L, sparsity, n_caches, reps):
    """Fused step (kernel + merge), the fused kernel alone and the three-launch stages at batch `bs`."""
    nq, nkv, D = 32, 8, 128
    g, Bkv, Bq = nq // nkv, bs * nkv, bs * nq
    kth = ops.kth_from_sparsity(sparsity, D)
    caches, _ = build_caches(torch, ops, dev, gen, Bkv, L, D, kth, n_caches)
    kb, vb = compressed_bytes(caches[0][0]), compressed_bytes(caches[0][1])
    q = torch.randn((Bq, D), generator=gen, device=dev, dtype=torch.float32).half()
    o = torch.empty((Bq, D), dtype=torch.float16, device=dev)
    s = torch.empty((Bq, 1, L), dtype=torch.float16, device=dev)
    p = torch.empty((Bq, 1, L), dtype=torch.float16, device=dev)
    ws = ops.Workspace(dev)
    step = ring_time_us(torch, lambda i: ops.decode_attention(caches[i][0], caches[i][1], q, g, out=o, ws=ws), n_caches, reps)
    kern = ring_time_us(torch, lambda i: ops.decode_attention_partial(caches[i][0], caches[i][1], q, g, ws=ws), n_caches, reps)
    key = ring_time_us(torch, lambda i: ops.key_spmv(caches[i][0], q.view(Bq, 1, D), g, out=s), n_caches, reps)
    sm = ring_time_us(torch, lambda i: ops.scale_softmax(s, D, out=p), n_caches, reps)
    val = ring_time_us(torch, lambda i: ops.value_spmv(caches[i][1], p, g, out=o.view(Bq, 1, D), ws=ws), n_caches, reps)
    alg = kb + vb + 2 * Bq * D * 2
    return {"batch": bs, "ctx": L, "sparsity": sparsity, "step_us": round(step, 2), "fused_kernel_us": round(kern, 2),
            "fused_kernel_gbs": round(alg / kern / 1e3, 1), "fused_kernel_frac_of_peak": round(alg / kern / 1e3 / HBM_PEAK_GBS, 4),
            "key_spmv_us": round(key, 2), "scale_softmax_us": round(sm, 2), "value_spmv_us": round(val, 2),
            "algorithmic_bytes": int(alg), "tokens_per_s": round(bs / (step * 1e-6), 1)}


def compress_record(torch, ops, dev, gen, bs, L, sparsity, reps):
    """configs[2]: prune + compress of the whole context, keys and values (two launches per call: the clearing of the
    status words and the one-pass kernel), calls replayed from a captured graph."""
    nkv, D = 8, 128
    Bkv = bs * nkv
    kth = ops.kth_from_sparsity(sparsity, D)
    copies, slots = 2, 4   # the graph holds four calls on two rotating inputs: the time of one call, not of a replay
    Ks, Vs = zip(*[make_kv(torch, dev, Bkv, L, D, gen) for _ in range(copies)])
    ws = ops.Workspace(dev)
    out = {"batch": bs, "ctx": L, "sparsity": sparsity}
    for name, xs, is_value in (("key", Ks, False), ("value", Vs, True)):
        keep = [None] * slots
        x = xs[0]

        def run(i):
            keep[i] = ops.compress(xs[i % copies], is_value, kth=kth, capacity_halfs=x.numel(), ws=ws)
        us = ring_time_us(torch, run, slots, reps)
        written = compressed_bytes(keep[0])
        read = x.numel() * 2
        out[name] = {"us": round(us, 1), "read_bytes": int(read), "written_bytes": int(written),
                     "gbs": round((read + written) / us / 1e3, 1),
                     "frac_of_peak": round((read + written) / us / 1e3 / HBM_PEAK_GBS, 4)}
    # keys and values of the context in one call (one clearing launch, one kernel over both sides)
    keep = [None] * slots

    def run_kv(i):
        keep[i] = ops.compress_kv(Ks[i % copies], Vs[i % copies], kth, kth, capacity_halfs=Ks[0].numel(), ws=ws)
    us = ring_time_us(torch, run_kv, slots, reps)
    moved = out["key"]["read_bytes"] + out["key"]["written_bytes"] + out["value"]["read_bytes"] + out["value"]["written_bytes"]
    out["key_and_value_one_call"] = {"us": round(us, 1), "us_per_side": round(us / 2, 1), "gbs": round(moved / us / 1e3, 1),
                                     "frac_of_peak": round(moved / us / 1e3 / HBM_PEAK_GBS, 4)}
    return out


def quant_record(torch, ops, dev, gen, bs, L, sparsity, bit, group_size, reps):
    """configs[3]: decode over the quantised cache - key SpMV, value SpMV (one row per head) and the fused launch."""
    from mustafar_amd import compression_quant as cq
    from mustafar_amd import mustafar_package_quant as mpq
    from mustafar_amd._lib import lib, check
    nq, nkv, D = 32, 8, 128
    g, Bkv, Bq = nq // nkv, bs * nkv, bs * nq
    kth = ops.kth_from_sparsity(sparsity, D)
    Lh = lib()
    n_caches = 2
    sides = []
    for _ in range(n_caches):
        K, V = make_kv(torch, dev, Bkv, L, D, gen)
        Kp = ops.prune_rows(K.view(-1, D), kth).view(Bkv, L, D)
        Vp = ops.prune_rows(V.view(-1, D), kth).view(Bkv, L, D)
        sides.append((cq.convert_key_batched_quant(Kp, return_metadata=True, bit=bit, group_size=group_size),
                      cq.convert_value_batched_quant(Vp, bit=bit, group_size=group_size)))
        del K, V, Kp, Vp
    q = torch.randn((Bq, D), generator=gen, device=dev, dtype=torch.float32).half()
    p1 = torch.softmax(torch.randn((Bq, L), generator=gen, device=dev), -1).half()
    s1 = torch.empty((Bq, L), dtype=torch.float16, device=dev)
    o = torch.empty((Bq, D), dtype=torch.float16, device=dev)
    ws = ops.Workspace(dev)
    wsv = ws.get(Lh.mstf_value_spmv_quant_workspace_bytes(D, L, Bq, g, 1))
    def qkey(i):
        st = torch.cuda.current_stream().cuda_stream   # the capturing stream while a graph is recorded
        kq = sides[i][0]
        check(Lh.mstf_key_spmv_quant_grouped(st, kq[0].data_ptr(), kq[2].data_ptr(), kq[1].data_ptr(), kq[5].data_ptr(),
                                             kq[6].data_ptr(), q.data_ptr(), s1.data_ptr(), L, D, Bq, g, 1, bit, 32 // bit,
                                             0, group_size), "mstf_key_spmv_quant_grouped")

    def qval(i):
        st = torch.cuda.current_stream().cuda_stream
        vq = sides[i][1]
        check(Lh.mstf_value_spmv_quant_grouped(st, vq[0].data_ptr(), vq[2].data_ptr(), vq[1].data_ptr(), vq[5].data_ptr(),
                                               vq[6].data_ptr(), p1.data_ptr(), o.data_ptr(), D, L, Bq, g, 1, bit,
                                               32 // bit, 0, group_size, wsv.data_ptr(), wsv.numel()),
              "mstf_value_spmv_quant_grouped")

    def side_bytes(t):
        return sum(x.numel() * x.element_size() for x in (t[0], t[1], t[2], t[5], t[6]))
    kb, vb = side_bytes(sides[0][0]), side_bytes(sides[0][1])

    # the producer on the pruned rows (what convert_*_batched_quant runs: kth = 0), outputs pre-allocated for the worst case
    T = L * D // 64
    Kp = ops.prune_rows(make_kv(torch, dev, Bkv, L, D, gen)[0].view(-1, D), kth).view(Bkv, L, D)
    pshape = (Bkv, T) if group_size == 64 else (Bkv, T, 2)
    pb = dict(bmp=torch.empty((Bkv, T), dtype=torch.int64, device=dev), off=torch.empty((Bkv, T), dtype=torch.int32, device=dev),
              cnt=torch.empty((Bkv, T), dtype=torch.int32, device=dev), units=torch.empty((Bkv, T), dtype=torch.int32, device=dev),
              sc=torch.empty(pshape, dtype=torch.float16, device=dev), zp=torch.empty(pshape, dtype=torch.float16, device=dev),
              tot=torch.empty((1,), dtype=torch.int64, device=dev),
              room=torch.empty((Bkv * T * (64 * bit // 32),), dtype=torch.int32, device=dev))
    wsp = ws.get(Lh.mstf_compress_quant_workspace_bytes(Bkv, L, D))

    def produce(is_value):
        def run(i):
            check(Lh.mstf_compress_quant_grouped(torch.cuda.current_stream().cuda_stream, Kp.data_ptr(), is_value, Bkv, L, D, 0,
                                                 bit, group_size, pb["bmp"].data_ptr(), pb["off"].data_ptr(),
                                                 pb["cnt"].data_ptr(), pb["units"].data_ptr(), pb["sc"].data_ptr(),
                                                 pb["zp"].data_ptr(), pb["tot"].data_ptr(), pb["room"].data_ptr(),
                                                 pb["room"].numel(), wsp.data_ptr(), wsp.numel()), "mstf_compress_quant_grouped")
        return ring_time_us(torch, run, 2, reps)
    prod_k, prod_v = produce(0), produce(1)
    del Kp, pb
    key = ring_time_us(torch, qkey, n_caches, reps)
    val = ring_time_us(torch, qval, n_caches, reps)
    fused = ring_time_us(torch, lambda i: mpq.decode_attention_quant(sides[i][0], sides[i][1], q, g, bit, out=o, ws=ws),
                         n_caches, reps)
    alg = kb + vb + 2 * Bq * D * 2
    return {"batch": bs, "ctx": L, "sparsity": sparsity, "bit": bit, "group_size": group_size,
            "key_spmv_us": round(key, 2), "value_spmv_us": round(val, 2), "fused_step_us": round(fused, 2),
            "producer_key_us": round(prod_k, 1), "producer_value_us": round(prod_v, 1),
            "key_spmv_gbs": round((kb + Bq * D * 2 + Bq * L * 2) / key / 1e3, 1),
            "value_spmv_gbs": round((vb + Bq * D * 2 + Bq * L * 2) / val / 1e3, 1),
            "fused_step_gbs": round(alg / fused / 1e3, 1), "fused_step_frac_of_peak": round(alg / fused / 1e3 / HBM_PEAK_GBS, 4),
            "bytes_per_token_per_kv_head": {"key": round(kb / Bkv / L, 2), "value": round(vb / Bkv / L, 2)}}


def decode_loop_record(torch, dev, layers, batch, prompt, new_tokens, cache="sparse"):
    """configs[4]: random-init Llama-3-8B shape, greedy decoding of new_tokens tokens with the step replayed from a
    HIP graph (tokens/s; the 256-token chunk that the window sheds on the way is pruned, compressed and appended
    inside the timed region) and a few eager steps with events around the cache's attention (its share of the step)."""
    import time as _time
    from mustafar_amd.harness import Config, Decoder, GraphedGreedyLoop, pool_tokens
    cfg = Config(layers=layers)
    eager_steps, warm_eager, warm_graph = 6, 2, 4
    total = prompt + warm_eager + eager_steps + warm_graph + new_tokens
    dec = Decoder(cfg, dev, cache=cache, sparsity=0.7, residual_length=256, max_tokens=pool_tokens(total))
    g = torch.Generator(device=dev)
    g.manual_seed(1)
    ids = torch.randint(0, cfg.vocab, (batch, prompt), generator=g, device=dev)
    dec.prefill(ids)                 # untimed: library start-up and kernel selection
    dec.reset_caches()
    torch.cuda.synchronize()
    t0 = _time.perf_counter()
    logits = dec.prefill(ids)
    torch.cuda.synchronize()
    t_prefill = _time.perf_counter() - t0
    nxt = logits[:, -1].argmax(-1, keepdim=True)
    for t in range(warm_eager):
        nxt = dec.step(nxt, prompt + t)[:, -1].argmax(-1, keepdim=True)
    torch.cuda.synchronize()
    t0 = _time.perf_counter()
    for t in range(warm_eager, warm_eager + eager_steps):
        nxt = dec.step(nxt, prompt + t, timed=True)[:, -1].argmax(-1, keepdim=True)
    torch.cuda.synchronize()
    t_eager = (_time.perf_counter() - t0) / eager_steps
    attn_ms = sum(a.elapsed_time(b) for a, b in dec.attn_events) / eager_steps
    loop = GraphedGreedyLoop(dec, nxt, prompt + warm_eager + eager_steps)
    loop.append_events = []
    for _ in range(warm_graph):
        loop.step()
    torch.cuda.synchronize()
    t0 = _time.perf_counter()
    for _ in range(new_tokens):
        loop.step()
    torch.cuda.synchronize()
    t_step = (_time.perf_counter() - t0) / new_tokens
    appends = [a.elapsed_time(b) for a, b in loop.append_events]
    pool_b = sum(c.kv_bytes()[0] for c in dec.caches)
    win_b = sum(c.kv_bytes()[1] for c in dec.caches)
    heads = batch * cfg.n_kv
    dense_pool = 2 * layers * heads * dec.caches[0].max_tokens * cfg.head_dim * 2       # the pools' token capacity, dense
    dense_all = 2 * layers * heads * total * cfg.head_dim * 2        # every token of the run, dense
    return {"cache": cache, "layers": layers, "batch": batch, "prompt": prompt, "new_tokens_timed": new_tokens,
            "prefill_s": round(t_prefill, 3),
            "graphed_decode_ms_per_step": round(1e3 * t_step, 3), "tokens_per_s": round(batch / t_step, 1),
            "graph_captures": loop.captures, "eager_decode_ms_per_step": round(1e3 * t_eager, 3),
            "eager_attention_over_cache_ms_per_step": round(attn_ms, 3),
            "eager_attention_share": round(attn_ms / (1e3 * t_eager), 4),
            "chunk_appends_in_timed_region": len(appends),
            "chunk_append_ms_all_layers": [round(a, 3) for a in appends],
            "compressed_tokens_at_end": dec.caches[0].compressed_length,
            "kv_bytes_allocated": int(pool_b), "kv_bytes_dense": int(dense_pool),
            "kv_allocated_over_dense": round(pool_b / dense_pool, 4),
            "kv_bytes_window_buffers": int(win_b),
            "kv_pools_plus_windows_over_dense_of_all_tokens": round((pool_b + win_b) / dense_all, 4),
            "pool_growths": sum(c.k_pool.generation + c.v_pool.generation for c in dec.caches)}


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
    ap.add_argument("--no-quant", action="store_true", help="skip the quantised format at the headline shape")
    ap.add_argument("--no-dense", action="store_true", help="skip the dense fp16 attention timed beside the sparse path")
    ap.add_argument("--no-configs", action="store_true", help="skip the other benchmark configurations (configs sub-records)")
    ap.add_argument("--loop-layers", type=int, default=32, help="layers of the configs[4] decode loop (0 = skip it)")
    ap.add_argument("--calibrate", action="store_true",
                    help="instead of the benchmark: time plain 16-byte-per-lane reads of buffers of the sizes the "
                         "kernels stream (one JSON line), the practical floor their times are read against")
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
    if args.calibrate:
        print(json.dumps(read_calibration(torch)))
        return
    bs, nq, nkv, D, L = args.batch, 32, 8, 128, args.ctx
    groups = nq // nkv
    Bkv, Bq = bs * nkv, bs * nq
    kth = ops.kth_from_sparsity(args.sparsity, D)
    gen = torch.Generator(device=dev)
    gen.manual_seed(20260312)
    reps = max(5, args.steps // args.caches)

    # ---- the rotating compressed caches of the headline workload
    caches, dense = build_caches(torch, ops, dev, gen, Bkv, L, D, kth, args.caches, keep_dense=not args.no_dense)
    kbytes, vbytes = compressed_bytes(caches[0][0]), compressed_bytes(caches[0][1])

    q = torch.randn((Bq, 1, D), generator=gen, device=dev, dtype=torch.float32).half()
    q2 = q.view(Bq, D)
    s = torch.empty((Bq, 1, L), dtype=torch.float16, device=dev)
    p = torch.empty((Bq, 1, L), dtype=torch.float16, device=dev)
    o = torch.empty((Bq, 1, D), dtype=torch.float16, device=dev)
    o2 = o.view(Bq, D)
    ws = ops.Workspace(dev)
    it = [0]

    def launch(i):
        ck, cv = caches[i % args.caches]
        if args.unfused:
            ops.key_spmv(ck, q, groups, out=s)
            ops.scale_softmax(s, D, out=p)
            ops.value_spmv(cv, p, groups, out=o, ws=ws)
        else:
            ops.decode_attention(ck, cv, q2, groups, out=o2, ws=ws)

    # The launches are captured once and replayed, so that the timed region measures the GPU work of a step
    # rather than the Python call overhead of its launches: one graph holds RING_ROUNDS passes of one step on each
    # of the rotating caches back to back (as a decode iteration holds the attention of consecutive layers in one
    # graph), and one single-step graph per cache serves the remainder when K is not a multiple of its length.
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
                for _ in range(RING_ROUNDS):
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
            if i == 0 and k >= args.caches * RING_ROUNDS:
                ring.replay()
                it[0] += args.caches * RING_ROUNDS
                k -= args.caches * RING_ROUNDS
            else:
                graphs[i].replay()
                it[0] += 1
                k -= 1

    # steady state first (see settle), then the W warm-up steps and the K timed ones
    settle(torch, lambda: run_steps(args.caches * RING_ROUNDS if ring is not None else 1), 0.1)
    it[0] = 0
    run_steps(args.warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run_steps(args.steps)
    torch.cuda.synchronize()
    wall_us = (time.perf_counter() - t0) * 1e6 / args.steps

    # the same step on ONE cache over and over: its compressed bytes stay in the last-level cache between steps.
    # Reported beside `value` (which rotates the caches so that every step reads from HBM), never instead of it.
    warm_us = ring_time_us(torch, lambda i: launch(0), args.caches, reps)

    # ---- per-kernel GPU times, every one from launches replayed out of a HIP graph on the rotating caches
    fused_us = ring_time_us(torch, lambda i: ops.decode_attention_partial(caches[i][0], caches[i][1], q2, groups, ws=ws),
                            args.caches, reps)
    wsm = ops.decode_attention_partial(caches[0][0], caches[0][1], q2, groups, ws=ws)
    merge_us = ring_time_us(torch, lambda i: ops.decode_attention_merge(wsm, L, D, Bq, groups, out=o2), args.caches, reps)
    key_us = ring_time_us(torch, lambda i: ops.key_spmv(caches[i][0], q, groups, out=s), args.caches, reps)
    val_us = ring_time_us(torch, lambda i: ops.value_spmv(caches[i][1], p, groups, out=o, ws=ws), args.caches, reps)
    sm_us = ring_time_us(torch, lambda i: ops.scale_softmax(s, D, out=p), args.caches, reps)

    # the compressors at the headline shape: prune + compress of the whole context
    comp = compress_record(torch, ops, dev, gen, args.batch, L, args.sparsity, 5)

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
            w = torch.matmul(q5, Kd.view(bs, nkv, L, D).transpose(2, 3)) / math.sqrt(D)
            return torch.matmul(torch.softmax(w, -1, dtype=torch.float32).half(), Vd.view(bs, nkv, L, D))

        def dense_sdpa(i):
            Kd, Vd = dense[i]
            return F.scaled_dot_product_attention(q4, Kd.view(bs, nkv, L, D), Vd.view(bs, nkv, L, D), enable_gqa=True)

        # the floor any dense kernel has: a plain read of the same K and V bytes (16 bytes per lane, nothing else)
        from mustafar_amd._lib import lib as _lib_, check as _check_
        sink = torch.zeros(1 << 16, dtype=torch.int32, device=dev)
        nb = Bkv * L * D * 2

        def dense_read(i):
            st = torch.cuda.current_stream().cuda_stream
            for t in dense[i]:
                _check_(_lib_().mstf_probe_read(st, t.data_ptr(), nb, sink.data_ptr(), 4096), "mstf_probe_read")

        dense_us = {"matmul_softmax_matmul": round(ring_time_us(torch, dense_matmul, args.caches, reps), 2),
                    "sdpa": round(ring_time_us(torch, dense_sdpa, args.caches, reps), 2),
                    "plain_read_of_k_and_v": round(ring_time_us(torch, dense_read, args.caches, reps), 2),
                    "bytes": int(2 * Bkv * L * D * 2)}
    del dense

    quant_here = {}
    if not args.no_quant:
        for bit in (2, 4):
            r = quant_record(torch, ops, dev, gen, bs, L, args.sparsity, bit, 64, 10)
            quant_here["%dbit" % bit] = {k: r[k] for k in ("key_spmv_us", "value_spmv_us", "fused_step_us",
                                                           "fused_step_gbs", "bytes_per_token_per_kv_head")}

    # ---- the other benchmark configurations, in the same run (skipped for a non-default workload)
    configs = None
    default_workload = (args.batch, args.ctx, args.sparsity, args.unfused) == (8, 4096, 0.7, False)
    if not args.no_configs and default_workload:
        del caches
        torch.cuda.empty_cache()
        configs = {"configs1_bs8_sparsity50": fp16_decode_record(torch, ops, dev, gen, 8, 4096, 0.5, 6, 20)}
        configs["configs2_compress_bs16"] = [compress_record(torch, ops, dev, gen, 16, 4096, sp, 5) for sp in (0.5, 0.7, 0.9)]
        torch.cuda.empty_cache()
        configs["configs3_fp16_bs32_for_comparison"] = fp16_decode_record(torch, ops, dev, gen, 32, 4096, 0.7, 3, 20)
        torch.cuda.empty_cache()
        configs["configs3_quant_bs32"] = [quant_record(torch, ops, dev, gen, 32, 4096, 0.7, bit, gs, 10)
                                          for bit, gs in ((2, 64), (4, 64), (2, 32), (4, 32))]
        torch.cuda.empty_cache()
        if args.loop_layers > 0:
            try:
                configs["configs4_decode_loop"] = decode_loop_record(torch, dev, args.loop_layers, 16, 4096, 256)
                torch.cuda.empty_cache()
                configs["configs4_decode_loop_2bit"] = decode_loop_record(torch, dev, args.loop_layers, 16, 4096, 256,
                                                                          cache="sparse_quant2")
            except Exception as e:  # pragma: no cover - e.g. out of memory on a shared box; reported, not fatal
                configs.setdefault("configs4_decode_loop", {"error": str(e)[:200]})
                configs.setdefault("configs4_decode_loop_2bit", {"error": str(e)[:200]})
        torch.cuda.empty_cache()

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
                           "steps replayed from HIP graphs (%d consecutive steps per graph)" % (args.caches * RING_ROUNDS) if graphs is not None else "steps launched from Python"),
            "compressed_bytes_per_token_per_kv_head": {"key": round(kbytes / Bkv / L, 2),
                                                       "value": round(vbytes / Bkv / L, 2)},
        },
        "tokens_per_s": round(bs / (wall_us * 1e-6), 1),
        "warm_cache_us_per_layer": round(warm_us, 2),
        # GPU time of each kernel, replayed from HIP graphs on the rotating caches (no Python launch gaps inside)
        "stages_us": {"fused_decode_attention": round(fused_us, 2), "fused_merge": round(merge_us, 2),
                      "key_spmv": round(key_us, 2), "scale_softmax": round(sm_us, 2), "value_spmv": round(val_us, 2),
                      "prune_compress_key_ctx": comp["key"]["us"], "prune_compress_value_ctx": comp["value"]["us"],
                      "prune_compress_key_and_value_ctx_one_call": comp["key_and_value_one_call"]["us"]},
        # BASELINE configs[1] asks for the compression of the cached context timed with the step: their sum
        "configs1_total_us": round(comp["key_and_value_one_call"]["us"] + wall_us, 2),
        "configs1_total_us_separate_calls": round(comp["key"]["us"] + comp["value"]["us"] + wall_us, 2),
        "compress": comp,
        "quant_stages_us": quant_here,
        "dense_fp16_attention_us": dense_us,
        "hbm_gbs_on_compressed_bytes": {"fused_decode_attention": round(fused_alg / fused_us / 1e3, 1),
                                        "key_spmv": round(key_alg / key_us / 1e3, 1),
                                        "value_spmv": round(val_alg / val_us / 1e3, 1),
                                        "whole_step": round(fused_alg / wall_us / 1e3, 1)},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": measured_traffic(args),
                     "traffic_source": "profiles/decode_attention_bs8_ctx4096_s70_traffic.txt (rocprofv3 --pmc runs of this "
                                       "command, calibrated on the copy this run ends with)",
                     "algorithmic_bytes": int(dom_bytes), "avg_launch_us": round(dom_us, 2),
                     "avg_launch_us_source": "HIP events over graph replays in this run",
                     "rocprof_avg_launch_us": profiled_launch_us(args),
                     "rocprof_source": "profiles/decode_attention_bs8_ctx4096_s70_kernel_stats.md (rocprofv3 "
                                       "--kernel-trace --stats of this command)"},
        "configs": configs,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args, bs, nkv, groups, L, D, kth)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
