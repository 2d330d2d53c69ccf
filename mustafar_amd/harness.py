"""Decode-loop harness: a random-init Llama-3 style decoder in plain PyTorch (library GEMMs, RMSNorm, RoPE, SDPA
prefill) around the sparse KV cache, after the reference's benchmark/mem_spd_test.py:109-187 and
benchmark/low_memory_generation.py: prompt -> prefill (the first Lc tokens are pruned and compressed per layer) ->
greedy decode, reporting tokens/s and the share of the step spent in attention over the cache.

The model is only the carrier of the measurement: weights are N(0, 0.02) and nothing is loaded from disk.
`cache="sparse"` uses SparseKVCache (compressed tokens and window in three launches, pooled storage);
`cache="sparse_quant2"` / `"sparse_quant4"` use QuantSparseKVCache (pruned + 2- or 4-bit codes, the same three launches
over the quantised format); `cache="dense_masked"` keeps the pruned tokens
dense and attends with torch ops - the reference's own dense path (models/llama_mustafar_Kt_Mag_Vt_Mag.py:836-1026) -
and is what the sparse run is compared against.

    python -m mustafar_amd.harness --layers 32 --batch 16 --prompt 4096 --new-tokens 256
"""
import argparse
import json
import math
import time

import torch
import torch.nn.functional as F

from . import ops
from .cache import CHUNK, QuantSparseKVCache, SparseKVCache, _repeat_kv


class Config:
    def __init__(self, hidden=4096, layers=32, n_q=32, n_kv=8, head_dim=128, ffn=14336, vocab=128256,
                 rope_theta=500000.0, rms_eps=1e-5):
        self.hidden, self.layers, self.n_q, self.n_kv, self.head_dim = hidden, layers, n_q, n_kv, head_dim
        self.ffn, self.vocab, self.rope_theta, self.rms_eps = ffn, vocab, rope_theta, rms_eps


class DenseMaskedCache:
    """Same state machine as SparseKVCache with the compressed range kept as pruned dense tensors.  The tokens live in
    buffers that grow geometrically (a decode step appends one row instead of re-concatenating the cache) and the
    query heads of a KV head are multiplied as one batch, so K and V are read once per KV head."""

    def __init__(self, groups, head_dim, k_sparsity, v_sparsity, residual_length, capacity=0):
        self.groups, self.head_dim, self.residual_length = groups, head_dim, residual_length
        self.kth_k = ops.kth_from_sparsity(k_sparsity, head_dim)
        self.kth_v = ops.kth_from_sparsity(v_sparsity, head_dim)
        self.capacity = capacity
        self._k = self._v = None
        self.compressed_length = self.kv_len = 0

    @property
    def k(self):
        return self._k[:, :, :self.kv_len]

    @property
    def v(self):
        return self._v[:, :, :self.kv_len]

    @staticmethod
    def _prune(x, kth):
        a = x.abs().float()
        thr = torch.kthvalue(a, kth, dim=-1, keepdim=True).values
        return torch.where(a >= thr, x, torch.zeros_like(x))

    def _compressed_form(self, K, V):
        """What the cache holds for a range of tokens that leaves the dense window: K, V [bs, n_kv, M, D], M % 256 == 0."""
        return self._prune(K, self.kth_k), self._prune(V, self.kth_v)

    def _room(self, n):
        if self._k is not None and self._k.shape[2] >= n:
            return
        cap = max(n, self.capacity, int(1.5 * self._k.shape[2]) if self._k is not None else 0)
        for name in ("_k", "_v"):
            old = getattr(self, name)
            new = torch.empty(old.shape[:2] + (cap,) + old.shape[3:], dtype=old.dtype, device=old.device)
            new[:, :, :self.kv_len] = old[:, :, :self.kv_len]
            setattr(self, name, new)

    def prefill(self, K, V):
        L = K.shape[2]
        Lc = ((L - self.residual_length) // CHUNK) * CHUNK if L > self.residual_length else 0
        cap = max(L, self.capacity)
        self._k = torch.empty(K.shape[:2] + (cap, K.shape[3]), dtype=K.dtype, device=K.device)
        self._v = torch.empty_like(self._k)
        self._k[:, :, :L], self._v[:, :, :L] = K, V
        if Lc > 0:
            self._k[:, :, :Lc], self._v[:, :, :Lc] = self._compressed_form(K[:, :, :Lc], V[:, :, :Lc])
        self.compressed_length, self.kv_len = Lc, L

    def decode(self, q, k_new, v_new):
        D, g = self.head_dim, self.groups
        bs, n_q = q.shape[0], q.shape[1]
        self._room(self.kv_len + 1)
        self._k[:, :, self.kv_len], self._v[:, :, self.kv_len] = k_new[:, :, 0], v_new[:, :, 0]
        self.kv_len += 1
        s = torch.matmul(q.view(bs, n_q // g, g, D), self.k.transpose(2, 3))
        p = torch.softmax((s / math.sqrt(D)).float(), -1).half()
        out = torch.matmul(p, self.v).view(bs, n_q, 1, D)
        Lc = self.compressed_length
        if (self.kv_len - self.residual_length - Lc) % CHUNK == 0 and self.kv_len - Lc >= CHUNK:
            kc, vc = self._compressed_form(self._k[:, :, Lc:Lc + CHUNK], self._v[:, :, Lc:Lc + CHUNK])
            self._k[:, :, Lc:Lc + CHUNK], self._v[:, :, Lc:Lc + CHUNK] = kc, vc
            self.compressed_length += CHUNK
        return out


def _rms_norm(x, w, eps):
    return F.rms_norm(x, (x.shape[-1],), w, eps)


def _rope_tables(pos, D, theta, dtype):
    """cos and signed sin of the rotary embedding for positions pos [L]: [L, D] each, sin negated in the first half,
    so that x * cos + roll(x, D/2) * sin_signed == x * cos + rotate_half(x) * sin product by product."""
    inv = 1.0 / (theta ** (torch.arange(0, D, 2, device=pos.device, dtype=torch.float32) / D))
    ang = pos.float()[:, None] * inv[None, :]
    cos = torch.cat([ang.cos(), ang.cos()], -1).to(dtype)
    sin = torch.cat([-ang.sin(), ang.sin()], -1).to(dtype)
    return cos, sin


def _rope(x, tables):
    """x: [bs, heads, L, D]; tables from _rope_tables for the L positions."""
    cos, sin = tables
    return x * cos + torch.roll(x, x.shape[-1] // 2, -1) * sin


class Decoder:
    def __init__(self, cfg, device, seed=0, cache="sparse", sparsity=0.7, residual_length=256, max_tokens=0,
                 proj_prefill=True, weights_of=None, dense_cache=None):
        """proj_prefill: the sparse caches take the keys and values of the prompt straight from the projection output
        (keys rotated by the compressor's own kernel; the fp16 cache also compresses them where they lie, without
        transposed or contiguous copies).  max_tokens: capacity of the compressed part of the sparse caches (0: caches
        that re-concatenate), of all tokens for the dense cache.  weights_of: another Decoder whose weight tensors
        this one shares.  dense_cache: class used for cache="dense_masked" (default DenseMaskedCache).
        shadow (attribute, a list of caches, one per layer): every layer's attention inputs - the projection output of
        the step, the prompt's keys and values - are also given to these caches and shadow_check(layer, output of the
        model's cache, output of the shadow cache) is called; the model goes on with its own cache's output, so the
        shadow caches are teacher-forced layer by layer."""
        self.cfg, self.dev = cfg, device
        self.proj_prefill = proj_prefill
        self.shadow, self.shadow_check = None, None
        self._dense_cache = dense_cache or DenseMaskedCache
        if weights_of is not None:
            self.embed, self.layers, self.norm, self.lm_head = (weights_of.embed, weights_of.layers, weights_of.norm,
                                                                weights_of.lm_head)
            self._cache_args = (cache, sparsity, residual_length, max_tokens)
            self.reset_caches()
            self.attn_events = []
            return
        g = torch.Generator(device=device)
        g.manual_seed(seed)

        def w(*shape):
            return (torch.randn(shape, generator=g, device=device, dtype=torch.float32) * 0.02).half()

        c = cfg
        self.embed = w(c.vocab, c.hidden)
        self.layers = []
        for _ in range(c.layers):
            self.layers.append({
                "qkv": w((c.n_q + 2 * c.n_kv) * c.head_dim, c.hidden), "o": w(c.hidden, c.n_q * c.head_dim),
                "gate_up": w(2 * c.ffn, c.hidden), "down": w(c.hidden, c.ffn),
                "ln1": torch.ones(c.hidden, device=device, dtype=torch.float16),
                "ln2": torch.ones(c.hidden, device=device, dtype=torch.float16)})
        self.norm = torch.ones(c.hidden, device=device, dtype=torch.float16)
        self.lm_head = w(c.vocab, c.hidden)
        self._cache_args = (cache, sparsity, residual_length, max_tokens)
        self.reset_caches()
        self.attn_events = []   # (start, end) pairs around the cache's decode of every layer of timed steps

    def reset_caches(self):
        """Fresh, empty caches for every layer (a new prompt)."""
        self.caches = self.make_caches(*self._cache_args)

    def make_caches(self, cache, sparsity=0.7, residual_length=256, max_tokens=0):
        """One cache per layer of the kind `cache` (what reset_caches installs; also how a shadow set is made)."""
        c = self.cfg
        groups = c.n_q // c.n_kv
        if cache == "sparse":
            return [SparseKVCache(groups, c.head_dim, sparsity, sparsity, residual_length, fused=True,
                                         max_tokens=max_tokens, window_kernel=True) for _ in range(c.layers)]
        if cache in ("sparse_quant2", "sparse_quant4"):
            return [QuantSparseKVCache(groups, c.head_dim, sparsity, sparsity, residual_length,
                                       bit=int(cache[-1]), fused=True, window_kernel=True, max_tokens=max_tokens)
                    for _ in range(c.layers)]
        # the dense cache holds every token: the compressed capacity plus the largest window
        total = max_tokens + residual_length + CHUNK if max_tokens > 0 else 0
        return [self._dense_cache(groups, c.head_dim, sparsity, sparsity, residual_length, capacity=total)
                for _ in range(c.layers)]

    def _mlp(self, lw, x):
        # two products over the halves of the stacked weight: both results are contiguous, so the activation and
        # the gating run as vectorised elementwise kernels
        ffn = self.cfg.ffn
        gate, up = F.linear(x, lw["gate_up"][:ffn]), F.linear(x, lw["gate_up"][ffn:])
        return F.linear(F.silu(gate) * up, lw["down"])

    def _qkv(self, lw, x, tables, proj=None):
        """proj: the projection output of x, if the caller already has it (decode steps)."""
        c = self.cfg
        bs, L, _ = x.shape
        if L == 1:
            # decode step: one contiguous pass over all heads; the value heads go through with cos = 1, sin = 0
            cos, sin = tables
            H = c.n_q + 2 * c.n_kv
            if cos.shape[0] != H:
                one = torch.ones((c.n_kv, c.head_dim), dtype=cos.dtype, device=cos.device)
                cos = torch.cat([cos.expand(c.n_q + c.n_kv, -1), one], 0)
                sin = torch.cat([sin.expand(c.n_q + c.n_kv, -1), torch.zeros_like(one)], 0)
                tables[0], tables[1] = cos, sin        # built by the first layer of the step, reused by the others
            proj = F.linear(x, lw["qkv"]) if proj is None else proj
            qkv = _rope(proj.view(bs, H, c.head_dim), (cos, sin)).unsqueeze(2)
            return qkv[:, : c.n_q], qkv[:, c.n_q: c.n_q + c.n_kv], qkv[:, c.n_q + c.n_kv:]
        qkv = F.linear(x, lw["qkv"]).view(bs, L, c.n_q + 2 * c.n_kv, c.head_dim).transpose(1, 2)
        qk = _rope(qkv[:, : c.n_q + c.n_kv], tables)   # query and key heads in one pass; contiguous [bs, heads, L, D]
        return qk[:, : c.n_q], qk[:, c.n_q:], qkv[:, c.n_q + c.n_kv:].contiguous()

    @torch.no_grad()
    def prefill(self, ids, seq_chunk=4):
        """ids: [bs, L].  Returns the logits of the last position; fills the caches."""
        c = self.cfg
        bs, L = ids.shape
        tables = _rope_tables(torch.arange(L, device=self.dev), c.head_dim, c.rope_theta, torch.float16)
        half = c.head_dim // 2
        usin = torch.cat([-tables[1][:, :half], tables[1][:, half:]], -1)   # sin itself: the kernel rotates with rotate_half
        x = self.embed[ids]
        for li, (lw, cache) in enumerate(zip(self.layers, self.caches)):
            h = _rms_norm(x, lw["ln1"], c.rms_eps)
            # every cache of the layer gets the same keys and values: the model's own and, if set, its shadow
            takers = [cache] + ([self.shadow[li]] if self.shadow is not None else [])
            from_proj = [t for t in takers if self.proj_prefill and isinstance(t, SparseKVCache)]
            if from_proj:
                qkv = F.linear(h, lw["qkv"]).view(bs, L, c.n_q + 2 * c.n_kv, c.head_dim)
                q = _rope(qkv[:, :, : c.n_q].transpose(1, 2), tables)
                k, v = from_proj[0].prefill_proj(qkv[:, :, c.n_q: c.n_q + c.n_kv], qkv[:, :, c.n_q + c.n_kv:], tables[0],
                                                 usin)
            else:
                q, k, v = self._qkv(lw, h, tables)
                k = k.contiguous()
            outs = []
            for b0 in range(0, bs, seq_chunk):   # bounded working set of the prefill attention
                outs.append(F.scaled_dot_product_attention(q[b0:b0 + seq_chunk], k[b0:b0 + seq_chunk], v[b0:b0 + seq_chunk],
                                                           is_causal=True, enable_gqa=True))
            a = torch.cat(outs, 0).transpose(1, 2).reshape(bs, L, c.n_q * c.head_dim)
            for t in takers:
                if not (from_proj and t is from_proj[0]):
                    t.prefill(k, v)      # (rotated keys)
            x = x + F.linear(a, lw["o"])
            h = _rms_norm(x, lw["ln2"], c.rms_eps)
            for b0 in range(0, bs, seq_chunk):
                x[b0:b0 + seq_chunk] += self._mlp(lw, h[b0:b0 + seq_chunk])
        return F.linear(_rms_norm(x[:, -1:], self.norm, c.rms_eps), self.lm_head)

    @torch.no_grad()
    def step(self, ids, position, timed=False):
        """ids: [bs, 1] -> logits [bs, 1, vocab]."""
        pos = torch.tensor([position], device=self.dev)
        if all(getattr(c, "window_kernel", False) for c in self.caches):
            # the caches take the projection output as it is (one launch for rotation, query layout and window append)
            logits = self._layers(ids, pos, timed, None, from_proj=True)
            for cache in self.caches:
                cache.advance()
        else:
            logits = self._layers(ids, pos, timed, lambda cache, q, k, v: cache.decode(q, k, v))
        for cache in self.shadow or ():
            cache.advance()
        return logits

    def _layers(self, ids, pos, timed, attend, from_proj=False):
        """from_proj: the cache takes the new token's projection output as it is (decode_device_proj: rotation, window
        append and query layout in one launch); otherwise q, k, v are rotated here and handed over as tensors."""
        c = self.cfg
        tables = list(_rope_tables(pos, c.head_dim, c.rope_theta, torch.float16))   # once per step, shared by the layers
        shadow = self.shadow
        if from_proj or shadow is not None:
            half, nq, nk = c.head_dim // 2, c.n_q * c.head_dim, c.n_kv * c.head_dim
            cos = tables[0]
            usin = torch.cat([-tables[1][:, :half], tables[1][:, half:]], -1)   # sin itself, for rotate_half
        x = self.embed[ids]
        for li, (lw, cache) in enumerate(zip(self.layers, self.caches)):
            h = _rms_norm(x, lw["ln1"], c.rms_eps)
            proj = F.linear(h, lw["qkv"])
            qkv = proj.view(x.shape[0], -1)
            if not from_proj:
                q, k, v = self._qkv(lw, h, tables, proj=proj)
            if timed:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
            if from_proj:
                a = cache.decode_device_proj(qkv[:, :nq], qkv[:, nq: nq + nk], qkv[:, nq + nk:], cos, usin)
            else:
                a = attend(cache, q.contiguous(), k, v)
            if timed:
                e1.record()
                self.attn_events.append((e0, e1))
            if shadow is not None:
                sa = shadow[li].decode_device_proj(qkv[:, :nq], qkv[:, nq: nq + nk], qkv[:, nq + nk:], cos, usin)
                self.shadow_check(li, a, sa)
            x = x + F.linear(a.transpose(1, 2).reshape(x.shape[0], 1, c.n_q * c.head_dim), lw["o"])
            x = x + self._mlp(lw, _rms_norm(x, lw["ln2"], c.rms_eps))
        return F.linear(_rms_norm(x, self.norm, c.rms_eps), self.lm_head)


class GraphedGreedyLoop:
    """Greedy decoding with the whole step - embedding to argmax - replayed from a HIP graph.

    Everything that changes from step to step lives in device memory and is updated inside the graph: the token
    ids, the position (RoPE), the window length (one counter for all layers) and the compressed-token count of every
    layer's cache.  The host only counts (SparseKVCache.advance) and, every 256 tokens, lets the caches compress a chunk between two
    replays.  Pooled caches (max_tokens > 0) grow in place and the graph stays valid; a cache whose arrays move
    (the quantised one) reports it and the graph is captured again."""

    def __init__(self, dec, first_ids, position):
        self.dec = dec
        self.ids = first_ids.clone()
        self.pos = torch.tensor([position], device=dec.dev)
        self.graph = None
        self.captures = 0
        self.append_events = None    # a list: (start, end) HIP events around every chunk append are collected in it
        # the layers' windows grow in lockstep: one device counter, advanced by the first layer's cache
        for cache in dec.caches[1:]:
            cache.share_clock(dec.caches[0])

    @torch.no_grad()
    def _device_step(self):
        logits = self.dec._layers(self.ids, self.pos, False, None, from_proj=True)
        self.ids.copy_(logits[:, -1].argmax(-1, keepdim=True))
        self.pos += 1

    def _advance(self):
        grew = False
        before = self.dec.caches[0].compressed_length
        if self.append_events is not None:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
        for cache in self.dec.caches:
            grew |= cache.advance()
        if self.append_events is not None and self.dec.caches[0].compressed_length != before:
            e1.record()
            self.append_events.append((e0, e1))
        if grew:
            self.graph = None

    def step(self):
        """One token for every sequence; returns nothing (self.ids holds the new tokens on the device)."""
        if self.graph is None:
            # one eager step warms allocations up, then the next step is captured and replayed from then on
            self._device_step()
            self._advance()
            if self.graph is None:
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    self._device_step()
                self.graph = g
                self.captures += 1
            return
        self.graph.replay()
        self._advance()


def pool_tokens(total_tokens, residual_length=256):
    """Capacity of the compressed part of a cache that will hold total_tokens tokens: the compressed length is a
    multiple of the chunk and leaves at least residual_length tokens dense."""
    return max(CHUNK, ((total_tokens - residual_length) // CHUNK) * CHUNK)


def generate(dec, prompt_ids, new_tokens, forced=None):
    """Greedy decode (or teacher-forced with `forced` [bs, new_tokens]).  Returns (tokens, logits per step)."""
    logits = dec.prefill(prompt_ids)
    L = prompt_ids.shape[1]
    toks, all_logits = [], []
    for t in range(new_tokens):
        nxt = logits[:, -1].argmax(-1, keepdim=True) if forced is None else forced[:, t:t + 1]
        toks.append(nxt)
        logits = dec.step(nxt, L + t)
        all_logits.append(logits[:, 0].float())
    return torch.cat(toks, 1), all_logits


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--prompt", type=int, default=4096)
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--sparsity", type=float, default=0.7)
    ap.add_argument("--residual", type=int, default=256)
    ap.add_argument("--cache", default="sparse", choices=["sparse", "sparse_quant2", "sparse_quant4", "dense_masked"])
    ap.add_argument("--graph", action="store_true", help="replay the decode step from a HIP graph (sparse cache only)")
    ap.add_argument("--copy-prefill", action="store_true",
                    help="prefill through rotated, transposed, contiguous copies of K and V instead of compressing "
                         "them where the projection left them")
    args = ap.parse_args()
    dev = torch.device("cuda:0")
    cfg = Config(layers=args.layers)
    max_tokens = pool_tokens(args.prompt + args.new_tokens, args.residual)
    dec = Decoder(cfg, dev, cache=args.cache, sparsity=args.sparsity, residual_length=args.residual, max_tokens=max_tokens,
                  proj_prefill=not args.copy_prefill)
    g = torch.Generator(device=dev)
    g.manual_seed(1)
    ids = torch.randint(0, cfg.vocab, (args.batch, args.prompt), generator=g, device=dev)
    dec.prefill(ids)            # untimed: the first pass also pays for library start-up and kernel selection
    dec.reset_caches()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    logits = dec.prefill(ids)
    torch.cuda.synchronize()
    t_prefill = time.perf_counter() - t0
    nxt = logits[:, -1].argmax(-1, keepdim=True)
    warm = min(8, args.new_tokens // 4)
    loop = None
    if args.graph:
        assert args.cache.startswith("sparse")
        loop = GraphedGreedyLoop(dec, nxt, args.prompt)
        for t in range(warm):
            loop.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for t in range(warm, args.new_tokens):
            loop.step()
        torch.cuda.synchronize()
        t_dec = time.perf_counter() - t0
    else:
        for t in range(warm):
            nxt = dec.step(nxt, args.prompt + t)[:, -1].argmax(-1, keepdim=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for t in range(warm, args.new_tokens):
            nxt = dec.step(nxt, args.prompt + t, timed=True)[:, -1].argmax(-1, keepdim=True)
        torch.cuda.synchronize()
        t_dec = time.perf_counter() - t0
    steps = args.new_tokens - warm
    attn_ms = sum(a.elapsed_time(b) for a, b in dec.attn_events)
    print(json.dumps({
        "workload": "random-init Llama-3-8B shape, %d layers, batch %d, prompt %d, %d greedy tokens, residual %d, "
                    "%d-token chunks, %.0f%% K/V sparsity, cache=%s (%s)"
                    % (args.layers, args.batch, args.prompt, args.new_tokens, args.residual, CHUNK,
                       100 * args.sparsity, args.cache,
                       "decode step replayed from a HIP graph" if loop is not None
                       else "eager PyTorch around the cache operators"),
        "prefill_s": round(t_prefill, 3), "decode_ms_per_step": round(1e3 * t_dec / steps, 3),
        "tokens_per_s": round(args.batch * steps / t_dec, 1),
        "attention_over_cache_ms_per_step": round(attn_ms / steps, 3) if loop is None else None,
        "attention_share": round(attn_ms / (1e3 * t_dec), 4) if loop is None else None,
        "graph_captures": loop.captures if loop is not None else 0,
        "compressed_tokens_at_end": dec.caches[0].compressed_length}))


if __name__ == "__main__":
    main()
