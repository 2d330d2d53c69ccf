"""The decode-loop harness on a small model: the sparse cache (fused launch, pooled storage) against the dense masked
cache with the same weights and the same forced tokens - the logits of every step agree, across a chunk append."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_sparse_cache_tracks_dense_masked_cache_in_the_decode_loop():
    from mustafar_amd.harness import Config, Decoder, generate
    dev = torch.device("cuda:0")
    cfg = Config(hidden=512, layers=2, n_q=4, n_kv=2, head_dim=128, ffn=1024, vocab=1000)
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    bs, prompt, new = 2, 600, 180                      # Lc = 256 after prefill, one append at kv_len 768
    ids = torch.randint(0, cfg.vocab, (bs, prompt), generator=g, device=dev)
    ref = Decoder(cfg, dev, seed=11, cache="dense_masked")
    toks, ref_logits = generate(ref, ids, new)
    sp = Decoder(cfg, dev, seed=11, cache="sparse", max_tokens=1024)
    toks2, sp_logits = generate(sp, ids, new, forced=toks)
    assert sp.caches[0].compressed_length == ref.caches[0].compressed_length == 512
    assert int(sp.caches[0].k_pool.overflow) == 0
    worst = 0.0
    for a, b in zip(sp_logits, ref_logits):
        worst = max(worst, float((a - b).abs().max() / b.abs().max()))
    assert worst < 1e-2, worst
    # the greedy choice agrees wherever the reference's margin between its two best logits is not a rounding matter
    agree = total = 0
    for a, b in zip(sp_logits, ref_logits):
        top2 = b.topk(2, -1).values
        clear = (top2[:, 0] - top2[:, 1]) > 2e-2 * b.abs().max()
        agree += int((a.argmax(-1) == b.argmax(-1))[clear].sum())
        total += int(clear.sum())
    assert total > 0 and agree == total


def test_graphed_loop_generates_the_same_tokens_as_the_eager_loop():
    """The decode step replayed from a HIP graph (device-resident ids, position, window length and compressed-token
    count; the pooled cache grows in place, so ONE capture serves the whole loop, chunk append included) against the
    eager loop on the same model: same tokens."""
    from mustafar_amd.harness import Config, Decoder, GraphedGreedyLoop, generate
    dev = torch.device("cuda:0")
    cfg = Config(hidden=512, layers=2, n_q=4, n_kv=2, head_dim=128, ffn=1024, vocab=1000)
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    bs, prompt, new = 2, 600, 200                      # a chunk is appended at kv_len 768, between two replays
    ids = torch.randint(0, cfg.vocab, (bs, prompt), generator=g, device=dev)
    eager = Decoder(cfg, dev, seed=21, cache="sparse", max_tokens=1024)
    toks, _ = generate(eager, ids, new)
    graphed = Decoder(cfg, dev, seed=21, cache="sparse", max_tokens=1024)
    logits = graphed.prefill(ids)
    loop = GraphedGreedyLoop(graphed, logits[:, -1].argmax(-1, keepdim=True), prompt)
    got = [loop.ids.clone()]
    for t in range(new - 1):
        loop.step()
        got.append(loop.ids.clone())
    got = torch.cat(got, 1)
    assert loop.captures == 1 and graphed.caches[0].compressed_length == eager.caches[0].compressed_length == 512
    assert torch.equal(got, toks)


def test_prefill_from_the_projection_output_fills_the_same_cache():
    """Prompt keys / values compressed where the projection left them (keys rotated in the compressor's kernel)
    against the route through rotated, transposed, contiguous copies: the first layer's cache is identical bit for
    bit (its inputs are), the logits agree."""
    from mustafar_amd.harness import Config, Decoder
    dev = torch.device("cuda:0")
    cfg = Config(hidden=512, layers=2, n_q=4, n_kv=2, head_dim=128, ffn=1024, vocab=1000)
    g = torch.Generator(device=dev)
    g.manual_seed(9)
    ids = torch.randint(0, cfg.vocab, (3, 600), generator=g, device=dev)
    a = Decoder(cfg, dev, seed=4, cache="sparse", max_tokens=1024, proj_prefill=False)
    b = Decoder(cfg, dev, seed=4, cache="sparse", max_tokens=1024, proj_prefill=True)
    la, lb = a.prefill(ids), b.prefill(ids)
    ca, cb = a.caches[0], b.caches[0]
    assert ca.compressed_length == cb.compressed_length == 256
    for sa, sb in ((ca.k, cb.k), (ca.v, cb.v)):
        assert torch.equal(sa.bmp, sb.bmp) and torch.equal(sa.idx, sb.idx)
        assert torch.equal(sa.nz.view(torch.int16), sb.nz.view(torch.int16))
    assert torch.equal(ca.k_win.view(torch.int16), cb.k_win.view(torch.int16))
    assert torch.equal(ca.v_win.view(torch.int16), cb.v_win.view(torch.int16))
    assert float((la - lb).abs().max() / la.abs().max()) < 1e-2


def test_graphed_loop_over_the_quantised_pooled_cache_needs_one_capture():
    """The quantised cache in pooled form (per-tile arrays and packed words pre-allocated, chunks quantised in place):
    the graphed loop generates the eager loop's tokens with ONE capture across a chunk append."""
    from mustafar_amd.harness import Config, Decoder, GraphedGreedyLoop, generate
    dev = torch.device("cuda:0")
    cfg = Config(hidden=512, layers=2, n_q=4, n_kv=2, head_dim=128, ffn=1024, vocab=1000)
    g = torch.Generator(device=dev)
    g.manual_seed(6)
    bs, prompt, new = 2, 600, 200                      # a chunk is appended at kv_len 768, between two replays
    ids = torch.randint(0, cfg.vocab, (bs, prompt), generator=g, device=dev)
    eager = Decoder(cfg, dev, seed=23, cache="sparse_quant2", max_tokens=1024)
    toks, _ = generate(eager, ids, new)
    graphed = Decoder(cfg, dev, seed=23, cache="sparse_quant2", max_tokens=1024)
    logits = graphed.prefill(ids)
    loop = GraphedGreedyLoop(graphed, logits[:, -1].argmax(-1, keepdim=True), prompt)
    got = [loop.ids.clone()]
    for t in range(new - 1):
        loop.step()
        got.append(loop.ids.clone())
    got = torch.cat(got, 1)
    assert loop.captures == 1 and graphed.caches[0].compressed_length == eager.caches[0].compressed_length == 512
    assert torch.equal(got, toks)
