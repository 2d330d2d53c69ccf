"""Compressed KV cache of one attention layer: the state machine of the reference caller
(models/llama_mustafar_kernel.py:371-568) over the fused device operators.

  prefill : Lc = ((L - residual_length) // 256) * 256 tokens are pruned + compressed (:540-557),
            the rest stays dense as the local window (:550,558);
  decode  : the new token joins the window; scores = [key SpMV over the compressed part | q.K_win^T],
            / sqrt(d), fp32 softmax, output = value SpMV + P_win.V_win (:391-441); when
            (kv_len - residual_length - Lc) % 256 == 0 the oldest 256 window tokens are pruned,
            compressed and appended and Lc grows by 256 (:445-519).

The appended cache is byte-identical to a one-shot compression of the same tokens (per head the new
tiles, offsets and values follow the old ones, :461-511).
"""
import math

import torch

from . import ops
from ._lib import check, lib

CHUNK = 256


def _repeat_kv(x, groups):
    if groups == 1:
        return x
    bs, n_kv, L, D = x.shape
    return x[:, :, None].expand(bs, n_kv, groups, L, D).reshape(bs, n_kv * groups, L, D)


def append_compressed(old, new):
    """Concatenates two compressed ranges of the same heads (old tokens first)."""
    assert old.heads == new.heads and old.head_dim == new.head_dim and old.is_value == new.is_value
    bmp = torch.cat([old.bmp, new.bmp], dim=1)
    base = old.idx[:, -1:]
    idx = torch.cat([old.idx[:, :-1], new.idx + base], dim=1).contiguous()
    old_sz = (2 * old.idx[:, -1].to(torch.int64)).tolist()      # one host read per appended chunk
    new_sz = (2 * new.idx[:, -1].to(torch.int64)).tolist()
    pieces = []
    for a, b in zip(torch.split(old.packed(), old_sz), torch.split(new.packed(), new_sz)):
        pieces += [a, b]
    nz = torch.cat(pieces) if pieces else old.nz
    total = sum(old_sz) + sum(new_sz)
    if nz.numel() < 8:
        nz = torch.zeros(8, dtype=torch.float16, device=bmp.device)
    per_head = torch.tensor([a + b for a, b in zip(old_sz, new_sz)], dtype=torch.int64, device=bmp.device) // 8
    nz_off = torch.zeros_like(per_head)
    nz_off[1:] = torch.cumsum(per_head, 0)[:-1]
    return ops.CompressedKV(bmp, idx, nz, nz_off.to(torch.int32), old.tokens + new.tokens, old.head_dim, old.is_value,
                            total)


def slab_fraction_for(kth, head_dim):
    """Slab size, relative to the dense size, that holds any cache pruned to rank kth whose rows have no ties at the
    threshold: D - kth + 1 survivors per row plus the worst padding of every 64-element tile (7 values).  Ties add
    survivors (an all-equal row keeps everything), so a pool this size can still overflow: it then grows."""
    keep = (head_dim - int(kth) + 1) / head_dim if kth > 0 else 1.0
    return min(1.0, keep + 7.0 / 64.0)


class CompressedPool:
    """One side (keys or values) of a compressed cache that grows in place.

    Every head owns a slab of the packed-value pool (nz_off[b] = start of slab b, which the format allows); a chunk
    is compressed straight to the end of each head's values by mstf_append_*_f16, so appending re-copies no packed
    values and launches the same kernels whatever the cache holds.  The per-tile arrays are pre-allocated for
    max_tokens too (bmp_store [heads, tile_capacity], idx_store [heads, tile_capacity + 1]) and a chunk's bitmaps and
    offsets are written behind the ones that are there; the number of tokens held is mirrored in device memory
    (tokens_dev) for consumers recorded into a HIP graph (ops.decode_attention_window_pool).

    slab_fraction: slab size relative to the dense size of max_tokens tokens.  1.0 can never overflow; smaller saves
    memory (slab_fraction_for(kth, head_dim) holds every cache without ties at the pruning threshold: 0.42 of dense at
    70 % sparsity, so that values + bitmaps + offsets come to 0.52 of the dense bytes).  Every append reads the call's
    flag word back once (the host is between two decode steps there anyway): a chunk that did not fit a head's slab
    makes the pool grow - new, larger slabs, the old ones copied over, the same chunk appended again - and
    `generation` counts such moves (a HIP graph that holds the pool's addresses must then be captured again); a
    producer workgroup that gave up its bounded wait raises."""

    def __init__(self, heads, head_dim, max_tokens, is_value, device, slab_fraction=1.0):
        assert max_tokens % 64 == 0 and 0.0 < slab_fraction <= 1.0
        self.heads, self.head_dim, self.is_value, self.max_tokens = heads, head_dim, is_value, max_tokens
        self.device = device
        self.dense16 = max_tokens * head_dim * 2 // 16
        self.generation = 0
        self._alloc_slabs(max(1, min(self.dense16, (int(math.ceil(max_tokens * head_dim * 2 * slab_fraction)) + 15) // 16)))
        self.tile_capacity = max_tokens * head_dim // 64
        self.bmp_store = torch.zeros((heads, self.tile_capacity), dtype=torch.int64, device=device)
        self.idx_store = torch.zeros((heads, self.tile_capacity + 1), dtype=torch.int32, device=device)
        self.overflow = torch.zeros(1, dtype=torch.int32, device=device)
        self.tokens_dev = torch.zeros(1, dtype=torch.int32, device=device)
        self.tokens = 0

    def _alloc_slabs(self, slab16):
        self.slab16 = slab16
        self.slab_fraction = slab16 / self.dense16
        self.nz = torch.zeros(self.heads * slab16 * 8, dtype=torch.float16, device=self.device)
        self.nz_off = (torch.arange(self.heads, device=self.device, dtype=torch.int64) * slab16).to(torch.int32)
        self.limit = (self.nz_off.to(torch.int64) + slab16).to(torch.int32)

    @property
    def tiles(self):
        return self.tokens * self.head_dim // 64

    @property
    def bmp(self):
        """Bitmaps of the tokens held, [heads, tiles] (a view of the pre-allocated array: rows are tile_capacity apart)."""
        return self.bmp_store[:, :self.tiles]

    @property
    def idx(self):
        return self.idx_store[:, :self.tiles + 1]

    def allocated_bytes(self):
        """Device bytes the pool holds: packed values, bitmaps, offsets."""
        return self.nz.numel() * 2 + self.bmp_store.numel() * 8 + self.idx_store.numel() * 4 + self.nz_off.numel() * 8

    def _publish(self, bmp_c, idx_c, M):
        """Writes a chunk's bitmaps and offsets (counted from the chunk's first value) behind the ones held."""
        T0, Tc = self.tiles, bmp_c.shape[1]
        self.bmp_store[:, T0:T0 + Tc] = bmp_c
        self.idx_store[:, T0 + 1:T0 + Tc + 1] = idx_c[:, 1:] + self.idx_store[:, T0:T0 + 1]
        self.tokens += M
        self.tokens_dev += M

    def _grow_slabs(self):
        """After a chunk that did not fit: slabs large enough for what the heads hold now (the chunk's offsets were
        published although its values were not written), scaled to the capacity in tokens, at least a quarter more."""
        need16 = (int(self.idx_store[:, self.tiles].max().item()) + 3) // 4
        scaled = int(math.ceil(need16 * (self.max_tokens / self.tokens) * 1.0625))
        new16 = min(self.dense16, max(scaled, int(math.ceil(self.slab16 * 1.25)), need16))
        if new16 <= self.slab16:
            raise RuntimeError("compressed pool overflow at the dense slab size: the appended rows are not [*, %d] fp16 "
                               "tokens of this pool" % self.head_dim)
        old, old16 = self.nz, self.slab16
        self._alloc_slabs(new16)
        self.nz.view(self.heads, new16 * 8)[:, :old16 * 8].copy_(old.view(self.heads, old16 * 8))
        self.generation += 1

    def _append_checked(self, launch, M):
        """launch(): one append call for the chunk at the pool's current end, published.  Reads the flag word back,
        grows and appends again on overflow."""
        launch()
        for attempt in range(2):
            flag = int(self.overflow.item())
            if flag & 2:
                raise RuntimeError("the compressor gave up waiting for an earlier workgroup; the appended chunk is "
                                   "incomplete and the pool is no longer usable")
            if not (flag & 1):
                return
            if attempt == 1:
                raise RuntimeError("compressed pool overflow after growing")
            self.overflow.zero_()
            self._grow_slabs()
            self.tokens -= M          # the chunk is appended again at the same place
            self.tokens_dev -= M
            launch()

    def append(self, x, kth, ws=None):
        """x: [heads, M, head_dim] fp16, M % 64 == 0.  ws: the caller's ops.Workspace (default: the stream's)."""
        B, M, N = x.shape
        assert B == self.heads and N == self.head_dim and M % 64 == 0 and self.tokens + M <= self.max_tokens
        x = x.contiguous()
        L = lib()
        Tc = M * N // 64
        wsb = L.mstf_compress_workspace_bytes(B, M, N)
        fn = L.mstf_append_value_f16 if self.is_value else L.mstf_append_key_f16

        def launch():
            bmp_c = torch.empty((B, Tc), dtype=torch.int64, device=x.device)
            idx_c = torch.empty((B, Tc + 1), dtype=torch.int32, device=x.device)
            dst = self.nz_off + self.idx_store[:, self.tiles] // 4          # 16-byte units; idx counts 4-byte units
            w = ops.workspace(x.device, wsb, ws)
            check(fn(torch.cuda.current_stream().cuda_stream, x.data_ptr(), B, M, N, int(kth), bmp_c.data_ptr(),
                     idx_c.data_ptr(), dst.data_ptr(), self.limit.data_ptr(), self.nz.data_ptr(), self.overflow.data_ptr(),
                     w.data_ptr(), w.numel()), "mstf_append_f16")
            self._publish(bmp_c, idx_c, M)
        self._append_checked(launch, M)

    def append_proj(self, x, kth, M, cos=None, sin=None, rot=None, ws=None):
        """The first M tokens of x [batch, rows, heads per batch entry, head_dim] (a view of the projection output,
        ops.proj_source) without a contiguous copy; with cos / sin all rows are rotated into rot (default: in place)
        before the first M are compressed."""
        import ctypes
        src, rot = ops.proj_source(x, cos, sin, rot)
        B, N = x.shape[0] * x.shape[2], x.shape[3]
        assert B == self.heads and N == self.head_dim and M % 64 == 0 and self.tokens + M <= self.max_tokens
        L = lib()
        Tc = M * N // 64
        wsb = L.mstf_compress_workspace_bytes(B, max(M, 64), N)
        state = {"src": src}

        def launch():
            bmp_c = torch.empty((B, Tc), dtype=torch.int64, device=x.device)
            idx_c = torch.empty((B, Tc + 1), dtype=torch.int32, device=x.device)
            dst = self.nz_off + self.idx_store[:, self.tiles] // 4
            w = ops.workspace(x.device, wsb, ws)
            check(L.mstf_append_proj_f16(torch.cuda.current_stream().cuda_stream, ctypes.byref(state["src"]),
                                         int(self.is_value), M, N, int(kth), bmp_c.data_ptr(), idx_c.data_ptr(),
                                         dst.data_ptr(), self.limit.data_ptr(), self.nz.data_ptr(),
                                         self.overflow.data_ptr(), w.data_ptr(), w.numel()), "mstf_append_proj_f16")
            if M > 0:
                self._publish(bmp_c, idx_c, M)
            # a second attempt (after growing) finds the rows already rotated where `rot` put them
            if cos is not None:
                state["src"], _ = ops.proj_source(rot)
        if M > 0:
            self._append_checked(launch, M)
        else:
            launch()
        return rot

    def view(self):
        """The cache as the operators take it (ops.key_spmv / value_spmv / decode_attention)."""
        return ops.CompressedKV(self.bmp.contiguous(), self.idx.contiguous(), self.nz, self.nz_off, self.tokens,
                                self.head_dim, self.is_value, None)

    def head_values(self, b):
        """Packed values of head b (a host read: for tests and debugging)."""
        n = 2 * int(self.idx[b, -1])
        start = 8 * int(self.nz_off[b])
        return self.nz[start:start + n]


def packed_fraction_for(kth, head_dim, bit):
    """Word-buffer size of a QuantPool, relative to the worst case (every element kept), that holds any cache pruned
    to rank kth without ties at the threshold: per 64-token block 64 * (D - kth + 1) codes in D tiles, each tile
    rounded up to whole words of 32 / bit codes."""
    if kth <= 0:
        return 1.0
    cap = 32 // bit
    tiles = head_dim                # tiles of one side of a 64-token block
    codes = 64 * (head_dim - int(kth) + 1)
    words = codes / cap + tiles * (cap - 1) / cap
    return min(1.0, words / (tiles * 64 / cap))


def append_pair(k_pool, v_pool, xk, xv, kth_k, kth_v, ws=None):
    """k_pool.append(xk, kth_k) and v_pool.append(xv, kth_v) of the same tokens as one call (mstf_append_kv_f16: both
    sides in one launch, identical results).  The sides share one flag word; should a slab overflow, the chunk is
    taken back and appended again side by side, where each pool grows its own slabs."""
    B, M, N = xk.shape
    assert xv.shape == xk.shape and not k_pool.is_value and v_pool.is_value
    for p in (k_pool, v_pool):
        assert B == p.heads and N == p.head_dim and M % 64 == 0 and p.tokens + M <= p.max_tokens
    xk, xv = xk.contiguous(), xv.contiguous()
    L = lib()
    Tc = M * N // 64
    dev = xk.device
    chunk = [(torch.empty((B, Tc), dtype=torch.int64, device=dev), torch.empty((B, Tc + 1), dtype=torch.int32, device=dev),
              p.nz_off + p.idx_store[:, p.tiles] // 4) for p in (k_pool, v_pool)]
    w = ops.workspace(dev, L.mstf_compress_kv_workspace_bytes(B, M, N), ws)
    (kb, ki, kd), (vb, vi, vd) = chunk
    check(L.mstf_append_kv_f16(torch.cuda.current_stream().cuda_stream, xk.data_ptr(), xv.data_ptr(), B, M, N, int(kth_k),
                               int(kth_v), kb.data_ptr(), ki.data_ptr(), kd.data_ptr(), k_pool.limit.data_ptr(),
                               k_pool.nz.data_ptr(), vb.data_ptr(), vi.data_ptr(), vd.data_ptr(), v_pool.limit.data_ptr(),
                               v_pool.nz.data_ptr(), k_pool.overflow.data_ptr(), w.data_ptr(), w.numel()),
          "mstf_append_kv_f16")
    k_pool._publish(kb, ki, M)
    v_pool._publish(vb, vi, M)
    flag = int(k_pool.overflow.item())
    if flag & 2:
        raise RuntimeError("the compressor gave up waiting for an earlier workgroup; the appended chunk is incomplete "
                           "and the pools are no longer usable")
    if flag & 1:
        k_pool.overflow.zero_()
        for p in (k_pool, v_pool):
            p.tokens -= M
            p.tokens_dev -= M
        k_pool.append(xk, kth_k, ws)
        v_pool.append(xv, kth_v, ws)


class QuantPool:
    """One side (keys or values) of a quantised cache that grows in place.

    Bitmaps, word offsets, counts, units, scales and zero-points are pre-allocated for max_tokens tokens
    ([heads, tile_capacity] each) and so is the buffer of packed words, sized `packed_fraction` of the worst case
    (every element kept; packed_fraction_for(kth, head_dim, bit) holds every cache without ties at the pruning
    threshold: 0.55 of the worst case for 2-bit codes at 70 % sparsity).  A chunk is quantised straight behind the
    words of the chunks before it - the producer's word total is read back once per append, which also tells a
    producer that gave up - and its per-tile arrays are written behind the ones held, the offsets shifted by the
    chunk's start.  A chunk that does not fit makes the buffer grow (a larger one, the old words copied, the chunk
    quantised again; `generation` counts such moves); otherwise no array ever moves (the reference concatenates all
    seven per chunk, models/llama_mustafar_quant_kernel.py:322-345).  The number of tokens held is mirrored in device
    memory (tokens_dev) for consumers recorded into a HIP graph
    (mustafar_package_quant.decode_attention_window_quant_pool)."""

    SLACK_WORDS = 64     # behind the last word: the consumers fetch a block's words in 16-byte pieces

    def __init__(self, heads, head_dim, max_tokens, is_value, bit, device, packed_fraction=1.0):
        assert max_tokens % 64 == 0 and bit in (2, 4, 8) and 0.0 < packed_fraction <= 1.0
        self.heads, self.head_dim, self.is_value, self.max_tokens, self.bit = heads, head_dim, is_value, max_tokens, bit
        self.tile_capacity = max_tokens * head_dim // 64
        T = self.tile_capacity

        def store(dtype):
            return torch.zeros((heads, T), dtype=dtype, device=device)

        self.bmp_store, self.off_store = store(torch.int64), store(torch.int32)
        self.counts_store, self.units_store = store(torch.int32), store(torch.int32)
        self.scales_store, self.zeros_store = store(torch.float16), store(torch.float16)
        self.worst_words = heads * max_tokens * head_dim * bit // 32
        assert self.worst_words < 2 ** 31, "tile offsets are 32-bit word offsets into one buffer, as in the reference's format"
        self.capacity_words = max(1, min(self.worst_words, int(math.ceil(self.worst_words * packed_fraction))))
        self.packed = torch.zeros(self.capacity_words + self.SLACK_WORDS, dtype=torch.int32, device=device)
        self.generation = 0
        self.reserved = 0            # words in use
        self.tokens_dev = torch.zeros(1, dtype=torch.int32, device=device)
        self.tokens = 0

    @property
    def tiles(self):
        return self.tokens * self.head_dim // 64

    def allocated_bytes(self):
        """Device bytes the pool holds: packed words and the six per-tile arrays."""
        per_tile = sum(t.numel() * t.element_size() for t in (self.bmp_store, self.off_store, self.counts_store,
                                                               self.units_store, self.scales_store, self.zeros_store))
        return self.packed.numel() * 4 + per_tile

    def _grow_packed(self, need_words, tokens_after):
        scaled = int(math.ceil(need_words * (self.max_tokens / tokens_after) * 1.0625))
        new_cap = min(self.worst_words, max(scaled, int(math.ceil(self.capacity_words * 1.25)), need_words))
        if new_cap < need_words:
            raise RuntimeError("quantised pool overflow at the worst-case buffer size")
        old = self.packed
        self.packed = torch.zeros(new_cap + self.SLACK_WORDS, dtype=torch.int32, device=old.device)
        self.packed[:self.reserved].copy_(old[:self.reserved])
        self.capacity_words = new_cap
        self.generation += 1

    def append(self, x, kth, ws=None):
        """x: [heads, M, head_dim] fp16, M % 64 == 0, pruned here to rank kth (0: already pruned)."""
        from . import compression_quant as cq
        B, M, N = x.shape
        assert B == self.heads and N == self.head_dim and M % 64 == 0 and self.tokens + M <= self.max_tokens
        for attempt in range(2):
            room = self.packed[self.reserved:self.capacity_words]
            bmp, off, _, counts, units, scales, zeros, total = cq._produce(x, self.is_value, self.bit, kth, 64, ws, room)
            words = cq.words_written(total)      # one host read; raises if the producer gave up
            if words <= room.numel():
                break
            if attempt == 1:
                raise RuntimeError("quantised pool overflow after growing")
            self._grow_packed(self.reserved + words, self.tokens + M)   # the tiles that did not fit were left unwritten
        T0, Tc = self.tiles, bmp.shape[1]
        self.bmp_store[:, T0:T0 + Tc] = bmp
        self.off_store[:, T0:T0 + Tc] = off + self.reserved
        self.counts_store[:, T0:T0 + Tc] = counts
        self.units_store[:, T0:T0 + Tc] = units
        self.scales_store[:, T0:T0 + Tc] = scales
        self.zeros_store[:, T0:T0 + Tc] = zeros
        self.reserved += words
        self.tokens += M
        self.tokens_dev += M

    def check(self):
        """Kept for callers of the earlier interface: every append already checks its own producer call."""

    def view(self):
        """The side as the reference's operators take it: [bitmaps, tile_offsets, packed, counts, units, scales,
        zeros] with contiguous per-tile arrays of the tokens held (copies; the packed buffer is the pool's own)."""
        T = self.tiles
        return [self.bmp_store[:, :T].contiguous(), self.off_store[:, :T].contiguous(), self.packed,
                self.counts_store[:, :T].contiguous(), self.units_store[:, :T].contiguous(),
                self.scales_store[:, :T].contiguous(), self.zeros_store[:, :T].contiguous()]


class SparseKVCache:
    def __init__(self, groups, head_dim=128, k_sparsity=0.7, v_sparsity=0.7, residual_length=256, fused=False,
                 max_tokens=0, window_kernel=False, pool_fraction=None):
        """fused: the compressed part of a decode step is one launch (ops.decode_attention) whose (max, sum) joins
        the dense window under one softmax, instead of the reference's key SpMV / softmax / value SpMV sequence.
        max_tokens > 0: the compressed part lives in pre-allocated pools (CompressedPool) and grows in place.
        pool_fraction: size of the pools' value buffers relative to the dense / worst-case size (None: what the
        sparsities need when no row has ties at its threshold - slab_fraction_for / packed_fraction_for; a pool that
        turns out too small grows, see CompressedPool).
        window_kernel: the dense window lives in a pre-allocated buffer and the whole attention of a step - compressed
        tokens and window - is ops.decode_attention_window (three launches, no torch operators)."""
        self.groups, self.head_dim, self.residual_length = groups, head_dim, residual_length
        self.fused = fused or window_kernel
        self.window_kernel = window_kernel
        self._kbuf = self._vbuf = None      # [bs * n_kv, residual_length + CHUNK, D], first _wlen tokens valid
        self._wlen = 0
        self.max_tokens = max_tokens
        # decode_device_proj over a pooled cache as mstf_decode_step_pool_f16 (two launches) instead of the append call
        # followed by the attention call (four); the results are identical
        self.step_launch = True
        self.pool_fraction = pool_fraction
        self._pool_gen = (0, 0)
        self.k_pool = self.v_pool = None
        self.kth_k = ops.kth_from_sparsity(k_sparsity, head_dim)
        self.kth_v = ops.kth_from_sparsity(v_sparsity, head_dim)
        self.k = self.v = None              # CompressedKV
        self.k_win = self.v_win = None      # [bs, n_kv, Lw, D] dense
        self.compressed_length = 0
        self.kv_len = 0
        self.ws = None                      # ops.Workspace of this cache: never shared with another cache or stream

    def _workspace(self, device):
        if self.ws is None:
            self.ws = ops.Workspace(device)
        return self.ws

    def _make_pools(self, heads, D, device):
        fk = self.pool_fraction if self.pool_fraction is not None else slab_fraction_for(self.kth_k, D)
        fv = self.pool_fraction if self.pool_fraction is not None else slab_fraction_for(self.kth_v, D)
        self.k_pool = CompressedPool(heads, D, self.max_tokens, False, device, fk)
        self.v_pool = CompressedPool(heads, D, self.max_tokens, True, device, fv)

    def pools_moved(self):
        """True once after a pool replaced its value buffer (it had to grow): addresses a HIP graph captured are stale."""
        gen = (self.k_pool.generation, self.v_pool.generation) if self.k_pool is not None else (0, 0)
        moved = gen != self._pool_gen
        self._pool_gen = gen
        return moved

    def kv_bytes(self):
        """(bytes the compressed part holds on the device, bytes of the dense window buffers)."""
        pool = self.k_pool.allocated_bytes() + self.v_pool.allocated_bytes() if self.k_pool is not None else 0
        win = 2 * self._kbuf.numel() * 2 if self._kbuf is not None else 0
        return pool, win

    def _grow(self, K, V):
        """Adds the tokens K, V [bs, n_kv, M, D] to the compressed part."""
        bs, n_kv, M, D = K.shape
        if self.max_tokens > 0:
            if self.k_pool is None:
                self._make_pools(bs * n_kv, D, K.device)
            ws = self._workspace(K.device)
            append_pair(self.k_pool, self.v_pool, K.reshape(bs * n_kv, M, D), V.reshape(bs * n_kv, M, D), self.kth_k,
                        self.kth_v, ws)
            self._pool_views()
            return
        ck, cv = self._compress(K, V)
        self.k = ck if self.k is None else append_compressed(self.k, ck)
        self.v = cv if self.v is None else append_compressed(self.v, cv)

    def _pool_views(self):
        """After an append to the pools.  With window_kernel the attention reads the pools themselves (nothing to
        rebuild); the operator-by-operator paths take contiguous per-tile arrays, copied here."""
        if self.window_kernel:
            self.k, self.v = self.k_pool, self.v_pool
        else:
            self.k, self.v = self.k_pool.view(), self.v_pool.view()

    def _compress(self, K, V):
        bs, n_kv, L, D = K.shape
        ws = self._workspace(K.device)
        ck = ops.compress(K.reshape(bs * n_kv, L, D), False, kth=self.kth_k, ws=ws)
        cv = ops.compress(V.reshape(bs * n_kv, L, D), True, kth=self.kth_v, ws=ws)
        return ck, cv

    def prefill_proj(self, kx, vx, cos, sin):
        """Prefill straight from the projection outputs kx, vx [bs, L, n_kv, D] (views of [bs, L, n_kv * D]; the keys
        not yet rotated) and the rotary factors cos, sin [L, D] or [bs, L, D]: the keys are rotated in place, the
        first Lc tokens of both sides are compressed from where they lie (no transposed or contiguous copy), the rest
        becomes the dense window.  Returns the rotated keys and the values as [bs, n_kv, L, D] views for the prefill
        attention (models/llama_mustafar_kernel.py:373-374, 531-560 in one pass over K and one over V)."""
        bs, L, n_kv, D = kx.shape
        Lc = ((L - self.residual_length) // CHUNK) * CHUNK if L > self.residual_length else 0
        if self.max_tokens > 0:
            if self.k_pool is None:
                self._make_pools(bs * n_kv, D, kx.device)
            ws = self._workspace(kx.device)
            self.k_pool.append_proj(kx, self.kth_k, Lc, cos, sin, ws=ws)
            if Lc > 0:
                self.v_pool.append_proj(vx, self.kth_v, Lc, ws=ws)
                self._pool_views()
        else:
            ws = self._workspace(kx.device)
            ck, _ = ops.compress_proj(kx, False, self.kth_k, Lc, cos, sin, ws=ws)
            if Lc > 0:
                cv, _ = ops.compress_proj(vx, True, self.kth_v, Lc, ws=ws)
                self.k, self.v = ck, cv
        K, V = kx.transpose(1, 2), vx.transpose(1, 2)
        self._prefill_window(K, V, Lc)
        return K, V

    def prefill(self, K, V):
        """K, V: [bs, n_kv, L, D] fp16 (after RoPE)."""
        L = K.shape[2]
        Lc = ((L - self.residual_length) // CHUNK) * CHUNK if L > self.residual_length else 0
        if Lc > 0:
            self._grow(K[:, :, :Lc].contiguous(), V[:, :, :Lc].contiguous())
        self._prefill_window(K, V, Lc)

    def _prefill_window(self, K, V, Lc):
        L = K.shape[2]
        self.compressed_length, self.kv_len = Lc, L
        if self.window_kernel:
            bs, n_kv, _, D = K.shape
            if self.max_tokens > 0 and self.k_pool is None:
                # nothing compressed yet: the (empty) pools exist from the start, so the attention call never changes form
                self._make_pools(bs * n_kv, D, K.device)
            cap = max(self.residual_length + CHUNK, L - Lc)   # the window never holds more before a chunk leaves
            self._kbuf = torch.empty((bs * n_kv, cap, D), dtype=torch.float16, device=K.device)
            self._vbuf = torch.empty_like(self._kbuf)
            self._wlen = L - Lc
            self._wlen_dev = torch.full((1,), self._wlen, dtype=torch.int32, device=K.device)   # valid rows
            self._owns_clock, self._clock_shared = True, False
            self._wovf = torch.zeros((1,), dtype=torch.int32, device=K.device)   # set by an append past the buffer
            self._kbuf[:, :self._wlen] = K[:, :, Lc:].reshape(bs * n_kv, self._wlen, D)
            self._vbuf[:, :self._wlen] = V[:, :, Lc:].reshape(bs * n_kv, self._wlen, D)
            self._shape = (bs, n_kv, D)
            self._window_views()
            return
        self.k_win = K[:, :, Lc:].contiguous().clone()
        self.v_win = V[:, :, Lc:].contiguous().clone()

    def _window_views(self):
        bs, n_kv, D = self._shape
        self.k_win = self._kbuf[:, :self._wlen].view(bs, n_kv, self._wlen, D)
        self.v_win = self._vbuf[:, :self._wlen].view(bs, n_kv, self._wlen, D)

    def share_clock(self, other):
        """Caches that advance in lockstep (the layers of one model) can read the window length from one device
        counter: this cache takes `other`'s and no longer advances it - the owner's decode_device does, once per step,
        before any of the sharers runs."""
        self._wlen_dev = other._wlen_dev
        self._owns_clock = False
        other._clock_shared = True

    def decode_device(self, q, k_new, v_new):
        """The device work of a decode step in window_kernel mode: append the token to the window, attend.  Only
        device memory changes (the window length is a device counter), so the call can be captured in a HIP graph and
        replayed; the host-side bookkeeping of the step is advance()."""
        bs, n_q, _, D = q.shape
        n_kv = self._shape[1]
        if self._owns_clock:
            self._wlen_dev += 1
        ops.window_append(k_new.reshape(bs, n_kv * D), v_new.reshape(bs, n_kv * D), self._kbuf, self._vbuf,
                          self._wlen + 1, win_len_dev=self._wlen_dev, overflow=self._wovf)
        return self._attend_device(q.reshape(bs * n_q, D).contiguous()).view(bs, n_q, 1, D)

    def decode_device_proj(self, q_in, k_in, v_in, cos, sin):
        """decode_device straight from the projection outputs of the new token, q_in [bs, n_q * D], k_in / v_in
        [bs, n_kv * D] (slices of one fused projection are fine), not yet rotated: rotation of query and key heads
        with cos, sin [D] or [bs, D] (sin itself, for rotate_half), the append to the window and the query layout are
        one launch (ops.window_append) in front of the attention.  Returns [bs, n_q, 1, D]."""
        bs, D = q_in.shape[0], self._shape[2]
        n_q = q_in.shape[1] // D
        if self._owns_clock:
            self._wlen_dev += 1
        if self.step_launch and self.k_pool is not None:
            # rotation, append and the attention over the window inside the launch of the compressed tokens
            return self._step_device(q_in, k_in, v_in, cos, sin).view(bs, n_q, 1, D)
        q2 = ops.window_append(k_in, v_in, self._kbuf, self._vbuf, self._wlen + 1, q_in=q_in, cos=cos, sin=sin,
                               win_len_dev=self._wlen_dev, overflow=self._wovf)
        return self._attend_device(q2).view(bs, n_q, 1, D)

    def _step_device(self, q_in, k_in, v_in, cos, sin):
        """The cache side of a step from the projection outputs in two launches; returns [Bq, D]."""
        return ops.decode_step_pool(self.k_pool, self.v_pool, q_in, k_in, v_in, self._kbuf, self._vbuf,
                                    self._kbuf.shape[1], cos, sin, win_len_dev=self._wlen_dev, overflow=self._wovf,
                                    ws=self._workspace(q_in.device))

    def _attend_device(self, q2):
        """Attention of the query rows q2 [Bq, D] over [compressed | window buffer] (three launches)."""
        if self.k_pool is not None:
            return ops.decode_attention_window_pool(self.k_pool, self.v_pool, q2, self._kbuf, self._vbuf,
                                                    self._kbuf.shape[1], self.groups, self._wlen_dev,
                                                    ws=self._workspace(q2.device))
        return ops.decode_attention_window(self.k, self.v, q2, self._kbuf, self._vbuf, self._kbuf.shape[1], self.groups,
                                           win_len_dev=self._wlen_dev, ws=self._workspace(q2.device))

    def advance(self):
        """Host-side bookkeeping after decode_device (or a replay of it): counts the token and, when the window holds
        residual_length + 256 tokens, compresses its oldest 256.  Returns True when arrays of the compressed part moved
        (a captured graph must then be captured again): with pools (max_tokens > 0), which grow in place, only when a
        pool's value buffer turned out too small and was replaced by a larger one."""
        bs, n_kv, D = self._shape
        self.kv_len += 1
        self._wlen += 1
        grew = False
        if (self.kv_len - self.residual_length - self.compressed_length) % CHUNK == 0 and self._wlen >= CHUNK:
            self._grow(self._kbuf[:, :CHUNK].reshape(bs, n_kv, CHUNK, D), self._vbuf[:, :CHUNK].reshape(bs, n_kv, CHUNK, D))
            rest = self._wlen - CHUNK
            self._kbuf[:, :rest] = self._kbuf[:, CHUNK:self._wlen].clone()
            self._vbuf[:, :rest] = self._vbuf[:, CHUNK:self._wlen].clone()
            if int(self._wovf.item()) != 0:
                raise RuntimeError("a token was appended past the end of the window buffer")
            self._wlen = rest
            self._wlen_dev.fill_(rest)
            self.compressed_length += CHUNK
            grew = self.k_pool is None or self.pools_moved()
        self._window_views()
        return grew

    def _decode_window_kernel(self, q, k_new, v_new):
        if not self._owns_clock or self._clock_shared:
            raise RuntimeError("caches that share a window counter advance together: decode_device on every cache, "
                               "then advance on every cache")
        out = self.decode_device(q, k_new, v_new)
        self.advance()
        return out

    def _decode_fused(self, q, s_loc):
        """One launch over the compressed tokens, then a log-sum-exp merge with the dense window."""
        bs, n_q, _, D = q.shape
        g = self.groups
        lse = torch.empty((bs * n_q, 2), dtype=torch.float32, device=q.device)
        o_c = ops.decode_attention(self.k, self.v, q.reshape(bs * n_q, D).contiguous(), g, lse=lse,
                                   ws=self._workspace(q.device))
        m_c = lse[:, 0].view(bs, n_q, 1, 1)
        l_c = lse[:, 1].view(bs, n_q, 1, 1)
        w = (s_loc / ops.sqrt_head_dim(D)).float()        # fp16 division first, as for the compressed scores
        M = torch.maximum(m_c, w.amax(-1, keepdim=True))
        p = torch.exp(w - M)
        a = l_c * torch.exp(m_c - M)
        num = a * o_c.view(bs, n_q, 1, D).float() + torch.matmul(p, _repeat_kv(self.v_win, g).float())
        return (num / (a + p.sum(-1, keepdim=True))).half()

    def decode(self, q, k_new, v_new):
        """q: [bs, n_q, 1, D]; k_new, v_new: [bs, n_kv, 1, D].  Returns the attention output [bs, n_q, 1, D]."""
        if self.window_kernel:
            return self._decode_window_kernel(q, k_new, v_new)
        bs, n_q, _, D = q.shape
        g, Lc = self.groups, self.compressed_length
        self.kv_len += 1
        self.k_win = torch.cat([self.k_win, k_new], dim=2)
        self.v_win = torch.cat([self.v_win, v_new], dim=2)
        s_loc = torch.matmul(q, _repeat_kv(self.k_win, g).transpose(2, 3))            # [bs, n_q, 1, Lw]
        if self.fused and Lc > 0:
            out = self._decode_fused(q, s_loc)
        elif Lc > 0:
            s_cmp = ops.key_spmv(self.k, q.reshape(bs * n_q, 1, D).contiguous(), g).view(bs, n_q, 1, Lc)
            s = torch.cat([s_cmp, s_loc], dim=-1)
        else:
            s = s_loc
        if not (self.fused and Lc > 0):
            p = ops.scale_softmax(s.contiguous(), D)
            out = torch.matmul(p[..., Lc:], _repeat_kv(self.v_win, g))
            if Lc > 0:
                o_cmp = ops.value_spmv(self.v, p[..., :Lc].reshape(bs * n_q, 1, Lc).contiguous(), g,
                                       ws=self._workspace(q.device))
                out = out + o_cmp.view(bs, n_q, 1, D)
        if (self.kv_len - self.residual_length - Lc) % CHUNK == 0 and self.k_win.shape[2] >= CHUNK:
            self._grow(self.k_win[:, :, :CHUNK].contiguous(), self.v_win[:, :, :CHUNK].contiguous())
            self.k_win = self.k_win[:, :, CHUNK:].contiguous()
            self.v_win = self.v_win[:, :, CHUNK:].contiguous()
            self.compressed_length += CHUNK
        return out


class QuantSparseKVCache(SparseKVCache):
    """The quantised caller's state machine (models/llama_mustafar_quant_kernel.py:305-345, 425-575): prefill split,
    a dense local window, 256-token chunks pruned + quantised + appended, decode over [compressed | window].

    The compressed sides are the reference's 7-element lists [bitmaps, tile_offsets, packed, counts, units, scales,
    zeros]; a chunk is appended as the reference does it (:322-345): its packed words go behind the existing ones
    and its tile offsets are shifted by the old size, the per-tile arrays are concatenated along the tile axis.  A
    head's tiles are then no longer contiguous across chunks, which the consumers allow: they only rely on the
    words of one 64-token block being contiguous.

    fused: the compressed part of a step is one launch (decode_attention_quant) whose (max, sum) joins the dense
    window under one softmax; otherwise the reference's key formulation -> softmax -> value formulation sequence.
    window_kernel: as in SparseKVCache - the window in a pre-allocated buffer, the whole attention of a step as
    decode_attention_window_quant (three launches, capturable with decode_device / advance)."""

    def __init__(self, groups, head_dim=128, k_sparsity=0.7, v_sparsity=0.7, residual_length=256, bit=2,
                 dequant_mode=0, fused=False, window_kernel=False, max_tokens=0, pool_fraction=None):
        """max_tokens > 0: the compressed part lives in pre-allocated pools (QuantPool) and grows in place, pruning
        fused into the producer; with window_kernel the attention reads the pools themselves and a captured decode
        step stays valid across chunk appends."""
        super().__init__(groups, head_dim, k_sparsity, v_sparsity, residual_length, fused=fused,
                         window_kernel=window_kernel, max_tokens=max_tokens, pool_fraction=pool_fraction)
        self.bit, self.dequant_mode = bit, dequant_mode
        # self.k / self.v: 7-element lists [bitmaps, tile_offsets, packed, counts, units, scales, zeros]

    def _step_device(self, q_in, k_in, v_in, cos, sin):
        from . import mustafar_package_quant as mpq
        return mpq.decode_step_quant_pool(self.k_pool, self.v_pool, q_in, k_in, v_in, self._kbuf, self._vbuf,
                                          self._kbuf.shape[1], cos, sin, self.dequant_mode, win_len_dev=self._wlen_dev,
                                          overflow=self._wovf, ws=self._workspace(q_in.device))

    def _attend_device(self, q2):
        from . import mustafar_package_quant as mpq
        if self.k_pool is not None:
            return mpq.decode_attention_window_quant_pool(self.k_pool, self.v_pool, q2, self._kbuf, self._vbuf,
                                                          self._kbuf.shape[1], self.groups, self.dequant_mode,
                                                          win_len_dev=self._wlen_dev, ws=self._workspace(q2.device))
        return mpq.decode_attention_window_quant(self.k, self.v, q2, self._kbuf, self._vbuf, self._kbuf.shape[1],
                                                 self.groups, self.bit, self.dequant_mode, win_len_dev=self._wlen_dev,
                                                 ws=self._workspace(q2.device))

    def prefill_proj(self, kx, vx, cos, sin):
        """As SparseKVCache.prefill_proj for the rotation - the keys are rotated in place by the compressor's kernel,
        in the projection's own layout - while the quantised producer, which takes contiguous rows like the
        reference's, goes through prefill on the transposed views."""
        ops.compress_proj(kx, False, self.kth_k, 0, cos, sin, ws=self._workspace(kx.device))      # M = 0: rotation only
        K, V = kx.transpose(1, 2), vx.transpose(1, 2)
        self.prefill(K, V)
        return K, V

    def _compress(self, K, V):
        from . import compression_quant as cq
        bs, n_kv, M, D = K.shape
        ws = self._workspace(K.device)   # the pruning runs inside the producer: one read of the dense rows
        return (list(cq.convert_key_batched_quant(K.reshape(bs * n_kv, M, D), return_metadata=True, bit=self.bit, ws=ws,
                                                  kth=self.kth_k)),
                list(cq.convert_value_batched_quant(V.reshape(bs * n_kv, M, D), bit=self.bit, ws=ws, kth=self.kth_v)))

    @staticmethod
    def _append(old, new):
        """models/llama_mustafar_quant_kernel.py:322-345."""
        shifted = new[1] + old[2].numel()
        return [torch.cat([old[0], new[0]], 1), torch.cat([old[1], shifted], 1), torch.cat([old[2], new[2]], 0),
                torch.cat([old[3], new[3]], 1), torch.cat([old[4], new[4]], 1), torch.cat([old[5], new[5]], 1),
                torch.cat([old[6], new[6]], 1)]

    def _make_pools(self, heads, D, device):
        fk = self.pool_fraction if self.pool_fraction is not None else packed_fraction_for(self.kth_k, D, self.bit)
        fv = self.pool_fraction if self.pool_fraction is not None else packed_fraction_for(self.kth_v, D, self.bit)
        self.k_pool = QuantPool(heads, D, self.max_tokens, False, self.bit, device, fk)
        self.v_pool = QuantPool(heads, D, self.max_tokens, True, self.bit, device, fv)

    def _grow(self, K, V):
        if self.max_tokens > 0:
            bs, n_kv, M, D = K.shape
            if self.k_pool is None:
                self._make_pools(bs * n_kv, D, K.device)
            ws = self._workspace(K.device)
            self.k_pool.append(K.reshape(bs * n_kv, M, D), self.kth_k, ws)
            self.v_pool.append(V.reshape(bs * n_kv, M, D), self.kth_v, ws)
            if not self.window_kernel:
                self.k, self.v = self.k_pool.view(), self.v_pool.view()
            return
        ck, cv = self._compress(K, V)
        self.k = ck if self.k is None else self._append(self.k, ck)
        self.v = cv if self.v is None else self._append(self.v, cv)

    def decode(self, q, k_new, v_new):
        """q: [bs, n_q, 1, D]; k_new, v_new: [bs, n_kv, 1, D].  Returns the attention output [bs, n_q, 1, D]."""
        from . import mustafar_package_quant as mpq
        if self.window_kernel:
            return self._decode_window_kernel(q, k_new, v_new)
        bs, n_q, _, D = q.shape
        g, Lc, cap = self.groups, self.compressed_length, 32 // self.bit
        Bq = bs * n_q
        self.kv_len += 1
        self.k_win = torch.cat([self.k_win, k_new], dim=2)
        self.v_win = torch.cat([self.v_win, v_new], dim=2)
        s_loc = torch.matmul(q, _repeat_kv(self.k_win, g).transpose(2, 3))            # [bs, n_q, 1, Lw]
        if Lc > 0 and self.fused:
            lse = torch.empty((Bq, 2), dtype=torch.float32, device=q.device)
            o_c = mpq.decode_attention_quant(self.k, self.v, q.reshape(Bq, D).contiguous(), g, self.bit,
                                             self.dequant_mode, lse=lse, ws=self._workspace(q.device))
            m_c, l_c = lse[:, 0].view(bs, n_q, 1, 1), lse[:, 1].view(bs, n_q, 1, 1)
            w = (s_loc / ops.sqrt_head_dim(D)).float()
            M = torch.maximum(m_c, w.amax(-1, keepdim=True))
            p = torch.exp(w - M)
            a = l_c * torch.exp(m_c - M)
            num = a * o_c.view(bs, n_q, 1, D).float() + torch.matmul(p, _repeat_kv(self.v_win, g).float())
            out = (num / (a + p.sum(-1, keepdim=True))).half()
        else:
            if Lc > 0:
                k = self.k
                padded_query = torch.nn.functional.pad(q.view(Bq, -1, D), (0, 0, 0, 7))
                s_cmp = mpq.mustafar_key_formulation_quant_meta(k[0], k[2], k[1], k[3], k[4], k[5], k[6], padded_query, Lc,
                                                                D, Bq, g, self.bit, cap, self.dequant_mode)
                s = torch.cat([s_cmp[:, 0:1, :].view(bs, n_q, 1, Lc), s_loc], dim=-1)
            else:
                s = s_loc
            p = ops.scale_softmax(s.contiguous(), D)
            out = torch.matmul(p[..., Lc:], _repeat_kv(self.v_win, g))
            if Lc > 0:
                v = self.v
                score = p[..., :Lc].reshape(Bq, Lc).contiguous()
                o_cmp = mpq.mustafar_value_formulation_quant_decode_n1(v[0], v[2], v[1], v[3], v[4], v[5], v[6], score,
                                                                       None, D, Lc, Bq, g, self.bit, cap,
                                                                       self.dequant_mode)
                out = out + o_cmp.view(bs, n_q, 1, D)
        if (self.kv_len - self.residual_length - Lc) % CHUNK == 0 and self.k_win.shape[2] >= CHUNK:
            self._grow(self.k_win[:, :, :CHUNK].contiguous(), self.v_win[:, :, :CHUNK].contiguous())
            self.k_win = self.k_win[:, :, CHUNK:].contiguous()
            self.v_win = self.v_win[:, :, CHUNK:].contiguous()
            self.compressed_length += CHUNK
        return out
