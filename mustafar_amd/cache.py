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
import torch

from . import ops

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


class SparseKVCache:
    def __init__(self, groups, head_dim=128, k_sparsity=0.7, v_sparsity=0.7, residual_length=256, fused=False):
        """fused: the compressed part of a decode step is one launch (ops.decode_attention) whose (max, sum) joins
        the dense window under one softmax, instead of the reference's key SpMV / softmax / value SpMV sequence."""
        self.groups, self.head_dim, self.residual_length = groups, head_dim, residual_length
        self.fused = fused
        self.kth_k = ops.kth_from_sparsity(k_sparsity, head_dim)
        self.kth_v = ops.kth_from_sparsity(v_sparsity, head_dim)
        self.k = self.v = None              # CompressedKV
        self.k_win = self.v_win = None      # [bs, n_kv, Lw, D] dense
        self.compressed_length = 0
        self.kv_len = 0

    def _compress(self, K, V):
        bs, n_kv, L, D = K.shape
        ck = ops.compress(K.reshape(bs * n_kv, L, D), False, kth=self.kth_k)
        cv = ops.compress(V.reshape(bs * n_kv, L, D), True, kth=self.kth_v)
        return ck, cv

    def prefill(self, K, V):
        """K, V: [bs, n_kv, L, D] fp16 (after RoPE)."""
        L = K.shape[2]
        Lc = ((L - self.residual_length) // CHUNK) * CHUNK if L > self.residual_length else 0
        if Lc > 0:
            self.k, self.v = self._compress(K[:, :, :Lc].contiguous(), V[:, :, :Lc].contiguous())
        self.k_win = K[:, :, Lc:].contiguous().clone()
        self.v_win = V[:, :, Lc:].contiguous().clone()
        self.compressed_length, self.kv_len = Lc, L

    def _decode_fused(self, q, s_loc):
        """One launch over the compressed tokens, then a log-sum-exp merge with the dense window."""
        bs, n_q, _, D = q.shape
        g = self.groups
        lse = torch.empty((bs * n_q, 2), dtype=torch.float32, device=q.device)
        o_c = ops.decode_attention(self.k, self.v, q.reshape(bs * n_q, D).contiguous(), g, lse=lse)
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
                o_cmp = ops.value_spmv(self.v, p[..., :Lc].reshape(bs * n_q, 1, Lc).contiguous(), g)
                out = out + o_cmp.view(bs, n_q, 1, D)
        if (self.kv_len - self.residual_length - Lc) % CHUNK == 0 and self.k_win.shape[2] >= CHUNK:
            ck, cv = self._compress(self.k_win[:, :, :CHUNK].contiguous(), self.v_win[:, :, :CHUNK].contiguous())
            self.k = ck if self.k is None else append_compressed(self.k, ck)
            self.v = cv if self.v is None else append_compressed(self.v, cv)
            self.k_win = self.k_win[:, :, CHUNK:].contiguous()
            self.v_win = self.v_win[:, :, CHUNK:].contiguous()
            self.compressed_length += CHUNK
        return out
