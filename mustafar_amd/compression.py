"""Drop-in for the reference's kernel/compression.py (convert_key_batched :249-342,
convert_value_batched :344-435): same arguments, same return types and shapes.

inputs: [B, M, N] fp16 on the GPU, already pruned (zeros are the holes), M % 64 == 0.
returns (bitmaps int64 [B, T], accum_counts int32 [B, T+1], [fp16 packed values per batch entry]).
"""
import torch

from . import ops


def _convert(inputs, is_value):
    assert inputs.is_cuda
    assert inputs.dim() == 3
    B, M, N = inputs.shape
    assert M % 64 == 0
    if inputs.dtype != torch.float16:
        raise RuntimeError("inputs must be float16")
    ck = ops.compress(inputs, is_value, kth=0)
    sizes = (2 * ck.idx[:, -1].to(torch.int64)).tolist()   # the reference also syncs here (.item())
    packed = [t.clone() for t in torch.split(ck.packed(), sizes)]
    return ck.bmp, ck.idx, packed


def convert_key_batched(inputs: torch.Tensor):
    return _convert(inputs, False)


def convert_value_batched(inputs: torch.Tensor):
    return _convert(inputs, True)


def nz_offsets(accum_counts):
    """NZ_Offset of the caller (models/llama_mustafar_kernel.py:450-452): running idx[b][-1] // 4."""
    last = accum_counts.view(accum_counts.shape[0], -1)[:, -1].to(torch.int64) // 4
    off = torch.zeros_like(last)
    off[1:] = torch.cumsum(last, 0)[:-1]
    return off.to(torch.int32)
