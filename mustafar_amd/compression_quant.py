"""Drop-in for the reference's kernel_quant/compression_quant.py (convert_key_batched_quant :159-264,
convert_value_batched_quant :425-529): same arguments and return tuples.  The reference hard-codes
2-bit codes; `bit` is exposed here as an extra keyword (2, 4 or 8; capacity = 32 // bit), and `group_size`
(64 = one scale / zero pair per tile as in the reference; 32 = two, scales and zeros then [B, T, 2]).

inputs: [B, M, N] fp16 on the GPU, already pruned (or pruned here: `kth`), M % 64 == 0.
"""
import torch

from . import ops
from ._lib import check, lib


def _produce(inputs, is_value, bit, kth=0, group_size=64, ws=None, room=None):
    """One call of the producer.  room: int32 tensor that takes the packed words (tile offsets count from its start;
    a tile whose words would pass its end is not written, and the total then exceeds room.numel());
    default: a fresh buffer with room for the worst case.  Returns the per-tile arrays, the buffer and the word total
    as a device tensor (all ones should a wait of the one-pass producer have run out) - nothing is read on the host."""
    assert inputs.is_cuda
    assert inputs.dim() == 3
    B, M, N = inputs.shape
    assert M % 64 == 0
    if inputs.dtype != torch.float16:
        raise RuntimeError("inputs must be float16")
    x = inputs.contiguous()
    dev = x.device
    T = M * N // 64
    L = lib()
    bmp = torch.empty((B, T), dtype=torch.int64, device=dev)
    tile_off = torch.empty((B, T), dtype=torch.int32, device=dev)
    counts = torch.empty((B, T), dtype=torch.int32, device=dev)
    units = torch.empty((B, T), dtype=torch.int32, device=dev)
    if group_size not in (32, 64):
        raise RuntimeError("group_size must be 32 or 64")
    meta_shape = (B, T) if group_size == 64 else (B, T, 2)
    scales = torch.empty(meta_shape, dtype=torch.float16, device=dev)
    zeros = torch.empty(meta_shape, dtype=torch.float16, device=dev)
    total = torch.empty((1,), dtype=torch.int64, device=dev)
    ws = ops.workspace(dev, L.mstf_compress_quant_workspace_bytes(B, M, N), ws)
    st = torch.cuda.current_stream().cuda_stream
    # one pass with room for the worst case (every element kept: 64 // capacity words per tile)
    cap_words = B * T * (64 * int(bit) // 32)
    if room is None:
        room = torch.empty((max(cap_words, 1),), dtype=torch.int32, device=dev)
    else:
        cap_words = room.numel()
    assert room.dtype == torch.int32 and room.is_contiguous()
    check(L.mstf_compress_quant_grouped(st, x.data_ptr(), int(bool(is_value)), B, M, N, int(kth), int(bit), int(group_size),
                                        bmp.data_ptr(), tile_off.data_ptr(), counts.data_ptr(), units.data_ptr(),
                                        scales.data_ptr(), zeros.data_ptr(), total.data_ptr(), room.data_ptr(), cap_words,
                                        ws.data_ptr(), ws.numel()), "mstf_compress_quant_grouped")
    return bmp, tile_off, room, counts, units, scales, zeros, total


def words_written(total):
    """The producer's word total on the host (one read, as the reference's .item()); raises if the producer gave up."""
    n = int(total.item())
    if n < 0:   # all ones: a workgroup of the one-pass producer gave up waiting (ruled out by the dispatch order)
        raise RuntimeError("the quantised producer gave up waiting for an earlier workgroup; the packed words are incomplete")
    return n


def _convert(inputs, is_value, bit, kth=0, group_size=64, ws=None):
    bmp, tile_off, room, counts, units, scales, zeros, total = _produce(inputs, is_value, bit, kth, group_size, ws)
    # the used part is copied out so that the large buffer goes back to the allocator
    packed = room[:words_written(total)].clone()
    return bmp, tile_off, packed, counts, units, scales, zeros


def convert_key_batched_quant(inputs: torch.Tensor, return_metadata: bool = False, bit: int = 2, group_size: int = 64,
                              ws=None, kth: int = 0):
    """kth > 0 (an extra of this build): the rows are pruned to that rank inside the producer, as dh_prune_key would
    have done in front of it (models/llama_mustafar_quant_kernel.py), with one read of the dense rows."""
    bmp, tile_off, packed, counts, units, scales, zeros = _convert(inputs, False, bit, kth, group_size, ws)
    if return_metadata:
        return bmp, tile_off, packed, counts, units, scales, zeros
    return bmp, tile_off, packed, scales, zeros


def convert_value_batched_quant(inputs: torch.Tensor, bit: int = 2, group_size: int = 64, ws=None, kth: int = 0):
    return _convert(inputs, True, bit, kth, group_size, ws)
