"""Drop-in for the reference's `mustafar_package` extension (kernel/kernel_wrapper/pybind.cpp:7-10,
mustafar_wrapper.cu:19-263): same positional arguments, same checks (RuntimeError), same output
shape [Batch_Size, 8, M_Global] fp16, launched on the current stream without synchronising."""
import torch

from . import ops
from ._lib import check, lib


def _checks(bmp, NZ, idx, NZ_Offset, B, need_b_contiguous):
    dev = B.device
    if any(t.device != dev for t in (bmp, NZ, idx, NZ_Offset)):
        raise RuntimeError("All input tensors must be on the same device.")
    if B.dtype != torch.float16:
        raise RuntimeError("Tensor B must be of type float16.")
    if NZ.dtype != torch.float16:
        raise RuntimeError("Tensor NZ must be of type float16.")
    if bmp.dtype != torch.int64:
        raise RuntimeError("Tensor bmp must be of type int64.")
    if idx.dtype != torch.int32:
        raise RuntimeError("Tensor idx must be of type int.")
    if NZ_Offset.dtype != torch.int32:
        raise RuntimeError("Tensor NZ_Offset must be of type int.")
    tensors = [bmp, NZ, idx, NZ_Offset] + ([B] if need_b_contiguous else [])
    if not all(t.is_contiguous() for t in tensors):
        raise RuntimeError("bmp, NZ, idx, B, C, and Reduction_Workspace tensors must be contiguous.")
    if not all(t.is_cuda for t in (bmp, NZ, idx, NZ_Offset, B)):
        raise RuntimeError("bmp, NZ, idx, B, C, and (not)Reduction_Workspace tensors must be on CUDA device.")


def mustafar_key_formulation(bmp, NZ, idx, NZ_Offset, B, M_Global, K_Global, Batch_Size, num_key_value_groups):
    """C[bq, n, m] = sum_k Ktilde[bq // groups][m, k] * B[bq, n, k];  B: [Batch_Size, 8, K_Global]."""
    _checks(bmp, NZ, idx, NZ_Offset, B, True)
    if B.numel() != Batch_Size * 8 * K_Global:
        raise RuntimeError("Tensor B must hold Batch_Size x 8 x K_Global elements.")
    C = torch.empty((Batch_Size, 8, M_Global), dtype=torch.float16, device=B.device)
    check(lib().mstf_key_spmv_f16(torch.cuda.current_stream().cuda_stream, bmp.data_ptr(), NZ.data_ptr(),
                                  idx.data_ptr(), NZ_Offset.data_ptr(), B.data_ptr(), C.data_ptr(), int(M_Global),
                                  int(K_Global), int(Batch_Size), int(num_key_value_groups), 8),
          "mustafar_key_formulation")
    return C


def mustafar_value_formulation(bmp, NZ, idx, NZ_Offset, B, Reduction_Workspace, M_Global, K_Global, Batch_Size,
                               num_key_value_groups):
    """C[bq, n, m] = sum_k Vtilde[bq // groups][k, m] * B[bq, n, k];  B: [Batch_Size, 8, K_Global].

    Reduction_Workspace is accepted for signature compatibility (the reference passes a one-element
    dummy); the fp32 split partials live in the package's own scratch tensor."""
    _checks(bmp, NZ, idx, NZ_Offset, B, False)
    if B.numel() != Batch_Size * 8 * K_Global:
        raise RuntimeError("Tensor B must hold Batch_Size x 8 x K_Global elements.")
    B = B.contiguous()
    L = lib()
    C = torch.empty((Batch_Size, 8, M_Global), dtype=torch.float16, device=B.device)
    wsb = L.mstf_value_spmv_workspace_bytes(int(M_Global), int(K_Global), int(Batch_Size), int(num_key_value_groups), 8)
    ws = ops.workspace(B.device, wsb)
    check(L.mstf_value_spmv_f16(torch.cuda.current_stream().cuda_stream, bmp.data_ptr(), NZ.data_ptr(),
                                idx.data_ptr(), NZ_Offset.data_ptr(), B.data_ptr(), C.data_ptr(), int(M_Global),
                                int(K_Global), int(Batch_Size), int(num_key_value_groups), 8, ws.data_ptr(),
                                ws.numel()), "mustafar_value_formulation")
    return C
