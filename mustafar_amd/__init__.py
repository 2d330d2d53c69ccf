"""MI355X-native sparse-KV decode-attention path of Mustafar.

Host-side mirror of the reference operator interface over the C ABI of libmustafar_hip.so:

    mustafar_amd.compression            ~ kernel/compression.py          (convert_{key,value}_batched)
    mustafar_amd.mustafar_package       ~ kernel/kernel_wrapper          (mustafar_{key,value}_formulation)
    mustafar_amd.compression_quant      ~ kernel_quant/compression_quant.py
    mustafar_amd.mustafar_package_quant ~ kernel_quant/kernel_wrapper
    mustafar_amd.ops                    the zero-copy decode path (flat cache, one query row per head)
"""
import sys
import types

from . import _lib  # noqa: F401

__all__ = ["compression", "mustafar_package", "compression_quant", "mustafar_package_quant", "ops", "install_aliases"]


def install_aliases():
    """Registers this package's mirrors under the module names the reference's model files import
    (models/llama_mustafar_kernel.py:15,20: `mustafar_package`, `kernel.compression`;
    models/llama_mustafar_quant_kernel.py:15,20: `mustafar_package_quant`, `kernel_quant.compression_quant`),
    so that those files run unchanged on PyTorch-ROCm.  Call it before importing them."""
    from . import compression, compression_quant, mustafar_package, mustafar_package_quant
    sys.modules["mustafar_package"] = mustafar_package                # was: kernel/kernel_wrapper (pybind.cpp:7-10)
    sys.modules["mustafar_package_quant"] = mustafar_package_quant    # was: kernel_quant/kernel_wrapper
    kernel = types.ModuleType("kernel")
    kernel.compression = compression
    sys.modules["kernel"], sys.modules["kernel.compression"] = kernel, compression   # was: Triton, kernel/compression.py
    kernel_quant = types.ModuleType("kernel_quant")
    kernel_quant.compression_quant = compression_quant
    sys.modules["kernel_quant"], sys.modules["kernel_quant.compression_quant"] = kernel_quant, compression_quant
