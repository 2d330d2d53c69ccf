"""MI355X-native sparse-KV decode-attention path of Mustafar.

Host-side mirror of the reference operator interface over the C ABI of libmustafar_hip.so:

    mustafar_amd.compression            ~ kernel/compression.py          (convert_{key,value}_batched)
    mustafar_amd.mustafar_package       ~ kernel/kernel_wrapper          (mustafar_{key,value}_formulation)
    mustafar_amd.compression_quant      ~ kernel_quant/compression_quant.py
    mustafar_amd.mustafar_package_quant ~ kernel_quant/kernel_wrapper
    mustafar_amd.ops                    the zero-copy decode path (flat cache, one query row per head)
"""
from . import _lib  # noqa: F401

__all__ = ["compression", "mustafar_package", "compression_quant", "mustafar_package_quant", "ops"]
