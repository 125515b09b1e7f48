"""compressed_tensors_amd — MI355X (gfx950) implementation of the
compressed-tensors weight compress / decompress hot path.

The Python layer mirrors the reference's operator and plug-in interface
(quantize / dequantize / fake_quantize, pack_to_int32, the per-format
compressors, ModelCompressor, Hadamard transforms); all tensor work happens in
hand-written HIP kernels reached through the C ABI of libctmi.so.
"""
from compressed_tensors_amd import _lib  # noqa: F401
from compressed_tensors_amd.config import *  # noqa: F401,F403
from compressed_tensors_amd.quantization import *  # noqa: F401,F403
from compressed_tensors_amd.utils import *  # noqa: F401,F403
from compressed_tensors_amd.compressors import *  # noqa: F401,F403
from compressed_tensors_amd.linear import *  # noqa: F401,F403

__version__ = "0.1.0"
