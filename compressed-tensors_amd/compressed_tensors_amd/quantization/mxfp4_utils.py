"""MXFP4 group scales on the GPU: powers of two stored as uint8 exponents.

Reference: quantization/utils/mxfp4_utils.py (convert_mxfp4_exp_scale :24-38,
round_to_power_2 :41-73, generate_mxfp4_scales :76-97).
"""
import torch

from compressed_tensors_amd import _lib

__all__ = ["convert_mxfp4_exp_scale", "generate_mxfp4_scales", "round_to_power_2"]


def convert_mxfp4_exp_scale(scale: torch.Tensor, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """uint8 exponents -> 2 ** (e - 127) in `dtype`"""
    assert scale.dtype == torch.uint8
    _lib.require_gpu(scale)
    s = scale.contiguous()
    out = torch.empty(s.shape, dtype=dtype, device=s.device)
    _lib.check(_lib.load().ctmi_mxfp4_convert_exp_scale(
        s.data_ptr(), out.data_ptr(), _lib.dtype_code(dtype), s.numel(), _lib.stream_of(s.device)))
    return out


def round_to_power_2(x: torch.Tensor) -> torch.Tensor:
    """bfloat16 values -> the power of two kept after adding half an e2m1 mantissa step"""
    assert x.dtype == torch.bfloat16
    _lib.require_gpu(x)
    v = x.contiguous()
    out = torch.empty_like(v)
    _lib.check(_lib.load().ctmi_mxfp4_round_to_power_2(
        v.data_ptr(), out.data_ptr(), v.numel(), _lib.stream_of(v.device)))
    return out


def generate_mxfp4_scales(x: torch.Tensor) -> torch.Tensor:
    """bfloat16 group maxima -> uint8 exponents of the group scales"""
    assert x.dtype == torch.bfloat16
    _lib.require_gpu(x)
    v = x.contiguous()
    out = torch.empty(v.shape, dtype=torch.uint8, device=v.device)
    _lib.check(_lib.load().ctmi_mxfp4_generate_scales(
        v.data_ptr(), out.data_ptr(), v.numel(), _lib.stream_of(v.device)))
    return out
