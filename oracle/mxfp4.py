"""TEST INFRASTRUCTURE ONLY: CPU restatement of the reference's MXFP4 scale helpers
(quantization/utils/mxfp4_utils.py), as the torch op chains they are.  Pinned by the
literal vectors of the reference's tests/test_quantization/test_utils/test_mxfp4_utils.py
(tests/golden/mxfp4.json) and by the closed form "biased exponent - 2"."""
import torch


def convert_mxfp4_exp_scale(scale, dtype=torch.bfloat16):
    # mxfp4_utils.py:24-38
    assert scale.dtype == torch.uint8
    scale_exp = scale.to(torch.int32) - 127
    return (2.00 ** (scale_exp.to(torch.float))).to(dtype)


def round_to_power_2(x):
    # mxfp4_utils.py:41-73: bf16 has 7 mantissa bits, e2m1 has 1
    assert x.dtype == torch.bfloat16
    bits = x.view(torch.uint16).to(torch.int32)
    val_to_add = 1 << (7 - 1 - 1)
    sign_exponent_mask = ((1 << (8 + 1)) - 1) << 7
    kept = torch.bitwise_and(bits + val_to_add, sign_exponent_mask)
    return kept.to(torch.uint16).view(torch.bfloat16)


def generate_mxfp4_scales(x):
    # mxfp4_utils.py:76-97
    scale_power_2 = round_to_power_2(x)
    scale_exp = 127 + torch.floor(torch.log2(scale_power_2)).to(torch.int32) - 2
    scale_exp = torch.clamp(scale_exp, max=255, min=0)
    return scale_exp.to(torch.uint8)
