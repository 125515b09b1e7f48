"""Oracle: bitmask sparsity formats.

Follows utils/helpers.py:302-339, compressors/sparse_compressors/sparse_bitmask.py:131-169
and sparse_24_bitmask.py:162-260 of the reference.
"""
import numpy
import torch

FP8 = torch.float8_e4m3fn


def pack_bitmasks(bytemasks):
    # helpers.py:302-313
    return torch.from_numpy(numpy.packbits(bytemasks.numpy(), axis=-1, bitorder="little"))


def unpack_bitmasks(packed, original_shape):
    # helpers.py:316-339
    bits = numpy.unpackbits(packed.cpu().numpy(), axis=-1, count=original_shape[-1],
                            bitorder="little")
    return torch.from_numpy(bits.reshape(original_shape).astype(bool))


def _masked_values(tensor, mask):
    if tensor.dtype == FP8:
        return tensor.view(torch.int8)[mask].view(FP8)
    return tensor[mask]


def bitmask_compress(tensor):
    # sparse_bitmask.py:131-149
    mask = tensor != 0
    counts = mask.sum(dim=-1)
    row_offsets = torch.cumsum(counts, 0) - counts
    return _masked_values(tensor, mask), pack_bitmasks(mask), row_offsets


def bitmask_decompress(values, bitmasks, original_shape):
    # sparse_bitmask.py:152-169
    mask = unpack_bitmasks(bitmasks, original_shape)
    out = torch.zeros(original_shape, dtype=values.dtype)
    if values.dtype == FP8:
        out.view(torch.int8)[mask] = values.view(torch.int8)
    else:
        out[mask] = values
    return out


def get_24_bytemasks(tensor):
    # sparse_24_bitmask.py:227-260
    if tensor.dtype == FP8:
        tensor = tensor.view(torch.int8)
    shape = tensor.shape
    if tensor.numel() % 4 != 0:
        raise ValueError("Tensor size must be a multiple of 4 for TWO_FOUR sparsity")
    groups = tensor.reshape(-1, 4)
    keep = groups.abs().topk(2, dim=1).indices
    mask = torch.zeros_like(groups, dtype=torch.bool)
    mask.scatter_(1, keep, True)
    return mask.reshape(shape)


def sparse24_bitmask_compress(tensor):
    # sparse_24_bitmask.py:162-203
    assert len(tensor.shape) == 2, "Only 2D tensors are supported"
    mask = get_24_bytemasks(tensor)
    rows, cols = tensor.shape
    values = _masked_values(tensor, mask).reshape(rows, cols // 2)
    return values, pack_bitmasks(mask)


def sparse24_bitmask_decompress(values, bitmasks, original_shape):
    # sparse_24_bitmask.py:206-224
    return bitmask_decompress(values.flatten(), bitmasks, list(original_shape))
