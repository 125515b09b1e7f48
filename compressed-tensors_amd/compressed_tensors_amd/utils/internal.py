import torch

__all__ = ["InternalModule"]


class InternalModule(torch.nn.Module):
    """Marks modules this library adds to a model (hooked attention, caches): they are
    never matched as quantization or transform targets (reference: utils/internal.py)."""
