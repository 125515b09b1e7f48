"""Oracle: Hadamard matrix construction and transform apply.

Follows transform/utils/hadamard.py:33-163, transform/utils/matrix.py:65-171 and
transform/factory/hadamard.py:46-121 of the reference on CPU tensors.

The reference ends its butterfly recursion in a table of known Hadamard
matrices (hadamards.safetensors) that does not travel with this repository.
For a power of two n other than 32 the table entry it picks (the largest K in
{256, 128, 64, 16, 8, 4, 2, 1} with n / K a power of two) is Sylvester's matrix of
that order - tests/test_oracle_hadamard.py checks this against the reference's file
when it is present - so `known_block` rebuilds it.  Other sizes take the table as an
argument ({K: K x K matrix}); the tests pass the blocks of
tests/golden/hadamard_blocks.safetensors, which cover the sizes of the reference's
own Hadamard tests.
"""
import math
from typing import Optional

import torch


def deterministic_hadamard_matrix(size, dtype=torch.bfloat16, device=torch.device("cpu")):
    # hadamard.py:33-62
    if size <= 0:
        raise ValueError("Cannot construct deterministic hadamard of size <= 0")
    log2 = int(math.log2(size))
    if size != 2**log2:
        raise ValueError("Cannot construct deterministic hadamard of size != 2^n")
    h = torch.tensor([[1]], dtype=dtype, device=device)
    for _ in range(log2):
        h = torch.vstack((torch.hstack((h, h)), torch.hstack((h, -h))))
    return h


def known_block(n: int, dtype, table=None) -> torch.Tensor:
    """_fetch_hadamard_divisor (hadamard.py:102-129): the largest K of the table with n / K
    a power of two.  Without a table: powers of two other than 32, whose entries are
    Sylvester's matrices."""
    if table is not None:
        for k in sorted(table, reverse=True):
            if n % k == 0 and (n // k) & (n // k - 1) == 0:
                return table[k].to(dtype)
    elif n & (n - 1) == 0 and n != 32:
        return deterministic_hadamard_matrix(min(n, 256), dtype)
    raise ValueError(f"Cannot construct random hadamard matrix of size {n}")


def matmul_hadU(x: torch.Tensor, table=None) -> torch.Tensor:
    # hadamard.py:132-163: butterfly stages down to the known block, then the block
    size = x.size(0)
    had_k = known_block(size, x.dtype, table)
    k = had_k.size(0)
    inp = x.clone().view(-1, size, 1)
    out = inp.clone()
    while inp.shape[1] > k:
        inp = inp.view(inp.shape[0], inp.shape[1] // 2, 2, inp.shape[2])
        out = out.view(inp.shape)
        out[:, :, 0, :] = inp[:, :, 0, :] + inp[:, :, 1, :]
        out[:, :, 1, :] = inp[:, :, 0, :] - inp[:, :, 1, :]
        out = out.view(inp.shape[0], inp.shape[1], -1)
        inp, out = out, inp
    assert inp.shape[1] == k
    inp = had_k.view(1, k, k).to(inp) @ inp
    return inp.view(x.shape)


def random_hadamard_matrix(size, dtype=torch.bfloat16, gen: Optional[torch.Generator] = None,
                           table=None):
    # hadamard.py:65-89
    q = torch.randint(low=0, high=2, size=(size,), generator=gen, dtype=dtype)
    q = q * 2 - 1
    return matmul_hadU(torch.diag(q), table)


def multihead_matmul(a, b):
    # matrix.py:137-171
    if a.shape[-1] > b.shape[-2]:
        h = b.shape[-2]
        return (a.unflatten(-1, (a.shape[-1] // h, h)) @ b).flatten(-2, -1)
    if a.shape[-1] < b.shape[-2]:
        h = a.shape[-1]
        return (a @ b.unflatten(-2, (b.shape[-2] // h, h))).flatten(-3, -2)
    return a @ b


def apply_transform_weight(weight, value, location: str, module_type):
    # matrix.py:65-134
    assert weight.shape[0] == weight.shape[1]
    if location not in ("weight_input", "weight_output"):
        return multihead_matmul(value, weight)
    if module_type == torch.nn.Linear:
        if location == "weight_input":
            return multihead_matmul(value, weight.T)
        return multihead_matmul(weight.T, value)
    if module_type == torch.nn.Embedding:
        if location == "weight_input":
            return multihead_matmul(weight, value)
        return multihead_matmul(value, weight)
    raise NotImplementedError()


def hadamard_forward(weight, value, location: str, module_type=torch.nn.Linear, inverse=False,
                     perm=None):
    # factory/hadamard.py:104-121
    scale = torch.tensor(weight.size(0), dtype=torch.float64).sqrt()
    if perm is not None:
        weight = weight[perm][:, perm]
    if inverse:
        weight = weight.T
    return (apply_transform_weight(weight, value.to(weight.dtype), location, module_type)
            / scale).to(value.dtype)
