"""Hadamard transforms on the GPU.

Reference surface mirrored here:
  deterministic_hadamard_matrix / random_hadamard_matrix / is_pow2
      transform/utils/hadamard.py:33-99
  apply_transform_weight / _multihead_matmul
      transform/utils/matrix.py:65-171
  HadamardFactory / RandomHadamardFactory / HadamardTransform
      transform/factory/hadamard.py:31-121, transform/factory/random_hadamard.py:21-40
  TransformLocation / TransformArgs / TransformScheme
      transform/transform_args.py:24-85, transform/transform_scheme.py:26-55

A Hadamard transform object remembers how its matrix was built,
    W = diag(signs) * Sylvester(n)          (signs = 1 for the deterministic kind),
so `forward` never touches the n x n matrix: the signs are applied on the way
in or out and Sylvester(n) = Sylvester(a) (x) Sylvester(b) runs as two small
products on the matrix cores (ctmi_hadamard_apply).  `weight` materialises the
dense matrix on demand for callers that want to look at it.  Explicit dense
matrices (anything that is not such a product) go through torch.matmul on the
GPU, as in the reference.
"""
import math
from enum import Enum
from typing import Dict, List, Optional, Tuple

import torch
from torch import Tensor

from compressed_tensors_amd import _lib
from compressed_tensors_amd.compressors.base import to_gpu
from compressed_tensors_amd.registry import RegistryMixin

__all__ = [
    "is_pow2",
    "deterministic_hadamard_matrix",
    "random_hadamard_matrix",
    "random_hadamard_signs",
    "hadamard_factors",
    "hadamard_apply",
    "hadamard_quantize_pack",
    "hadamard_apply_many",
    "hadamard_quantize_pack_many",
    "apply_transform_weight",
    "TransformLocation",
    "TransformArgs",
    "TransformScheme",
    "TransformFactory",
    "HadamardFactory",
    "RandomHadamardFactory",
    "HadamardTransform",
]

_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


def is_pow2(n: int) -> bool:
    return n > 0 and (n & (n - 1) == 0)


def deterministic_hadamard_matrix(
    size: int, dtype: torch.dtype = torch.bfloat16, device=torch.device("cpu")
) -> Tensor:
    """Sylvester's construction; entry (i, j) = (-1)^popcount(i & j)."""
    if size <= 0:
        raise ValueError("Cannot construct deterministic hadamard of size <= 0")
    if not is_pow2(size):
        raise ValueError("Cannot construct deterministic hadamard of size != 2^n")
    idx = torch.arange(size, device=device)
    both = idx.unsqueeze(0) & idx.unsqueeze(1)
    parity = torch.zeros_like(both)
    for bit in range(max(size.bit_length() - 1, 1)):
        parity ^= (both >> bit) & 1
    return (1 - 2 * parity).to(dtype)


def random_hadamard_signs(size: int, gen: Optional[torch.Generator] = None) -> Tensor:
    """The +-1 diagonal the reference draws (on the CPU, from `gen`) for a random
    Hadamard matrix: Q = 2 * randint(0, 2, (size,)) - 1  (hadamard.py:85-88)."""
    q = torch.randint(low=0, high=2, size=(size,), generator=gen, dtype=torch.float32)
    return q * 2 - 1


def random_hadamard_matrix(
    size: int,
    dtype: torch.dtype = torch.bfloat16,
    device=torch.device("cpu"),
    gen: Optional[torch.Generator] = None,
) -> Tensor:
    """diag(Q) * H.  For a power of two of at least 64 the reference's butterfly
    stages end in a stored Sylvester block, so H = Sylvester(size); other sizes
    need the reference's table of known Hadamard matrices and are not built."""
    if not (is_pow2(size) and size >= 64):
        raise NotImplementedError(
            f"random Hadamard matrices are built for powers of two >= 64, got {size}"
        )
    q = random_hadamard_signs(size, gen).to(device=device)
    h = deterministic_hadamard_matrix(size, torch.float32, device)
    return (q.unsqueeze(1) * h).to(dtype)


# ------------------------------------------------------------------ kernel plumbing
_KRON = {32: (1, 32), 64: (1, 64), 128: (1, 128), 1024: (32, 32), 2048: (32, 64),
         4096: (64, 64), 8192: (64, 128)}
_factor_cache: Dict[Tuple[int, str], Tensor] = {}


def hadamard_factors(n: int) -> Optional[Tuple[int, int]]:
    """(a, b) with Sylvester(n) = Sylvester(a) (x) Sylvester(b), if an MFMA kernel exists"""
    return _KRON.get(n)


def _sylvester_bf16(size: int, device) -> Tensor:
    key = (size, str(device))
    if key not in _factor_cache:
        _factor_cache[key] = deterministic_hadamard_matrix(size, torch.bfloat16, device).contiguous()
    return _factor_cache[key]


def hadamard_apply(
    value: Tensor,
    n: int,
    sign_in: Optional[Tensor] = None,
    sign_out: Optional[Tensor] = None,
    matrix_t: Optional[Tensor] = None,
) -> Tensor:
    """every run of n elements x of the last dim becomes
    (x * sign_in) @ M * sign_out / sqrt(n), M = Sylvester(n) or, for n <= 128,
    the explicit matrix whose transpose is `matrix_t` (bf16, entries exact in bf16)."""
    x = to_gpu(value).contiguous()
    if x.dtype not in _FLOATS:
        raise NotImplementedError(f"transforms of dtype {x.dtype} are not supported")
    if x.shape[-1] % n != 0:
        raise ValueError(f"{n} must divide the last dimension {x.shape[-1]}")
    fac = hadamard_factors(n)
    lib = _lib.load()
    code = _lib.dtype_code(x.dtype)
    if fac is None or not lib.ctmi_hadamard_supported(fac[0], fac[1], code):
        raise NotImplementedError(f"no MFMA Hadamard kernel for size {n} and dtype {x.dtype}")
    a, b = fac
    dev = x.device
    if matrix_t is not None:
        if a != 1:
            raise NotImplementedError("explicit matrices are supported for sizes 32, 64 and 128")
        mb_t = matrix_t.to(device=dev, dtype=torch.bfloat16).contiguous()
        ma_t = None
    else:
        mb_t = _sylvester_bf16(b, dev)
        ma_t = _sylvester_bf16(a, dev) if a > 1 else None
    s_in = None if sign_in is None else sign_in.to(device=dev, dtype=torch.float32).contiguous()
    s_out = None if sign_out is None else sign_out.to(device=dev, dtype=torch.float32).contiguous()
    out = torch.empty_like(x)
    _lib.check(
        lib.ctmi_hadamard_apply(
            x.data_ptr(), out.data_ptr(), code, x.numel(), a, b, _lib.ptr(ma_t), mb_t.data_ptr(),
            _lib.ptr(s_in), _lib.ptr(s_out), _lib.stream_of(dev),
        )
    )
    return out


def hadamard_quantize_pack(
    value: Tensor,
    n: int,
    quantization_args,
    sign_in: Optional[Tensor] = None,
    sign_out: Optional[Tensor] = None,
    matrix_t: Optional[Tensor] = None,
    return_rotated: bool = False,
) -> Dict[str, Tensor]:
    """hadamard_apply, the min-max observer and pack-quantized compression in one
    pass over a bf16 [rows, cols] tensor, for block size n (32, 64 or 128) equal
    to the group size of a symmetric 4-bit integer scheme.  Returns what the
    three steps return, bit for bit: weight_packed int32 [rows, cols / 8],
    weight_scale bf16 [rows, cols / n], weight_shape int64 [2] (and the rotated
    tensor under "rotated" if asked for)."""
    x = to_gpu(value).contiguous()
    args = quantization_args
    if x.ndim != 2 or x.dtype != torch.bfloat16:
        raise NotImplementedError("the fused path takes 2-D bfloat16 tensors")
    if not (args.num_bits == 4 and str(getattr(args.type, "value", args.type)) == "int" and args.symmetric
            and str(getattr(args.strategy, "value", args.strategy)) == "group" and args.group_size == n):
        raise NotImplementedError(
            "the fused path covers symmetric int4 group quantization with group_size == block size")
    if n not in (32, 64, 128):
        raise NotImplementedError("block size must be 32, 64 or 128")
    rows, cols = x.shape
    if cols % n != 0:
        raise ValueError(f"{n} must divide the last dimension {cols}")
    dev = x.device
    mb_t = (_sylvester_bf16(n, dev) if matrix_t is None
            else matrix_t.to(device=dev, dtype=torch.bfloat16).contiguous())
    s_in = None if sign_in is None else sign_in.to(device=dev, dtype=torch.float32).contiguous()
    s_out = None if sign_out is None else sign_out.to(device=dev, dtype=torch.float32).contiguous()
    packed = torch.empty((rows, cols // 8), dtype=torch.int32, device=dev)
    scale = torch.empty((rows, cols // n), dtype=torch.bfloat16, device=dev)
    rotated = torch.empty_like(x) if return_rotated else None
    _lib.check(
        _lib.load().ctmi_hadamard_quant_pack(
            x.data_ptr(), _lib.dtype_code(x.dtype), x.numel(), n, mb_t.data_ptr(), _lib.ptr(s_in),
            _lib.ptr(s_out), 4, 1, packed.data_ptr(), scale.data_ptr(), _lib.ptr(rotated),
            _lib.stream_of(dev),
        )
    )
    out = {"weight_packed": packed, "weight_scale": scale, "weight_shape": torch.tensor(x.shape)}
    if return_rotated:
        out["rotated"] = rotated
    return out


def hadamard_apply_many(
    values: List[Tensor],
    n: int,
    sign_in: Optional[Tensor] = None,
    sign_out: Optional[Tensor] = None,
    matrix_t: Optional[Tensor] = None,
) -> List[Tensor]:
    """hadamard_apply on several tensors of one dtype that share the matrix and the
    signs (the weights of a model under one transform scheme), from one call: the
    kernels take 8 tensors per launch."""
    if not values:
        return []
    xs = [to_gpu(v).contiguous() for v in values]
    dtype, dev = xs[0].dtype, xs[0].device
    if dtype not in _FLOATS:
        raise NotImplementedError(f"transforms of dtype {dtype} are not supported")
    for x in xs:
        if x.dtype != dtype or x.device != dev:
            raise ValueError("tensors of one call share dtype and device")
        if x.shape[-1] % n != 0:
            raise ValueError(f"{n} must divide the last dimension {x.shape[-1]}")
    fac = hadamard_factors(n)
    lib = _lib.load()
    code = _lib.dtype_code(dtype)
    if fac is None or not lib.ctmi_hadamard_supported(fac[0], fac[1], code):
        raise NotImplementedError(f"no MFMA Hadamard kernel for size {n} and dtype {dtype}")
    a, b = fac
    if matrix_t is not None:
        if a != 1:
            raise NotImplementedError("explicit matrices are supported for sizes 32, 64 and 128")
        mb_t, ma_t = matrix_t.to(device=dev, dtype=torch.bfloat16).contiguous(), None
    else:
        mb_t = _sylvester_bf16(b, dev)
        ma_t = _sylvester_bf16(a, dev) if a > 1 else None
    s_in = None if sign_in is None else sign_in.to(device=dev, dtype=torch.float32).contiguous()
    s_out = None if sign_out is None else sign_out.to(device=dev, dtype=torch.float32).contiguous()
    outs = [torch.empty_like(x) for x in xs]
    jobs = (_lib.HadamardJob * len(xs))()
    for job, x, out in zip(jobs, xs, outs):
        job.x, job.out, job.numel = x.data_ptr(), out.data_ptr(), x.numel()
    _lib.check(
        lib.ctmi_hadamard_apply_many(jobs, len(xs), code, a, b, _lib.ptr(ma_t), mb_t.data_ptr(),
                                     _lib.ptr(s_in), _lib.ptr(s_out), _lib.stream_of(dev))
    )
    return outs


def hadamard_quantize_pack_many(
    values: List[Tensor],
    n: int,
    quantization_args,
    sign_in: Optional[Tensor] = None,
    sign_out: Optional[Tensor] = None,
    matrix_t: Optional[Tensor] = None,
) -> List[Dict[str, Tensor]]:
    """hadamard_quantize_pack on several bf16 [rows, cols] tensors from one call (8 per
    launch); one dict per tensor, as hadamard_quantize_pack returns it"""
    if not values:
        return []
    xs = [to_gpu(v).contiguous() for v in values]
    args = quantization_args
    if not (args.num_bits == 4 and str(getattr(args.type, "value", args.type)) == "int" and args.symmetric
            and str(getattr(args.strategy, "value", args.strategy)) == "group" and args.group_size == n):
        raise NotImplementedError(
            "the fused path covers symmetric int4 group quantization with group_size == block size")
    if n not in (32, 64, 128):
        raise NotImplementedError("block size must be 32, 64 or 128")
    dev = xs[0].device
    for x in xs:
        if x.ndim != 2 or x.dtype != torch.bfloat16 or x.device != dev:
            raise NotImplementedError("the fused path takes 2-D bfloat16 tensors on one device")
        if x.shape[1] % n != 0:
            raise ValueError(f"{n} must divide the last dimension {x.shape[1]}")
    mb_t = (_sylvester_bf16(n, dev) if matrix_t is None
            else matrix_t.to(device=dev, dtype=torch.bfloat16).contiguous())
    s_in = None if sign_in is None else sign_in.to(device=dev, dtype=torch.float32).contiguous()
    s_out = None if sign_out is None else sign_out.to(device=dev, dtype=torch.float32).contiguous()
    jobs = (_lib.HadamardPackJob * len(xs))()
    results = []
    for job, x in zip(jobs, xs):
        rows, cols = x.shape
        packed = torch.empty((rows, cols // 8), dtype=torch.int32, device=dev)
        scale = torch.empty((rows, cols // n), dtype=torch.bfloat16, device=dev)
        job.x, job.packed, job.scale, job.rotated, job.numel = (
            x.data_ptr(), packed.data_ptr(), scale.data_ptr(), None, x.numel())
        results.append({"weight_packed": packed, "weight_scale": scale,
                        "weight_shape": torch.tensor(x.shape)})
    _lib.check(
        _lib.load().ctmi_hadamard_quant_pack_many(
            jobs, len(xs), _lib.dtype_code(torch.bfloat16), n, mb_t.data_ptr(), _lib.ptr(s_in),
            _lib.ptr(s_out), 4, 1, _lib.stream_of(dev))
    )
    return results


# ------------------------------------------------------------------ vocabulary
class TransformLocation(str, Enum):
    INPUT = "input"
    WEIGHT_INPUT = "weight_input"
    WEIGHT_OUTPUT = "weight_output"
    OUTPUT = "output"
    K_CACHE = "k_cache"
    Q_ATTN = "q_attn"

    def is_online(self) -> bool:
        return self not in (TransformLocation.WEIGHT_INPUT, TransformLocation.WEIGHT_OUTPUT)


class TransformArgs:
    def __init__(self, targets: List[str], location, inverse: bool = False,
                 ignore: Optional[List[str]] = None):
        self.targets = [targets] if isinstance(targets, str) else list(targets)
        self.location = TransformLocation(location)
        self.inverse = bool(inverse)
        self.ignore = list(ignore or [])

    def is_online(self) -> bool:
        return self.location.is_online()


class TransformScheme:
    def __init__(self, type: str, apply: Optional[List[TransformArgs]] = None,
                 randomize: bool = False, requires_grad: bool = False,
                 head_dim: Optional[int] = None, precision: torch.dtype = torch.float32):
        self.type = type
        self.apply = list(apply or [])
        self.randomize = randomize
        self.requires_grad = requires_grad
        self.head_dim = head_dim
        self.precision = precision


def _matmul_blocks(a: Tensor, b: Tensor) -> Tensor:
    """A @ B where the smaller square operand acts block-diagonally (matrix.py:137-171)"""
    if a.shape[-1] > b.shape[-2]:
        h = b.shape[-2]
        return (a.unflatten(-1, (a.shape[-1] // h, h)) @ b).flatten(-2, -1)
    if a.shape[-1] < b.shape[-2]:
        h = a.shape[-1]
        return (a @ b.unflatten(-2, (b.shape[-2] // h, h))).flatten(-3, -2)
    return a @ b


def apply_transform_weight(
    transform_weight: Tensor, value: Tensor, location, module_type: type
) -> Tensor:
    """Explicit-matrix form (matrix.py:65-134): a library GEMM on the GPU.  The
    structured, matrix-free path is HadamardTransform.forward."""
    assert transform_weight.shape[0] == transform_weight.shape[1]
    w, v = to_gpu(transform_weight), to_gpu(value)
    location = TransformLocation(location)
    if location.is_online():
        return _matmul_blocks(v, w)
    if module_type == torch.nn.Linear:
        if location == TransformLocation.WEIGHT_INPUT:
            return _matmul_blocks(v, w.T)
        if location == TransformLocation.WEIGHT_OUTPUT:
            return _matmul_blocks(w.T, v)
    elif module_type == torch.nn.Embedding:
        if location == TransformLocation.WEIGHT_INPUT:
            return _matmul_blocks(w, v)
        if location == TransformLocation.WEIGHT_OUTPUT:
            return _matmul_blocks(v, w)
    raise NotImplementedError(f"Applying transforms to {module_type} {location} is not supported")


def _orientation(location: TransformLocation, module_type: type) -> Tuple[bool, bool]:
    """(left_multiply, transposed): the value is multiplied by W or W^T, from the
    right (along its last dim) or from the left (along its first dim)."""
    if location.is_online():
        return False, False
    if module_type == torch.nn.Linear:
        if location == TransformLocation.WEIGHT_INPUT:
            return False, True
        if location == TransformLocation.WEIGHT_OUTPUT:
            return True, True
    elif module_type == torch.nn.Embedding:
        if location == TransformLocation.WEIGHT_INPUT:
            return True, False
        if location == TransformLocation.WEIGHT_OUTPUT:
            return False, False
    raise NotImplementedError(f"Applying transforms to {module_type} {location} is not supported")


class HadamardTransform(torch.nn.Module):
    """W = diag(signs) * Sylvester(size), optionally row/column permuted by `perm`
    (W[perm][:, perm]); forward(value) applies it at `args.location`, divides by
    sqrt(size) and returns value.dtype (hadamard.py:85-121)."""

    def __init__(self, size: int, signs: Optional[Tensor], perm: Optional[Tensor],
                 scheme: TransformScheme, args: TransformArgs, module_type: type,
                 precision: torch.dtype = torch.float32):
        super().__init__()
        if not is_pow2(size):
            raise ValueError("Cannot construct deterministic hadamard of size != 2^n")
        self.size = size
        self.signs = signs
        self.perm = perm
        self.scheme = scheme
        self.args = args
        self.module_type = module_type
        self.precision = precision
        self._scale = torch.tensor(size, dtype=torch.float64).sqrt()

    @property
    def weight(self) -> Tensor:
        """the dense matrix the reference would hold (before `perm`)"""
        h = deterministic_hadamard_matrix(self.size, self.precision, torch.device("cpu"))
        if self.signs is not None:
            h = self.signs.to(self.precision).cpu().unsqueeze(1) * h
        return h

    def forward(self, value: Tensor) -> Tensor:
        left, transposed = _orientation(self.args.location, self.module_type)
        if self.args.inverse:
            transposed = not transposed
        if left:
            # M @ V = (V^T @ M^T)^T: the transposed value is multiplied by the other orientation
            transposed = not transposed
        value = to_gpu(value)
        n = self.size
        fast = hadamard_factors(n) is not None and value.dtype in _FLOATS and bool(
            _lib.load().ctmi_hadamard_supported(*hadamard_factors(n), _lib.dtype_code(value.dtype))
        )
        if not fast:
            w = self.weight.to(value.device)
            if self.perm is not None:
                w = w[self.perm.to(w.device)][:, self.perm.to(w.device)]
            if self.args.inverse:
                w = w.T
            out = apply_transform_weight(w, value.to(w.dtype), self.args.location, self.module_type)
            return (out / self._scale).to(value.dtype)

        x = value.transpose(0, -1) if left else value  # left multiply = right multiply of the transpose
        # W   = diag(q) H  ->  x W   = (x * q) H
        # W^T = H diag(q)  ->  x W^T = (x H) * q
        s_in = s_out = None
        if self.signs is not None:
            if transposed:
                s_out = self.signs
            else:
                s_in = self.signs
        if self.perm is not None:
            # W' = W[p][:, p]:  x W' = ((x scattered to p) W) gathered at p
            p = self.perm.to(x.device)
            blocks = x.unflatten(-1, (x.shape[-1] // n, n))
            x = blocks.index_select(-1, torch.argsort(p)).flatten(-2, -1)
        y = hadamard_apply(x, n, sign_in=s_in, sign_out=s_out)
        if self.perm is not None:
            y = y.unflatten(-1, (y.shape[-1] // n, n)).index_select(-1, p).flatten(-2, -1)
        return y.transpose(0, -1).contiguous() if left else y


class TransformFactory(RegistryMixin):
    """name -> factory registry with the reference's `from_scheme` entry
    (transform/factory/base.py:53-92); module hooking is left to the caller."""

    def __init__(self, name: str, scheme: TransformScheme, seed: Optional[int] = None):
        self.name = name
        self.scheme = scheme
        self.generator = torch.Generator()
        if seed is not None:
            self.generator.manual_seed(seed)

    @classmethod
    def from_scheme(cls, scheme: TransformScheme, **kwargs):
        return cls.get_value_from_registry(scheme.type)(scheme=scheme, **kwargs)


def _transform_size(module: torch.nn.Module, location: TransformLocation,
                    head_dim: Optional[int]) -> int:
    size = None
    if isinstance(module, torch.nn.Linear):
        size = (module.in_features
                if location in (TransformLocation.INPUT, TransformLocation.WEIGHT_INPUT)
                else module.out_features)
    elif isinstance(module, torch.nn.Embedding):
        size = (module.num_embeddings
                if location in (TransformLocation.INPUT, TransformLocation.WEIGHT_INPUT)
                else module.embedding_dim)
    elif head_dim is None:
        raise NotImplementedError(
            f"Transforms on {type(module)} are not supported without head_dim"
        )
    if head_dim is not None:
        if size is not None and size % head_dim != 0:
            raise ValueError(f"{head_dim} must divide {size} for {type(module)} at {location}")
        size = head_dim
    return size


@TransformFactory.register("hadamard")
class HadamardFactory(TransformFactory):
    def __init__(self, name: str, scheme: TransformScheme, seed: Optional[int] = None):
        super().__init__(name, scheme, seed)
        self._signs: Dict[int, Optional[Tensor]] = {}
        self._perms: Dict[int, Tensor] = {}

    def _create_signs(self, size: int) -> Optional[Tensor]:
        return None

    def create_transform(self, module: torch.nn.Module, args: TransformArgs) -> HadamardTransform:
        size = _transform_size(module, args.location, self.scheme.head_dim)
        if size not in self._signs:  # one draw per size, as the reference's weight cache
            self._signs[size] = self._create_signs(size)
        perm = None
        if self.scheme.randomize:
            if size not in self._perms:
                self._perms[size] = torch.randperm(size, generator=self.generator)
            perm = self._perms[size]
        precision = self.scheme.precision if args.is_online() else torch.float64
        return HadamardTransform(size, self._signs[size], perm, self.scheme, args, type(module),
                                 precision=precision)


@TransformFactory.register("random-hadamard")
class RandomHadamardFactory(HadamardFactory):
    def _create_signs(self, size: int) -> Optional[Tensor]:
        if not (is_pow2(size) and size >= 64):
            raise NotImplementedError(
                f"random Hadamard matrices are built for powers of two >= 64, got {size}"
            )
        return random_hadamard_signs(size, self.generator)
