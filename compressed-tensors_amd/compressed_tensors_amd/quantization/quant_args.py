"""Quantization argument vocabulary (host side, plain Python).

Mirrors the fields, defaults, validation rules and error types of the
reference's QuantizationArgs (quantization/quant_args.py:148-381) so that
configs written for the reference read the same here.  No pydantic: a slotted
class with explicit validation.
"""
import warnings
from enum import Enum
from typing import Any, Dict, List, Optional, Union

import torch

from compressed_tensors_amd.utils.helpers import Aliasable

__all__ = [
    "FP8_DTYPE",
    "FP8_E4M3_DATA",
    "FP4_E2M1_DATA",
    "BFLOAT16_DATA",
    "FloatArgs",
    "round_to_quantized_type",
    "QuantizationType",
    "QuantizationStrategy",
    "DynamicType",
    "ActivationOrdering",
    "QuantizationArgs",
]

FP8_DTYPE = torch.float8_e4m3fn


class FloatArgs:
    """the fields a floating-point format is described by (quant_args.py:39-45)"""
    exponent: int
    mantissa: int
    bits: Optional[int] = None
    max: Optional[float] = None
    min: Optional[float] = None
    dtype: Optional[torch.dtype] = None


class FP4_E2M1_DATA(FloatArgs):
    exponent, mantissa, bits = 2, 1, 4
    max, min = 6.0, -6.0

    @staticmethod
    def cast_to_fp4(x: torch.Tensor) -> torch.Tensor:
        """every element to the nearest e2m1 value, in x's dtype (quant_args.py:55-68); on
        the GPU, into a new tensor"""
        return _round_on_gpu(x, 1, 4)


class FP8_E4M3_DATA(FloatArgs):
    exponent, mantissa, bits = 4, 3, 8
    max = torch.finfo(FP8_DTYPE).max  # 448
    min = torch.finfo(FP8_DTYPE).min
    dtype = FP8_DTYPE


class BFLOAT16_DATA(FloatArgs):
    exponent, mantissa = 8, 7


def _round_on_gpu(tensor: torch.Tensor, qtype: int, num_bits: int) -> torch.Tensor:
    from compressed_tensors_amd import _lib

    _lib.require_gpu(tensor)
    x = tensor.contiguous()
    if x.data_ptr() % 16:  # a view that starts inside a buffer: the kernel reads 16 bytes a lane
        x = x.clone()
    out = torch.empty_like(x)
    _lib.check(_lib.load().ctmi_round_to_quantized_type(
        x.data_ptr(), out.data_ptr(), _lib.dtype_code(x.dtype), x.numel(), qtype, num_bits,
        _lib.stream_of(x.device)))
    return out


def round_to_quantized_type(tensor: torch.Tensor, args: "QuantizationArgs") -> torch.Tensor:
    """every element to the nearest value of the quantized type, in the tensor's dtype
    (quant_args.py:384-408): one kernel, the tensor read once"""
    qtype = args.type.value if isinstance(args.type, Enum) else args.type
    if qtype == QuantizationType.FLOAT.value:
        if args.num_bits not in (4, 8):
            raise NotImplementedError("Only num_bits in (4, 8) are supported")
        return _round_on_gpu(tensor, 1, args.num_bits)
    if qtype == QuantizationType.INT.value:
        return _round_on_gpu(tensor, 0, args.num_bits)
    raise ValueError(f"Invalid quantization type {args.type}")


class QuantizationType(str, Enum):
    INT = "int"
    FLOAT = "float"


class QuantizationStrategy(str, Enum):
    TENSOR = "tensor"
    CHANNEL = "channel"
    GROUP = "group"
    BLOCK = "block"
    TOKEN = "token"
    TENSOR_GROUP = "tensor_group"
    ATTN_HEAD = "attn_head"


class DynamicType(str, Enum):
    LOCAL = "local"


class ActivationOrdering(Aliasable, str, Enum):
    """group: groups and weight are reordered; weight: the weight only; dynamic and static
    are other names for the two and compare equal to them (quant_args.py:123-145)"""
    GROUP = "group"
    WEIGHT = "weight"
    DYNAMIC = "dynamic"
    STATIC = "static"

    @staticmethod
    def get_aliases() -> Dict[str, str]:
        return {"dynamic": "group", "static": "weight"}

    @classmethod
    def parse(cls, value: str) -> "ActivationOrdering":
        return cls(value.lower())


_GROUPED = (QuantizationStrategy.GROUP.value, QuantizationStrategy.TENSOR_GROUP.value)
_DYNAMIC_OK = (
    QuantizationStrategy.TOKEN.value,
    QuantizationStrategy.TENSOR.value,
    QuantizationStrategy.TENSOR_GROUP.value,
    QuantizationStrategy.GROUP.value,
)


def _enum_value(v):
    return v.value if isinstance(v, Enum) else v


class QuantizationArgs:
    """num_bits / type / symmetric / group_size / strategy / block_structure /
    dynamic / actorder / observer / observer_kwargs.  Enum-valued fields are
    stored as their string values (the reference uses `use_enum_values`)."""

    __slots__ = (
        "num_bits",
        "type",
        "symmetric",
        "group_size",
        "strategy",
        "block_structure",
        "dynamic",
        "actorder",
        "observer",
        "observer_kwargs",
    )

    def __init__(
        self,
        num_bits: int = 8,
        type: Union[QuantizationType, str] = QuantizationType.INT,
        symmetric: bool = True,
        group_size: Optional[int] = None,
        strategy: Union[QuantizationStrategy, str, None] = None,
        block_structure: Union[List[int], str, None] = None,
        dynamic: Union[DynamicType, bool, str] = False,
        actorder: Union[ActivationOrdering, bool, str, None] = None,
        observer: Optional[str] = None,
        observer_kwargs: Optional[Dict[str, Any]] = None,
    ):
        self.num_bits = int(num_bits)
        self.type = QuantizationType(_enum_value(type).lower()).value
        self.symmetric = bool(symmetric)

        if group_size is not None and group_size < -1:
            raise ValueError(
                f"Invalid group size {group_size}. Use group_size > 0 for "
                "strategy='group' and group_size = -1 for 'channel'"
            )
        self.group_size = group_size

        if isinstance(block_structure, str):
            try:
                block_structure = [int(p) for p in block_structure.split("x")]
            except Exception:
                raise ValueError(
                    f"Invalid block_structure '{block_structure}'. Must be a list of ints "
                    "[rows, cols]."
                )
        if block_structure is not None:
            if (
                not isinstance(block_structure, (list, tuple))
                or len(block_structure) != 2
                or not all(isinstance(v, int) for v in block_structure)
            ):
                raise ValueError(
                    f"Invalid block_structure '{block_structure}'. Must be a list of ints "
                    "[rows, cols]."
                )
            block_structure = list(block_structure)
        self.block_structure = block_structure

        if isinstance(dynamic, str):
            dynamic = DynamicType(dynamic.lower()).value
        self.dynamic = _enum_value(dynamic)

        if isinstance(actorder, bool):
            actorder = ActivationOrdering.GROUP if actorder else None
        elif isinstance(actorder, str):
            actorder = ActivationOrdering.parse(actorder)
        self.actorder = _enum_value(actorder)

        if strategy is not None:
            strategy = QuantizationStrategy(_enum_value(strategy).lower()).value
        self.observer = observer
        self.observer_kwargs = dict(observer_kwargs or {})
        self.strategy = strategy
        self._finish()

    def _finish(self) -> None:
        strategy, group_size = self.strategy, self.group_size
        if strategy is None:
            if group_size is None:
                strategy = QuantizationStrategy.TENSOR.value
            elif group_size > 0:
                strategy = QuantizationStrategy.GROUP.value
            elif group_size == -1:
                strategy = QuantizationStrategy.CHANNEL.value
            else:
                raise ValueError(
                    f"Invalid group size {group_size}. Use group_size > 0 for "
                    "strategy='group' and group_size = -1 for 'channel'"
                )
        if strategy == QuantizationStrategy.TOKEN.value and not self.dynamic:
            raise ValueError("Cannot perform static token quantization, please use `dynamic=True`")
        if strategy in _GROUPED and (group_size is None or group_size <= 0):
            raise ValueError(f"strategy {strategy} requires group_size to be set to a positive value")
        if group_size is not None and group_size > 0 and strategy not in _GROUPED:
            raise ValueError("group_size requires strategy to be set to 'group'")
        is_block = strategy == QuantizationStrategy.BLOCK.value
        if is_block and self.block_structure is None:
            raise ValueError("Block strategy requires block structure")
        if self.block_structure is not None and not is_block:
            raise ValueError("Block structure requires block strategy")
        if self.actorder is not None and strategy != QuantizationStrategy.GROUP.value:
            raise ValueError(
                "Must use group quantization strategy in order to apply activation ordering"
            )
        observer = self.observer
        if self.dynamic:
            if strategy not in _DYNAMIC_OK:
                raise ValueError(f"One of {_DYNAMIC_OK} must be used for dynamic quant.")
            if self.dynamic == DynamicType.LOCAL.value and (
                strategy != QuantizationStrategy.TENSOR_GROUP.value
            ):
                raise ValueError("local is only supported for strategy tensor_group")
            if observer is not None:
                if self.dynamic is True:
                    if observer != "memoryless":
                        warnings.warn("No observer is used for dynamic quant., setting to None")
                    observer = None
            elif self.dynamic == DynamicType.LOCAL.value:
                observer = "minmax"
        elif observer is None:
            observer = "minmax"
        self.strategy = strategy
        self.observer = observer

    # ------------------------------------------------------------------
    def pytorch_dtype(self) -> torch.dtype:
        if self.type == QuantizationType.FLOAT.value:
            if self.num_bits == 8:
                return FP8_DTYPE
            raise NotImplementedError("Only num_bits in (8) are supported")
        if self.type == QuantizationType.INT.value:
            if self.num_bits <= 8:
                return torch.int8
            if self.num_bits <= 16:
                return torch.int16
            return torch.int32
        raise ValueError(f"Invalid quantization type {self.type}")

    def model_dump(self) -> Dict[str, Any]:
        return {k: getattr(self, k) for k in self.__slots__}

    @classmethod
    def model_validate(cls, data: Union["QuantizationArgs", Dict[str, Any]]) -> "QuantizationArgs":
        if isinstance(data, cls):
            return data
        unknown = set(data) - set(cls.__slots__)
        if unknown:
            raise ValueError(f"Unknown QuantizationArgs fields: {sorted(unknown)}")
        return cls(**data)

    def __eq__(self, other) -> bool:
        return isinstance(other, QuantizationArgs) and self.model_dump() == other.model_dump()

    def __repr__(self) -> str:
        return "QuantizationArgs(" + ", ".join(f"{k}={v!r}" for k, v in self.model_dump().items()) + ")"
