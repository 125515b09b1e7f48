"""`dense`: the identity compressor (reference: compressors/sparse_compressors/dense.py:28-67)."""
from typing import Dict, Generator, Tuple

from torch import Tensor

from compressed_tensors_amd.compressors.base import BaseCompressor
from compressed_tensors_amd.config import CompressionFormat
from compressed_tensors_amd.utils.helpers import load_safetensors_state_dict

__all__ = ["DenseCompressor"]


@BaseCompressor.register(name=CompressionFormat.dense.value)
class DenseCompressor(BaseCompressor):
    @property
    def compression_param_names(self) -> Tuple[str]:
        return ()

    def compress(self, model_state: Dict[str, Tensor], **kwargs) -> Dict[str, Tensor]:
        return model_state

    def decompress(
        self, path_to_model_or_tensors, device: str = "cpu", **kwargs
    ) -> Generator[Tuple[str, Tensor], None, None]:
        state = (
            path_to_model_or_tensors
            if isinstance(path_to_model_or_tensors, dict)
            else load_safetensors_state_dict(path_to_model_or_tensors, device=device)
        )
        yield from state.items()

    def decompress_from_state_dict(self, state_dict: Dict[str, Tensor]):
        yield from state_dict.items()

    def decompress_module_from_state_dict(self, prefix, state_dict, scheme):
        return dict(state_dict)
