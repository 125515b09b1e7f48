"""A transform configuration and its application to a model (reference:
src/compressed_tensors/transform/transform_config.py, transform/apply.py)."""
from typing import Dict

import torch

from compressed_tensors_amd.config import TRANSFORM_CONFIG_NAME

from .hadamard import TransformFactory, TransformScheme

__all__ = ["TransformConfig", "apply_transform_config"]


class TransformConfig:
    """named transform schemes, as written into a model's config.json
    (transform_config.py:23-35)"""

    def __init__(self, config_groups: Dict[str, TransformScheme]):
        self.config_groups = {name: TransformScheme.model_validate(scheme)
                              for name, scheme in config_groups.items()}

    def model_dump(self) -> Dict:
        return {"config_groups": {name: s.model_dump() for name, s in self.config_groups.items()}}

    @classmethod
    def model_validate(cls, data) -> "TransformConfig":
        if isinstance(data, cls):
            return data
        extra = set(data) - {"config_groups"}
        if extra:
            raise ValueError(f"TransformConfig: unexpected field(s) {sorted(extra)}")
        return cls(config_groups=data["config_groups"])

    def __eq__(self, other) -> bool:
        return isinstance(other, TransformConfig) and self.model_dump() == other.model_dump()

    def __repr__(self) -> str:
        return f"TransformConfig({self.model_dump()})"


def apply_transform_config(model: torch.nn.Module, config: TransformConfig) -> None:
    """Every scheme of the configuration goes into the model: transforms of weights are
    multiplied into the weights (on the GPU, several weights per launch), transforms of
    activations become submodules called from hooks; the configuration is left on the model
    for the compressor to write out (transform/apply.py:27-49)."""
    for name, scheme in config.config_groups.items():
        TransformFactory.from_scheme(scheme, name=name).apply_to_model(model)
    setattr(model, TRANSFORM_CONFIG_NAME, config)
