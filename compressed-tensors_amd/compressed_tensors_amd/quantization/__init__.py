from .quant_args import *  # noqa: F401,F403
from .quant_scheme import *  # noqa: F401,F403
from .helpers import *  # noqa: F401,F403
from .forward import *  # noqa: F401,F403
from .initialize import *  # noqa: F401,F403
from .mxfp4_utils import *  # noqa: F401,F403
from .lifecycle import *  # noqa: F401,F403
from .quant_metadata import *  # noqa: F401,F403
from compressed_tensors_amd.config import (  # noqa: F401
    DEFAULT_QUANTIZATION_FORMAT, DEFAULT_QUANTIZATION_METHOD, LIFECYCLE_ORDER, QuantizationStatus,
)
