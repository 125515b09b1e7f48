from .helpers import *  # noqa: F401,F403
from .safetensors_io import *  # noqa: F401,F403
from .internal import *  # noqa: F401,F403
from .match import *  # noqa: F401,F403
