from .hadamard import *  # noqa: F401,F403
from .matrix_multiply import *  # noqa: F401,F403
from .apply import *  # noqa: F401,F403
