from .hadamard import *  # noqa: F401,F403
