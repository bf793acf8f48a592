from .quant_args import *  # noqa: F401,F403
from .lifecycle import *  # noqa: F401,F403
