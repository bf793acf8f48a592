from .base import GPTQModifier  # noqa: F401
from .gptq_quantize import *  # noqa: F401,F403
