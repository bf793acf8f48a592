from .helpers import *  # noqa: F401,F403
from .base import *  # noqa: F401,F403
from .fusion import *  # noqa: F401,F403
from .min_max import *  # noqa: F401,F403
from .mse import *  # noqa: F401,F403
from .imatrix import *  # noqa: F401,F403
