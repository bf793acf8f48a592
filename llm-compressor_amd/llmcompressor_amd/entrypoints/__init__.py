from .oneshot import Oneshot, oneshot  # noqa: F401
from .model_free import model_free_ptq  # noqa: F401,E402
