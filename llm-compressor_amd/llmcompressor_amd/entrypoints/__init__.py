from .oneshot import Oneshot, oneshot  # noqa: F401
