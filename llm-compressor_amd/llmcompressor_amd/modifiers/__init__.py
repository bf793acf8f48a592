from .modifier import Modifier  # noqa: F401
from .factory import ModifierFactory  # noqa: F401
