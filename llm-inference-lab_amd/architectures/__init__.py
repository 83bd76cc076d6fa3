"""Architectures known to the framework; importing this package registers them."""
from . import qwen2  # noqa: F401
from . import vivevik  # noqa: F401
from . import ruvalorn  # noqa: F401
from . import minodra  # noqa: F401
from . import ninisun  # noqa: F401
