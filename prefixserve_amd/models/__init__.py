"""Architectures known to the registry. Importing this package registers them."""

from . import fubelorn  # noqa: F401
from . import gokolix  # noqa: F401
from . import larupel  # noqa: F401
from . import llama  # noqa: F401
from . import radivik  # noqa: F401
