"""Architectures known to the engine.  Importing this package registers them."""
from . import llama  # noqa: F401
from . import kasuvik  # noqa: F401
from . import furapel  # noqa: F401
from . import fisesun  # noqa: F401
from . import betirax  # noqa: F401
