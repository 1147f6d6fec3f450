"""Architectures.  Importing this package registers them."""
from . import llama  # noqa: F401
from . import sagalorn  # noqa: F401
from . import dekinex  # noqa: F401
from . import vumalix  # noqa: F401
from . import tekilix  # noqa: F401
