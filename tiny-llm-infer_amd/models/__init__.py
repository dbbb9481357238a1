"""Architectures this engine knows.  Importing the package registers them."""
from . import qwen3  # noqa: F401
from . import sinepel  # noqa: F401
from . import kapanex  # noqa: F401
from . import gimipel  # noqa: F401
from . import defosun  # noqa: F401
