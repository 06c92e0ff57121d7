"""Parts a layer is put together from; importing this package registers the built-in kinds."""
from . import base, linear, norm, rotary, attention, mlp, block  # noqa: F401
