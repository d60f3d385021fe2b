from . import state  # noqa: F401
from .base import Tensor, Parameter  # noqa: F401
