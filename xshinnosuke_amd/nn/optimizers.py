"""``xs.nn.optimizers`` is the import path the reference's README uses; the classes live in ``optim``."""
from ..optim import Optimizer, SGD, get_optimizer  # noqa: F401
