from ..core.base import Tensor, Parameter
from ..core import state as GLOBAL
from . import functional
from .objectives import MSELoss, CrossEntropyLoss
from .models import Sequential, Model, Module
