from .base import Layer
from .linear import Dense, Flatten
from .convolutional import Conv2D
from .pooling import MaxPooling2D, AvgPooling2D
from .normalize import BatchNormalization
from .activators import ReLU, Sigmoid, Tanh, Activation, get_activator
from .ops import Input, Add
