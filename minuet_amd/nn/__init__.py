from . import functional
from .kernel_map import *
from .convolutions import *
from .activations import *
from .normalizations import *
from .pooling import *
from .fused import *
