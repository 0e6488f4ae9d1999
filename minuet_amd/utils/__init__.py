from . import typing
from . import random
from . import helpers
