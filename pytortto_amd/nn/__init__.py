from .modules import *
from .parameter import Parameter
from . import functional
from . import init
