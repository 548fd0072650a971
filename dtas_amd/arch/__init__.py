from .arch_base import Arch
from .MI355X import MI355X
from .RTX3090 import RTX3090
