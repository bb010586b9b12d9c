from .build import BuildError, all_units, ensure
from .ops import HipOps, KernelError
from .tuning import Tuning
