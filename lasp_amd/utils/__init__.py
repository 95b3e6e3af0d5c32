from .module_utils import *  # noqa: F401,F403
from .seq_parallel_manager import *  # noqa: F401,F403
