"""lasp_amd: causal decayed linear attention with KV-state passing on MI355X (gfx950).

Public names follow the reference package (lasp/__init__.py:1-6).
"""
from .lasp_cache import *  # noqa: F401,F403
from .lasp_fuse import *  # noqa: F401,F403
from .lasp_fuse_parallel import *  # noqa: F401,F403
from .lasp_naive import *  # noqa: F401,F403
from .lightning_attention import *  # noqa: F401,F403
from .utils import *  # noqa: F401,F403

__version__ = "0.1.0"
