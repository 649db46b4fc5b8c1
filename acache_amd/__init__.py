"""acache_amd — MI355X (gfx950) implementation of ACache's affix-KV reuse hot path.

Host side (same names and signatures as the reference's nano-vdllm modules):
``Sequence``, ``BlockManager``, ``Scheduler``, ``Config``, ``Context`` helpers,
and the operator functions in :mod:`acache_amd.ops`, which call hand-written HIP
kernels in ``libacache_hip.so`` through a C ABI.
"""
from .block_manager import BlockManager
from .config import Config
from .scheduler import Scheduler
from .sequence import Sequence, SequenceStatus
from .utils import Context, get_context, reset_context, set_context

__all__ = [
    "BlockManager", "Config", "Scheduler", "Sequence", "SequenceStatus",
    "Context", "get_context", "reset_context", "set_context",
]
