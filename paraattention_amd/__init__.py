"""paraattention_amd: the attention op layer of ParaAttention for MI355X (gfx950).

Importing the package registers the ``torch.ops.para_attn.*`` operators; the HIP
library itself is loaded on first use and its absence is an error, not a
fallback.
"""
from . import config  # noqa: F401
from . import ops  # noqa: F401  (registers torch.ops.para_attn.*)
from . import fbcache, interface, merge, sparse, taylorseer  # noqa: F401
from .interface import (  # noqa: F401
    InBatchAttnMode, RingAttnMode, SparseKVAttnMode, UlyssesAttnMode, UnifiedAttnMode, in_batch_attn_func,
    ring_attn_func, sparse_kv_attn_func, ulysses_attn_func,
)
from .merge import SDPAMerger, ring_sweep  # noqa: F401
from .taylorseer import TaylorSeer  # noqa: F401
from .sparse import StructSparseAttnMode, struct_sparse_attn_func  # noqa: F401

__all__ = [
    "config", "ops", "merge", "sparse", "fbcache", "taylorseer", "TaylorSeer", "interface",
    "UnifiedAttnMode", "SparseKVAttnMode", "RingAttnMode", "UlyssesAttnMode", "InBatchAttnMode",
    "sparse_kv_attn_func", "ring_attn_func", "ulysses_attn_func", "in_batch_attn_func",
    "SDPAMerger", "ring_sweep", "StructSparseAttnMode", "struct_sparse_attn_func",
]
