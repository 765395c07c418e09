"""The two behaviour flags of the reference's config module (src/para_attn/config.py:12-17).

``attention.force_dispatch_to_custom_ops``: route plain SDPA calls of the modes to
``para_attn::attention_forward`` (src/para_attn/para_attn_interface.py:469-470).
``attention.allow_reduced_precision_compute``: merge partial results in the
activation dtype instead of fp32 (src/para_attn/para_attn_interface.py:132-137,
src/para_attn/sparse_attn.py:175).
"""
import contextlib
import os


class _Attention:
    force_dispatch_to_custom_ops = os.getenv("PARA_ATTN_FORCE_DISPATCH_TO_CUSTOM_OPS") == "1"
    allow_reduced_precision_compute = os.getenv("PARA_ATTN_ALLOW_REDUCED_PRECISION_COMPUTE") == "1"


attention = _Attention()


@contextlib.contextmanager
def patch(**kwargs):
    """``with config.patch(**{"attention.allow_reduced_precision_compute": True}): ...``"""
    saved = {}
    try:
        for key, val in kwargs.items():
            key = key.replace("__", ".")
            group, _, name = key.rpartition(".")
            if group != "attention" or not hasattr(attention, name):
                raise AttributeError(f"unknown config entry {key!r}")
            saved[name] = getattr(attention, name)
            setattr(attention, name, val)
        yield
    finally:
        for name, val in saved.items():
            setattr(attention, name, val)
