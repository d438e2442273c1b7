"""MI355X-native GridNeRF render path (hand-written HIP behind a C ABI)."""
from .params import GridNeRFParams  # noqa: F401

__all__ = ["GridNeRFParams", "GridNeRFHIP", "renderer_fn", "MultiBlockParallelHIP"]


def __getattr__(name):
    if name in ("GridNeRFHIP", "from_reference_model"):
        from . import model

        return getattr(model, name)
    if name in ("renderer_fn", "MultiBlockParallelHIP"):
        from . import render

        return getattr(render, name)
    raise AttributeError(name)
