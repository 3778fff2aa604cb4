"""Stage ranges of the layer for rocprofv3 (``--marker-trace``) and other roctx consumers.

The reference wraps the stages of ``topk_moe_forward`` in profiler scopes named "router",
"get_token_indices", "fused_grouped_glu", "down_grouped_gemm", "scale_and_reduce" and
"shared_expert" (``functional/topk_moe.py:16-57``).  Here the same names are pushed as roctx
ranges (``torch.cuda.nvtx`` is roctx on ROCm).  Off by default, since a range costs two host
calls a stage: switch on with ``MOE_EXPLORE_TRACE=1`` or ``enable(True)``.
"""
import contextlib
import os

_enabled = os.environ.get("MOE_EXPLORE_TRACE", "0") not in ("", "0")


def enable(on=True):
    global _enabled
    _enabled = bool(on)


def enabled():
    return _enabled


class _Null:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NULL = _Null()


@contextlib.contextmanager
def _range(name):
    import torch
    torch.cuda.nvtx.range_push(name)
    try:
        yield
    finally:
        torch.cuda.nvtx.range_pop()


def scope(name):
    """Context manager: a roctx range called ``name`` when tracing is on, else nothing."""
    return _range(name) if _enabled else _NULL
