"""MI355X-native (gfx950) implementation of the xKV compressed-KV decode path.

Sub-packages mirror the reference project's module tree so they drop in for it:
``flash_recontruction`` (sic) - qAB / qAB_no_pe / rope / fused_attention, and
``flash_decoding`` - gqa.py, mla.py, mla2.  Put this directory on ``sys.path`` to import them
under their original top-level names.  All compute runs in hand-written HIP kernels loaded from
``libxkv_hip.so`` through the C ABI declared in ``include/xkv_hip.h``.
"""
from . import _lib  # noqa: F401

__all__ = ["_lib"]


def install_aliases() -> None:
    """Register ``flash_recontruction`` and ``flash_decoding`` as top-level module names bound to
    this package's mirrors, so code written against the reference (``from flash_recontruction
    import qAB_rope_v1``) runs unchanged."""
    import importlib
    import sys
    for name in ("flash_recontruction", "flash_decoding"):
        mod = importlib.import_module(f"{__name__}.{name}")
        sys.modules.setdefault(name, mod)
