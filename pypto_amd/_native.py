"""Loads the native extension.  There is no fallback: when the HIP library or its pybind11 module
is missing the operators raise, naming the build command."""
from __future__ import annotations

_C = None
_ERR = None


def load():
    global _C, _ERR
    if _C is not None:
        return _C
    try:
        from . import _C as mod  # noqa: WPS433  (pybind11 module built by pypto_amd.build)
    except ImportError as exc:  # pragma: no cover - exercised only on a broken install
        _ERR = exc
        raise RuntimeError(
            "pypto_amd: the native HIP extension is not built or not loadable "
            f"({exc}); build it in-tree with `python -m pypto_amd.build`") from exc
    _C = mod
    return _C
