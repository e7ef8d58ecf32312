"""flashquant_amd: the TurboQuant TQ4 KV-cache hot path on MI355X (gfx950).

The package holds hand-written HIP kernels behind a C ABI (libfq_hip.so,
include/fq_hip.h), the pybind11 module ``_C`` that exposes them under the
operator names the reference's Python layer looks for, and a Python layer with
the reference's operator signatures (``flashquant_amd.kernels``).  There is no
CPU fallback: every operator raises if the native module is missing or a
tensor is not on the GPU.
"""
from __future__ import annotations

__version__ = "0.1.0"


def load_native():
    """Imports and returns the pybind11 module, with a clear error if it has not
    been built (``python -m flashquant_amd.build``)."""
    try:
        from flashquant_amd import _C  # type: ignore[attr-defined]
    except ImportError as exc:  # pragma: no cover - exercised only on a broken install
        raise ImportError(
            "flashquant_amd._C is not built or cannot be loaded; run "
            "`python -m flashquant_amd.build` from the repository root "
            f"(original error: {exc})"
        ) from exc
    return _C
