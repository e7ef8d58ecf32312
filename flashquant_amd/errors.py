"""Exception types of the package (names of src/flashquant/errors.py:25-60)."""
from __future__ import annotations


class FlashQuantError(Exception):
    """Base class of the package's own errors."""


class FlashQuantCompatError(FlashQuantError):
    """The installed vLLM (or one of the internals the plugin hooks into) is not one the plugin supports."""
