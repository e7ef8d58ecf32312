"""vLLM version gate (src/flashquant/vllm/compat.py:49-90): the plugin hooks into vLLM internals that
move between releases, so a version outside [VLLM_MIN, VLLM_MAX) is refused with a message that says
what to install, instead of failing later with an import error somewhere inside vLLM."""
from __future__ import annotations

import re
from typing import Tuple

from flashquant_amd.errors import FlashQuantCompatError

VLLM_MIN = "0.18.0"
VLLM_MAX = "0.22.0"


def parse_version(text: str) -> Tuple[int, ...]:
    """Leading integers of the dot-separated fields: '0.20.1.dev0+rocm' -> (0, 20, 1)."""
    fields = []
    for part in text.split("."):
        m = re.match(r"\d+", part)
        if m is None:
            break
        fields.append(int(m.group()))
    return tuple(fields)


def check_vllm_version() -> str:
    """The installed vLLM's version string; raises FlashQuantCompatError when vLLM is missing or its
    version lies outside the supported range."""
    wanted = f"vLLM >= {VLLM_MIN}, < {VLLM_MAX}"
    try:
        import vllm
    except ImportError:
        raise FlashQuantCompatError(f"vLLM is not installed; the FlashQuant attention backend needs {wanted}") from None
    found = str(getattr(vllm, "__version__", "0.0.0"))
    version = parse_version(found)
    if version < parse_version(VLLM_MIN):
        raise FlashQuantCompatError(f"vLLM {found} is older than the plugin supports ({wanted})")
    if version >= parse_version(VLLM_MAX):
        raise FlashQuantCompatError(f"vLLM {found} is newer than the plugin was written against ({wanted})")
    return found
