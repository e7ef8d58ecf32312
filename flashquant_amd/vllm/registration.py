"""Registration of the backend with vLLM (src/flashquant/vllm/registration.py:29-134): the version
gate, the CUSTOM slot of the backend registry, the block allocator's spec map, and the patch that
makes decoder attention layers report the packed uint8 cache spec.  Called by the
``vllm.general_plugins`` entry point or by hand before vLLM starts; calling it again does nothing."""
from __future__ import annotations

import logging

from flashquant_amd.errors import FlashQuantCompatError
from flashquant_amd.vllm.compat import check_vllm_version

logger = logging.getLogger(__name__)

_registered = False
_stock_get_kv_cache_spec = None


def register_flashquant_backend() -> None:
    global _registered, _stock_get_kv_cache_spec
    if _registered:
        return
    found = check_vllm_version()
    try:
        import torch
        from vllm.v1.attention.backends.registry import AttentionBackendEnum, register_backend
        from vllm.v1.kv_cache_interface import FullAttentionSpec
    except ImportError as exc:
        raise FlashQuantCompatError(f"vLLM {found} lacks an internal the plugin hooks into: {exc}") from exc

    from flashquant_amd.vllm.backend import get_flashquant_backend_class
    from flashquant_amd.vllm.spec import get_flashquant_attention_spec

    backend = get_flashquant_backend_class()
    register_backend(AttentionBackendEnum.CUSTOM, f"{backend.__module__}.{backend.__qualname__}")

    spec_class = get_flashquant_attention_spec()
    try:
        from vllm.v1.core.single_type_kv_cache_manager import spec_manager_map
        spec_manager_map.setdefault(spec_class, spec_manager_map[FullAttentionSpec])
    except ImportError:
        logger.warning("vLLM's spec_manager_map not found: pages of the packed size may not be allocated")

    try:
        from dataclasses import fields

        from vllm.model_executor.layers.attention.attention import Attention

        if _stock_get_kv_cache_spec is None:
            _stock_get_kv_cache_spec = Attention.get_kv_cache_spec
        stock = _stock_get_kv_cache_spec

        def packed_get_kv_cache_spec(self, vllm_config):
            spec = stock(self, vllm_config)
            if isinstance(spec, FullAttentionSpec) and not isinstance(spec, spec_class):
                values = {f.name: getattr(spec, f.name) for f in fields(spec)}
                values["dtype"] = torch.uint8
                return spec_class(**values)
            return spec

        Attention.get_kv_cache_spec = packed_get_kv_cache_spec
    except ImportError:
        logger.warning("vLLM's Attention layer not found: configure the packed cache spec by hand")

    _registered = True
    logger.info("FlashQuant attention backend registered as CUSTOM (packed TQ4 cache, vLLM %s)", found)
