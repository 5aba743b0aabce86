"""vLLM plugin entry point (reference: aither_kvcache/vllm/plugin.py:18-53).

vLLM calls `register()` at start-up in every process (API server and engine workers) for each
entry point listed under `vllm.general_plugins`; a packaging file would name
`aitherkvcache_amd.vllm.plugin:register` there.  It registers the TurboQuant attention backend
under the CUSTOM slot (`--attention-backend CUSTOM`) and the tq::decode_step /
tq::hybrid_decode_step ops.  The reference's second registration, its graph-aware block eviction,
is a scheduler policy and no part of this package.
"""
import logging
import sys

logger = logging.getLogger("turboquant.vllm.plugin")


def register() -> bool:
    """Returns True when the backend was registered with vLLM.  Never raises: a process without
    vLLM (or with a release whose registry differs) keeps running without the backend."""
    print("[aitherkvcache-amd] plugin register() called", file=sys.stderr, flush=True)
    try:
        from vllm.v1.attention.backends.registry import AttentionBackendEnum, register_backend
    except ImportError:
        return False
    try:
        register_backend(AttentionBackendEnum.CUSTOM, "aitherkvcache_amd.vllm.backend.TurboQuantBackend")
    except Exception as e:
        print(f"[aitherkvcache-amd] backend registration failed: {e}", file=sys.stderr, flush=True)
        return False
    try:
        from .hooks import register_custom_ops
        register_custom_ops()
    except Exception as e:      # the impl calls the plain functions when the ops are missing
        logger.warning("custom op registration failed: %s", e)
    print("[aitherkvcache-amd] registered TurboQuant CUSTOM backend", file=sys.stderr, flush=True)
    return True
