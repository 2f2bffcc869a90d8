"""MI355X-native forest cascade decode attention (ZoRRo inference path) and the trainer's
split attention over deduplicated batches (ZoRRo Train)."""

from .config import ModelConfig, build_model_config, parse_arctic_inference_rollout, validate_fca_support
from .kv_layout import BLOCK_SIZE, convert_cache, kv_cache_shape, pack_blocks, unpack_blocks

__all__ = [
    "BLOCK_SIZE",
    "ModelConfig",
    "build_model_config",
    "parse_arctic_inference_rollout",
    "validate_fca_support",
    "kv_cache_shape",
    "pack_blocks",
    "unpack_blocks",
    "convert_cache",
    "build_forest_metadata",
    "forest_cascade_decode",
    "append_kv",
    "SplitLayout",
    "split_attention_forward",
    "split_attention_backward",
    "reconstruct_sequences",
    "deduplicate_sequences",
]


def __getattr__(name):
    # operators need the HIP library; resolve them lazily so the flag parser and layout
    # helpers stay importable in a process that only builds or inspects
    if name in ("build_forest_metadata", "ForestMetadata"):
        from . import forest

        return getattr(forest, name)
    if name in ("forest_cascade_decode", "prefix_pass", "suffix_pass", "forest_pass", "merge_partials"):
        from . import ops

        return getattr(ops, name)
    if name in ("ForestCascadeAttentionBackend", "ForestCascadeMetadataBuilder", "ForestCascadeAttentionImpl"):
        from . import backend

        return getattr(backend, name)
    if name in ("SplitLayout", "split_attention_forward", "split_attention_backward", "split_attention_padded"):
        # (the operator `split_attention` itself is reached as split_attention.split_attention:
        # the name belongs to the submodule)
        import importlib

        return getattr(importlib.import_module(".split_attention", __name__), name)
    if name in ("reconstruct_sequences", "deduplicate_sequences"):
        from . import reconstruct

        return getattr(reconstruct, name)
    if name == "append_kv":
        from . import cache

        return cache.append_kv
    raise AttributeError(name)
