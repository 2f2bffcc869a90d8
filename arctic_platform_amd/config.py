"""Feature-flag path of forest cascade attention.

Mirrors the platform's translation of ``arctic_inference_config`` into engine fields:
``parse_arctic_inference_rollout`` and ``build_model_config``
(arctic_platform/common/utils/server_models.py:123-165).  An absent or empty config
leaves the feature off; an unsupported shape is rejected when the job is set up, not in
the middle of decoding (the fail-fast convention of
arctic_platform/model/patches/zorro_train.py:35-36).
"""

from __future__ import annotations

import dataclasses

from .kv_layout import BLOCK_SIZE


@dataclasses.dataclass
class ModelConfig:
    """The engine-side fields this build knows about (stand-in for the external
    engine's config model, which the platform imports at server_models.py:155)."""

    model: str = ""
    use_fca: bool = False
    spec_model: str | None = None
    tensor_parallel_size: int = 1
    max_num_seqs: int = 256
    block_size: int = BLOCK_SIZE
    kv_cache_dtype: str = "auto"
    extra_engine_kwargs: dict = dataclasses.field(default_factory=dict)

    @classmethod
    def field_names(cls) -> set:
        return {f.name for f in dataclasses.fields(cls)}


def parse_arctic_inference_rollout(arctic_inference_config, model_config_fields=None):
    """``{"zorro_inference": {"enable": True}}`` -> ``{"use_fca": True}`` when the engine
    config declares ``use_fca``; ``speculative_decoding.model`` -> ``spec_model`` likewise."""
    if not arctic_inference_config:
        return {}
    declared = set(model_config_fields or ())
    picked = {}
    section = arctic_inference_config.get("zorro_inference")
    if isinstance(section, dict) and section.get("enable") and "use_fca" in declared:
        picked["use_fca"] = True
    section = arctic_inference_config.get("speculative_decoding")
    if isinstance(section, dict):
        draft = (section.get("model") or "").strip()
        if draft and "spec_model" in declared:
            picked["spec_model"] = draft
    return picked


def build_model_config(model_name, vllm_config=None, arctic_inference_config=None) -> ModelConfig:
    declared = ModelConfig.field_names()
    merged = dict(vllm_config or {})
    merged["model"] = model_name
    merged.update(parse_arctic_inference_rollout(arctic_inference_config, declared))
    kwargs = {k: v for k, v in merged.items() if k in declared}
    rest = {k: v for k, v in merged.items() if k not in declared}
    if rest:
        kwargs["extra_engine_kwargs"] = rest
    cfg = ModelConfig(**kwargs)
    validate_fca_support(cfg)
    return cfg


def validate_fca_support(cfg: ModelConfig, *, head_dim=None, num_q_heads=None, num_kv_heads=None) -> None:
    """Raise at set-up time for shapes the kernels do not cover."""
    if not cfg.use_fca:
        return
    if cfg.block_size != BLOCK_SIZE:
        raise ValueError(f"forest cascade attention needs block_size={BLOCK_SIZE}, got {cfg.block_size}")
    if cfg.kv_cache_dtype not in ("auto", "bfloat16", "fp8", "fp8_e4m3"):
        raise ValueError(f"forest cascade attention supports bf16 and fp8 e4m3 KV caches, got {cfg.kv_cache_dtype!r}")
    if head_dim is not None and head_dim not in (64, 128, 256):
        raise ValueError(f"forest cascade attention supports head_dim 64, 128 or 256, got {head_dim}")
    if num_q_heads is not None and num_kv_heads is not None:
        # (a member's query heads must fit one row tile: 32 rows by default, 64 at most)
        if num_q_heads % num_kv_heads or num_q_heads // num_kv_heads > 64:
            raise ValueError("num_q_heads must be a multiple of num_kv_heads with at most 64 query heads per KV head")
