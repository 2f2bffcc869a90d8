"""Restatement of the platform's rollout feature-flag translation.

``parse_arctic_inference_rollout`` (arctic_platform/common/utils/server_models.py:123-140):
an absent or empty config yields nothing; ``zorro_inference.enable`` truthy yields
``use_fca = True`` only when the engine's config model declares that field;
``speculative_decoding.model`` (stripped, non-empty) yields ``spec_model`` under the same
condition.  ``build_model_config`` (:143-165) overlays those on the user's engine dict,
sets ``model``, and moves every key the config model does not declare into
``extra_engine_kwargs``.
"""

from __future__ import annotations


def rollout_flags(arctic_inference_config, model_config_fields=None):
    if not arctic_inference_config:
        return {}
    known = set(model_config_fields or ())
    found = {}
    zorro = arctic_inference_config.get("zorro_inference")
    if isinstance(zorro, dict) and zorro.get("enable") and "use_fca" in known:
        found["use_fca"] = True
    spec = arctic_inference_config.get("speculative_decoding")
    if isinstance(spec, dict):
        name = (spec.get("model") or "").strip()
        if name and "spec_model" in known:
            found["spec_model"] = name
    return found


def model_config_kwargs(model_name, vllm_config, arctic_inference_config, known_fields):
    merged = dict(vllm_config or {})
    merged["model"] = model_name
    merged.update(rollout_flags(arctic_inference_config, known_fields))
    declared = {k: v for k, v in merged.items() if k in known_fields}
    other = {k: v for k, v in merged.items() if k not in known_fields}
    if other:
        declared["extra_engine_kwargs"] = other
    return declared
