"""Feature-flag path: the package's parser against the oracle's restatement and the
literal cases of arctic_platform/common/utils/server_models.py:123-165."""

import pytest

from arctic_platform_amd.config import ModelConfig, build_model_config, parse_arctic_inference_rollout, validate_fca_support
from oracle.flags import model_config_kwargs, rollout_flags

FIELDS = {"use_fca", "spec_model", "model"}
CASES = [
    (None, FIELDS, {}),
    ({}, FIELDS, {}),
    ({"zorro_inference": {"enable": True}}, FIELDS, {"use_fca": True}),
    ({"zorro_inference": {"enable": True}}, {"model"}, {}),
    ({"zorro_inference": {"enable": False}}, FIELDS, {}),
    ({"zorro_inference": True}, FIELDS, {}),
    ({"speculative_decoding": {"model": " x "}}, FIELDS, {"spec_model": "x"}),
    ({"speculative_decoding": {"model": "   "}}, FIELDS, {}),
    ({"speculative_decoding": {"model": None}}, FIELDS, {}),
    ({"speculative_decoding": {"model": "d"}}, {"use_fca"}, {}),
    ({"zorro_inference": {"enable": 1}, "speculative_decoding": {"model": "d"}}, FIELDS, {"use_fca": True, "spec_model": "d"}),
    ({"zorro_inference": {"enable": True}}, None, {}),
]


@pytest.mark.parametrize("cfg,fields,want", CASES)
def test_rollout_flags(cfg, fields, want):
    assert rollout_flags(cfg, fields) == want
    assert parse_arctic_inference_rollout(cfg, fields) == want


def test_build_model_config_splits_unknown_keys():
    vllm = {"tensor_parallel_size": 1, "forest_cascade_attn_configs": "{}", "max_num_seqs": 256}
    cfg = build_model_config("Qwen/Qwen3-4B", vllm, {"zorro_inference": {"enable": True}})
    assert cfg.model == "Qwen/Qwen3-4B" and cfg.use_fca is True and cfg.max_num_seqs == 256
    assert cfg.extra_engine_kwargs == {"forest_cascade_attn_configs": "{}"}
    want = model_config_kwargs("Qwen/Qwen3-4B", vllm, {"zorro_inference": {"enable": True}}, ModelConfig.field_names())
    got = {k: getattr(cfg, k) for k in want}
    assert got == want


def test_feature_stays_off_without_config():
    assert build_model_config("m").use_fca is False
    assert build_model_config("m", {"max_num_seqs": 8}, {}).use_fca is False


def test_unsupported_shapes_fail_at_setup():
    with pytest.raises(ValueError):
        build_model_config("m", {"block_size": 32}, {"zorro_inference": {"enable": True}})
    build_model_config("m", {"block_size": 32}, None)  # feature off: nothing to reject
    cfg = ModelConfig(model="m", use_fca=True)
    with pytest.raises(ValueError):
        validate_fca_support(cfg, head_dim=96)
    with pytest.raises(ValueError):
        validate_fca_support(cfg, num_q_heads=12, num_kv_heads=5)
    validate_fca_support(cfg, head_dim=128, num_q_heads=32, num_kv_heads=8)
