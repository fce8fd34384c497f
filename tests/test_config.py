"""Configuration and registry (vectors of the reference's tests/unit/test_model_config.py:41-199,
with sliding-window attention supported instead of rejected)."""

from __future__ import annotations

import json

import pytest
import torch

import tiny
from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
from turboserve_amd.config.model_config import Qwen2Config, UnsupportedModelError, read_config_json
from turboserve_amd.config.registry import ARCHITECTURES, architecture_of, parse_model_config
from turboserve_amd.sampling.params import SamplingParams

QWEN2_RAW = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "hidden_size": 64,
    "num_hidden_layers": 2,
    "num_attention_heads": 8,
    "num_key_value_heads": 2,
    "intermediate_size": 128,
    "vocab_size": 512,
    "max_position_embeddings": 4096,
    "rms_norm_eps": 1e-6,
    "rope_theta": 1000000.0,
    "hidden_act": "silu",
    "tie_word_embeddings": False,
    "torch_dtype": "bfloat16",
    "eos_token_id": 151645,
}


def test_bias_placement_and_derived_shapes():
    config = Qwen2Config.from_dict(QWEN2_RAW)
    assert (config.qkv_bias, config.o_proj_bias, config.mlp_bias) == (True, False, False)
    assert config.head_dim == 8 and config.num_kv_groups == 4 and config.is_gqa
    assert config.q_proj_size == 64 and config.kv_proj_size == 16
    assert config.attn_scale == pytest.approx(8 ** -0.5)
    big = Qwen2Config.from_dict({**QWEN2_RAW, "head_dim": 128})
    assert big.head_dim == 128 and big.q_proj_size == 8 * 128
    assert Qwen2Config.from_dict({**QWEN2_RAW, "attention_bias": False}).qkv_bias is True  # architectural
    minimal = {k: QWEN2_RAW[k] for k in ("architectures", "hidden_size", "num_hidden_layers", "num_attention_heads",
                                         "intermediate_size", "vocab_size")}
    defaults = Qwen2Config.from_dict(minimal)
    assert defaults.num_key_value_heads == 8 and defaults.rms_norm_eps == 1e-6 and defaults.rope_theta == 10000.0
    assert defaults.max_position_embeddings == 2048 and defaults.tie_word_embeddings is False
    assert defaults.hidden_act == "silu" and defaults.torch_dtype is None and defaults.eos_token_ids == ()


def test_rope_spellings_and_scaling():
    flat = Qwen2Config.from_dict({**QWEN2_RAW, "rope_theta": 5000.0})
    nested_raw = {k: v for k, v in QWEN2_RAW.items() if k != "rope_theta"}
    nested = Qwen2Config.from_dict({**nested_raw, "rope_parameters": {"rope_type": "default", "rope_theta": 5000.0}})
    assert flat.rope_theta == nested.rope_theta == 5000.0
    assert flat.rope_scaling_factor == nested.rope_scaling_factor == 1.0
    linear = Qwen2Config.from_dict({**QWEN2_RAW, "rope_scaling": {"rope_type": "linear", "factor": 4.0}})
    assert linear.rope_scaling_factor == 4.0
    assert Qwen2Config.from_dict({**QWEN2_RAW, "rope_scaling": {"type": "linear", "factor": 2.0}}).rope_scaling_factor == 2.0
    for kind in ("dynamic", "llama3", "yarn"):
        with pytest.raises(UnsupportedModelError, match="rope_type"):
            Qwen2Config.from_dict({**QWEN2_RAW, "rope_scaling": {"rope_type": kind, "factor": 8.0}})
    with pytest.raises(UnsupportedModelError, match="rope_theta"):
        Qwen2Config.from_dict({**QWEN2_RAW, "rope_theta": 0})
    with pytest.raises(UnsupportedModelError, match="factor"):
        Qwen2Config.from_dict({**QWEN2_RAW, "rope_scaling": {"rope_type": "linear", "factor": 0}})


def test_rejections():
    with pytest.raises(UnsupportedModelError, match="architecture"):
        parse_model_config({**QWEN2_RAW, "architectures": ["MixtralForCausalLM"]})
    with pytest.raises(UnsupportedModelError, match="architecture"):
        parse_model_config({k: v for k, v in QWEN2_RAW.items() if k != "architectures"})
    with pytest.raises(UnsupportedModelError, match="hidden_act"):
        Qwen2Config.from_dict({**QWEN2_RAW, "hidden_act": "relu2"})
    with pytest.raises(UnsupportedModelError, match="GQA"):
        Qwen2Config.from_dict({**QWEN2_RAW, "num_key_value_heads": 3})
    with pytest.raises(UnsupportedModelError, match="hidden_size"):
        Qwen2Config.from_dict({k: v for k, v in QWEN2_RAW.items() if k != "hidden_size"})
    with pytest.raises(UnsupportedModelError, match="must be an int"):
        Qwen2Config.from_dict({**QWEN2_RAW, "vocab_size": "512"})
    with pytest.raises(UnsupportedModelError, match="must be an int"):
        Qwen2Config.from_dict({**QWEN2_RAW, "num_hidden_layers": True})
    with pytest.raises(UnsupportedModelError, match="must be positive"):
        Qwen2Config.from_dict({**QWEN2_RAW, "num_hidden_layers": 0})
    with pytest.raises(UnsupportedModelError, match="head_dim must be even"):
        Qwen2Config.from_dict({**QWEN2_RAW, "head_dim": 7})
    with pytest.raises(UnsupportedModelError, match="eos_token_id"):
        Qwen2Config.from_dict({**QWEN2_RAW, "eos_token_id": "x"})


def test_dtype_and_eos_spellings():
    assert Qwen2Config.from_dict(QWEN2_RAW).torch_dtype is torch.bfloat16
    renamed = {k: v for k, v in QWEN2_RAW.items() if k != "torch_dtype"}
    assert Qwen2Config.from_dict({**renamed, "dtype": "float16"}).torch_dtype is torch.float16
    assert Qwen2Config.from_dict(renamed).torch_dtype is None
    with pytest.raises(UnsupportedModelError, match="dtype"):
        Qwen2Config.from_dict({**renamed, "dtype": "int4"})
    assert Qwen2Config.from_dict(QWEN2_RAW).eos_token_ids == (151645,)
    assert Qwen2Config.from_dict({**QWEN2_RAW, "eos_token_id": [1, 2]}).eos_token_ids == (1, 2)


def test_sliding_window_is_described_not_rejected():
    config = Qwen2Config.from_dict({**QWEN2_RAW, "use_sliding_window": True, "sliding_window": 4096, "max_window_layers": 1})
    assert [config.layer_window(layer) for layer in range(2)] == [None, 4096]
    off = Qwen2Config.from_dict({**QWEN2_RAW, "use_sliding_window": False, "sliding_window": 4096})
    assert off.layer_window(1) is None
    every = Qwen2Config.from_dict({**QWEN2_RAW, "use_sliding_window": True, "sliding_window": 8})
    assert [every.layer_window(layer) for layer in range(2)] == [8, 8]
    with pytest.raises(UnsupportedModelError, match="sliding_window"):
        Qwen2Config.from_dict({**QWEN2_RAW, "use_sliding_window": True, "sliding_window": "wide"})
    windowed = {**QWEN2_RAW, "use_sliding_window": True, "sliding_window": 8}
    assert Qwen2Config.from_dict({**windowed, "max_window_layers": None}).max_window_layers == 0
    with pytest.raises(UnsupportedModelError, match="max_window_layers.*non-negative"):
        Qwen2Config.from_dict({**windowed, "max_window_layers": -1})
    with pytest.raises(UnsupportedModelError, match="max_window_layers.*must be an int"):
        Qwen2Config.from_dict({**windowed, "max_window_layers": "2"})


def test_kv_bytes_and_round_trip(tmp_path):
    config = Qwen2Config.from_dict(QWEN2_RAW)
    assert config.kv_bytes_per_token(torch.float16) == 2 * 2 * 2 * 8 * 2
    shape7b = Qwen2Config.from_dict({**QWEN2_RAW, "hidden_size": 3584, "num_hidden_layers": 28, "num_attention_heads": 28,
                                     "num_key_value_heads": 4, "intermediate_size": 18944, "vocab_size": 152064})
    assert shape7b.kv_bytes_per_token(torch.bfloat16) == 57344
    again = Qwen2Config.from_dict(config.to_hf_dict())
    assert again == Qwen2Config.from_dict(QWEN2_RAW)
    json.dumps(config.to_dict())
    for name, (raw, _, _) in tiny.TINY.items():
        parsed = Qwen2Config.from_dict(raw)
        assert Qwen2Config.from_dict(parsed.to_hf_dict()) == parsed, name
    (tmp_path / "config.json").write_text(json.dumps(QWEN2_RAW))
    assert read_config_json(tmp_path)["vocab_size"] == 512
    from_folder = Qwen2Config.from_hf(tmp_path)
    assert from_folder.name_or_path == str(tmp_path)
    assert from_folder.to_hf_dict() == Qwen2Config.from_dict(QWEN2_RAW).to_hf_dict()
    with pytest.raises(UnsupportedModelError, match="no config.json"):
        read_config_json(tmp_path / "nowhere")
    (tmp_path / "config.json").write_text("[1, 2]")
    with pytest.raises(UnsupportedModelError, match="JSON object"):
        read_config_json(tmp_path)


def test_registry_maps_the_name_to_config_and_plan():
    arch = architecture_of(QWEN2_RAW)
    assert arch.name == "Qwen2ForCausalLM" and "Qwen2ForCausalLM" in ARCHITECTURES
    config = arch.parse_config(QWEN2_RAW)
    plan = arch.build_plan(config)
    assert len(plan.layers) == 2 and [c.layer for c in plan.schedule] == [0, 1]
    assert plan.layers[1].prefix == "model.layers.1"
    assert plan.embedding.kind == "token_table" and plan.head.kind == "norm_linear" and plan.head.params["tied_to"] is None
    mixer = plan.layers[0].block.params["mixer"]
    assert mixer.kind == "gqa_attention" and mixer.params["num_kv_heads"] == 2 and mixer.params["qkv_bias"] is True
    assert mixer.params["position"].kind == "rope" and mixer.params["position"].params["theta"] == 1000000.0


def test_engine_and_sampling_options():
    assert SchedulerConfig().max_num_seqs == 64 and SchedulerConfig().max_num_batched_tokens == 2048
    assert SchedulerConfig().block_size == 16 and SchedulerConfig().enable_chunked_prefill is True
    with pytest.raises(ValueError, match="power of two"):
        SchedulerConfig(block_size=12)
    with pytest.raises(ValueError, match="at least one block"):
        SchedulerConfig(block_size=16, max_num_batched_tokens=8)
    # What the reference has and this engine does not is accepted switched off, refused switched on.
    assert SchedulerConfig(enable_prefix_caching=False, policy="fcfs").enable_prefix_caching is False
    with pytest.raises(ValueError, match="no prefix cache"):
        SchedulerConfig(enable_prefix_caching=True)
    with pytest.raises(ValueError, match="fcfs"):
        SchedulerConfig(policy="priority")
    from turboserve_amd.engine.outputs import RequestOutput

    assert RequestOutput(request_id="r").cached_prompt_tokens == 0
    with pytest.raises(ValueError, match="not built"):
        EngineConfig(model="m", speculative={"model": "draft"})
    env = {"TURBOSERVE_MODEL": "/models/q", "TURBOSERVE_DTYPE": "float32", "TURBOSERVE_MAX_NUM_SEQS": "12",
           "TURBOSERVE_BLOCK_SIZE": "32", "TURBOSERVE_ENABLE_CHUNKED_PREFILL": "false", "TURBOSERVE_NUM_BLOCKS": ""}
    from_env = EngineConfig.from_env(env, seed=7)
    assert (from_env.model, from_env.dtype, from_env.seed) == ("/models/q", "float32", 7)
    assert (from_env.scheduler.max_num_seqs, from_env.block_size, from_env.num_blocks) == (12, 32, None)
    assert from_env.scheduler.enable_chunked_prefill is False and from_env.scheduler.max_num_batched_tokens == 2048
    with pytest.raises(ValueError, match="TURBOSERVE_MODEL"):
        EngineConfig.from_env({})
    config = EngineConfig(model="m")
    assert config.resolved_dtype() == "bfloat16" and config.resolved_device() == "cuda:0"
    assert config.gpu_memory_utilization == 0.9 and config.block_size == 16 and config.num_blocks is None
    with pytest.raises(ValueError, match="dtype"):
        EngineConfig(model="m", dtype="float16")
    with pytest.raises(ValueError, match="GPU only"):
        EngineConfig(model="m", device="cpu")
    params = SamplingParams()
    assert (params.max_tokens, params.temperature, params.top_p, params.top_k) == (128, 1.0, 1.0, 0)
    assert SamplingParams(temperature=0).is_greedy and not params.is_greedy
    for bad in (dict(max_tokens=0), dict(temperature=-1.0), dict(top_p=0.0), dict(top_p=1.5), dict(top_k=-1),
                dict(repetition_penalty=0.0)):
        with pytest.raises(ValueError):
            SamplingParams(**bad)
