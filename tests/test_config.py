"""Configuration: engine sections and overrides, the typed model config, the registries."""

import dataclasses

import pytest

from clockwork_amd.config.engine import CacheConfig, EngineConfig, SchedulerConfig
from clockwork_amd.config.spec import KVPagesSpec, LayerSpec, ModelSpec, RunEntry
from clockwork_amd.models.qwen2 import Qwen2Config, build_spec, weight_plan
from clockwork_amd.parts.specs import AttentionSpec, RMSNormSpec, RopeNeoxSpec, SwiGLUSpec
from clockwork_amd.registry import resolve_architecture
from tests.configs import TINY_A, TINY_B, TINY_C


def test_engine_defaults_match_the_reference():
    cfg = EngineConfig.defaults("some/dir")
    # clockwork/config.py:17-47
    assert (cfg.model.dtype, cfg.model.max_model_len, cfg.model.seed) == ("float32", 4096, 0)
    cache = dataclasses.asdict(cfg.cache)
    assert cache.pop("memory_fraction") == 0.8  # this engine's own: sizes the pools when num_blocks is 0
    assert cache == dict(block_size=16, num_blocks=512, enable_prefix_cache=True, watermark=0.01)
    assert (cfg.scheduler.max_num_seqs, cfg.scheduler.max_num_batched_tokens) == (64, 2048)
    assert cfg.scheduler.enable_chunked_prefill and cfg.scheduler.max_prefill_chunk == 0


def test_overrides_are_routed_by_field_name():
    cfg = EngineConfig.defaults("m", num_blocks=7, max_num_seqs=3, dtype="bfloat16", max_model_len=99)
    assert cfg.cache.num_blocks == 7 and cfg.scheduler.max_num_seqs == 3 and cfg.model.dtype == "bfloat16"
    # max_model_len lives on two sections and is set on both (clockwork/config.py:76-86)
    assert cfg.model.max_model_len == 99 and cfg.scheduler.max_model_len == 99
    with pytest.raises(ValueError, match="unknown config override 'nonsense'"):
        EngineConfig.defaults("m", nonsense=1)


def test_key_value_overrides_are_read_as_yaml():
    cfg = EngineConfig.defaults("m")
    cfg.apply_overrides(["num_blocks=1024", "enable_prefix_cache=false", "watermark=0.25", "dtype=bfloat16"])
    assert cfg.cache.num_blocks == 1024 and cfg.cache.enable_prefix_cache is False
    assert cfg.cache.watermark == 0.25 and cfg.model.dtype == "bfloat16"
    with pytest.raises(ValueError, match="not KEY=VALUE"):
        cfg.apply_overrides(["oops"])


def test_yaml_sections(tmp_path):
    path = tmp_path / "engine.yaml"
    path.write_text("model:\n  model: /m\n  dtype: bfloat16\ncache:\n  block_size: 8\nscheduler:\n  max_num_seqs: 5\n")
    cfg = EngineConfig.from_yaml(path)
    assert cfg.model.model == "/m" and cfg.cache.block_size == 8 and cfg.scheduler.max_num_seqs == 5
    assert cfg.cache.num_blocks == CacheConfig().num_blocks
    assert cfg.scheduler.max_num_batched_tokens == SchedulerConfig().max_num_batched_tokens
    bad = tmp_path / "bad.yaml"
    bad.write_text("cache:\n  block_size: 8\n")
    with pytest.raises(ValueError, match="top-level 'model' section"):
        EngineConfig.from_yaml(bad)


def test_the_example_configuration_loads():
    from pathlib import Path

    cfg = EngineConfig.from_yaml(Path(__file__).resolve().parent.parent / "configs" / "qwen2.5-1.5b-instruct.yaml")
    assert cfg.model.dtype == "bfloat16" and cfg.model.tune_products is True
    assert cfg.cache.num_blocks == 0 and cfg.cache.memory_fraction == 0.8 and cfg.cache.block_size == 16
    assert cfg.scheduler.max_num_batched_tokens == 2048 and cfg.scheduler.max_model_len == cfg.model.max_model_len


def test_dtype_whitelist():
    import torch

    assert EngineConfig.defaults("m", dtype="bfloat16").model.torch_dtype() == torch.bfloat16
    assert EngineConfig.defaults("m").model.torch_dtype() == torch.float32
    with pytest.raises(ValueError, match="unknown dtype"):
        EngineConfig.defaults("m", dtype="int8").model.torch_dtype()
    with pytest.raises(ValueError, match="float16"):
        EngineConfig.defaults("m", dtype="float16").model.torch_dtype()


def test_random_weights_are_a_mode_of_the_configuration_and_of_the_command_line(tmp_path):
    """clockwork/engine/loader.py:82-103 builds a model from a seed without a checkpoint; here that
    is ``weights: random`` + ``weight_seed`` in the model section, ``--random-weights SEED`` on
    the command line, and ``model`` may then name a bare config.json."""
    import json

    from clockwork_amd import cli
    from clockwork_amd.weights.loader import read_config_json

    cfg = EngineConfig.defaults("m")
    assert (cfg.model.weights, cfg.model.weight_seed) == ("checkpoint", 0)
    cfg.apply_overrides(["weights=random", "weight_seed=7"])
    assert (cfg.model.weights, cfg.model.weight_seed) == ("random", 7)
    with pytest.raises(ValueError, match="weights 'noise'"):
        cfg.set("weights", "noise")
    assert cfg.model.weights == "random"  # a refused value changes nothing
    with pytest.raises(ValueError, match="weights 'noise'"):
        EngineConfig.defaults("m", weights="noise")
    path = tmp_path / "engine.yaml"
    path.write_text("model:\n  model: /m/config.json\n  weights: random_device\n  weight_seed: 3\n")
    from_yaml = EngineConfig.from_yaml(path)
    assert (from_yaml.model.weights, from_yaml.model.weight_seed) == ("random_device", 3)

    config_json = tmp_path / "tiny.json"
    config_json.write_text(json.dumps(TINY_B))
    args, cfg, prompts = cli.parse_generate(["--model", str(config_json), "--random-weights", "2", "--prompt-ids", "5,17,3",
                                             "--max-tokens", "8"])
    assert (cfg.model.model, cfg.model.weights, cfg.model.weight_seed) == (str(config_json), "random", 2)
    assert prompts == [[5, 17, 3]] and args.max_tokens == 8
    _, cfg, _ = cli.parse_generate(["--model", "/some/dir", "--prompt-ids", "1"])
    assert cfg.model.weights == "checkpoint"
    # a file stands for itself, a folder for the config.json inside it
    assert read_config_json(config_json) == TINY_B
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    assert read_config_json(tmp_path) == TINY_A
    with pytest.raises(FileNotFoundError):
        read_config_json(tmp_path / "nothing")


# ------------------------------------------------------------------ the model's own keys
def test_qwen2_config_reads_every_size_from_the_dict():
    for d in (TINY_A, TINY_B, TINY_C):
        cfg = Qwen2Config.from_dict(d)
        for key in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                    "num_key_value_heads", "intermediate_size", "rms_norm_eps", "rope_theta"):
            assert getattr(cfg, key) == d[key]
        assert cfg.tie_word_embeddings == d.get("tie_word_embeddings", False)
    # clockwork/engine/model.py:17-18: head_dim defaults to hidden // heads, an explicit key wins
    assert Qwen2Config.from_dict(TINY_A).head_dim == 16
    assert Qwen2Config.from_dict(TINY_C).head_dim == 48
    assert Qwen2Config.from_dict(dict(TINY_A, head_dim=None)).head_dim == 16


def test_qwen2_config_refuses_what_is_not_built():
    with pytest.raises(NotImplementedError, match="hidden_act"):
        Qwen2Config.from_dict(dict(TINY_A, hidden_act="gelu"))
    with pytest.raises(NotImplementedError, match="sliding-window"):
        Qwen2Config.from_dict(dict(TINY_A, use_sliding_window=True))
    with pytest.raises(NotImplementedError, match="rope_type"):
        Qwen2Config.from_dict(dict(TINY_A, rope_parameters={"rope_type": "yarn", "rope_theta": 1e4}))
    with pytest.raises(ValueError, match="not a multiple"):
        Qwen2Config.from_dict(dict(TINY_A, num_key_value_heads=3))
    missing = dict(TINY_A)
    del missing["rms_norm_eps"]
    with pytest.raises(ValueError, match="rms_norm_eps"):
        Qwen2Config.from_dict(missing)
    # clockwork/engine/model.py:21-29: theta inside rope_parameters
    d = dict(TINY_A, rope_parameters={"rope_type": "default", "rope_theta": 12345.0})
    assert Qwen2Config.from_dict(d).rope_theta == 12345.0
    assert Qwen2Config.from_dict(dict(TINY_A, eos_token_id=[5, 6])).eos_token_ids == (5, 6)
    assert Qwen2Config.from_dict(dict(TINY_A, eos_token_id=5)).eos_token_ids == (5,)


def test_registry_picks_by_architecture_or_model_type_and_rejects_the_rest():
    assert resolve_architecture({"architectures": ["Qwen2ForCausalLM"]}).name == "Qwen2ForCausalLM"
    assert resolve_architecture({"model_type": "qwen2"}).name == "Qwen2ForCausalLM"
    # clockwork/engine/loader.py:70-71: whatever is not the built architecture is refused; the
    # registry names what it was given and what it knows, the architecture itself keeps the
    # reference's words for a config that reaches it under a wrong model_type
    with pytest.raises(ValueError, match="no architecture is registered for model_type='llama'.*Qwen2ForCausalLM"):
        resolve_architecture({"model_type": "llama", "architectures": ["LlamaForCausalLM"]})
    with pytest.raises(ValueError, match="expected a qwen2 model, got model_type='llama'"):
        Qwen2Config.from_dict(dict(TINY_A, model_type="llama"))


def test_spec_carries_the_config_layer_by_layer():
    cfg = Qwen2Config.from_dict(TINY_B)
    spec = build_spec(cfg)
    assert len(spec.layers) == 3 and [e.layer for e in spec.run] == [0, 1, 2]
    mixer = spec.layers[0].mixer
    assert isinstance(mixer, AttentionSpec)
    assert (mixer.num_heads, mixer.num_kv_heads, mixer.head_dim) == (6, 1, 32)
    assert mixer.scale == 32 ** -0.5 and mixer.qkv_bias and not mixer.out_bias and mixer.window is None
    assert mixer.position == RopeNeoxSpec(rotary_dim=32, theta=1e6)
    assert spec.layers[0].feed_forward == SwiGLUSpec(192, 384)
    assert spec.final_norm == RMSNormSpec(192, 1e-5)
    assert not spec.tie_embeddings and build_spec(Qwen2Config.from_dict(TINY_A)).tie_embeddings


def test_weight_plan_names_and_shapes():
    cfg = Qwen2Config.from_dict(TINY_C)
    plan = {t.param: t for t in weight_plan(cfg, build_spec(cfg))}
    qkv = plan["layers.1.mixer.qkv_weight"]
    assert qkv.sources == tuple(f"model.layers.1.self_attn.{n}_proj.weight" for n in "qkv")
    assert qkv.source_shapes == ((144, 80), (144, 80), (144, 80))
    # o_proj reads num_heads * head_dim columns, not hidden_size (clockwork/engine/model.py:77)
    assert plan["layers.0.mixer.out_weight"].source_shapes == ((80, 144),)
    assert plan["layers.0.feed_forward.gate_up_weight"].source_shapes == ((100, 80), (100, 80))
    assert not plan["lm_head.weight"].optional
    cfg_a = Qwen2Config.from_dict(TINY_A)
    assert {t.param: t for t in weight_plan(cfg_a, build_spec(cfg_a))}["lm_head.weight"].optional


def test_run_list_is_checked():
    norm = RMSNormSpec(8, 1e-6)
    layer = LayerSpec("prenorm", AttentionSpec(8, 1, 1, 16, False, False, 0.25), SwiGLUSpec(8, 16), norm, norm)
    ok = ModelSpec("toy", 10, 8, [layer], [RunEntry(0), RunEntry(0), RunEntry(0, cache_from=0)], norm)
    ok.validate()
    for run in ([RunEntry(1)], [RunEntry(0, cache_from=0)], [RunEntry(0), RunEntry(0, cache_from=0), RunEntry(0, cache_from=1)]):
        with pytest.raises(ValueError):
            ModelSpec("toy", 10, 8, [layer], run, norm).validate()


def test_attention_spec_refuses_sizes_the_kernels_do_not_take():
    with pytest.raises(ValueError, match="multiples of 16"):
        AttentionSpec(64, 4, 2, 24, True, False, 1.0)
    with pytest.raises(ValueError, match="not a multiple"):
        AttentionSpec(64, 5, 2, 16, True, False, 1.0)
    assert KVPagesSpec(2, 16).group_key() != KVPagesSpec(2, 16, window=8).group_key()


def test_bench_refuses_more_than_one_gpu_with_one_line():
    """The benchmark is a one-GPU program: asked for more it says so in one line and exits with 2,
    before anything touches a GPU."""
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parent.parent
    run = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2", "--steps", "3", "--warmup", "1"],
                         capture_output=True, text=True, timeout=120)
    assert run.returncode == 2
    assert len(run.stdout.strip().splitlines()) == 1 and "one GPU" in run.stdout
