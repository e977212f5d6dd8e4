"""Weights by tensor name: one clear error for missing, unexpected and misshapen tensors;
dtype rules; tied heads; the random-weights mode."""

import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from clockwork_amd.models.qwen2 import Qwen2Config, build_spec, weight_plan
from clockwork_amd.parts.model import model_param_specs
from clockwork_amd.weights import WeightMismatchError, load_parameters, write_random_model
from clockwork_amd.weights.random_init import random_checkpoint_tensors
from tests.configs import TINY_A, TINY_B


def _plan(config):
    cfg = Qwen2Config.from_dict(config)
    spec = build_spec(cfg)
    return weight_plan(cfg, spec), model_param_specs(spec)


def _load(model_dir, config, dtype=torch.bfloat16):
    plan, specs = _plan(config)
    return load_parameters(model_dir, plan, specs, dtype, "cpu")


def test_random_model_folder_round_trip(tmp_path):
    d = write_random_model(tmp_path / "m", TINY_B, seed=1)
    assert json.loads((d / "config.json").read_text())["hidden_size"] == 192
    params = _load(d, TINY_B)
    plan, specs = _plan(TINY_B)
    assert set(params) == set(specs)
    for name, spec in specs.items():
        assert tuple(params[name].shape) == tuple(spec.shape), name
        assert params[name].dtype == torch.bfloat16
    raw = load_file(str(d / "model.safetensors"))
    # fused projections are the stored tensors stacked along the output dimension
    qkv = params["layers.2.mixer.qkv_weight"]
    stacked = torch.cat([raw[f"model.layers.2.self_attn.{n}_proj.weight"] for n in "qkv"])
    assert torch.equal(qkv, stacked)
    gate_up = params["layers.0.feed_forward.gate_up_weight"]
    assert torch.equal(gate_up[:384], raw["model.layers.0.mlp.gate_proj.weight"])
    assert torch.equal(gate_up[384:], raw["model.layers.0.mlp.up_proj.weight"])


def test_random_weights_follow_the_stated_distributions_and_the_seed():
    a = random_checkpoint_tensors(TINY_B, seed=1)
    b = random_checkpoint_tensors(TINY_B, seed=1)
    c = random_checkpoint_tensors(TINY_B, seed=2)
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    w = a["model.embed_tokens.weight"].float()
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.001
    bias = a["model.layers.0.self_attn.q_proj.bias"].float()
    assert 0.01 < float(bias.std()) < 0.03
    norm = a["model.layers.1.input_layernorm.weight"].float()
    assert float(norm.min()) >= 0.89 and float(norm.max()) <= 1.11 and float(norm.std()) > 0.02
    assert "lm_head.weight" in a  # untied
    assert "lm_head.weight" not in random_checkpoint_tensors(TINY_A, seed=0)  # tied: left out


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = write_random_model(tmp_path / "m", TINY_A, seed=0)
    tensors = load_file(str(d / "model.safetensors"))
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["model.layers.0.self_attn.k_proj.bias"] = torch.zeros(33, dtype=torch.bfloat16)
    save_file(tensors, str(d / "model.safetensors"))
    with pytest.raises(WeightMismatchError) as err:
        _load(d, TINY_A)
    e = err.value
    assert sorted(e.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert len(e.wrong_shape) == 1 and "k_proj.bias" in e.wrong_shape[0] and "(33,)" in e.wrong_shape[0]
    text = str(e)
    assert "state dict mismatch" in text and "missing=" in text and "unexpected=" in text and "wrong_shape=" in text


def test_tied_head_may_be_absent_untied_may_not(tmp_path):
    d = write_random_model(tmp_path / "tied", TINY_A, seed=0)
    params = _load(d, TINY_A)
    assert "lm_head.weight" not in params  # the model aliases the embedding (clockwork/engine/loader.py:60-62)
    tensors = load_file(str(d / "model.safetensors"))
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    save_file(tensors, str(d / "model.safetensors"))
    assert "lm_head.weight" in _load(d, TINY_A)  # present in a tied checkpoint: taken, not "unexpected"
    d2 = write_random_model(tmp_path / "untied", TINY_B, seed=1)
    tensors = load_file(str(d2 / "model.safetensors"))
    del tensors["lm_head.weight"]
    save_file(tensors, str(d2 / "model.safetensors"))
    with pytest.raises(WeightMismatchError) as err:
        _load(d2, TINY_B)
    assert err.value.missing == ["lm_head.weight"]


def test_a_tied_checkpoint_that_carries_its_head_keeps_one_table(tmp_path):
    """clockwork/engine/model.py:217-218: a tied head is the embedding's parameter, so a head
    tensor in the file can only be that table again. It is checked and let go (one matrix in
    memory, one in the step's byte count); a head that differs from the table is an error."""
    from clockwork_amd.models.qwen2 import Qwen2Config, build_spec
    from clockwork_amd.parts.model import DecoderModel

    d = write_random_model(tmp_path / "tied", TINY_A, seed=0)
    tensors = load_file(str(d / "model.safetensors"))
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    save_file(tensors, str(d / "model.safetensors"))
    spec = build_spec(Qwen2Config.from_dict(TINY_A))
    model = DecoderModel(spec)
    params = _load(d, TINY_A)
    assert "lm_head.weight" in params
    model.bind(params, torch.device("cpu"), torch.float32)
    assert model.head.weight is model.embedding.weight and "lm_head.weight" not in model.params
    alone = DecoderModel(spec)
    without = {k: v for k, v in params.items() if k != "lm_head.weight"}
    alone.bind(without, torch.device("cpu"), torch.float32)
    assert model.weight_bytes_per_step() == alone.weight_bytes_per_step()
    params["lm_head.weight"] = params["lm_head.weight"].clone()
    params["lm_head.weight"][3, 5] += 1.0
    with pytest.raises(ValueError, match="differs from the embedding table"):
        DecoderModel(spec).bind(params, torch.device("cpu"), torch.float32)
    # an untied model keeps a head of its own and counts it
    from tests.configs import TINY_B as B

    spec_b = build_spec(Qwen2Config.from_dict(B))
    model_b = DecoderModel(spec_b)
    model_b.bind(_load(write_random_model(tmp_path / "untied", B, seed=1), B), torch.device("cpu"), torch.float32)
    assert model_b.head.weight is not model_b.embedding.weight
    assert model_b.weight_bytes_per_step() == sum(
        t.numel() * t.element_size() for k, t in model_b.params.items() if k != "embed.weight")


def test_dtype_rules(tmp_path):
    """Matrices take the engine's dtype; small vectors that the file holds in 32-bit stay 32-bit."""
    d = write_random_model(tmp_path / "m", TINY_A, seed=0)
    tensors = load_file(str(d / "model.safetensors"))
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float()
    for n in "qkv":
        key = f"model.layers.0.self_attn.{n}_proj.bias"
        tensors[key] = tensors[key].float()
    tensors["model.layers.0.mlp.down_proj.weight"] = tensors["model.layers.0.mlp.down_proj.weight"].float()
    save_file(tensors, str(d / "model.safetensors"))
    bf = _load(d, TINY_A, torch.bfloat16)
    assert bf["final_norm.weight"].dtype == torch.float32
    assert bf["layers.0.mixer.qkv_bias"].dtype == torch.float32
    assert bf["layers.1.mixer.qkv_bias"].dtype == torch.bfloat16
    assert bf["layers.0.feed_forward.down_weight"].dtype == torch.bfloat16
    f32 = _load(d, TINY_A, torch.float32)
    assert all(t.dtype == torch.float32 for t in f32.values())
    # bfloat16 values survive the upcast exactly
    assert torch.equal(f32["embed.weight"], tensors["model.embed_tokens.weight"].float())


def test_several_files_are_merged_and_an_empty_folder_is_an_error(tmp_path):
    d = write_random_model(tmp_path / "m", TINY_A, seed=0)
    tensors = load_file(str(d / "model.safetensors"))
    names = sorted(tensors)
    (d / "model.safetensors").unlink()
    save_file({k: tensors[k] for k in names[:10]}, str(d / "model-00001-of-00002.safetensors"))
    save_file({k: tensors[k] for k in names[10:]}, str(d / "model-00002-of-00002.safetensors"))
    assert torch.equal(_load(d, TINY_A)["embed.weight"], tensors["model.embed_tokens.weight"])
    empty = tmp_path / "empty"
    empty.mkdir()
    with pytest.raises(FileNotFoundError, match="no .safetensors files"):
        _load(empty, TINY_A)


def test_a_checkpoint_tensor_may_be_transposed_or_split_on_its_way_in(tmp_path):
    """A parameter's sources go through the target's ``transform`` before they are stacked: a
    matrix the file holds the other way round, a slice of a tensor that holds several
    projections, or both; an architecture may register steps of its own."""
    from clockwork_amd.config.spec import ParamSpec, WeightTarget
    from clockwork_amd.weights.transforms import apply_transform, register_transform, steps_of, transformed_shape

    stored = {"down_t": torch.arange(24.0).reshape(4, 6), "qkv": torch.arange(36.0).reshape(9, 4),
              "a": torch.arange(8.0).reshape(2, 4), "b_t": torch.full((4, 3), 2.0)}
    save_file({k: v.to(torch.bfloat16) for k, v in stored.items()}, str(tmp_path / "model.safetensors"))
    specs = {"down": ParamSpec((6, 4)), "k": ParamSpec((3, 4)), "v_t": ParamSpec((4, 3)), "ab": ParamSpec((5, 4)),
             "reversed": ParamSpec((2, 4))}
    plan = [
        WeightTarget("down", ("down_t",), ((4, 6),), transform=("transpose",)),
        WeightTarget("k", ("qkv",), ((9, 4),), transform=("split_rows", 1, 3)),
        WeightTarget("v_t", ("qkv",), ((9, 4),), transform=(("split_rows", 2, 3), ("transpose",))),
        WeightTarget("reversed", ("a",), ((2, 4),), transform=("flip_rows",)),
    ]
    assert transformed_shape(("transpose",), (4, 6)) == (6, 4) and steps_of(("transpose",)) == (("transpose",),)
    assert transformed_shape((("split_rows", 2, 3), ("transpose",)), (9, 4)) == (4, 3)
    del specs["ab"]
    with pytest.raises(KeyError, match="no weight transform is registered under 'flip_rows'"):
        load_parameters(tmp_path, plan + [WeightTarget("ab", ("b_t",), ((4, 3),), optional=True)], specs, torch.float32, "cpu")
    register_transform("flip_rows", lambda t: t.flip(0))   # an architecture's own step
    # the steps apply to every source, then the sources are stacked; sources that do not stack
    # afterwards are a fault of the plan, said as such
    unstackable = WeightTarget("ab", ("a", "b_t"), ((2, 4), (4, 3)), transform=("transpose",))
    with pytest.raises(RuntimeError, match="weight plan for ab stacks sources whose rows differ"):
        load_parameters(tmp_path, plan + [unstackable], dict(specs, ab=ParamSpec((7, 2))), torch.float32, "cpu")
    params = load_parameters(tmp_path, plan + [WeightTarget("ab", ("b_t",), ((4, 3),), optional=True)],
                             dict(specs, ab=ParamSpec((4, 3))), torch.float32, "cpu")
    assert torch.equal(params["reversed"], stored["a"].flip(0)) and torch.equal(params["ab"], stored["b_t"])
    assert torch.equal(params["down"], stored["down_t"].t())
    assert torch.equal(params["k"], stored["qkv"][3:6]) and torch.equal(params["v_t"], stored["qkv"][6:9].t())
    assert params["down"].is_contiguous() and params["v_t"].is_contiguous()
    with pytest.raises(KeyError, match="no weight transform is registered under 'rotate'"):
        apply_transform(("rotate",), stored["a"])
    with pytest.raises(ValueError, match="does not divide"):
        apply_transform(("split_rows", 0, 2), stored["qkv"])
    # a shape that differs from the file's is still named, in the file's terms
    bad = [WeightTarget("down", ("down_t",), ((6, 4),), transform=("transpose",))]
    with pytest.raises(WeightMismatchError) as err:
        load_parameters(tmp_path, bad, {"down": ParamSpec((4, 6))}, torch.float32, "cpu")
    assert "down_t: checkpoint (4, 6), model (6, 4)" in str(err.value)
