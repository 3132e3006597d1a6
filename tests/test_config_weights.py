"""Configuration, registry, safetensors reading, weight errors and the random-weights mode."""
import json
import os

import pytest
import torch

import tiny_configs
from macllm_infer_amd.config import (ConfigError, FalconH1Config, config_from_dict, load_config,
                                     registered_architectures)
from macllm_infer_amd.engine.model import DecoderModel
from macllm_infer_amd.weights import WeightError, WeightSource, bind, write_safetensors
from macllm_infer_amd.weights.random_init import random_tensors


def test_config_reads_its_own_keys_and_defaults():
    config = FalconH1Config.from_dict(tiny_configs.TINY_B)
    assert (config.hidden_size, config.num_hidden_layers, config.head_dim) == (96, 3, 32)
    assert config.num_attention_heads * config.head_dim != config.hidden_size      # heads*dim need not be the width
    assert config.ssm_multipliers == (0.8, 1.4, 0.6, 1.5, 1.1) and config.mlp_multipliers == (1.25, 0.75)
    minimal = FalconH1Config.from_dict(dict(
        model_type="falcon_h1", hidden_size=32, num_hidden_layers=1, num_attention_heads=4,
        intermediate_size=48, vocab_size=50, max_position_embeddings=64, mamba_n_heads=2, mamba_d_ssm=16,
        mamba_d_state=8))
    assert minimal.head_dim == 8 and minimal.num_key_value_heads == 4 and minimal.mamba_d_head == 8
    assert minimal.mamba_d_conv == 4 and minimal.mamba_n_groups == 1 and minimal.rope_theta == 1e11
    assert minimal.rms_norm_eps == 1e-5 and minimal.mamba_conv_bias and not minimal.tie_word_embeddings
    spec = minimal.to_model_spec()
    assert [slot.name for slot in spec.layers[0].mixers] == ["self_attn", "mamba"]
    assert spec.layers[0].mixers[0].spec.scale == pytest.approx(8 ** -0.5)
    assert [entry.layer for entry in spec.schedule] == [0]


def test_state_and_cache_sizes_match_the_reference_gate():
    """Sizes asserted by the reference for Falcon-H1-Tiny-90M (tests/falcon_h1_gguf_reference.rs:50-114):
    kv bytes/token 12288 at 16-bit, fixed state 4 976 640 B with a float32 conv tail."""
    config = FalconH1Config.from_dict(dict(
        model_type="falcon_h1", hidden_size=512, num_hidden_layers=24, num_attention_heads=8,
        num_key_value_heads=2, head_dim=64, intermediate_size=1024, vocab_size=32768,
        max_position_embeddings=2048, mamba_n_heads=24, mamba_d_head=32, mamba_d_state=64, mamba_n_groups=1,
        mamba_d_conv=4))
    assert config.kv_bytes_per_token(2) == 12288
    assert config.fixed_state_bytes(4) == 4976640


@pytest.mark.parametrize("change, word", [
    ({"hidden_size": None}, "hidden_size"),
    ({"num_key_value_heads": 4}, "num_key_value_heads"),
    ({"mamba_n_groups": 4}, "mamba_n_groups"),
    ({"mamba_d_ssm": 100}, "mamba_d_ssm"),
    ({"ssm_multipliers": [1.0, 2.0]}, "ssm_multipliers"),
    ({"rms_norm_eps": 0.0}, "eps"),
    ({"head_dim": 31}, "head_dim"),
    ({"rope_scaling": {"type": "linear", "factor": 2}}, "rope_scaling"),
    ({"sliding_window": 128}, "sliding_window"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"mamba_norm_before_gate": True, "mamba_rms_norm": True}, "mamba_norm_before_gate"),
    ({"time_step_limit": [0.001, 0.1]}, "time_step_limit"),
    ({"time_step_limit": [0.0, 100.0]}, "time_step_limit"),
    ({"time_step_limit": "none"}, "time_step_limit"),
    ({"rope_parameters": {"rope_type": "yarn", "rope_theta": 1e6, "factor": 4.0}}, "rope_type"),
    ({"rope_parameters": {"rope_theta": 1e6}, "rope_theta": 1e4}, "disagree"),
    ({"rope_parameters": [1e6]}, "rope_parameters"),
    ({"vocab_size": "many"}, "vocab_size"),
    ({"max_position_embeddings": 1 << 21}, "max_position_embeddings"),
])
def test_config_errors_name_the_field(change, word):
    raw = dict(tiny_configs.TINY_B)
    raw.update(change)
    if change.get("hidden_size", 0) is None:
        del raw["hidden_size"]
    with pytest.raises(ConfigError, match=word):
        FalconH1Config.from_dict(raw)


def test_the_model_spec_refuses_a_cap_on_the_logits_that_is_no_positive_number():
    from dataclasses import replace
    from macllm_infer_amd.config import ConfigError
    spec = tiny_configs.config("A").to_model_spec()
    assert spec.logit_softcap is None
    replace(spec, logit_softcap=30.0).validate()
    for cap in (0.0, -1.0, float("inf"), float("nan")):
        with pytest.raises(ConfigError, match="cap on the logits"):
            replace(spec, logit_softcap=cap).validate()


def test_registry_maps_names_and_lists_them_for_an_unknown_one(tmp_path):
    assert "FalconH1ForCausalLM" in registered_architectures() and "falcon_h1" in registered_architectures()
    assert isinstance(config_from_dict(tiny_configs.TINY_A), FalconH1Config)
    only_type = {k: v for k, v in tiny_configs.TINY_A.items() if k != "architectures"}
    assert isinstance(config_from_dict(only_type), FalconH1Config)
    with pytest.raises(ConfigError, match="FalconH1ForCausalLM"):
        config_from_dict({"architectures": ["SomethingElse"], "hidden_size": 8})
    with pytest.raises(ConfigError, match="names no architecture"):
        config_from_dict({"hidden_size": 8})
    with pytest.raises(ConfigError, match="does not exist"):
        load_config(str(tmp_path))


def test_config_as_the_family_tooling_writes_it():
    """What checkpoints of the family carry in config.json beyond this engine's own keys: the rope base inside
    a ``rope_parameters`` table, ``mamba_norm_before_gate`` (which says nothing when there is no gated norm),
    an unclamped ``time_step_limit``, and keys that do not change the computation.  The result is the same
    typed configuration, and so the same model, as the engine's own spelling gives."""
    own = dict(tiny_configs.TINY_A, rope_theta=5e5)
    theirs = {key: value for key, value in own.items() if key != "rope_theta"}
    theirs.update(rope_parameters={"rope_theta": 5e5, "rope_type": "default"}, mamba_norm_before_gate=True,
                  time_step_limit=[0.0, float("inf")], time_step_min=0.001, time_step_max=0.1, time_step_floor=1e-4,
                  mamba_expand=2, mamba_use_mlp=True, projectors_bias=False, rope_scaling=None, sliding_window=None,
                  num_logits_to_keep=1, bos_token_id=1, pad_token_id=0, use_cache=True, initializer_range=0.02,
                  attention_dropout=0.0, transformers_version="5.0.0", dtype="bfloat16")
    config = FalconH1Config.from_dict(json.loads(json.dumps(theirs)))         # through text, Infinity included
    assert config == FalconH1Config.from_dict(own) and config.rope_theta == 5e5
    assert config.to_model_spec() == FalconH1Config.from_dict(own).to_model_spec()
    both = dict(own, rope_parameters={"rope_theta": 5e5})
    assert FalconH1Config.from_dict(both).rope_theta == 5e5
    # the flag matters only beside the gated norm
    gated = dict(tiny_configs.TINY_B, mamba_norm_before_gate=False)
    assert FalconH1Config.from_dict(gated) == FalconH1Config.from_dict(tiny_configs.TINY_B)
    # and the engine's own spelling round-trips through its own writer
    assert FalconH1Config.from_dict(config.to_dict()) == config


def test_unknown_keys_are_ignored():
    raw = dict(tiny_configs.TINY_A, some_future_key=3, torch_dtype="bfloat16")
    assert FalconH1Config.from_dict(raw) == FalconH1Config.from_dict(tiny_configs.TINY_A)


def test_random_model_folder_round_trips_and_keeps_dtypes(tmp_path):
    folder = tiny_configs.make_model_dir("B", tmp_path / "b", torch.bfloat16)
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    config = load_config(folder)
    assert config == tiny_configs.config("B")
    source = WeightSource.from_dir(folder)
    bound = bind(source, DecoderModel.expected_tensors(config.to_model_spec()))
    assert bound["model.layers.0.mamba.in_proj.weight"].dtype == torch.bfloat16
    assert bound["model.layers.0.mamba.A_log"].dtype == torch.float32          # stored in 32-bit, stays so
    assert bound["model.layers.2.mamba.norm.weight"].shape == (2, 48)
    # the library reads the same bytes
    from safetensors.torch import load_file
    theirs = load_file(os.path.join(folder, "model.safetensors"))
    assert set(theirs) == set(bound)
    for name, tensor in theirs.items():
        assert torch.equal(tensor.reshape(bound[name].shape), bound[name]) and tensor.dtype == bound[name].dtype
    # same seed, same bits; another seed, other bits
    again = random_tensors(config, 1, torch.bfloat16, "unit")
    assert all(torch.equal(again[name], bound[name]) for name in bound)
    other = random_tensors(config, 2, torch.bfloat16, "unit")
    assert not torch.equal(other["lm_head.weight"], bound["lm_head.weight"])


def test_baseline_preset_distributions():
    tensors = random_tensors(tiny_configs.config("B"), 3, torch.float32, "baseline")
    assert abs(tensors["lm_head.weight"].std().item() - 0.02) < 0.002
    assert abs(tensors["model.norm.weight"].mean().item() - 1.0) < 0.05
    a = torch.exp(tensors["model.layers.0.mamba.A_log"])
    assert (a >= 1).all() and (a <= 16).all()
    step = torch.nn.functional.softplus(tensors["model.layers.1.mamba.dt_bias"])
    assert (step >= 1e-3 * 0.999).all() and (step <= 0.1 * 1.001).all()


def test_weight_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    config = tiny_configs.config("A")
    expectations = DecoderModel.expected_tensors(config.to_model_spec())
    tensors = random_tensors(config, 0, torch.float32)
    del tensors["model.layers.1.mamba.D"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.mlp.extra.weight"] = torch.zeros(2)
    tensors["lm_head.weight"] = torch.zeros(256, 64)                       # tied model: not expected
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64)
    tensors["model.layers.0.mamba.dt_bias"] = torch.zeros(8, dtype=torch.int32)
    path = tmp_path / "model.safetensors"
    write_safetensors(str(path), tensors)
    with pytest.raises(WeightError) as caught:
        bind(WeightSource.from_dir(str(tmp_path)), expectations)
    error = caught.value
    assert error.missing == ["model.layers.1.mamba.D", "model.norm.weight"]
    assert error.unexpected == ["lm_head.weight", "model.layers.0.mlp.extra.weight"]
    assert [(name, got) for name, _, got in error.wrong_shape] == [("model.layers.0.self_attn.k_proj.weight", (16, 64))]
    assert error.wrong_dtype[0][0] == "model.layers.0.mamba.dt_bias"
    text = str(error)
    for word in ("model.layers.1.mamba.D", "lm_head.weight", "expected [32, 64], got [16, 64]"):
        assert word in text


def test_a_tied_model_saved_with_its_output_head_binds_if_the_head_is_the_embedding():
    config = tiny_configs.config("A")
    spec = config.to_model_spec()
    assert spec.tied_embeddings
    tensors = random_tensors(config, 0, torch.float32)
    expectations, copies = DecoderModel.expected_tensors(spec), DecoderModel.tensor_copies(spec)
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    bound = bind(WeightSource.from_tensors(tensors), expectations, copies)
    assert "lm_head.weight" not in bound and len(bound) == len(tensors) - 1
    tensors["lm_head.weight"][3, 5] += 1.0
    with pytest.raises(WeightError, match="differs") as caught:
        bind(WeightSource.from_tensors(tensors), expectations, copies)
    assert len(caught.value.unexpected) == 1 and not caught.value.missing
    tensors["lm_head.weight"] = torch.zeros(7, 64)
    with pytest.raises(WeightError, match="differs"):
        bind(WeightSource.from_tensors(tensors), expectations, copies)
    # an untied model binds its head and allows no copy
    untied = tiny_configs.config("B").to_model_spec()
    assert DecoderModel.tensor_copies(untied) == {}


def test_alternative_shapes_and_widening(tmp_path):
    config = tiny_configs.config("A")
    tensors = random_tensors(config, 0, torch.float32)
    tensors["model.layers.0.mamba.conv1d.weight"] = tensors["model.layers.0.mamba.conv1d.weight"].reshape(96, 1, 4)
    tensors["model.layers.0.mamba.A_log"] = tensors["model.layers.0.mamba.A_log"].reshape(8, 1).double()
    tensors["model.layers.0.mamba.D"] = tensors["model.layers.0.mamba.D"].half()
    from macllm_infer_amd.weights import Float16Narrowed
    with pytest.warns(Float16Narrowed, match="1 tensors stored in float16.*model.layers.0.mamba.D"):   # not silently
        bound = bind(WeightSource.from_tensors(tensors), DecoderModel.expected_tensors(config.to_model_spec()))
    assert bound["model.layers.0.mamba.conv1d.weight"].shape == (96, 4)
    assert bound["model.layers.0.mamba.A_log"].shape == (8,) and bound["model.layers.0.mamba.A_log"].dtype == torch.float32
    assert bound["model.layers.0.mamba.D"].dtype == torch.bfloat16


def test_sharded_checkpoint(tmp_path):
    config = tiny_configs.config("A")
    tensors = random_tensors(config, 0, torch.float32)
    names = sorted(tensors)
    half = len(names) // 2
    write_safetensors(str(tmp_path / "model-00001-of-00002.safetensors"), {n: tensors[n] for n in names[:half]})
    write_safetensors(str(tmp_path / "model-00002-of-00002.safetensors"), {n: tensors[n] for n in names[half:]})
    weight_map = {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
                  for i, n in enumerate(names)}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    bound = bind(WeightSource.from_dir(str(tmp_path)), DecoderModel.expected_tensors(config.to_model_spec()))
    assert all(torch.equal(bound[n], tensors[n]) for n in names)


def _respell(tensors, pairs, strip=""):
    out = {}
    for name, tensor in tensors.items():
        for ours, other in pairs:
            name = name.replace(ours, other)
        if strip and name.startswith(strip):
            name = name[len(strip):]
        out[name] = tensor
    return out


CHECKPOINT_SPELLING = ((".attn_norm.", ".input_layernorm."), (".ffn_norm.", ".pre_ff_layernorm."),
                       (".mlp.", ".feed_forward."), ("model.norm.", "model.final_layernorm."))


def test_the_other_spelling_of_the_tensor_names_binds_to_the_same_tensors():
    config = tiny_configs.config("B")
    spec = config.to_model_spec()
    tensors = random_tensors(config, 3, torch.float32, "unit")
    plain = bind(WeightSource.from_tensors(tensors), DecoderModel.expected_tensors(spec))
    for strip in ("", "model."):                   # with the namespace, and saved from the inner model
        source = WeightSource.from_tensors(_respell(tensors, CHECKPOINT_SPELLING, strip))
        assert "model.layers.0.input_layernorm.weight"[len(strip):] in source.names()
        source.apply_aliases(spec.tensor_aliases, root_prefix=spec.root_namespace)
        bound = bind(source, DecoderModel.expected_tensors(spec))
        assert bound.keys() == plain.keys()
        assert all(torch.equal(bound[name], plain[name]) for name in plain)


def test_a_tensor_under_both_spellings_and_a_stranger_are_reported_by_their_stored_names():
    config = tiny_configs.config("A")
    spec = config.to_model_spec()
    tensors = _respell(random_tensors(config, 3, torch.float32, "unit"), CHECKPOINT_SPELLING)
    tensors["model.layers.1.ffn_norm.weight"] = tensors["model.layers.1.pre_ff_layernorm.weight"]
    tensors["model.layers.0.feed_forward.router.weight"] = torch.zeros(2, 2)
    source = WeightSource.from_tensors(tensors)
    source.apply_aliases(spec.tensor_aliases, root_prefix=spec.root_namespace)
    with pytest.raises(WeightError) as caught:
        bind(source, DecoderModel.expected_tensors(spec))
    assert not caught.value.missing
    assert "model.layers.0.feed_forward.router.weight" in caught.value.unexpected
    assert any("pre_ff_layernorm" in name and "ffn_norm" in name for name in caught.value.unexpected)


def test_command_line_writes_and_inspects_a_random_model(tmp_path, capsys):
    """``random-weights`` writes a model folder from a config.json and a seed (the same tensors as the
    Python call with that seed); ``inspect`` prints the geometry the cache manager sizes itself by."""
    from macllm_infer_amd import cli
    (tmp_path / "config.json").write_text(json.dumps(tiny_configs.TINY_B))
    folder = tmp_path / "model"
    assert cli.main(["random-weights", "--config", str(tmp_path / "config.json"), "--seed", "3", "--out", str(folder),
                     "--dtype", "f32"]) == 0
    config = load_config(str(folder))
    assert config == tiny_configs.config("B")
    bound = bind(WeightSource.from_dir(str(folder)), DecoderModel.expected_tensors(config.to_model_spec()))
    assert all(torch.equal(bound[name], tensor) for name, tensor in random_tensors(config, 3, torch.float32).items())
    capsys.readouterr()
    assert cli.main(["inspect", "-m", str(folder)]) == 0
    report = json.loads(capsys.readouterr().out)
    assert report["layers"] == 3 and report["kv_bytes_per_token_bf16"] == config.kv_bytes_per_token(2)
    assert report["fixed_state_bytes_per_request_f32"] == config.fixed_state_bytes(4)
