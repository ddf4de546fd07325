"""Configuration, registry, safetensors reading and writing, weight errors."""
import json
import os

import pytest
import torch

from wllm_amd.architectures import GemmaConfig
from wllm_amd.config import ConfigError, read_config_json, register_architecture, resolve_architecture
from wllm_amd.parts import build_model, load_model, write_random_model_folder
from wllm_amd.weights import Checkpoint, SafetensorsFile, WeightError, write_safetensors
from helpers import TINY

RAW = dict(vocab_size=100, hidden_size=48, intermediate_size=96, num_hidden_layers=2, num_attention_heads=4)


def test_defaults_follow_the_reference():
    c = GemmaConfig.from_dict(RAW)
    assert (c.num_key_value_heads, c.head_dim, c.rms_norm_eps, c.rope_theta) == (4, 12, 1e-6, 10000.0)
    assert c.max_position_embeddings == 4096 and c.tie_word_embeddings is True and c.attention_bias is False


def test_head_dim_key_wins():
    raw = dict(RAW, hidden_size=3072, num_attention_heads=16)
    assert GemmaConfig.from_dict(raw).head_dim == 192
    assert GemmaConfig.from_dict(dict(raw, head_dim=256)).head_dim == 256


def test_rope_theta_may_live_under_rope_parameters():
    assert GemmaConfig.from_dict(dict(RAW, rope_parameters={"rope_theta": 500})).rope_theta == 500.0
    assert GemmaConfig.from_dict(dict(RAW, rope_theta=77, rope_parameters={"rope_theta": 500})).rope_theta == 77.0


@pytest.mark.parametrize("bad", [
    {"num_key_value_heads": 3}, {"head_dim": 7}, {"vocab_size": 0}, {"hidden_size": -1},
    {"num_hidden_layers": 1.5}, {"rms_norm_eps": -1.0}, {"rope_theta": 0},
])
def test_invalid_values_are_refused(bad):
    with pytest.raises(ConfigError):
        GemmaConfig.from_dict(dict(RAW, **bad))


def test_missing_keys_are_named():
    raw = dict(RAW)
    del raw["vocab_size"], raw["intermediate_size"]
    with pytest.raises(ConfigError, match="vocab_size.*intermediate_size|intermediate_size.*vocab_size"):
        GemmaConfig.from_dict(raw)


def test_config_round_trips_through_json(tmp_path):
    c = TINY["B"]["config"]
    (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
    raw = read_config_json(str(tmp_path))
    assert raw["architectures"] == ["GemmaForCausalLM"]
    assert GemmaConfig.from_dict(raw) == c


def test_registry_takes_the_first_known_name_and_names_what_it_knows():
    assert resolve_architecture(["Nope", "GemmaForCausalLM"]).name == "GemmaForCausalLM"
    with pytest.raises(ConfigError, match="GemmaForCausalLM"):
        resolve_architecture(["LlamaForCausalLM"])
    with pytest.raises(ConfigError):
        resolve_architecture(None)
    with pytest.raises(ConfigError):
        register_architecture("GemmaForCausalLM", GemmaConfig.from_dict, lambda c: None)


def test_plan_takes_every_size_from_the_configuration():
    for name in ("A", "B", "C"):
        c = TINY[name]["config"]
        plan = build_model(c.to_dict()).plan
        assert len(plan.layers) == len(plan.schedule) == c.num_hidden_layers
        m = plan.layers[0].mixer
        assert (m.num_heads, m.num_kv_heads, m.head_dim) == (c.num_attention_heads, c.num_key_value_heads, c.head_dim)
        assert abs(m.scale - c.head_dim ** -0.5) < 1e-15 and m.position.theta == c.rope_theta
        assert plan.layers[0].mixer_norm.eps == c.rms_norm_eps and plan.layers[0].mixer_norm.weight_offset == 1.0
        assert plan.embedding.scale == c.hidden_size ** 0.5
        assert (plan.head.weight is None) == c.tie_word_embeddings


def test_safetensors_round_trip_and_agreement_with_the_safetensors_package(tmp_path):
    from safetensors import safe_open
    from safetensors.torch import save_file
    tensors = {"a": torch.randn(3, 5), "b.c": torch.randn(7).to(torch.bfloat16), "i": torch.arange(6, dtype=torch.int32).view(2, 3)}
    ours = str(tmp_path / "ours.safetensors")
    write_safetensors(ours, tensors, {"k": "v"})
    with safe_open(ours, framework="pt") as f:
        for n, t in tensors.items():
            assert torch.equal(f.get_tensor(n), t)
    theirs = str(tmp_path / "theirs.safetensors")
    save_file(tensors, theirs)
    f = SafetensorsFile(theirs)
    for n, t in tensors.items():
        assert f.dtype(n) == t.dtype and f.shape(n) == tuple(t.shape) and torch.equal(f.tensor(n), t)
    f.close()


def test_random_weights_do_not_depend_on_creation_order_and_are_bfloat16_exact(model_folders):
    ck = Checkpoint(model_folders["A"])
    t = ck.tensor("model.layers.1.mlp.up_proj.weight")
    from wllm_amd.weights import random_tensor
    assert torch.equal(t, random_tensor(TINY["A"]["seed"], "model.layers.1.mlp.up_proj.weight", t.shape, TINY["A"]["std"]))
    assert ck.stored_dtype("model.norm.weight") == torch.bfloat16
    assert 0.01 < t.float().std() < 0.03 and 0.05 < ck.tensor("model.norm.weight").float().std() < 0.2
    ck.close()


def _rewrite(folder, out, change):
    ck = Checkpoint(folder)
    tensors = {n: ck.tensor(n) for n in ck.names()}
    ck.close()
    change(tensors)
    os.makedirs(out, exist_ok=True)
    write_safetensors(os.path.join(out, "model.safetensors"), tensors)
    with open(os.path.join(folder, "config.json")) as f, open(os.path.join(out, "config.json"), "w") as g:
        g.write(f.read())
    return out


def test_one_error_lists_missing_unexpected_and_wrong_shapes(model_folders, tmp_path):
    def change(t):
        del t["model.layers.0.mlp.up_proj.weight"]
        del t["model.norm.weight"]
        t["model.layers.0.extra.weight"] = torch.zeros(2)
        t["model.layers.1.self_attn.q_proj.weight"] = torch.zeros(5, 5, dtype=torch.bfloat16)
    folder = _rewrite(model_folders["A"], str(tmp_path / "broken"), change)
    model = build_model(read_config_json(folder))
    with pytest.raises(WeightError) as e:
        model.load(Checkpoint(folder), torch.float32, torch.device("cpu"))
    err = e.value
    assert sorted(err.missing) == ["model.layers.0.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.extra.weight"]
    assert [w[0] for w in err.wrong_shape] == ["model.layers.1.self_attn.q_proj.weight"]
    for name in err.missing + err.unexpected + [err.wrong_shape[0][0]]:
        assert name in str(err)


def test_tied_model_accepts_a_stored_head_only_if_it_is_the_table(model_folders, tmp_path):
    same = _rewrite(model_folders["A"], str(tmp_path / "same"),
                    lambda t: t.__setitem__("lm_head.weight", t["model.embed_tokens.weight"].clone()))
    build_model(read_config_json(same)).load(Checkpoint(same), torch.float32, torch.device("cpu"))
    other = _rewrite(model_folders["A"], str(tmp_path / "other"),
                     lambda t: t.__setitem__("lm_head.weight", t["model.embed_tokens.weight"] + 1))
    with pytest.raises(WeightError, match="lm_head.weight"):
        build_model(read_config_json(other)).load(Checkpoint(other), torch.float32, torch.device("cpu"))


def test_untied_model_needs_its_head_and_rotary_frequencies_are_ignored(model_folders, tmp_path):
    def change(t):
        del t["lm_head.weight"]
        t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(10)
    folder = _rewrite(model_folders["C"], str(tmp_path / "nohead"), change)
    with pytest.raises(WeightError) as e:
        build_model(read_config_json(folder)).load(Checkpoint(folder), torch.float32, torch.device("cpu"))
    assert e.value.missing == ["lm_head.weight"] and not e.value.unexpected


def test_dtypes_after_loading(model_folders, tmp_path):
    # matrices take the model's dtype; norm weights and biases are float32 in every mode;
    # a float32 checkpoint stays float32 in a float32 run
    for dtype in (torch.bfloat16, torch.float32):
        m = build_model(read_config_json(model_folders["C"]))
        m.load(Checkpoint(model_folders["C"]), dtype, torch.device("cpu"))
        assert m.embed_table.dtype == dtype and m.blocks[0].mixer.w_qkv.dtype == dtype
        assert m.final_norm.weight.dtype == torch.float32 and m.blocks[0].mixer.b_qkv.dtype == torch.float32
        assert m.blocks[0].mixer.position.inv_freq.dtype == torch.float32
    folder = write_random_model_folder(str(tmp_path / "f32"), TINY["A"]["config"], 1, store_dtype=torch.float32)
    ck = Checkpoint(folder)
    assert ck.stored_dtype("model.norm.weight") == torch.float32
    ck.close()


def test_missing_files_are_clear_errors(tmp_path):
    with pytest.raises(ConfigError, match="config.json"):
        read_config_json(str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(TINY["A"]["config"].to_dict()))
    with pytest.raises(WeightError, match="safetensors"):
        load_model(str(tmp_path), "float32", "cpu")


def test_a_head_size_beyond_the_kernels_is_refused_when_the_model_is_built():
    from wllm_amd.parts import build_model
    c = TINY["A"]["config"].to_dict()
    c["head_dim"] = 272
    with pytest.raises(ValueError, match="head_dim 272"):
        build_model(c)


def test_the_index_file_names_files_of_its_own_folder_only(model_folders, tmp_path):
    """model.safetensors.index.json belongs to a folder that may come from anywhere: a weight_map
    entry that is absolute, climbs out of the folder or is no .safetensors file is refused; a plain
    name is honoured (two shards, loaded as one checkpoint)."""
    src = Checkpoint(model_folders["A"])
    tensors = {n: src.tensor(n) for n in src.names()}
    src.close()
    names = sorted(tensors)
    folder = tmp_path / "sharded"
    folder.mkdir()
    halves = {"part-1.safetensors": names[:5], "part-2.safetensors": names[5:]}
    for file, part in halves.items():
        write_safetensors(str(folder / file), {n: tensors[n] for n in part})
    (folder / "config.json").write_text(json.dumps(TINY["A"]["config"].to_dict()))
    (folder / "model.safetensors.index.json").write_text(
        json.dumps({"weight_map": {n: file for file, part in halves.items() for n in part}}))
    ck = Checkpoint(str(folder))
    assert sorted(ck.names()) == names and torch.equal(ck.tensor(names[7]), tensors[names[7]])
    ck.close()
    outside = tmp_path / "outside.safetensors"
    write_safetensors(str(outside), {"x": torch.zeros(1)})
    for bad in (str(outside), "../outside.safetensors", "sub/part-1.safetensors", "config.json"):
        (folder / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"x": bad}}))
        with pytest.raises(WeightError, match="weight_map"):
            Checkpoint(str(folder))
