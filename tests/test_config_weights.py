"""Configuration, registry, weight loading and the random-weights mode (CPU)."""

import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from helpers import TINY_A, TINY_B, TINY_C
from socrates_amd.config import (ConfigError, Qwen3Config, known_architectures, load_config,
                                 register_architecture)
from socrates_amd.config.specs import ModelPlan, RunStep
from socrates_amd.parts import expected_tensors
from socrates_amd.weights import WeightError, load_weights, write_random_model

# The reference's pinned configuration of Qwen3-4B (model/configs/qwen3-4b.json), with every key it
# carries, ignored ones included. Kept here as data so that the test runs wherever the
# repository is checked out; SOCRATES_REFERENCE may name a checkout of the reference to
# compare this copy with.
REFERENCE_4B = {
    "architectures": ["Qwen3ForCausalLM"], "attention_bias": False, "attention_dropout": 0.0,
    "bos_token_id": 151643, "eos_token_id": 151645, "head_dim": 128, "hidden_act": "silu",
    "hidden_size": 2560, "initializer_range": 0.02, "intermediate_size": 9728,
    "max_position_embeddings": 40960, "max_window_layers": 36, "model_type": "qwen3",
    "num_attention_heads": 32, "num_hidden_layers": 36, "num_key_value_heads": 8,
    "rms_norm_eps": 1e-06, "rope_scaling": None, "rope_theta": 1000000, "sliding_window": None,
    "tie_word_embeddings": True, "torch_dtype": "bfloat16", "transformers_version": "4.51.0",
    "use_cache": True, "use_sliding_window": False, "vocab_size": 151936}


def test_reads_every_size_from_its_own_keys():
    a, b = Qwen3Config.from_dict(TINY_A["cfg"]), Qwen3Config.from_dict(TINY_B["cfg"])
    c = Qwen3Config.from_dict(TINY_C["cfg"])
    for key in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                "num_key_value_heads", "head_dim", "intermediate_size", "rms_norm_eps", "rope_theta",
                "tie_word_embeddings"):
        assert getattr(a, key) == TINY_A["cfg"][key] and getattr(b, key) == TINY_B["cfg"][key]
        # B and C differ in every size and option; A differs from B in all but the kv heads
        assert getattr(b, key) != getattr(c, key), f"tiny B and C share {key}"
        assert getattr(a, key) != getattr(b, key) or key == "num_key_value_heads"
    assert TINY_A["block_size"] != TINY_B["block_size"] != TINY_C["block_size"]
    plan = b.plan()
    att = plan.layers[0].mixer
    assert (att.n_heads, att.n_kv_heads, att.head_dim) == (8, 2, 32)
    assert att.scale == 32 ** -0.5 and att.qk_norm.eps == 1e-5 and att.position.theta == 1e6
    assert att.window is None and plan.head_name == "lm_head.weight"
    assert a.plan().head_name is None                     # tied: the head is the embedding table
    assert len(plan.layers) == 3 and [s.layer for s in plan.order] == [0, 1, 2]


def test_reference_config_reads(tmp_path):
    import os
    (tmp_path / "config.json").write_text(json.dumps(REFERENCE_4B))
    cfg = Qwen3Config.from_json(tmp_path)                  # model/configs/qwen3-4b.json
    assert load_config(tmp_path) == cfg                    # through the registry too
    checkout = os.environ.get("SOCRATES_REFERENCE")
    if checkout:
        assert json.loads(open(os.path.join(checkout, "model/configs/qwen3-4b.json")).read()) == REFERENCE_4B
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.head_dim) == (36, 2560, 128)
    assert cfg.tie_word_embeddings and cfg.eos_token_ids == (151645,)
    counts = cfg.param_counts()
    assert abs(counts["total"] / 1e9 - 4.0225) < 0.001     # the survey's 4.0225 B parameters
    assert cfg.kv_bytes_per_token(2) == 147456


@pytest.mark.parametrize("change,needle", [
    ({"hidden_size": None}, "lacks"), ({"attention_bias": True}, "attention_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"), ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"),
    ({"use_sliding_window": True}, "sliding"), ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 24}, "head_dim"), ({"vocab_size": -5}, "positive")])
def test_rejects_what_it_does_not_compute(change, needle):
    d = dict(TINY_A["cfg"])
    for k, v in change.items():
        if v is None:
            d.pop(k)
        else:
            d[k] = v
    with pytest.raises(ConfigError, match=needle):
        Qwen3Config.from_dict(d)


def test_head_dim_falls_back_like_the_reference_analysis():
    d = dict(TINY_A["cfg"])
    d.pop("head_dim")
    assert Qwen3Config.from_dict(d).head_dim == 64 // 4    # analysis/arithmetic.py:68-72


def test_registry(tmp_path):
    assert "Qwen3ForCausalLM" in known_architectures()
    (tmp_path / "config.json").write_text(json.dumps(dict(TINY_A["cfg"], architectures=["NoSuchLM"])))
    with pytest.raises(ConfigError, match="unknown architecture.*Qwen3ForCausalLM"):
        load_config(tmp_path)

    class Other(Qwen3Config):
        pass
    register_architecture("OtherLM", Other)
    (tmp_path / "config.json").write_text(json.dumps(dict(TINY_A["cfg"], architectures=["OtherLM"])))
    assert type(load_config(tmp_path)) is Other


def test_plug_ins_named_in_the_environment(tmp_path, monkeypatch):
    """A module named in SOCRATES_AMD_PLUGINS is imported when a name is looked up that the
    registry does not know, and may register it; a module that cannot be imported is one
    clear error."""
    import socrates_amd.config.registry as registry
    (tmp_path / "plug_a.py").write_text(
        "from socrates_amd.config import Qwen3Config, register_architecture\n"
        "class Plugged(Qwen3Config):\n    pass\n"
        "register_architecture('PluggedLM', Plugged)\n")
    (tmp_path / "config.json").write_text(json.dumps(dict(TINY_A["cfg"], architectures=["PluggedLM"])))
    monkeypatch.syspath_prepend(str(tmp_path))
    monkeypatch.setattr(registry, "_plugins_loaded", False)
    monkeypatch.setenv("SOCRATES_AMD_PLUGINS", "no_such_module_anywhere")
    with pytest.raises(ConfigError, match="no_such_module_anywhere.*cannot be imported"):
        load_config(tmp_path)
    monkeypatch.setattr(registry, "_plugins_loaded", False)
    monkeypatch.setenv("SOCRATES_AMD_PLUGINS", " plug_a ,")
    assert type(load_config(tmp_path)).__name__ == "Plugged"
    registry._ARCHITECTURES.pop("PluggedLM")


def test_presets_that_come_with_the_package():
    """Five configuration files: the two tiny test shapes and Qwen3-4B, -8B and -32B sizes.
    Parameter counts of the big ones are the published model sizes; the 4B file says what the
    reference's pinned copy says, where that is present."""
    from socrates_amd.config import known_presets, load_preset, preset_path
    assert known_presets() == ["qwen3-32b", "qwen3-4b", "qwen3-8b", "tiny-a", "tiny-b"]
    for name, billions in (("qwen3-4b", 4.02), ("qwen3-8b", 8.19), ("qwen3-32b", 32.76)):
        assert abs(load_preset(name).param_counts()["total"] / 1e9 - billions) < 0.01, name
    a, b = load_preset("tiny-a"), load_preset("tiny-b")
    assert (a.head_dim, a.tie_word_embeddings, b.head_dim, b.tie_word_embeddings) == (16, True, 32, False)
    with pytest.raises(ConfigError, match="unknown preset.*qwen3-4b"):
        preset_path("qwen3-400b")
    ours, theirs = load_preset("qwen3-4b"), Qwen3Config.from_dict(REFERENCE_4B)
    for key in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
                "head_dim", "intermediate_size", "rms_norm_eps", "rope_theta", "tie_word_embeddings"):
        assert getattr(ours, key) == getattr(theirs, key), key


def test_run_order_is_data():
    plan = Qwen3Config.from_dict(TINY_B["cfg"]).plan()
    fields = {f: getattr(plan, f) for f in plan.__dataclass_fields__}
    # layer 1 runs twice; its second run reads the cache its first run wrote
    order = (RunStep(0, 0), RunStep(1, 1), RunStep(1, 1, write=False), RunStep(2, 2))
    assert ModelPlan(**dict(fields, order=order)).n_cache_slots == 3
    with pytest.raises(ValueError, match="before any step wrote"):
        ModelPlan(**dict(fields, order=(RunStep(0, 0, write=False),)))
    with pytest.raises(ValueError, match="written by two"):
        ModelPlan(**dict(fields, order=(RunStep(0, 0), RunStep(1, 0))))


def test_random_model_round_trip(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_B["cfg"])
    folder = write_random_model(tmp_path / "m", cfg, seed=5)
    assert load_config(folder) == cfg
    stored = load_file(str(folder / "model.safetensors"))
    plan = cfg.plan()
    expected = expected_tensors(plan)
    assert set(stored) == set(expected) and len(expected) == 11 * 3 + 3       # 11 per layer + 3
    assert all(t.dtype == torch.bfloat16 for t in stored.values())
    w16 = load_weights(folder, expected, torch.bfloat16, "cpu")
    w32 = load_weights(folder, expected, torch.float32, "cpu")
    q = "model.layers.1.self_attn.q_proj.weight"
    assert w16[q].dtype == torch.bfloat16 and w32[q].dtype == torch.float32
    assert torch.equal(w16[q].float(), w32[q])                               # bf16 -> fp32 is exact
    gain = "model.layers.0.input_layernorm.weight"
    assert w16[gain].dtype == torch.float32 and abs(w16[gain].mean() - 1) < 0.2   # gains near one
    again = write_random_model(tmp_path / "m2", cfg, seed=5)
    assert all(torch.equal(v, load_file(str(again / "model.safetensors"))[k]) for k, v in stored.items())
    other = write_random_model(tmp_path / "m3", cfg, seed=6)
    assert not torch.equal(stored[q], load_file(str(other / "model.safetensors"))[q])


def test_a_tensor_stored_in_32_bit_stays_so(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_A["cfg"])
    folder = write_random_model(tmp_path / "m", cfg, seed=1, dtype=torch.float32)
    with pytest.warns(UserWarning, match="stored in 32-bit"):         # and says so: those products are slow
        w = load_weights(folder, expected_tensors(cfg.plan()), torch.bfloat16, "cpu")
    assert all(t.dtype == torch.float32 for t in w.values())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_A["cfg"])
    folder = write_random_model(tmp_path / "m", cfg, seed=1)
    path = folder / "model.safetensors"
    t = load_file(str(path))
    del t["model.layers.1.mlp.up_proj.weight"], t["model.norm.weight"]
    t["lm_head.weight"] = torch.zeros(256, 64, dtype=torch.bfloat16)          # tied: unexpected
    t["model.layers.0.extra.bias"] = torch.zeros(3)
    t["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(32, 65, dtype=torch.bfloat16)
    t["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(16, dtype=torch.int32)
    save_file(t, str(path))
    with pytest.raises(WeightError) as e:
        load_weights(folder, expected_tensors(cfg.plan()), torch.bfloat16, "cpu")
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["lm_head.weight", "model.layers.0.extra.bias"]
    assert err.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (32, 64), (32, 65))]
    assert err.wrong_dtype == [("model.layers.0.self_attn.q_norm.weight", "I32")]
    for s in err.missing + err.unexpected + ["expected [32, 64], found [32, 65]"]:
        assert s in str(err)


def test_sharded_folder_with_index(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_A["cfg"])
    folder = write_random_model(tmp_path / "m", cfg, seed=2)
    t = load_file(str(folder / "model.safetensors"))
    names = sorted(t)
    half = len(names) // 2
    save_file({n: t[n] for n in names[:half]}, str(folder / "model-00001-of-00002.safetensors"))
    save_file({n: t[n] for n in names[half:]}, str(folder / "model-00002-of-00002.safetensors"))
    index = {"weight_map": {n: f"model-0000{1 if i < half else 2}-of-00002.safetensors"
                            for i, n in enumerate(names)}}
    (folder / "model.safetensors.index.json").write_text(json.dumps(index))
    (folder / "model.safetensors").unlink()
    w = load_weights(folder, expected_tensors(cfg.plan()), torch.bfloat16, "cpu")
    assert all(torch.equal(w[n].to(t[n].dtype) if w[n].dtype != t[n].dtype else w[n], t[n])
               for n in names if t[n].dim() == 2)
    with pytest.raises(FileNotFoundError):
        load_weights(tmp_path, expected_tensors(cfg.plan()), torch.bfloat16, "cpu")


def test_a_tied_checkpoint_may_store_its_head_if_it_is_the_embedding_table(tmp_path):
    """Some exporters write ``lm_head.weight`` beside the embedding although the two are tied:
    accepted if and only if the values are the same; never loaded twice."""
    from safetensors.torch import load_file, save_file
    cfg = Qwen3Config.from_dict(TINY_A["cfg"])
    plan = cfg.plan()
    folder = write_random_model(tmp_path / "m", cfg, seed=1)
    path = folder / "model.safetensors"
    t = load_file(str(path))
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    save_file(t, str(path))
    w = load_weights(folder, expected_tensors(plan), torch.bfloat16, "cpu", plan.duplicates)
    assert "lm_head.weight" not in w and set(w) == set(expected_tensors(plan))
    with pytest.raises(WeightError) as e:                    # without the plan's say-so it stays unexpected
        load_weights(folder, expected_tensors(plan), torch.bfloat16, "cpu")
    assert e.value.unexpected == ["lm_head.weight"]
    t["lm_head.weight"][3, 5] += 1
    save_file(t, str(path))
    with pytest.raises(WeightError) as e:
        load_weights(folder, expected_tensors(plan), torch.bfloat16, "cpu", plan.duplicates)
    assert e.value.unexpected == ["lm_head.weight"]
