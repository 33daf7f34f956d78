"""Configuration, registry, safetensors I/O and weight errors (no GPU)."""

from __future__ import annotations

import json

import pytest
import torch

from conftest import TINY_A, TINY_B
from lockstep_amd.config import (ConfigError, ModelConfig, Qwen3Config, config_from_dict, config_from_dir,
                                 known_architectures, register_architecture, unregister_architecture)
from lockstep_amd.engine.model import collect_ties, collect_weight_specs
from lockstep_amd.weights import (SafetensorsFile, WeightError, load_weights, random_tensors, save_file,
                                  write_random_model)


def test_config_reads_its_keys_and_has_no_defaults():
    cfg = config_from_dict(dict(TINY_B, model_type="qwen3", ignored_key=5))
    assert isinstance(cfg, Qwen3Config) and cfg.head_dim == 32 and cfg.tie_word_embeddings is False
    for key in TINY_A:
        raw = dict(TINY_A, model_type="qwen3")
        del raw[key]
        with pytest.raises(ConfigError, match=key):
            config_from_dict(raw)


def test_registry_finds_by_either_name_and_lists_known_names():
    assert isinstance(config_from_dict(dict(TINY_A, architectures=["Qwen3ForCausalLM"])), Qwen3Config)
    with pytest.raises(ConfigError, match="qwen3"):
        config_from_dict(dict(TINY_A, model_type="llama"))
    assert "qwen3" in known_architectures()


def test_config_rejects_impossible_values():
    for key, value in (("num_key_value_heads", 3), ("head_dim", 15), ("hidden_size", 0), ("rms_norm_eps", 0.0)):
        with pytest.raises(ConfigError):
            config_from_dict(dict(TINY_A, model_type="qwen3", **{key: value}))


def test_model_spec_states_the_architecture_as_data():
    spec = Qwen3Config.from_dict(TINY_B).model_spec()
    assert len(spec.layers) == 3 and [e.layer for e in spec.schedule] == [0, 1, 2]
    mixer = spec.layers[1].mixer
    assert mixer.kind == "attention" and mixer["num_heads"] == 6 and mixer["num_kv_heads"] == 3
    assert mixer["qk_norm"]["eps"] == 1e-5 and mixer["position"]["theta"] == 1e6 and mixer["window"] is None
    assert spec.layers[0].feed_forward["intermediate_size"] == 256
    assert spec.head["tied_to"] is None
    assert Qwen3Config.from_dict(TINY_A).model_spec().head["tied_to"] == "model.embed_tokens.weight"


def test_a_new_architecture_registers_without_touching_the_package():
    from dataclasses import dataclass

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        width: int
        architecture_names = ("toy-arch",)

    register_architecture(ToyConfig)
    try:
        assert config_from_dict({"model_type": "toy-arch", "width": 8}).width == 8
        with pytest.raises(ConfigError):
            register_architecture(type("Clash", (ToyConfig,), {"architecture_names": ("qwen3",)}))
    finally:
        unregister_architecture(ToyConfig)


def test_safetensors_round_trip_and_library_compatibility(tmp_path):
    from safetensors.torch import load_file, save_file as lib_save

    tensors = {"a": torch.randn(3, 5).to(torch.bfloat16), "b": torch.arange(7, dtype=torch.int64),
               "c": torch.randn(4), "d": torch.randn(2, 2).to(torch.float16)}
    save_file(tensors, tmp_path / "mine.safetensors")
    back = load_file(str(tmp_path / "mine.safetensors"))
    assert all(torch.equal(back[k], v) for k, v in tensors.items())
    lib_save(tensors, str(tmp_path / "theirs.safetensors"))
    handle = SafetensorsFile(tmp_path / "theirs.safetensors")
    assert sorted(handle.keys()) == ["a", "b", "c", "d"]
    assert all(torch.equal(handle.get(k), v) for k, v in tensors.items())


def test_random_model_folder_loads_and_is_seeded(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_A)
    folder = write_random_model(cfg, tmp_path / "m", seed=0)
    assert config_from_dir(folder) == cfg
    spec = cfg.model_spec()
    store = load_weights(folder, collect_weight_specs(spec), collect_ties(spec))
    assert "lm_head.weight" in store and "lm_head.weight" not in store.names()
    assert store.source_name("lm_head.weight") == "model.embed_tokens.weight"
    emb = store.get("model.embed_tokens.weight")
    assert emb.dtype is torch.bfloat16 and 0.015 < float(emb.float().std()) < 0.025
    assert torch.equal(store.get("model.norm.weight").float(), torch.ones(64))
    again = random_tensors(cfg, 0)
    assert torch.equal(again["model.embed_tokens.weight"], emb)
    other = random_tensors(cfg, 1)
    assert not torch.equal(other["model.embed_tokens.weight"], emb)
    b = random_tensors(Qwen3Config.from_dict(TINY_B), 2, std=0.05, norm_std=0.1)
    assert "lm_head.weight" in b and 0.05 < float(b["model.norm.weight"].float().std()) < 0.15


def test_dtypes_are_normalised_not_chosen(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_A)
    tensors = random_tensors(cfg, 0)
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float()          # stored in 32-bit: stays
    tensors["model.layers.0.mlp.up_proj.weight"] = tensors["model.layers.0.mlp.up_proj.weight"].to(torch.float16)
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    save_file(tensors, tmp_path / "model.safetensors")
    spec = cfg.model_spec()
    store = load_weights(tmp_path, collect_weight_specs(spec), collect_ties(spec))
    assert store.get("model.norm.weight").dtype is torch.float32
    assert store.get("model.layers.0.mlp.up_proj.weight").dtype is torch.float16  # kept as stored until it is used
    assert store.get("model.embed_tokens.weight").dtype is torch.bfloat16


def test_a_lossy_cast_of_the_checkpoint_is_measured():
    # reference engine/model/qwen3.py:176-216: element count, inexact count, largest errors
    from lockstep_amd.weights.cast import CastLedger

    ledger = CastLedger(torch.bfloat16)
    stored = torch.tensor([1.0, 1.0 + 2.0 ** -10, -3.0, 0.3330078125], dtype=torch.float16)
    used = ledger.cast(stored, torch.bfloat16)
    assert used.dtype is torch.bfloat16
    assert ledger.report["elements"] == 4 and ledger.report["lossy_tensors"] == 1
    assert ledger.report["inexact_elements"] == 2                 # 1 + 2^-10 and 0.333 need more than 8 bits
    assert ledger.report["max_abs_error"] == pytest.approx(2.0 ** -10, rel=0.5)
    assert 0 < ledger.report["max_rel_error"] < 2.0 ** -8
    before = dict(ledger.report)
    assert ledger.cast(torch.ones(5, dtype=torch.bfloat16), torch.bfloat16).dtype is torch.bfloat16
    assert ledger.report == before                                # same dtype: not a cast
    wide = CastLedger(torch.float32)
    assert torch.equal(wide.cast(stored, torch.float32), stored.float())
    assert wide.report["elements"] == 4 and wide.report["lossy_tensors"] == 0 and wide.report["inexact_elements"] == 0
    assert wide.cast(torch.tensor([3], dtype=torch.int32), torch.float32).dtype is torch.int32   # tables are left alone


def test_the_position_bound_comes_from_the_configuration():
    spec = Qwen3Config.from_dict(TINY_A).model_spec()
    assert spec.max_positions == TINY_A["max_position_embeddings"] == 256
    assert Qwen3Config.from_dict(TINY_B).model_spec().max_positions == 512


def test_engine_config_is_typed_and_checked():
    from lockstep_amd.engine.config import EngineConfig
    from lockstep_amd.engine.policy import DefaultPolicy, FixedChunkPolicy

    cfg = EngineConfig(page_size=8, num_pages=40, prefill_chunk=12, eos_token_ids=[3, 7])
    assert cfg.eos_token_ids == (3, 7) and isinstance(cfg.policy(), FixedChunkPolicy) and cfg.policy().chunk == 12
    assert isinstance(EngineConfig().policy(), DefaultPolicy) and EngineConfig().policy().max_running == 64
    assert cfg.with_(num_pages=9).num_pages == 9 and cfg.to_dict()["page_size"] == 8
    for bad in (dict(page_size=48), dict(dtype="float16"), dict(reserve="eager"), dict(num_pages=0),
                dict(prefill_chunk=0), dict(decode_burst=0)):
        with pytest.raises(ValueError):
            EngineConfig(**bad)


def test_one_error_lists_missing_unexpected_and_misshapen(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_B)
    tensors = random_tensors(cfg, 2)
    del tensors["model.layers.1.self_attn.k_norm.weight"]
    del tensors["lm_head.weight"]
    tensors["model.layers.7.extra.weight"] = torch.zeros(3)
    tensors["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(96, 192, dtype=torch.bfloat16)  # transposed
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    save_file(tensors, tmp_path / "model.safetensors")
    spec = cfg.model_spec()
    with pytest.raises(WeightError) as info:
        load_weights(tmp_path, collect_weight_specs(spec), collect_ties(spec))
    err = info.value
    assert err.missing == ["lm_head.weight", "model.layers.1.self_attn.k_norm.weight"]
    assert err.unexpected == ["model.layers.7.extra.weight"]
    assert [m[0] for m in err.mismatched] == ["model.layers.0.self_attn.q_proj.weight"]
    text = str(err)
    assert "missing (2)" in text and "unexpected (1)" in text and "expected [192, 96] found [96, 192]" in text


def test_tied_head_present_and_equal_is_accepted_and_differing_is_refused(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_A)
    spec = cfg.model_spec()
    tensors = random_tensors(cfg, 0)
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    save_file(tensors, tmp_path / "model.safetensors")
    store = load_weights(tmp_path, collect_weight_specs(spec), collect_ties(spec))
    assert store.source_name("lm_head.weight") == "model.embed_tokens.weight"
    tensors["lm_head.weight"] = tensors["lm_head.weight"] + 1
    save_file(tensors, tmp_path / "model.safetensors")
    with pytest.raises(WeightError, match="refusing to alias"):
        load_weights(tmp_path, collect_weight_specs(spec), collect_ties(spec))


def test_sharded_checkpoints_are_read_through_their_index(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_A)
    spec = cfg.model_spec()
    tensors = random_tensors(cfg, 0)
    names = sorted(tensors)
    half = len(names) // 2
    save_file({n: tensors[n] for n in names[:half]}, tmp_path / "model-00001-of-00002.safetensors")
    save_file({n: tensors[n] for n in names[half:]}, tmp_path / "model-00002-of-00002.safetensors")
    index = {"weight_map": {n: ("model-00001-of-00002.safetensors" if i < half else
                                "model-00002-of-00002.safetensors") for i, n in enumerate(names)}}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    store = load_weights(tmp_path, collect_weight_specs(spec), collect_ties(spec))
    assert torch.equal(store.get(names[-1]), tensors[names[-1]])


def test_graph_safety_is_asked_of_every_part_of_a_layer():
    """A layer may run inside a captured graph only if the arrangement, its mixer (and the mixer's
    position encoding), its feed-forward and its norms all say so."""
    from lockstep_amd.config.presets import preset
    from lockstep_amd.parts import part_class
    from lockstep_amd.parts.base import graph_safe_tree

    spec = preset("tiny-a").model_spec()
    layer = part_class(spec.layers[0].arrangement.kind)(spec.layers[0])
    assert graph_safe_tree(layer)
    for part in (layer.feed_forward, layer.mixer.position, layer.mixer_norm):
        part.graph_safe = False          # on the instance: the class keeps its value
        assert not graph_safe_tree(layer)
        del part.graph_safe
    assert graph_safe_tree(layer)
