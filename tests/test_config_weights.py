"""Configuration, registry, safetensors round trips and the loader's one error."""

import json
import os

import pytest
import torch

import paged_attention_engine_amd as pae
from paged_attention_engine_amd.config import ModelPlan, ScheduleEntry
from paged_attention_engine_amd.config.model_config import ConfigError as CfgErr
from paged_attention_engine_amd.weights import SafetensorsFile, save_file
from tests import helpers
from tests.plain import qwen2_plain as plain


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_config_reads_every_key(name):
    raw = helpers.TINY[name][0]
    cfg = pae.read_config_dict(raw)
    assert cfg.num_hidden_layers == raw["num_hidden_layers"] and cfg.hidden_size == raw["hidden_size"]
    assert cfg.num_attention_heads == raw["num_attention_heads"]
    assert cfg.num_key_value_heads == raw["num_key_value_heads"] and cfg.head_dim == raw["head_dim"]
    assert cfg.intermediate_size == raw["intermediate_size"] and cfg.vocab_size == raw["vocab_size"]
    assert cfg.rms_norm_eps == raw["rms_norm_eps"] and cfg.rope_theta == raw["rope_theta"]
    assert cfg.tie_word_embeddings == raw["tie_word_embeddings"]
    plan = cfg.plan()
    assert len(plan.layers) == raw["num_hidden_layers"] == len(plan.schedule)
    mixer = plan.layers[-1].mixer
    assert mixer.scale == raw["head_dim"] ** -0.5 and mixer.position.theta == raw["rope_theta"]
    assert (plan.head_name is None) == raw["tie_word_embeddings"]
    # a round trip through config.json keeps the typed config
    assert pae.read_config_dict(json.loads(json.dumps(cfg.to_json_dict()))) == cfg


def test_windows_are_chosen_layer_by_layer():
    plan = pae.read_config_dict(helpers.TINY_C).plan()
    assert [layer.mixer.window for layer in plan.layers] == [None, None, 24, 24]
    assert all(layer.mixer.window is None for layer in pae.read_config_dict(helpers.TINY_A).plan().layers)


def test_head_dim_falls_back_and_theta_may_be_nested():
    raw = dict(helpers.TINY_A)
    del raw["head_dim"], raw["rope_theta"]
    raw["rope_parameters"] = {"rope_theta": 5000.0, "rope_type": "default"}
    cfg = pae.read_config_dict(raw)  # engine/model.py:66-70,79 of the reference
    assert cfg.head_dim == 64 // 4 and cfg.rope_theta == 5000.0


@pytest.mark.parametrize("change,needle", [
    ({"architectures": ["LlamaForCausalLM"]}, "unknown architecture"),
    ({"architectures": None}, "architectures"),
    ({"hidden_size": None}, "hidden_size"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"rms_norm_eps": "x"}, "rms_norm_eps"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 4}}, "rope_scaling"),
    ({"use_sliding_window": True, "sliding_window": None}, "sliding_window"),
    ({"vocab_size": 0}, "vocab_size"),
])
def test_config_errors_name_the_key(change, needle):
    raw = dict(helpers.TINY_A)
    raw.update(change)
    with pytest.raises(pae.ConfigError) as err:
        pae.read_config_dict(raw)
    assert needle in str(err.value)


def test_unknown_architecture_lists_the_known_ones():
    with pytest.raises(pae.ConfigError) as err:
        pae.read_config_dict({"architectures": ["Nope"]})
    assert "Qwen2ForCausalLM" in str(err.value) and "Qwen2ForCausalLM" in pae.known_architectures()


def test_schedule_must_point_backwards():
    plan = pae.read_config_dict(helpers.TINY_A).plan()
    with pytest.raises(CfgErr):
        ModelPlan(**{**plan.__dict__, "schedule": (ScheduleEntry(0, cache_from=0),)})
    with pytest.raises(CfgErr):
        ModelPlan(**{**plan.__dict__, "schedule": (ScheduleEntry(5),)})


def test_expected_tensors_match_the_checkpoint_names():
    for name in ("A", "B", "C"):
        raw = helpers.TINY[name][0]
        want = plain.tensor_shapes(raw)  # names as the reference reads them, engine/model.py:198-227
        got = pae.expected_tensors(pae.read_config_dict(raw).plan())
        assert {k: tuple(v) for k, v in got.items()} == want


def test_safetensors_round_trip(tmp_path):
    tensors = {"a": torch.randn(3, 5).to(torch.bfloat16), "b": torch.randn(7), "c": torch.arange(6, dtype=torch.int64),
               "d": torch.randn(2, 2).to(torch.float16), "e": torch.zeros(0, 4)}
    path = str(tmp_path / "x.safetensors")
    save_file(tensors, path, {"k": "v"})
    f = SafetensorsFile(path)
    assert f.metadata == {"k": "v"} and set(f.names()) == set(tensors)
    for name, t in tensors.items():
        assert torch.equal(f.tensor(name), t) and f.dtype(name) == t.dtype
    # the file is what the safetensors package reads too
    from safetensors import safe_open
    with safe_open(path, "pt") as handle:
        assert torch.equal(handle.get_tensor("a"), tensors["a"])


def test_loader_keeps_stored_precision(tmp_path):
    folder = str(tmp_path)
    save_file({"w": torch.randn(2, 3).to(torch.bfloat16), "n": torch.ones(3), "h": torch.randn(3).to(torch.float16),
               "t": torch.arange(4, dtype=torch.int64)}, os.path.join(folder, "model.safetensors"))
    out = pae.load_weights(folder, {"w": (2, 3), "n": (3,), "h": (3,), "t": (4,)})
    assert out["w"].dtype == torch.bfloat16 and out["n"].dtype == torch.float32
    assert out["h"].dtype == torch.float32 and out["t"].dtype == torch.int32


def test_random_weights_mode_writes_a_loadable_folder(tmp_path):
    folder = helpers.make_model_folder(tmp_path, "B")
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    cfg = pae.read_config(folder)
    weights = pae.load_weights(folder, pae.expected_tensors(cfg.plan()))
    assert all(t.dtype == torch.bfloat16 for t in weights.values())
    q = weights["model.layers.0.self_attn.q_proj.weight"].float()
    assert 0.015 < float(q.std()) < 0.025
    assert float(weights["model.layers.0.self_attn.q_proj.bias"].float().abs().max()) > 0  # biases carry signal
    norm = weights["model.layers.1.input_layernorm.weight"].float()
    assert 0.05 < float(norm.std()) < 0.15 and abs(float(norm.mean()) - 1) < 0.05
    # same seed, same folder; another seed, other numbers
    again = helpers.make_model_folder(tmp_path / "again", "B")
    w2 = pae.load_weights(again, pae.expected_tensors(cfg.plan()))
    assert all(torch.equal(weights[k], w2[k]) for k in weights)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = helpers.make_model_folder(tmp_path, "A")
    _, tensors = helpers.read_folder_plain(folder)
    tensors = {k: v.to(torch.bfloat16) for k, v in tensors.items()}
    del tensors["model.layers.1.mlp.up_proj.weight"], tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(63, dtype=torch.bfloat16)
    tensors["model.layers.0.mlp.down_proj.weight"] = torch.zeros(176, 64, dtype=torch.bfloat16)
    tensors["model.layers.7.extra.weight"] = torch.zeros(2)
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    with pytest.raises(pae.WeightsError) as err:
        pae.load_weights(folder, pae.expected_tensors(pae.read_config(folder).plan()))
    e = err.value
    assert set(e.missing) == {"model.layers.1.mlp.up_proj.weight", "model.norm.weight"}
    assert e.unexpected == ("model.layers.7.extra.weight",)
    assert {w[0] for w in e.wrong_shape} == {"model.layers.0.self_attn.q_proj.bias", "model.layers.0.mlp.down_proj.weight"}
    text = str(e)
    for needle in ("missing (2)", "unexpected (1)", "wrong shape (2)", "model.norm.weight", "[176, 64]", "[64, 176]"):
        assert needle in text


def test_untied_config_needs_its_head_and_tied_tolerates_one(tmp_path):
    folder = helpers.make_model_folder(tmp_path, "A")  # tied
    _, tensors = helpers.read_folder_plain(folder)
    tensors = {k: v.to(torch.bfloat16) for k, v in tensors.items()}
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    plan = pae.read_config(folder).plan()
    pae.load_weights(folder, pae.expected_tensors(plan), optional=("lm_head.weight",))  # stored head is ignored
    raw = dict(helpers.TINY_A, tie_word_embeddings=False)
    del tensors["lm_head.weight"]
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    with pytest.raises(pae.WeightsError) as err:
        pae.load_weights(folder, pae.expected_tensors(pae.read_config_dict(raw).plan()))
    assert err.value.missing == ("lm_head.weight",)


def test_missing_files_are_reported(tmp_path):
    with pytest.raises(pae.ConfigError):
        pae.read_config(str(tmp_path))
    with pytest.raises(pae.WeightsError):
        pae.load_weights(str(tmp_path), {"a": (1,)})


def test_sharded_folder(tmp_path):
    folder = str(tmp_path)
    save_file({"a": torch.ones(2)}, os.path.join(folder, "model-00001-of-00002.safetensors"))
    save_file({"b": torch.zeros(3)}, os.path.join(folder, "model-00002-of-00002.safetensors"))
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as handle:
        json.dump({"weight_map": {"a": "model-00001-of-00002.safetensors", "b": "model-00002-of-00002.safetensors"}}, handle)
    out = pae.load_weights(folder, {"a": (2,), "b": (3,)})
    assert torch.equal(out["a"], torch.ones(2)) and torch.equal(out["b"], torch.zeros(3))


# ------------------------------------------------------------------ pool sizing, random weights, shards
def test_the_pool_is_sized_once_in_pages_or_bytes_or_a_share_of_free_memory():
    from paged_attention_engine_amd.config.engine_config import NUM_GPU_BLOCKS, EngineConfig

    asked = []

    def free():
        asked.append(1)
        return 1000

    assert EngineConfig().pages(100, free) == NUM_GPU_BLOCKS
    assert EngineConfig(num_blocks=7).pages(100, free) == 7
    assert EngineConfig(kv_bytes=1050).pages(100, free) == 10 and not asked
    assert EngineConfig(fill_hbm=0.55).pages(100, free) == 5 and asked
    with pytest.raises(ValueError, match="once"):
        EngineConfig(num_blocks=4, kv_bytes=100)
    with pytest.raises(ValueError):
        EngineConfig(fill_hbm=1.5)
    with pytest.raises(ValueError, match="one page"):
        EngineConfig(kv_bytes=99).pages(100, free)


def test_random_weights_are_drawn_at_the_lookup_and_repeat():
    from paged_attention_engine_amd.weights import RandomWeights

    from paged_attention_engine_amd.parts import ScaleShape

    # how a tensor is drawn is said where it is declared, not read off its name: the scale vector is
    # called `ln.scale` here, and a matrix whose name ends like a norm's weight stays a matrix
    shapes = {"a.q_proj.weight": (6, 4), "a.ln.scale": ScaleShape((4,)), "b.weight": (3, 3),
              "c.input_layernorm.weight": (64, 8)}
    assert shapes["a.ln.scale"] == (4,)
    drawn = RandomWeights(shapes, seed=5, std={"": 0.02, "q_proj.weight": 0.5}, norm_std=0.1, device="cpu")
    assert sorted(drawn) == sorted(shapes) and len(drawn) == 4
    first, again = drawn["a.q_proj.weight"], drawn["a.q_proj.weight"]
    assert first is not again and torch.equal(first, again) and first.dtype == torch.bfloat16
    assert float(first.float().std()) > 0.2 > float(drawn["b.weight"].float().std())  # the wider ending applies
    assert float((drawn["a.ln.scale"].float() - 1).abs().max()) < 0.5
    assert float((RandomWeights(shapes, seed=5, device="cpu")["a.ln.scale"].float() - 1).abs().max()) == 0.0
    assert float(drawn["c.input_layernorm.weight"].float().abs().max()) < 0.2  # about zero: it was declared a matrix
    assert not torch.equal(first, RandomWeights(shapes, seed=6, device="cpu")["a.q_proj.weight"])
    with pytest.raises(KeyError):
        drawn["c"]
    assert drawn.get("c") is None


def test_an_index_that_names_what_a_shard_lacks_is_a_weights_error(tmp_path):
    import json

    from paged_attention_engine_amd.weights import load_weights, save_file

    save_file({"a": torch.zeros(2, 2)}, str(tmp_path / "part1.safetensors"))
    index = {"weight_map": {"a": "part1.safetensors", "b": "part1.safetensors"}}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    with pytest.raises(pae.WeightsError, match="b \\(not in part1.safetensors\\)") as err:
        load_weights(str(tmp_path), {"a": (2, 2), "b": (2, 2)})
    assert err.value.missing == ("b",)
    index["weight_map"]["b"] = "part2.safetensors"
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    with pytest.raises(pae.WeightsError, match="part2.safetensors"):
        load_weights(str(tmp_path), {"a": (2, 2), "b": (2, 2)})


def test_a_shard_index_cannot_reach_outside_the_model_folder(tmp_path):
    import json

    from paged_attention_engine_amd.weights import load_weights, save_file

    outside = tmp_path / "elsewhere.safetensors"
    save_file({"a": torch.zeros(2, 2)}, str(outside))
    folder = tmp_path / "model"
    folder.mkdir()
    for shard in ("../elsewhere.safetensors", str(outside), "sub/x.safetensors", "..", ""):
        (folder / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": shard}}))
        with pytest.raises(pae.WeightsError, match="plain file name"):
            load_weights(str(folder), {"a": (2, 2)})


def test_loaded_weights_are_views_of_the_file(tmp_path):
    from paged_attention_engine_amd.weights import load_weights, save_file

    save_file({"a": torch.arange(6, dtype=torch.float32).view(2, 3), "h": torch.ones(2, dtype=torch.float16)},
              str(tmp_path / "model.safetensors"))
    weights = load_weights(str(tmp_path), {"a": (2, 3), "h": (2,)})
    assert not isinstance(weights, dict) and sorted(weights) == ["a", "h"]
    assert torch.equal(weights["a"], torch.arange(6, dtype=torch.float32).view(2, 3))
    assert weights["h"].dtype == torch.float32  # half precision is widened, nothing else is copied
    assert weights.get("zzz") is None


def test_the_default_precision_is_the_configs_own():
    from paged_attention_engine_amd.engine.model import default_dtype

    cfg = dict(helpers.TINY_A)
    assert default_dtype(pae.read_config_dict(cfg)) == "bfloat16"
    assert default_dtype(pae.read_config_dict(dict(cfg, torch_dtype="float32"))) == "float32"
    assert default_dtype(pae.read_config_dict(dict(cfg, torch_dtype="torch.float32"))) == "float32"
    assert default_dtype(pae.read_config_dict(dict(cfg, torch_dtype="float16"))) == "bfloat16"  # served in bfloat16
    assert pae.read_config_dict(dict(cfg, torch_dtype="float32")).to_json_dict()["torch_dtype"] == "float32"


def test_state_slots_bound_live_sequences_only_where_someone_said_so():
    from paged_attention_engine_amd.config.engine_config import EngineConfig

    assert EngineConfig(num_state_slots=5, max_num_seqs=9).state_slots_for(100, True) == 5
    assert EngineConfig(max_num_seqs=9).state_slots_for(100, False) == 9
    # nobody said: a model without per-request state gets a slot per page, which never binds
    assert EngineConfig().state_slots_for(100, False) == 100
    with pytest.raises(ValueError, match="max_num_seqs or num_state_slots"):
        EngineConfig().state_slots_for(100, True)


def test_a_plan_names_the_tensors_a_checkpoint_may_hold_unused():
    tied = pae.read_config_dict(dict(helpers.TINY_A, tie_word_embeddings=True)).plan()
    untied = pae.read_config_dict(dict(helpers.TINY_A, tie_word_embeddings=False)).plan()
    assert tied.optional_names == ("lm_head.weight",) and untied.optional_names == ()
