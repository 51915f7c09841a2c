"""Configuration, registry and weight loading (no GPU)."""
import json

import pytest
import torch
from safetensors.torch import save_file

from llm_infrence_engine_amd.config import (ConfigError, Qwen2Config, config_from_dict, known_architectures,
                                            load_config, register_architecture)
from llm_infrence_engine_amd.config.spec import ModelSpec, PartSpec, Run
from llm_infrence_engine_amd.parts import Model
from llm_infrence_engine_amd.weights import CheckpointReader, TensorSpec, WeightsError, place, write_random_model
from tests.conftest import TINY, plain_random_weights, write_plain_model

HALF_B = {  # Qwen2.5-0.5B's config.json keys
    "architectures": ["Qwen2ForCausalLM"], "hidden_size": 896, "intermediate_size": 4864, "num_hidden_layers": 24,
    "num_attention_heads": 14, "num_key_value_heads": 2, "vocab_size": 151936, "rms_norm_eps": 1e-6,
    "rope_theta": 1000000.0, "tie_word_embeddings": True, "use_sliding_window": False, "sliding_window": 32768,
    "max_position_embeddings": 32768, "hidden_act": "silu", "torch_dtype": "bfloat16"}


def test_config_reads_its_keys_and_derives_the_rest():
    c = config_from_dict(HALF_B)
    assert isinstance(c, Qwen2Config)
    assert (c.head_dim, c.num_params, c.kv_bytes_per_token(2)) == (64, 494032768, 12288)
    assert config_from_dict(TINY["C"]).head_dim == 48            # stated in config.json, not hidden / heads
    d = dict(TINY["A"]); del d["rope_theta"]
    assert config_from_dict(d).rope_theta == 10000.0             # the reference's default
    d["rope_parameters"] = {"rope_theta": 5e5}
    assert config_from_dict(d).rope_theta == 5e5                 # and its fallback
    d = dict(TINY["A"]); del d["tie_word_embeddings"]
    assert config_from_dict(d).tie_word_embeddings is False
    assert config_from_dict(c.to_dict()) == c                    # round trip through config.json


@pytest.mark.parametrize("change,match", [
    ({"hidden_size": None}, "hidden_size"), ({"num_key_value_heads": 3}, "multiple"),
    ({"hidden_size": 65}, "head_dim"), ({"rope_scaling": {"type": "yarn", "factor": 4}}, "rope_scaling"),
    ({"use_sliding_window": True}, "sliding_window"), ({"vocab_size": "many"}, "integer"),
    ({"head_dim": 15}, "even"), ({"architectures": ["LlamaForCausalLM"]}, "unknown architecture"),
])
def test_config_errors_name_the_key(change, match):
    d = dict(TINY["A"]); d.update(change)
    with pytest.raises(ConfigError, match=match):
        config_from_dict(d)


def test_registry_chooses_by_name(tmp_path):
    assert "Qwen2ForCausalLM" in known_architectures()
    d = dict(TINY["B"]); del d["architectures"]; d["model_type"] = "qwen2"
    assert isinstance(config_from_dict(d), Qwen2Config)
    (tmp_path / "config.json").write_text(json.dumps(TINY["B"]))
    assert load_config(tmp_path).num_hidden_layers == 3
    with pytest.raises(ConfigError, match="not found"):
        load_config(tmp_path / "nowhere")

    class Other:
        @classmethod
        def from_dict(cls, d): return cls()
        def to_dict(self): return {}
        def to_spec(self): return None
    register_architecture("OtherForCausalLM", Other)
    try:
        assert isinstance(config_from_dict({"architectures": ["OtherForCausalLM"]}), Other)
    finally:
        from llm_infrence_engine_amd.config import registry
        registry._ARCHITECTURES.pop("OtherForCausalLM")


def test_spec_is_data_and_checks_its_order():
    s = config_from_dict(TINY["B"]).to_spec()
    assert len(s.layers) == 3 and [r.layer for r in s.order] == [0, 1, 2]
    a = s.layers[1].mixer
    assert a.kind == "gqa_attention" and a.params["num_heads"] == 6 and a.params["qkv_bias"] and not a.params["out_bias"]
    assert s.layers[1].position.params["theta"] == 1e6 and s.layers[1].mixer_norm.params["eps"] == 1e-5
    assert s.head.params["tied_to"] is None
    assert config_from_dict(TINY["A"]).to_spec().head.params["tied_to"] == "model.embed_tokens.weight"
    kw = dict(architecture="x", hidden_size=s.hidden_size, vocab_size=s.vocab_size, embedding=s.embedding,
              layers=s.layers, final_norm=s.final_norm, head=s.head)
    ModelSpec(order=(Run(0), Run(1), Run(1), Run(2, cache_of=0)), **kw)      # a layer twice, a borrowed cache
    with pytest.raises(ValueError, match="layer 3"):
        ModelSpec(order=(Run(3),), **kw)
    with pytest.raises(ValueError, match="before"):
        ModelSpec(order=(Run(0, cache_of=0),), **kw)
    with pytest.raises(ValueError, match="none of its own"):
        ModelSpec(order=(Run(0), Run(1, cache_of=0), Run(2, cache_of=1)), **kw)


def test_model_lists_its_tensors():
    m = Model(config_from_dict(TINY["A"]).to_spec())
    names = [s.name for s in m.tensor_specs()]
    assert len(names) == len(set(names)) == 1 + 2 * 12 + 1      # tied: no lm_head.weight
    assert "lm_head.weight" not in names and m.ignorable_tensors() == ["lm_head.weight"]
    roles = {s.name: s.role for s in m.tensor_specs()}
    assert roles["model.layers.0.self_attn.q_proj.bias"] == "bias" and roles["model.norm.weight"] == "norm"
    m = Model(config_from_dict(TINY["B"]).to_spec())
    assert "lm_head.weight" in [s.name for s in m.tensor_specs()]
    assert sum(int(torch.tensor(s.shape).prod()) for s in Model(config_from_dict(HALF_B).to_spec()).tensor_specs()) == 494032768


def test_random_model_folder_round_trips(tmp_path):
    cfg = config_from_dict(TINY["B"])
    d = write_random_model(tmp_path / "m", cfg, seed=1, dtype="bfloat16")
    assert load_config(d) == cfg
    r = CheckpointReader(d)
    m = Model(cfg.to_spec())
    r.check(m.tensor_specs(), m.ignorable_tensors())
    assert r.stored_type("model.norm.weight") == "BF16"
    w = r.get("model.layers.2.mlp.down_proj.weight")
    assert w.shape == (192, 320) and 0.015 < w.float().std() < 0.025
    n = r.get("model.norm.weight").float()
    assert abs(n.mean() - 1) < 0.05 and 0.05 < n.std() < 0.15
    d2 = write_random_model(tmp_path / "m2", cfg, seed=1, dtype="bfloat16")
    assert torch.equal(CheckpointReader(d2).get("lm_head.weight"), r.get("lm_head.weight"))   # the seed decides
    d3 = write_random_model(tmp_path / "m3", cfg, seed=2, dtype="float32")
    assert not torch.equal(CheckpointReader(d3).get("lm_head.weight").bfloat16(), r.get("lm_head.weight"))
    assert CheckpointReader(d3).stored_type("lm_head.weight") == "F32"


def test_one_error_lists_missing_unexpected_and_misshapen(tmp_path):
    cfg = TINY["A"]
    w = plain_random_weights(cfg, 0)
    del w["model.layers.1.mlp.up_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.0.self_attn.o_proj.bias"] = torch.zeros(64)
    w["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64)
    w["model.layers.0.input_layernorm.weight"] = torch.zeros(64, dtype=torch.int32)
    write_plain_model(tmp_path, cfg, w)
    m = Model(config_from_dict(cfg).to_spec())
    with pytest.raises(WeightsError) as e:
        CheckpointReader(tmp_path).check(m.tensor_specs(), m.ignorable_tensors())
    err = e.value
    assert sorted(err.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.o_proj.bias"]
    assert [(n, list(want), list(got)) for n, want, got in err.wrong_shape] == \
        [("model.layers.0.self_attn.k_proj.weight", [32, 64], [16, 64])]
    assert err.wrong_type[0][0] == "model.layers.0.input_layernorm.weight"
    for needle in ("up_proj", "model.norm.weight", "o_proj.bias", "[16, 64]", "[32, 64]", "I32"):
        assert needle in str(err)


def test_shards_in_two_files_and_a_shard_the_index_names_but_the_folder_lacks(tmp_path):
    """Every ``*.safetensors`` file is read and merged by name; the index is only asked which files should be there."""
    import json

    from safetensors.torch import save_file

    cfg = TINY["A"]
    w = plain_random_weights(cfg, 0)
    names = sorted(w)
    half = len(names) // 2
    tmp_path.mkdir(exist_ok=True)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    shards = {"model-00001-of-00002.safetensors": names[:half], "model-00002-of-00002.safetensors": names[half:]}
    for f, ns in shards.items():
        save_file({n: w[n].contiguous() for n in ns}, str(tmp_path / f))
    (tmp_path / "model.safetensors.index.json").write_text(
        json.dumps({"metadata": {}, "weight_map": {n: f for f, ns in shards.items() for n in ns}}))
    m = Model(config_from_dict(cfg).to_spec())
    r = CheckpointReader(tmp_path)
    r.check(m.tensor_specs(), m.ignorable_tensors())
    assert torch.equal(r.get(names[0]), w[names[0]]) and torch.equal(r.get(names[-1]), w[names[-1]])
    (tmp_path / "model-00002-of-00002.safetensors").unlink()
    with pytest.raises(WeightsError, match="model-00002-of-00002.safetensors, named by model.safetensors.index.json"):
        CheckpointReader(tmp_path)


def test_tied_head_ignores_its_own_copy_and_untied_needs_it(tmp_path):
    cfg = TINY["A"]
    w = plain_random_weights(cfg, 0)
    w["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    write_plain_model(tmp_path / "tied", cfg, w)
    m = Model(config_from_dict(cfg).to_spec())
    CheckpointReader(tmp_path / "tied").check(m.tensor_specs(), m.ignorable_tensors())
    cfg_b = TINY["B"]
    w = plain_random_weights(cfg_b, 0)
    del w["lm_head.weight"]
    write_plain_model(tmp_path / "untied", cfg_b, w)
    m = Model(config_from_dict(cfg_b).to_spec())
    with pytest.raises(WeightsError, match="lm_head.weight"):
        CheckpointReader(tmp_path / "untied").check(m.tensor_specs())
    with pytest.raises(WeightsError, match="safetensors"):
        CheckpointReader(tmp_path / "empty")


def test_kept_types():
    """Matrices in the run's type, vectors in float, integer tables as int32, a 32-bit tensor that asks to stay so stays."""
    bf = torch.randn(4, 4).bfloat16()
    f32 = torch.randn(4, 4)
    assert place(bf, TensorSpec("a", (4, 4)), torch.bfloat16, "cpu").dtype == torch.bfloat16
    assert torch.equal(place(bf, TensorSpec("a", (4, 4)), torch.float32, "cpu"), bf.float())
    assert place(f32, TensorSpec("a", (4, 4)), torch.bfloat16, "cpu").dtype == torch.bfloat16
    assert place(f32, TensorSpec("a", (4, 4), keep32=True), torch.bfloat16, "cpu").dtype == torch.float32
    assert place(bf[0], TensorSpec("b", (4,), "bias"), torch.bfloat16, "cpu").dtype == torch.float32
    assert place(bf[0], TensorSpec("n", (4,), "norm"), torch.bfloat16, "cpu").dtype == torch.float32
    assert place(torch.arange(4), TensorSpec("t", (4,), "table"), torch.bfloat16, "cpu").dtype == torch.int32


def test_a_layer_names_its_parts_and_the_arrangement_says_which_it_takes():
    """``LayerSpec(block, parts)``: the arrangement builds the parts it names; a part it does not take, or a missing
    one, is an error that names it; a position encoding is optional and goes to the mixer."""
    from llm_infrence_engine_amd.config import layer, preset
    from llm_infrence_engine_amd.parts import CacheNeed, KVNeed, PageTensor

    spec = config_from_dict(preset("tinyA")).to_spec()
    ls = spec.layers[0]
    assert ls.block == "pre_norm_residual" and sorted(ls.parts) == ["feed_forward", "feed_forward_norm", "mixer",
                                                                    "mixer_norm", "position"]
    assert ls.mixer.kind == "gqa_attention" and ls.parts.get("no_such_part") is None
    with pytest.raises(AttributeError, match="no part named 'mixr'"):     # a misspelt name is an error, not None
        ls.mixr
    with pytest.raises(TypeError):
        ls.parts["mixer"] = ls.mixer                                       # the spec is read-only
    assert hash(spec) == hash(config_from_dict(preset("tinyA")).to_spec()) and spec == config_from_dict(preset("tinyA")).to_spec()
    block = Model(spec).layers[0]
    assert block.mixer.position is block.position and [type(p).__name__ for p in block.parts()] == \
        ["RMSNorm", "GQAttention", "RMSNorm", "SwiGLU"]
    # what a mixer declares does not depend on whether it is loaded or in which type: values may be kept
    # transposed for pages of a multiple of 16 tokens in bfloat16, and the pool decides
    need = CacheNeed((PageTensor("k", 2, 16), PageTensor("v", 2, 16, 16, torch.bfloat16)), None)
    assert block.cache_need() == need == KVNeed(2, 16, None, 16, torch.bfloat16)
    assert block.state_need() is None and block.graph_safe()

    def model_with(parts):
        return Model(ModelSpec(spec.architecture, spec.hidden_size, spec.vocab_size, spec.embedding,
                               (layer("pre_norm_residual", **parts),), (Run(0),), spec.final_norm, spec.head))

    parts = dict(ls.parts)
    with pytest.raises(KeyError, match="post_norm"):
        model_with({**parts, "post_norm": parts["mixer_norm"]})
    with pytest.raises(KeyError, match="feed_forward_norm"):
        model_with({k: v for k, v in parts.items() if k != "feed_forward_norm"})
    no_position = model_with({k: v for k, v in parts.items() if k != "position"})
    assert no_position.layers[0].position is None and no_position.layers[0].mixer.position is None
    assert no_position.spec.layers[0].parts.get("position") is None
    with pytest.raises(ValueError, match="each name once"):
        CacheNeed((PageTensor("k", 1, 8), PageTensor("k", 1, 8)))
