"""Configuration, registry and weight loading (CPU)."""

from __future__ import annotations

import json

import pytest
import torch

from pyre_amd.config import ConfigError, EngineConfig, Qwen2Config, preset
from pyre_amd.registry import (config_from_dict, get_architecture, known_architectures, load_config,
                               register_architecture, unregister_architecture)
from pyre_amd.weights import (WeightsError, adopt_state, checkpoint_index, load_weights, model_tensor_specs,
                              random_state, write_random_model)

RAW = {"architectures": ["Qwen2ForCausalLM"], "hidden_size": 64, "intermediate_size": 176,
       "num_hidden_layers": 2, "num_attention_heads": 4, "vocab_size": 512}


def test_defaults_are_the_references():
    """pyre/config.py:45-61: kv heads default to heads, eps 1e-6, theta 1e4, untied,
    32768 positions, head_dim = hidden // heads."""
    c = config_from_dict(RAW)
    assert isinstance(c, Qwen2Config)
    assert (c.num_key_value_heads, c.rms_norm_eps, c.rope_theta, c.tie_word_embeddings,
            c.max_position_embeddings, c.head_dim, c.n_rep) == (4, 1e-6, 1e4, False, 32768, 16, 1)
    assert config_from_dict({**RAW, "head_dim": 24}).q_dim == 96      # head_dim need not be hidden/heads
    assert config_from_dict({**RAW, "num_key_value_heads": 2}).n_rep == 2


@pytest.mark.parametrize("key", ["hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "vocab_size"])
def test_required_keys(key):
    raw = dict(RAW)
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        config_from_dict(raw)


@pytest.mark.parametrize("bad,match", [
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"use_sliding_window": True}, "sliding"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"),
    ({"rms_norm_eps": 0}, "rms_norm_eps"),
    ({"vocab_size": -5}, "vocab_size"),
    ({"hidden_size": "64"}, "hidden_size"),
])
def test_rejected_configs(bad, match):
    with pytest.raises(ConfigError, match=match):
        config_from_dict({**RAW, **bad})


def test_registry_is_exact():
    assert "Qwen2ForCausalLM" in known_architectures()
    for name in ("Qwen2MoeForCausalLM", "Qwen2", "LlamaForCausalLM"):   # pyre/config.py:38-43 would admit the first two
        with pytest.raises(ConfigError, match="unknown architecture"):
            get_architecture(name)
    with pytest.raises(ConfigError, match="architectures"):
        config_from_dict({k: v for k, v in RAW.items() if k != "architectures"})


def test_registering_another_architecture():
    register_architecture("ToyForCausalLM", Qwen2Config, get_architecture("Qwen2ForCausalLM").build)
    try:
        assert config_from_dict({**RAW, "architectures": ["ToyForCausalLM"]}).hidden_size == 64
    finally:
        unregister_architecture("ToyForCausalLM")


def test_config_round_trip(tmp_path):
    for name in ("tiny-a", "tiny-b", "qwen2.5-7b"):
        c = preset(name)
        c.save(tmp_path / name)
        assert load_config(tmp_path / name) == c
    with pytest.raises(FileNotFoundError):
        load_config(tmp_path / "nothing")


def test_presets_match_the_published_shapes():
    c = preset("qwen2.5-7b")
    assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim,
            c.intermediate_size, c.vocab_size, c.tie_word_embeddings) == (28, 3584, 28, 4, 128, 18944, 152064, False)
    n_params = sum(torch.Size(s.shape).numel() for s in model_tensor_specs(c) if s.alias_of is None)
    assert n_params == 7_615_616_512
    c = preset("qwen2.5-1.5b")
    assert sum(torch.Size(s.shape).numel() for s in model_tensor_specs(c) if s.alias_of is None) == 1_543_714_304


def test_engine_config_validation():
    assert EngineConfig(dtype="bf16").dtype == "bfloat16" and EngineConfig(dtype="fp32").dtype == "float32"
    with pytest.raises(ValueError):
        EngineConfig(dtype="float16")
    with pytest.raises(ValueError):
        EngineConfig(page_size=0)


# ----------------------------------------------------------------------------- weights

def test_manifest_names_are_the_checkpoints():
    """pyre/model.py:1-5,156-158: the names of a Qwen2 checkpoint."""
    names = {s.name: s.shape for s in model_tensor_specs(preset("tiny-b"))}
    assert names["model.embed_tokens.weight"] == (1000, 96)
    assert names["model.layers.2.self_attn.q_proj.weight"] == (96, 96)
    assert names["model.layers.2.self_attn.k_proj.bias"] == (24,)
    assert names["model.layers.0.self_attn.o_proj.weight"] == (96, 96)
    assert "model.layers.0.self_attn.o_proj.bias" not in names
    assert names["model.layers.1.mlp.gate_proj.weight"] == (256, 96)
    assert names["model.layers.1.mlp.down_proj.weight"] == (96, 256)
    assert names["model.layers.1.post_attention_layernorm.weight"] == (96,)
    assert names["model.norm.weight"] == (96,) and names["lm_head.weight"] == (1000, 96)
    assert len(names) == 3 * 12 + 3


def test_random_model_is_seeded_and_tied_head_is_left_out(tmp_path):
    a = write_random_model(tmp_path / "a", preset("tiny-a"), seed=0)
    b = write_random_model(tmp_path / "b", preset("tiny-a"), seed=0)
    c = write_random_model(tmp_path / "c", preset("tiny-a"), seed=1)
    ia = checkpoint_index(a)
    assert "lm_head.weight" not in ia            # tied: pyre/loader.py:58-61
    specs = model_tensor_specs(preset("tiny-a"))
    wa, wb, wc = (load_weights(d, specs, "cpu", torch.bfloat16) for d in (a, b, c))
    assert all(torch.equal(wa[k], wb[k]) for k in wa)
    assert not torch.equal(wa["model.embed_tokens.weight"], wc["model.embed_tokens.weight"])
    assert wa["lm_head.weight"].data_ptr() == wa["model.embed_tokens.weight"].data_ptr()
    assert torch.all(wa["model.norm.weight"] == 1)
    w = wa["model.layers.0.mlp.up_proj.weight"].float()
    assert abs(w.std().item() - 0.02) < 2e-3 and abs(w.mean().item()) < 1e-3


def test_element_types_follow_the_file(tmp_path):
    from safetensors.torch import save_file

    cfg = preset("tiny-a")
    specs = model_tensor_specs(cfg)
    state = random_state(specs, 0)
    state["model.norm.weight"] = state["model.norm.weight"].float()          # stored in 32 bits: stays so
    state["model.layers.0.self_attn.q_proj.bias"] = state["model.layers.0.self_attn.q_proj.bias"].half()
    cfg.save(tmp_path)
    save_file(state, str(tmp_path / "model.safetensors"))
    w16 = load_weights(tmp_path, specs, "cpu", torch.bfloat16)
    assert w16["model.norm.weight"].dtype == torch.float32
    assert w16["model.embed_tokens.weight"].dtype == torch.bfloat16
    assert w16["model.layers.0.self_attn.q_proj.bias"].dtype == torch.bfloat16
    w32 = load_weights(tmp_path, specs, "cpu", torch.float32)
    assert all(t.dtype == torch.float32 for t in w32.values())
    assert torch.equal(w32["model.embed_tokens.weight"], state["model.embed_tokens.weight"].float())


def test_one_error_lists_everything_that_is_wrong(tmp_path):
    from safetensors.torch import save_file

    cfg = preset("tiny-b")
    specs = model_tensor_specs(cfg)
    state = random_state(specs, 0)
    del state["model.layers.1.mlp.up_proj.weight"]
    del state["lm_head.weight"]                                   # untied: missing, not aliased
    state["model.layers.7.mlp.up_proj.weight"] = torch.zeros(2, 2)
    state["model.norm.weight"] = torch.zeros(95)
    state["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(96, 24)   # transposed
    cfg.save(tmp_path)
    save_file(state, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        load_weights(tmp_path, specs, "cpu", torch.bfloat16)
    err = e.value
    assert set(err.missing) == {"model.layers.1.mlp.up_proj.weight", "lm_head.weight"}
    assert err.unexpected == ["model.layers.7.mlp.up_proj.weight"]
    assert {n for n, _, _ in err.wrong_shape} == {"model.norm.weight", "model.layers.0.self_attn.k_proj.weight"}
    msg = str(err)
    for piece in ("missing", "unexpected", "wrong shape", "lm_head.weight", "(96, 24)", "(24, 96)"):
        assert piece in msg
    with pytest.raises(WeightsError):
        adopt_state(state, specs, "cpu", torch.float32)


def test_wrong_class_of_element_type_is_named(tmp_path):
    """Integers under a weight's name are refused at load, by name, in the same one error
    as everything else that is wrong (not later, inside a kernel call)."""
    from safetensors.torch import save_file

    cfg = preset("tiny-b")
    specs = model_tensor_specs(cfg)
    state = random_state(specs, 0)
    state["model.layers.2.mlp.down_proj.weight"] = torch.zeros(96, 256, dtype=torch.int64)
    state["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(96, dtype=torch.int8)
    state["model.norm.weight"] = torch.zeros(95)
    cfg.save(tmp_path)
    save_file(state, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        load_weights(tmp_path, specs, "cpu", torch.bfloat16)
    assert {n for n, _, _ in e.value.wrong_dtype} == {"model.layers.2.mlp.down_proj.weight",
                                                      "model.layers.0.self_attn.q_proj.bias"}
    assert [n for n, _, _ in e.value.wrong_shape] == ["model.norm.weight"]
    assert "wrong element type" in str(e.value) and "I64" in str(e.value) and "floating-point" in str(e.value)
    with pytest.raises(WeightsError) as e2:
        adopt_state(state, specs, "cpu", torch.float32)
    assert len(e2.value.wrong_dtype) == 2


def test_tied_head_that_the_file_also_holds_must_equal_the_embedding(tmp_path):
    from safetensors.torch import save_file

    cfg = preset("tiny-a")                                       # tie_word_embeddings
    specs = model_tensor_specs(cfg)
    state = random_state(specs, 0)
    assert "lm_head.weight" not in state
    state["lm_head.weight"] = state["model.embed_tokens.weight"].clone()
    cfg.save(tmp_path)
    save_file(state, str(tmp_path / "model.safetensors"))
    w = load_weights(tmp_path, specs, "cpu", torch.bfloat16)      # equal: accepted, and one memory
    assert w["lm_head.weight"].data_ptr() == w["model.embed_tokens.weight"].data_ptr()
    state["lm_head.weight"][3, 5] += 1.0
    save_file(state, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        load_weights(tmp_path, specs, "cpu", torch.bfloat16)
    assert e.value.tied_mismatch == [("lm_head.weight", "model.embed_tokens.weight")]
    assert "tied but different" in str(e.value)
    with pytest.raises(WeightsError):
        adopt_state(state, specs, "cpu", torch.float32)


def test_no_safetensors(tmp_path):
    preset("tiny-a").save(tmp_path)
    with pytest.raises(FileNotFoundError, match="safetensors"):      # pyre/loader.py:47-48
        load_weights(tmp_path, model_tensor_specs(preset("tiny-a")), "cpu", torch.float32)


def test_sharded_checkpoint(tmp_path):
    from safetensors.torch import save_file

    cfg = preset("tiny-a")
    specs = model_tensor_specs(cfg)
    state = random_state(specs, 3)
    names = sorted(state)
    cfg.save(tmp_path)
    save_file({n: state[n] for n in names[::2]}, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({n: state[n] for n in names[1::2]}, str(tmp_path / "model-00002-of-00002.safetensors"))
    w = load_weights(tmp_path, specs, "cpu", torch.bfloat16)
    assert all(torch.equal(w[n], state[n]) for n in names)


def test_model_spec_is_data():
    """Layers are descriptions chosen per layer; the order of layers is a list."""
    from pyre_amd.parts.base import AttentionSpec, SwiGLUSpec

    spec = get_architecture("Qwen2ForCausalLM").build(preset("tiny-b"))
    assert len(spec.layers) == 3 and [c.layer for c in spec.schedule] == [0, 1, 2]
    assert all(isinstance(b.mixer, AttentionSpec) and isinstance(b.feed_forward, SwiGLUSpec) for b in spec.layers)
    assert spec.layers[1].mixer.position.theta == 1e6 and spec.layers[1].mixer_norm.eps == 1e-5
    assert spec.head.tied_to is None
    assert get_architecture("Qwen2ForCausalLM").build(preset("tiny-a")).head.tied_to == "model.embed_tokens.weight"
    json.dumps(preset("tiny-a").to_dict())


def test_sizes_that_no_kernel_takes_are_refused_when_the_model_is_built():
    """A head of more than 256 elements is refused by the attention part's constructor, before
    any weight is read (no attention kernel takes it), with a message that names the size."""
    from pyre_amd.parts.model import LayeredModel

    cfg = config_from_dict({"architectures": ["Qwen2ForCausalLM"], "hidden_size": 64, "intermediate_size": 32,
                            "num_hidden_layers": 1, "num_attention_heads": 2, "vocab_size": 50, "head_dim": 288})
    with pytest.raises(ValueError, match="head_dim 288 is outside 1..256"):
        LayeredModel(get_architecture(cfg.architecture).build(cfg))
    ok = config_from_dict({"architectures": ["Qwen2ForCausalLM"], "hidden_size": 64, "intermediate_size": 32,
                           "num_hidden_layers": 1, "num_attention_heads": 2, "vocab_size": 50, "head_dim": 256})
    assert LayeredModel(get_architecture(ok.architecture).build(ok)).cache_specs()[0][0].tensors[0].token_shape == (2, 256)


def test_parts_take_their_tensors_and_let_the_originals_go():
    """Binding empties the dictionary it is given, and a tensor that its part copies (the fused
    q/k/v and gate/up weights) is dropped as soon as it has been copied: nothing but the model
    holds the weights afterwards."""
    import weakref

    from pyre_amd.parts.base import TensorBag, take
    from pyre_amd.parts.model import LayeredModel

    cfg = preset("tiny-b")
    model = LayeredModel(get_architecture(cfg.architecture).build(cfg))
    state = random_state(model.tensor_specs(), 0, dtype="float32")
    refs = {n: weakref.ref(t) for n, t in state.items()}
    model.bind(state, None)
    assert state == {}
    fused = [n for n in refs if any(k in n for k in ("q_proj", "k_proj", "v_proj", "gate_proj", "up_proj"))]
    assert len(fused) == 3 * 8 and all(refs[n]() is None for n in fused)           # copied, then let go
    assert refs["model.layers.0.mlp.down_proj.weight"]() is model.layers[0].feed_forward.down.weight
    # a tensor that two parts name stays until the second has it
    bag = TensorBag({"w": 1, "v": 2}, {"w": 2, "v": 1})
    assert take(bag, "w") == 1 and "w" in bag and take(bag, "w") == 1 and "w" not in bag
    assert take(bag, "v") == 2 and not bag and take({"x": 3}, "x") == 3
