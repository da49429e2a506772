"""Configuration, registry, safetensors container, loader errors, random weights."""
import json
import os

import pytest
import torch

import helpers as H
from llm_inference_lab_amd.config import (ConfigError, WeightError, Qwen2Config, read_config,
                                          registered_architectures, get_architecture)
from llm_inference_lab_amd.weights import (TensorSpec, VECTOR, MATRIX, INT_TABLE, load_tensors,
                                           save_safetensors, ModelFiles, kept_dtype)
from llm_inference_lab_amd import write_random_model


def test_config_reads_every_size_from_the_file():
    cfg = Qwen2Config.from_dict(dict(H.TINY_B))
    assert (cfg.vocab_size, cfg.hidden_size, cfg.intermediate_size, cfg.num_hidden_layers) == (515, 96, 320, 3)
    assert (cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim) == (3, 1, 32)
    assert cfg.rms_norm_eps == 1e-5 and cfg.rope_theta == 1e6 and not cfg.tie_word_embeddings
    assert cfg.eos_token_ids == (3, 4)
    assert [cfg.layer_window(i) for i in range(3)] == [None, 24, 24]
    assert Qwen2Config.from_dict(cfg.to_dict()) == cfg        # round trip through config.json


def test_head_dim_defaults_to_hidden_over_heads_and_may_differ():
    raw = dict(H.TINY_A)
    raw.pop("head_dim")
    assert Qwen2Config.from_dict(raw).head_dim == 16
    assert H.config_of("C").head_dim * H.config_of("C").num_attention_heads != H.config_of("C").hidden_size


def test_window_needs_the_switch():
    raw = dict(H.TINY_B, use_sliding_window=False)
    cfg = Qwen2Config.from_dict(raw)
    assert all(cfg.layer_window(i) is None for i in range(3))


@pytest.mark.parametrize("change,message", [
    (dict(hidden_size=None), "hidden_size"),
    (dict(rms_norm_eps=0.0), "rms_norm_eps"),
    (dict(rope_theta=-1.0), "rope_theta"),
    (dict(num_key_value_heads=3), "multiple"),
    (dict(hidden_act="gelu"), "hidden_act"),
    (dict(rope_scaling={"type": "yarn"}), "rope_scaling"),
    (dict(model_type="llama"), "model_type"),
    (dict(vocab_size="many"), "vocab_size"),
    (dict(use_sliding_window=True, sliding_window=None), "sliding_window"),
    (dict(tie_word_embeddings="yes"), "tie_word_embeddings"),
])
def test_config_errors_name_the_key(change, message):
    raw = dict(H.TINY_A)
    raw.update(change)
    with pytest.raises(ConfigError, match=message):
        Qwen2Config.from_dict(raw)


def test_registry_selects_by_architecture_name(tmp_path):
    assert "Qwen2ForCausalLM" in registered_architectures()
    (tmp_path / "config.json").write_text(json.dumps(H.TINY_A))
    arch, cfg = read_config(str(tmp_path))
    assert arch.name == "Qwen2ForCausalLM" and isinstance(cfg, Qwen2Config)
    (tmp_path / "config.json").write_text(json.dumps(dict(H.TINY_A, architectures=["NoSuchModel"])))
    with pytest.raises(ConfigError, match="unknown architecture 'NoSuchModel'.*Qwen2ForCausalLM"):
        read_config(str(tmp_path))


def test_spec_is_data_layer_by_layer():
    cfg = H.config_of("B")
    spec = get_architecture(cfg.architecture).build_spec(cfg)
    assert len(spec.blocks) == 3 and [e.block for e in spec.schedule] == [0, 1, 2]
    assert [b.parts["mixer"].params["window"] for b in spec.blocks] == [None, 24, 24]
    assert spec.head.tensors["weight"] == "lm_head.weight"
    tied = get_architecture("Qwen2ForCausalLM").build_spec(H.config_of("A"))
    assert tied.head.tensors["weight"] == tied.embedding.tensors["weight"]
    assert "lm_head.weight" not in H.expected_tensors(H.config_of("A"))


def test_safetensors_round_trip_keeps_bits(tmp_path):
    specials = torch.tensor([0.0, -0.0, float("inf"), float("-inf"), float("nan"), 1e-40, 1.5])
    tensors = {"a": specials.to(torch.bfloat16), "b": specials.clone(), "c": torch.arange(6, dtype=torch.int32).view(2, 3),
               "empty": torch.zeros(0, 4)}
    path = str(tmp_path / "model.safetensors")
    save_safetensors(path, tensors.items(), {"k": "v"})
    files = ModelFiles(str(tmp_path))
    assert sorted(files.names()) == sorted(tensors)
    for name, t in tensors.items():
        back = files.tensor(name)
        assert back.dtype == t.dtype and tuple(back.shape) == tuple(t.shape)
        assert torch.equal(back.view(torch.uint8), t.contiguous().view(torch.uint8))
    files.close()


def test_sharded_folder_reads_like_a_single_file(tmp_path):
    a, b = torch.randn(3, 4), torch.randn(5)
    save_safetensors(str(tmp_path / "s1.safetensors"), [("a", a)])
    save_safetensors(str(tmp_path / "s2.safetensors"), [("b", b)])
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}))
    files = ModelFiles(str(tmp_path))
    assert torch.equal(files.tensor("a"), a) and torch.equal(files.tensor("b"), b)
    files.close()
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {"a": "../s1.safetensors"}}))
    with pytest.raises(ValueError, match="plain"):
        ModelFiles(str(tmp_path))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = H.config_of("A")
    tensors = H.make_tensors(cfg, 0)
    del tensors["model.norm.weight"]
    del tensors["model.layers.1.mlp.up_proj.weight"]
    tensors["lm_head.weight"] = torch.zeros(256, 64, dtype=torch.bfloat16)     # tied: not expected
    tensors["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(63, dtype=torch.bfloat16)
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(64, 32, dtype=torch.bfloat16)
    save_safetensors(str(tmp_path / "model.safetensors"), tensors.items())
    with pytest.raises(WeightError) as err:
        load_tensors(str(tmp_path), H.expected_tensors(cfg), torch.float32, "cpu")
    e = err.value
    assert e.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["lm_head.weight"]
    assert sorted(n for n, _, _ in e.wrong_shape) == ["model.layers.0.self_attn.k_proj.weight",
                                                      "model.layers.0.self_attn.q_proj.bias"]
    text = str(e)
    for piece in ("missing (2)", "unexpected (1)", "wrong shape (2)", "model.norm.weight",
                  "expected [32, 64] found [64, 32]"):
        assert piece in text


def test_tensors_the_model_does_not_use_are_left_unread(tmp_path):
    """A file that holds all the model needs and more loads (the reference ignores extra
    tensors, rust/engine/src/runner/loader.rs:218): the extra names are reported, and an
    error only where the caller asks for strictness."""
    cfg = H.config_of("A")
    tensors = H.make_tensors(cfg, 0)
    tensors["lm_head.weight"] = torch.zeros(256, 64, dtype=torch.bfloat16)     # tied: not used
    tensors["model.rotary_emb.inv_freq"] = torch.zeros(8)
    save_safetensors(str(tmp_path / "model.safetensors"), tensors.items())
    said = []
    loaded = load_tensors(str(tmp_path), H.expected_tensors(cfg), torch.float32, "cpu", progress=said.append)
    assert sorted(loaded) == sorted(H.expected_tensors(cfg))
    assert any("lm_head.weight" in line and "left unread" in line for line in said)
    with pytest.raises(WeightError) as err:
        load_tensors(str(tmp_path), H.expected_tensors(cfg), torch.float32, "cpu", strict=True)
    assert err.value.unexpected == ["lm_head.weight", "model.rotary_emb.inv_freq"] and not err.value.missing


def test_kept_dtypes():
    bf, f32 = torch.bfloat16, torch.float32
    assert kept_dtype(MATRIX, bf, bf) == bf and kept_dtype(MATRIX, f32, bf) == bf
    assert kept_dtype(VECTOR, bf, bf) == bf
    assert kept_dtype(VECTOR, f32, bf) == f32          # stored in 32 bits: stays so
    assert kept_dtype(VECTOR, torch.float16, bf) == f32
    assert kept_dtype(INT_TABLE, torch.int64, bf) == torch.int32
    assert kept_dtype(MATRIX, bf, f32) == f32 and kept_dtype(VECTOR, bf, f32) == f32


def test_integer_tensor_is_refused_for_a_weight(tmp_path):
    cfg = H.config_of("A")
    tensors = H.make_tensors(cfg, 0)
    tensors["model.norm.weight"] = torch.ones(64, dtype=torch.int32)
    save_safetensors(str(tmp_path / "model.safetensors"), tensors.items())
    with pytest.raises(WeightError, match="wrong dtype"):
        load_tensors(str(tmp_path), H.expected_tensors(cfg), torch.float32, "cpu")


def test_random_model_folder_is_reproducible_and_loads(tmp_path):
    cfg = H.config_of("B")
    d1 = write_random_model(str(tmp_path / "m1"), cfg, seed=5)
    d2 = write_random_model(str(tmp_path / "m2"), cfg, seed=5)
    d3 = write_random_model(str(tmp_path / "m3"), cfg, seed=6)
    assert sorted(os.listdir(d1)) == ["config.json", "model.safetensors"]
    b1, b2, b3 = (open(os.path.join(d, "model.safetensors"), "rb").read() for d in (d1, d2, d3))
    assert b1 == b2 and b1 != b3
    arch, back = read_config(d1)
    assert back == cfg
    loaded = load_tensors(d1, H.expected_tensors(cfg), torch.bfloat16, "cpu")
    assert set(loaded) == set(H.expected_tensors(cfg))
    norm = loaded["model.norm.weight"].float()
    assert abs(norm.mean().item() - 1.0) < 0.05 and 0.05 < norm.std().item() < 0.15
    w = loaded["model.layers.0.mlp.gate_proj.weight"].float()
    assert abs(w.mean().item()) < 2e-3 and abs(w.std().item() - 0.02) < 2e-3
    assert cfg.parameter_count() == sum(t.numel() for t in loaded.values())


def test_engine_without_gpu_fails_loudly():
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    with pytest.raises(RuntimeError, match="no GPU|hipcc"):
        H.lab.Engine(config=H.config_of("A"), dtype="f32")
