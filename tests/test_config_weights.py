"""Configuration, registry, weight loading errors and the random-weights folder (no GPU)."""

import json
import os

import pytest
import torch

import tiny_models as tm
from miniinfer_amd.config import (ConfigError, EngineConfig, Qwen3Config, load_model_config, model_spec_of,
                                  resolve_architecture)
from miniinfer_amd.weights import (WeightsError, build_model, load_model, load_weights, write_random_model,
                                   write_safetensors, SafetensorsFile)


def test_config_reads_its_own_keys():
  cfg = Qwen3Config.from_dict(tm.TINY_B)
  assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim) == \
      (3, 96, 8, 2, 32)
  assert cfg.rms_norm_eps == 1e-5 and cfg.rope_theta == 1e6 and cfg.tie_word_embeddings is False
  spec = model_spec_of(cfg)
  assert len(spec.layers) == 3 and spec.run_order == (0, 1, 2)
  m = spec.layers[1].mixer
  assert (m.num_heads, m.num_kv_heads, m.head_dim, m.window) == (8, 2, 32, None)
  assert m.scale == 32 ** -0.5 and m.qk_norm.eps == 1e-5 and m.position.theta == 1e6
  assert spec.layers[0].feed_forward.intermediate_size == 160


def test_config_defaults_of_the_reference():
  raw = dict(tm.TINY_A)
  del raw["head_dim"]
  raw["num_key_value_heads"] = None
  cfg = Qwen3Config.from_dict(raw)
  assert cfg.head_dim == 64 // 4 and cfg.num_key_value_heads == 4   # qwen3.py:46-48,75-79


@pytest.mark.parametrize("change,match", [
  (dict(hidden_act="gelu"), "hidden_act"), (dict(attention_bias=True), "attention_bias"),
  (dict(rope_scaling={"rope_type": "yarn", "factor": 4}), "rope_scaling"),
  (dict(num_key_value_heads=3), "multiple"), (dict(head_dim=15), "even"), (dict(vocab_size=0), "positive")])
def test_config_refuses_what_it_cannot_honour(change, match):
  raw = dict(tm.TINY_A)
  raw.update(change)
  with pytest.raises(ConfigError, match=match):
    Qwen3Config.from_dict(raw)


def test_config_missing_key():
  raw = dict(tm.TINY_A)
  del raw["intermediate_size"]
  with pytest.raises(ConfigError, match="intermediate_size"):
    Qwen3Config.from_dict(raw)


def test_sliding_window_layers():
  raw = dict(tm.TINY_B, use_sliding_window=True, sliding_window=24, max_window_layers=1)
  cfg = Qwen3Config.from_dict(raw)
  assert cfg.layer_windows == (None, 24, 24)
  raw = dict(tm.TINY_B, sliding_window=16, layer_types=["sliding_attention", "full_attention", "sliding_attention"])
  cfg = Qwen3Config.from_dict(raw)
  assert cfg.layer_windows == (16, None, 16)
  assert Qwen3Config.from_dict(cfg.to_dict()) == cfg


def test_registry():
  name, cls = resolve_architecture({"architectures": ["Qwen3ForCausalLM"]})
  assert name == "Qwen3ForCausalLM" and cls is Qwen3Config
  assert resolve_architecture({"model_type": "qwen3"})[1] is Qwen3Config
  with pytest.raises(ValueError, match="Qwen3ForCausalLM"):
    resolve_architecture({"architectures": ["LlamaForCausalLM"], "model_type": "llama"})


def test_engine_config_rejects_unknown_and_bad_values():
  with pytest.raises(TypeError, match="unknown engine option"):
    EngineConfig.from_kwargs("x", max_modle_len=3)
  assert EngineConfig.from_kwargs("x", max_context_len=77).max_model_len == 77    # the reference's field name
  with pytest.raises(ValueError, match="power of two"):
    EngineConfig(model_path="x", page_size=24)
  with pytest.raises(ValueError, match="dtype"):
    EngineConfig(model_path="x", dtype="float16")
  assert EngineConfig(model_path="x", dtype=torch.bfloat16).dtype == "bfloat16"


def test_load_by_name_fuses_and_keeps_dtypes(tmp_path):
  cfg, w = tm.make_model(str(tmp_path), "B", seed=1, dtype=torch.bfloat16)
  model, mc = load_model(str(tmp_path), torch.bfloat16, "cpu")
  att = model.blocks[2].mixer
  p = "model.layers.2.self_attn."
  assert torch.equal(att.qkv_weight, torch.cat([w[p + "q_proj.weight"], w[p + "k_proj.weight"], w[p + "v_proj.weight"]]))
  ff = model.blocks[0].feed_forward
  assert torch.equal(ff.gate_up_weight, torch.cat([w["model.layers.0.mlp.gate_proj.weight"],
                                                   w["model.layers.0.mlp.up_proj.weight"]]))
  assert att.qkv_weight.dtype == torch.bfloat16 and model.embedding.dtype == torch.bfloat16
  assert att.q_norm.weight.dtype == torch.float32          # norm weights are held in 32-bit
  assert torch.equal(att.q_norm.weight, w[p + "q_norm.weight"].float())
  assert torch.equal(model.head, w["lm_head.weight"])
  # the 32-bit mode widens a bfloat16 file exactly
  model32, _ = load_model(str(tmp_path), torch.float32, "cpu")
  assert model32.embedding.dtype == torch.float32 and torch.equal(model32.embedding, w["model.embed_tokens.weight"].float())


def test_tied_head_is_an_alias_and_prefix_is_optional(tmp_path):
  cfg, w = tm.make_model(str(tmp_path / "a"), "A", seed=1)
  model, _ = load_model(str(tmp_path / "a"), torch.float32, "cpu")
  assert model.head is None      # the forward pass uses the embedding table itself: no second copy
  # untied configuration whose file has no lm_head: falls back to the table (layers/embedding.py:41-48)
  cfgb, wb = tm.make_model(str(tmp_path / "b"), "B", seed=1)
  wb.pop("lm_head.weight")
  tm.write_model(str(tmp_path / "b"), cfgb, wb)
  assert load_model(str(tmp_path / "b"), torch.float32, "cpu")[0].head is None
  # names without the "model." prefix (models/fused_qwen3.py:225-226)
  w2 = {(k[len("model."):] if k.startswith("model.") else k): v for k, v in w.items()}
  tm.write_model(str(tmp_path / "c"), cfg, w2)
  m2, _ = load_model(str(tmp_path / "c"), torch.float32, "cpu")
  assert torch.equal(m2.embedding, w["model.embed_tokens.weight"])


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
  cfg, w = tm.make_model(str(tmp_path), "A", seed=1)
  w.pop("model.layers.1.self_attn.k_proj.weight")
  w.pop("model.norm.weight")
  w["model.layers.0.mlp.extra.weight"] = torch.zeros(3)
  w["model.layers.0.self_attn.o_proj.weight"] = torch.zeros(64, 63)
  w["model.layers.1.self_attn.q_norm.weight"] = torch.zeros(8)
  tm.write_model(str(tmp_path), cfg, w)
  with pytest.raises(WeightsError) as ei:
    load_model(str(tmp_path), torch.float32, "cpu")
  e = ei.value
  assert e.missing == ["model.layers.1.self_attn.k_proj.weight", "model.norm.weight"]
  assert e.unexpected == ["model.layers.0.mlp.extra.weight"]
  assert [n for n, _, _ in e.wrong_shape] == ["model.layers.0.self_attn.o_proj.weight",
                                              "model.layers.1.self_attn.q_norm.weight"]
  msg = str(e)
  for needle in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (2)", "(64, 63)", "(64, 64)"):
    assert needle in msg


def test_no_files_and_no_config(tmp_path):
  with pytest.raises(FileNotFoundError, match="config.json"):
    load_model_config(str(tmp_path))
  with open(tmp_path / "config.json", "w") as f:
    json.dump(tm.TINY_A, f)
  with pytest.raises(FileNotFoundError, match="safetensors"):
    load_model(str(tmp_path), torch.float32, "cpu")


def test_random_weights_folder_round_trip(tmp_path):
  cfg = Qwen3Config.from_dict(tm.TINY_B)
  write_random_model(cfg, str(tmp_path / "r1"), seed=5, dtype=torch.bfloat16)
  write_random_model(cfg, str(tmp_path / "r2"), seed=5, dtype=torch.bfloat16)
  write_random_model(cfg, str(tmp_path / "r3"), seed=6, dtype=torch.bfloat16)
  assert load_model_config(str(tmp_path / "r1")) == Qwen3Config.from_dict(dict(tm.TINY_B, torch_dtype="bfloat16"))
  from safetensors import safe_open   # the library reads what the engine's writer wrote
  with safe_open(str(tmp_path / "r1" / "model.safetensors"), "pt") as f:
    names = set(f.keys())
    emb = f.get_tensor("model.embed_tokens.weight")
    nw = f.get_tensor("model.layers.0.input_layernorm.weight")
  assert "lm_head.weight" in names and "model.layers.2.self_attn.k_norm.weight" in names
  assert len(names) == 2 + 1 + 3 * 11
  assert emb.dtype == torch.bfloat16 and abs(float(emb.float().std()) - 0.02) < 2e-3
  assert abs(float(nw.float().mean()) - 1.0) < 0.05
  m1, _ = load_model(str(tmp_path / "r1"), torch.bfloat16, "cpu")
  m2, _ = load_model(str(tmp_path / "r2"), torch.bfloat16, "cpu")
  m3, _ = load_model(str(tmp_path / "r3"), torch.bfloat16, "cpu")
  assert torch.equal(m1.blocks[1].mixer.qkv_weight, m2.blocks[1].mixer.qkv_weight)
  assert not torch.equal(m1.blocks[1].mixer.qkv_weight, m3.blocks[1].mixer.qkv_weight)
  # a tied configuration writes no head
  cfga = Qwen3Config.from_dict(tm.TINY_A)
  write_random_model(cfga, str(tmp_path / "ra"), seed=1, dtype=torch.float32)
  assert "lm_head.weight" not in SafetensorsFile(str(tmp_path / "ra" / "model.safetensors")).keys()


def test_safetensors_reader_refuses_broken_files(tmp_path):
  p = tmp_path / "x.safetensors"
  write_safetensors(str(p), [("a", torch.arange(6, dtype=torch.int32).reshape(2, 3)), ("b", torch.ones(4, dtype=torch.bfloat16))])
  f = SafetensorsFile(str(p))
  assert f.shape("a") == (2, 3) and torch.equal(f.tensor("a"), torch.arange(6, dtype=torch.int32).reshape(2, 3))
  assert f.tensor("b").dtype == torch.bfloat16
  raw = p.read_bytes()
  (tmp_path / "short.safetensors").write_bytes(raw[:-3])
  with pytest.raises(ValueError, match="data_offsets"):
    SafetensorsFile(str(tmp_path / "short.safetensors"))
  (tmp_path / "tiny.safetensors").write_bytes(b"abc")
  with pytest.raises(ValueError, match="not a safetensors"):
    SafetensorsFile(str(tmp_path / "tiny.safetensors"))


def test_eos_of_generation_config(tmp_path):
  """generation_config.json names the end-of-sequence id (one or several); without the file there is none."""
  from miniinfer_amd.engine.llm_engine import LLMEngine
  d = tmp_path / "m"
  d.mkdir()
  assert LLMEngine._eos_of_folder(str(d)) is None
  (d / "generation_config.json").write_text(json.dumps({"eos_token_id": [7, 9], "temperature": 0.6}))
  assert LLMEngine._eos_of_folder(str(d)) == [7, 9]
  (d / "generation_config.json").write_text(json.dumps({"eos_token_id": 11}))
  assert LLMEngine._eos_of_folder(str(d)) == 11
  (d / "generation_config.json").write_text(json.dumps({"do_sample": True}))
  assert LLMEngine._eos_of_folder(str(d)) is None


def test_sampling_params_checks():
  from miniinfer_amd import SamplingParams
  sp = SamplingParams(stop_token_ids=(3, 5))
  assert sp.stop_token_ids == [3, 5] and SamplingParams().stop_token_ids == []
  for bad in (dict(temperature=-1), dict(max_tokens=0), dict(top_k=-1), dict(top_p=0.0), dict(stop_token_ids=[-2])):
    with pytest.raises(ValueError):
      SamplingParams(**bad)


def test_built_kernels_are_not_loaded_from_a_folder_others_can_write(tmp_path, monkeypatch):
  """The fallback folder for built kernels lies under the shared temp dir: it is used only when it belongs to
  this user and nobody else may write to it."""
  import tempfile
  from miniinfer_amd.kernels import jit
  monkeypatch.setattr(tempfile, "tempdir", str(tmp_path))
  shared = tmp_path / "shared"
  shared.mkdir()
  os.chmod(shared, 0o777)
  assert not jit._private_temp_dir(str(shared))
  mine = tmp_path / "mine"
  assert jit._private_temp_dir(str(mine)) and (os.stat(mine).st_mode & 0o777) == 0o700
  link = tmp_path / "link"
  os.symlink(shared, link)
  assert not jit._private_temp_dir(str(link))
  # the fallback of build_dirs() is refused as a place to write when someone else prepared it
  monkeypatch.delenv("MINIINFER_AMD_BUILD_DIR", raising=False)
  fallback = jit.build_dirs()[-1]
  assert fallback.startswith(str(tmp_path))
  os.makedirs(fallback)
  os.chmod(fallback, 0o777)
  assert not jit._usable(fallback)


def test_model_frame_options_are_data_of_the_spec():
  """The frame around the blocks (embedding factor, learned positions, logit factor and cap) is chosen by fields of
  the spec, and another frame class by its kind."""
  import dataclasses
  from miniinfer_amd.parts import FRAMES, BuildContext
  spec = model_spec_of(Qwen3Config.from_dict(tm.TINY_A))
  assert spec.kind == "decoder" and spec.embedding_scale == 1.0 and spec.logit_softcap is None
  spec2 = dataclasses.replace(spec, position_table_name="model.positions.weight", embedding_scale=8.0,
                              logit_softcap=30.0)
  model = FRAMES.build(spec2, BuildContext(device=torch.device("cpu"), dtype=torch.float32))
  names = {prefix + src.name for prefix, _, ps in model.named_params() for src in ps.sources}
  assert "model.positions.weight" in names
  with pytest.raises(KeyError, match="model frame"):
    FRAMES.build(dataclasses.replace(spec, kind="no_such_frame"), BuildContext(torch.device("cpu"), torch.float32))
  with pytest.raises(ValueError, match="logit_softcap"):
    FRAMES.build(dataclasses.replace(spec, logit_softcap=0.0), BuildContext(torch.device("cpu"), torch.float32))
  assert model.is_capturable()
