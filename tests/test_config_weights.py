"""Configuration, registry, weights: reading, errors, the random-weights folder."""
import json
import os
import warnings

import pytest
import torch

from tiny_configs import ALL, TINY_A, TINY_B
from yalis_amd.config.reader import ConfigError
from yalis_amd.config.registry import get_architecture, known_architectures, load_model_config
from yalis_amd.config.runtime import EngineConfig, InferenceConfig, ModelConfig
from yalis_amd.engine.factory import spec_from_config, tensor_specs_for
from yalis_amd.models.llama import LlamaConfig
from yalis_amd.weights.loader import TensorSpec, WeightsError, open_tensors, target_dtype


def load_tensors(folder, specs, engine_dtype, device, wide_tensors="auto"):
    """Every tensor of ``specs`` through the loader that generation uses (``open_tensors``:
    the folder is checked as a whole, then each tensor is read when asked for)."""
    source = open_tensors(folder, specs, {n: 1 for n in specs}, engine_dtype, device, wide_tensors=wide_tensors)
    return {n: source[n] for n in specs}
from yalis_amd.weights.random_init import write_random_model
from yalis_amd.weights.safetensors_io import SafetensorsError, index_folder, read_tensor, write_dict


def test_llama_config_reads_its_own_keys():
    c = LlamaConfig.from_dict(TINY_B)
    assert (c.hidden_size, c.num_hidden_layers, c.num_attention_heads, c.num_key_value_heads) == (128, 3, 4, 1)
    assert (c.head_dim, c.intermediate_size, c.vocab_size) == (32, 352, 384)
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 500000.0 and c.tie_word_embeddings
    assert c.rope_scaling.factor == 8.0 and c.rope_scaling.original_max_position_embeddings == 64
    # defaults: groups = heads, head_dim = hidden / heads (yalis/external/config.py:108-125)
    d = dict(TINY_A)
    del d["num_key_value_heads"], d["head_dim"]
    c2 = LlamaConfig.from_dict(d)
    assert c2.num_key_value_heads == 4 and c2.head_dim == 16
    # round trip through its own config.json
    assert LlamaConfig.from_dict(c.to_dict()) == c


@pytest.mark.parametrize("change,match", [
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "yarn"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0}}, "low_freq_factor"),
    ({"hidden_size": "64"}, "integer"),
    ({"rms_norm_eps": 0}, "rms_norm_eps"),
    ({"sliding_window": 128}, "sliding_window"),
    ({"head_dim": 15}, "even"),
])
def test_llama_config_refuses(change, match):
    with pytest.raises(ConfigError, match=match):
        LlamaConfig.from_dict({**TINY_A, **change})


def test_llama_config_missing_and_unknown_keys():
    d = dict(TINY_A)
    del d["intermediate_size"]
    with pytest.raises(ConfigError, match="intermediate_size"):
        LlamaConfig.from_dict(d)
    with pytest.warns(UserWarning, match="mystery_key"):
        LlamaConfig.from_dict({**TINY_A, "mystery_key": 1})
    with pytest.raises(ConfigError, match="mystery_key"):
        LlamaConfig.from_dict({**TINY_A, "mystery_key": 1}, strict=True)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        LlamaConfig.from_dict({**TINY_A, "transformers_version": "4.40", "bos_token_id": 1, "eos_token_id": [2, 3]})


def test_registry(tmp_path):
    assert "LlamaForCausalLM" in known_architectures()
    with pytest.raises(ConfigError, match="unknown architecture 'NoSuchModel'.*LlamaForCausalLM"):
        get_architecture("NoSuchModel")
    with open(tmp_path / "config.json", "w") as f:
        json.dump(TINY_A, f)
    arch, cfg = load_model_config(str(tmp_path))
    assert arch.name == "LlamaForCausalLM" and isinstance(cfg, LlamaConfig)
    with pytest.raises(FileNotFoundError):
        load_model_config(str(tmp_path / "nothing"))


def test_spec_has_every_constant_as_data():
    _, _, spec = spec_from_config(TINY_B)
    assert len(spec.layers) == 3 and [e.layer for e in spec.run_order] == [0, 1, 2]
    assert list(spec.layers[1].parts) == ["mixer_norm", "mixer", "feed_forward_norm", "feed_forward"] and spec.layers[1].block == "prenorm"
    m = spec.layers[1].part("mixer").params
    assert (m["num_heads"], m["num_kv_heads"], m["head_dim"], m["window"]) == (4, 1, 32, None)
    assert abs(m["scale"] - 32**-0.5) < 1e-12
    assert m["position"].params["theta"] == 500000.0 and m["position"].params["scaling"]["factor"] == 8.0
    assert spec.layers[1].part("mixer_norm").params["eps"] == 1e-6 and spec.layers[1].part("post_mixer_norm") is None
    assert spec.head.params["tied_to"] == "model.embed_tokens.weight"


def test_runtime_configs():
    with pytest.raises(ValueError, match="Invalid precision"):
        ModelConfig(model_path="/", precision="fp8")
    with pytest.raises(ValueError, match="does not exist"):
        ModelConfig(model_name="nope/none")
    with pytest.raises(ValueError, match="Either"):
        ModelConfig()
    assert ModelConfig(model_path="/", precision="bf16").dtype == "bfloat16"
    for bad in (dict(max_batch_size=0), dict(temperature=-1.0), dict(top_k=0), dict(top_p=1.5), dict(tp_dims=(2, 1, 1)), dict(attention_backend="flash")):
        with pytest.raises(ValueError):
            InferenceConfig(**bad)
    ic = InferenceConfig(max_batch_size=4, top_p=0.8)
    assert ic.max_length == 1024 and ic.temperature == 1.0 and ic.top_k is None
    with pytest.raises(ValueError, match="multiple of 16"):
        EngineConfig(page_size=24)
    assert EngineConfig(page_size=64, max_num_seqs=4, max_model_len=1000).resolved_num_pages() == 64


def test_safetensors_round_trip_and_errors(tmp_path):
    t = {
        "a": torch.randn(3, 5),
        "b": torch.randn(7).to(torch.bfloat16),
        "c": torch.arange(6, dtype=torch.int64).reshape(2, 3),
    }
    os.makedirs(tmp_path / "m")
    write_dict(str(tmp_path / "m" / "model.safetensors"), t)
    idx = index_folder(str(tmp_path / "m"))
    for k, v in t.items():
        assert torch.equal(read_tensor(idx[k]), v)
    # the same file read by the safetensors package
    from safetensors.torch import load_file

    lib = load_file(str(tmp_path / "m" / "model.safetensors"))
    assert all(torch.equal(lib[k], v) for k, v in t.items())
    # truncated file
    data = open(tmp_path / "m" / "model.safetensors", "rb").read()
    os.makedirs(tmp_path / "t")
    open(tmp_path / "t" / "model.safetensors", "wb").write(data[:-10])
    with pytest.raises(SafetensorsError, match="truncated|beyond"):
        index_folder(str(tmp_path / "t"))
    with pytest.raises(FileNotFoundError):
        index_folder(str(tmp_path / "none"))
    # shards with an index
    os.makedirs(tmp_path / "s")
    write_dict(str(tmp_path / "s" / "model-00001-of-00002.safetensors"), {"a": t["a"]})
    write_dict(str(tmp_path / "s" / "model-00002-of-00002.safetensors"), {"b": t["b"], "c": t["c"]})
    json.dump({"weight_map": {"a": "model-00001-of-00002.safetensors", "b": "model-00002-of-00002.safetensors", "c": "model-00002-of-00002.safetensors"}},
              open(tmp_path / "s" / "model.safetensors.index.json", "w"))
    idx = index_folder(str(tmp_path / "s"))
    assert torch.equal(read_tensor(idx["c"]), t["c"])


def test_precision_rule():
    assert target_dtype("BF16", "float", "bfloat16") == torch.bfloat16
    assert target_dtype("F16", "float", "bfloat16") == torch.bfloat16
    assert target_dtype("F32", "float", "bfloat16") == torch.float32, "a tensor stored in 32 bits stays so"
    assert target_dtype("BF16", "float", "float32") == torch.float32
    assert target_dtype("F32", "float", "bfloat16", keep_wide=False) == torch.bfloat16
    assert target_dtype("I64", "int", "bfloat16") == torch.int32


def test_random_folder_loads_back_bit_exact(tmp_path):
    folder = write_random_model(str(tmp_path / "b"), TINY_B, seed=1, dtype="bfloat16")
    specs = tensor_specs_for(TINY_B)
    assert "lm_head.weight" not in specs, "tied: the head reads the embedding table"
    loaded = load_tensors(folder, specs, "bfloat16", "cpu")
    again = write_random_model(str(tmp_path / "b2"), TINY_B, seed=1, dtype="bfloat16")
    other = write_random_model(str(tmp_path / "b3"), TINY_B, seed=2, dtype="bfloat16")
    l2 = load_tensors(again, specs, "bfloat16", "cpu")
    l3 = load_tensors(other, specs, "bfloat16", "cpu")
    for n, t in loaded.items():
        assert t.dtype == torch.bfloat16 and tuple(t.shape) == specs[n].shape
        assert torch.equal(t, l2[n]) and not torch.equal(t, l3[n])
    w = loaded["model.layers.0.self_attn.q_proj.weight"].float()
    assert abs(w.std().item() - 0.02) < 0.002 and abs(w.mean().item()) < 0.002
    n = loaded["model.norm.weight"].float()
    assert abs(n.mean().item() - 1.0) < 0.05 and 0.05 < n.std().item() < 0.15
    # the 32-bit engine widens
    assert load_tensors(folder, specs, "float32", "cpu")["model.norm.weight"].dtype == torch.float32
    assert json.load(open(os.path.join(folder, "config.json")))["architectures"] == ["LlamaForCausalLM"]


def test_sixteen_bit_floats_of_the_other_kind_and_wide_matrices(tmp_path, caplog):
    """A checkpoint stored in float16: the bfloat16 engine rounds it to bfloat16 (to nearest even, as
    the reference casts every tensor to its parameter's dtype, yalis/model_loading.py:172-173) and
    says so once; the float32 engine widens it exactly.  Matrices stored in 32 bits stay so in the
    bfloat16 engine when it is told to keep them, which it says once."""
    import logging

    specs = tensor_specs_for(TINY_A)
    folder = write_random_model(str(tmp_path / "h"), TINY_A, seed=0, dtype="float32")
    tensors = {n: read_tensor(e).to(torch.float16) for n, e in index_folder(folder).items()}
    write_dict(os.path.join(folder, "model.safetensors"), tensors)
    log = logging.getLogger("yalis_amd")
    log.propagate = True  # (the package's loggers keep to themselves; the test listens in)
    try:
        with caplog.at_level(logging.WARNING, logger="yalis_amd"):
            narrow = load_tensors(folder, specs, "bfloat16", "cpu")
        assert sum("stored in float16" in r.getMessage() for r in caplog.records) == 1
        assert all(t.dtype == torch.bfloat16 for t in narrow.values())
        assert torch.equal(narrow["lm_head.weight"], tensors["lm_head.weight"].to(torch.bfloat16))
        assert not torch.equal(narrow["lm_head.weight"].float(), tensors["lm_head.weight"].float()), "the test's weights must need the rounding"
        wide = load_tensors(folder, specs, "float32", "cpu")
        assert all(t.dtype == torch.float32 for t in wide.values())
        assert torch.equal(wide["lm_head.weight"], tensors["lm_head.weight"].float())
        f32 = write_random_model(str(tmp_path / "w"), TINY_A, seed=0, dtype="float32")
        caplog.clear()
        with caplog.at_level(logging.WARNING, logger="yalis_amd"):
            got = load_tensors(f32, specs, "bfloat16", "cpu", wide_tensors="keep")
    finally:
        log.propagate = False
    assert got["lm_head.weight"].dtype == torch.float32
    assert sum("stored in 32 bits" in r.getMessage() for r in caplog.records) == 1


def test_tensors_stored_in_32_bits(tmp_path):
    """The bfloat16 engine: a checkpoint stored wholly in 32 bits is narrowed (the reference
    casts every tensor to its parameter's dtype, yalis/model_loading.py:172-173), rounding to
    nearest even; single 32-bit tensors inside a 16-bit checkpoint stay 32-bit; "keep" and
    "cast" override both ways; the float32 engine is not affected."""
    specs = tensor_specs_for(TINY_A)
    f32 = write_random_model(str(tmp_path / "w"), TINY_A, seed=0, dtype="float32")
    stored = {n: read_tensor(e) for n, e in index_folder(f32).items()}
    got = load_tensors(f32, specs, "bfloat16", "cpu")
    assert all(t.dtype == torch.bfloat16 for t in got.values())
    assert torch.equal(got["lm_head.weight"], stored["lm_head.weight"].to(torch.bfloat16))
    assert all(t.dtype == torch.float32 for t in load_tensors(f32, specs, "bfloat16", "cpu", wide_tensors="keep").values())
    assert all(torch.equal(t, stored[n]) for n, t in load_tensors(f32, specs, "float32", "cpu").items())
    # a 16-bit checkpoint whose norm weights are stored wide
    mixed = {n: (t if n.endswith("norm.weight") else t.to(torch.bfloat16)) for n, t in stored.items()}
    os.makedirs(tmp_path / "m")
    json.dump(TINY_A, open(tmp_path / "m" / "config.json", "w"))
    write_dict(str(tmp_path / "m" / "model.safetensors"), mixed)
    got = load_tensors(str(tmp_path / "m"), specs, "bfloat16", "cpu")
    assert got["model.norm.weight"].dtype == torch.float32 and torch.equal(got["model.norm.weight"], stored["model.norm.weight"])
    assert got["lm_head.weight"].dtype == torch.bfloat16
    assert load_tensors(str(tmp_path / "m"), specs, "bfloat16", "cpu", wide_tensors="cast")["model.norm.weight"].dtype == torch.bfloat16
    with pytest.raises(ValueError, match="wide_tensors"):
        load_tensors(f32, specs, "bfloat16", "cpu", wide_tensors="sometimes")


def test_one_error_lists_everything_wrong(tmp_path):
    folder = write_random_model(str(tmp_path / "a"), TINY_A, seed=0, dtype="bfloat16")
    specs = tensor_specs_for(TINY_A)
    path = os.path.join(folder, "model.safetensors")
    tensors = {n: read_tensor(e) for n, e in index_folder(folder).items()}
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["lm_head.weight"]
    tensors["model.layers.0.extra.weight"] = torch.zeros(3)
    tensors["model.norm.weight"] = torch.zeros(65, dtype=torch.bfloat16)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)  # harmless, ignored
    tensors["model.layers.0.input_layernorm.weight"] = torch.zeros(64, dtype=torch.int32)
    write_dict(path, tensors)
    with pytest.raises(WeightsError) as e:
        load_tensors(folder, specs, "bfloat16", "cpu")
    err = e.value
    assert err.missing == ["lm_head.weight", "model.layers.1.mlp.up_proj.weight"]
    assert err.unexpected == ["model.layers.0.extra.weight"]
    assert err.wrong_shape == [("model.norm.weight", (65,), (64,))]
    assert err.wrong_kind[0][0] == "model.layers.0.input_layernorm.weight"
    msg = str(err)
    for piece in ("missing tensors (2)", "unexpected tensors (1)", "model.norm.weight has (65,), the model needs (64,)", "wrong type"):
        assert piece in msg


def test_tensors_are_made_when_a_part_asks(tmp_path):
    """The loader hands the model a source that reads a tensor when a part asks for it: each
    tensor is read once, a tied table is read once and shared by the embedding and the head,
    nothing is kept afterwards, and the folder is still checked as a whole first."""
    from kernel_refs import RefOps
    from yalis_amd.engine.factory import build_model, load_runner
    from yalis_amd.weights import loader

    folder = write_random_model(str(tmp_path / "m"), TINY_B, seed=5)
    eng = EngineConfig(page_size=16, num_pages=4, max_num_seqs=2, max_model_len=64, dtype="float32", device="cpu")
    model = build_model(TINY_B, eng, ops=RefOps())
    uses = model.tensor_uses()
    assert uses["model.embed_tokens.weight"] == 2 and uses["model.norm.weight"] == 1
    reads = []
    real = loader.read_tensor
    loader.read_tensor = lambda e: (reads.append(e.name), real(e))[1]
    try:
        src = loader.open_tensors(folder, model.tensor_specs(), uses, "float32", "cpu")
        model.load(src)
    finally:
        loader.read_tensor = real
    assert sorted(reads) == sorted(model.tensor_specs()), "every tensor is read exactly once"
    assert not src._kept, "nothing is held once every part has its tensors"
    assert model.head.weight.data_ptr() == model.embedding.table.data_ptr(), "the tied table is shared"
    # the same through the factory, and the one error still comes before anything is read
    runner = load_runner(folder, eng, ops=RefOps())
    assert runner.model.head.weight.data_ptr() == runner.model.embedding.table.data_ptr()
    t = {n: read_tensor(e) for n, e in index_folder(folder).items()}
    del t["model.norm.weight"]
    bad = str(tmp_path / "bad")
    os.makedirs(bad)
    json.dump(TINY_B, open(os.path.join(bad, "config.json"), "w"))
    write_dict(os.path.join(bad, "model.safetensors"), t)
    with pytest.raises(WeightsError, match="model.norm.weight"):
        load_runner(bad, eng, ops=RefOps())


def test_graphs_switch_follows_the_reference(monkeypatch):
    monkeypatch.delenv("YALIS_DISABLE_DECODE_CUDAGRAPHS", raising=False)
    assert EngineConfig().decode_graphs
    monkeypatch.setenv("YALIS_DISABLE_DECODE_CUDAGRAPHS", "1")
    assert not EngineConfig().decode_graphs and EngineConfig(decode_graphs=True).decode_graphs
