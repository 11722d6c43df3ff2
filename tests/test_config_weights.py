"""Configuration, registry and weight-file errors (CPU)."""
import json
import os

import pytest
import torch

import tiny
from swifttransformer_amd.config import (ConfigError, OptHyperParam, hyper_param_from_dir,
                                         registered_architectures, resolve_architecture)
from swifttransformer_amd.models.decoder import DecoderModel
from swifttransformer_amd.weights import (ModelFiles, WeightError, match_specs, save_safetensors,
                                          write_random_model)


def test_config_roundtrip_and_defaults(tmp_path):
    hp = tiny.hyper("B")
    d = write_random_model(hp, str(tmp_path / "m"), seed=0)
    arch, hp2 = hyper_param_from_dir(d)
    assert arch.name == "OPTForCausalLM"
    assert hp2 == hp
    assert hp2.head_dim == 32 and hp2.has_projection and not hp2.has_final_norm
    # defaults of keys a config.json may leave out
    minimal = {"architectures": ["OPTForCausalLM"], "vocab_size": 50, "max_position_embeddings": 16,
               "hidden_size": 32, "num_hidden_layers": 1, "num_attention_heads": 2, "ffn_dim": 64}
    hp3 = OptHyperParam.from_dict(minimal)
    assert hp3.word_embed_proj_dim == 32 and hp3.do_layer_norm_before and hp3.enable_bias
    assert hp3.layer_norm_eps == 1e-5 and hp3.position_offset == 2 and hp3.eos_token_id == 2


@pytest.mark.parametrize("change,match", [
    ({"num_attention_heads": 5}, "not a multiple"),
    ({"activation_function": "gelu"}, "activation_function"),
    ({"hidden_size": None}, "hidden_size"),
    ({"vocab_size": 0}, "vocab_size"),
    ({"do_layer_norm_before": "yes"}, "do_layer_norm_before"),
])
def test_config_errors(change, match):
    cfg = dict(tiny.TINY_A, architectures=["OPTForCausalLM"])
    for k, v in change.items():
        if v is None:
            cfg.pop(k)
        else:
            cfg[k] = v
    with pytest.raises(ConfigError, match=match):
        OptHyperParam.from_dict(cfg)


def test_registry():
    assert "OPTForCausalLM" in registered_architectures()
    with pytest.raises(ConfigError, match="unknown architecture"):
        resolve_architecture("LlamaForCausalLM")


def test_model_type_stands_in_for_a_missing_class_name(tmp_path):
    d = tmp_path / "m"
    d.mkdir()
    cfg = dict(tiny.TINY_A, model_type="opt")
    (d / "config.json").write_text(json.dumps(cfg))
    arch, hp = hyper_param_from_dir(str(d))
    assert arch.name == "OPTForCausalLM" and hp.hidden_size == 64
    (d / "config.json").write_text(json.dumps(dict(tiny.TINY_A, model_type="llama")))
    with pytest.raises(ConfigError, match="names no architecture"):
        hyper_param_from_dir(str(d))


def test_unknown_architecture_in_folder(tmp_path):
    d = tmp_path / "m"
    d.mkdir()
    (d / "config.json").write_text(json.dumps({"architectures": ["Foo"], "hidden_size": 8}))
    with pytest.raises(ConfigError, match="unknown architecture"):
        hyper_param_from_dir(str(d))


def _specs(name):
    arch = resolve_architecture("OPTForCausalLM")
    return DecoderModel(arch.build_spec(tiny.hyper(name)), torch.float32).tensor_specs()


def test_weight_names_match_file(tmp_path):
    for name in tiny.CONFIGS:
        d = tiny.write_model(name, str(tmp_path))
        files = ModelFiles(d)
        found = match_specs(_specs(name), {k: files.shape(k) for k in files.keys()})
        # everything in the file is used; a tied head is found absent and that is fine
        assert set(found.values()) == set(files.keys())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = tiny.write_model("A", str(tmp_path))
    files = ModelFiles(d)
    tensors = {k: files.tensor(k).clone() for k in files.keys()}
    del tensors["model.decoder.layers.1.fc1.bias"]
    del tensors["model.decoder.embed_positions.weight"]
    tensors["model.decoder.layers.0.self_attn.rotary.inv_freq"] = torch.zeros(4)
    tensors["model.decoder.layers.0.fc2.weight"] = torch.zeros(64, 255, dtype=torch.bfloat16)
    save_safetensors(os.path.join(d, "model.safetensors"), tensors)
    files = ModelFiles(d)
    with pytest.raises(WeightError) as ei:
        match_specs(_specs("A"), {k: files.shape(k) for k in files.keys()})
    e = ei.value
    assert e.missing == ["model.decoder.embed_positions.weight", "model.decoder.layers.1.fc1.bias"]
    assert e.unexpected == ["model.decoder.layers.0.self_attn.rotary.inv_freq"]
    assert e.wrong_shape == [("model.decoder.layers.0.fc2.weight", (64, 256), (64, 255))]
    msg = str(e)
    for part in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (1)",
                 "expected [64, 256], file has [64, 255]"):
        assert part in msg


def test_names_without_model_prefix_and_untied_head(tmp_path):
    d = tiny.write_model("C", str(tmp_path))      # untied head: lm_head.weight is in the file
    files = ModelFiles(d)
    assert "lm_head.weight" in files
    tensors = {k[len("model."):] if k.startswith("model.") else k: files.tensor(k).clone()
               for k in files.keys()}
    found = match_specs(_specs("C"), {k: tuple(v.shape) for k, v in tensors.items()})
    assert found["model.decoder.embed_tokens.weight"] == "decoder.embed_tokens.weight"


def test_projection_and_final_norm_presence(tmp_path):
    specs_a = {s.name for s in _specs("A")}
    specs_b = {s.name for s in _specs("B")}
    assert "model.decoder.final_layer_norm.weight" in specs_a
    assert "model.decoder.final_layer_norm.weight" not in specs_b      # post-norm: no final norm
    assert "model.decoder.project_in.weight" in specs_b and "model.decoder.project_out.weight" in specs_b
    assert "model.decoder.project_in.weight" not in specs_a
    assert not any(n.endswith(".bias") and "layer_norm" not in n for n in specs_b)   # enable_bias false


def test_safetensors_reader_rejects_garbage(tmp_path):
    from swifttransformer_amd.weights import SafetensorsError, SafetensorsFile
    p = tmp_path / "x.safetensors"
    p.write_bytes(b"\x10\x00\x00\x00\x00\x00\x00\x00not json at all!!")
    with pytest.raises(SafetensorsError):
        SafetensorsFile(str(p))
    p.write_bytes(b"\x01\x02")
    with pytest.raises(SafetensorsError):
        SafetensorsFile(str(p))


@pytest.mark.parametrize("offsets", [[-16, 0], [8, 0], [0, 32]])
def test_safetensors_reader_rejects_offsets_outside_the_data(tmp_path, offsets):
    """Offsets that would read the header's own bytes (negative start), run backwards, or pass
    the file's end are refused."""
    import json
    import struct
    from swifttransformer_amd.weights import SafetensorsError, SafetensorsFile
    header = json.dumps({"t": {"dtype": "F32", "shape": [4], "data_offsets": offsets}}).encode()
    header += b" " * (-len(header) % 8)
    p = tmp_path / "x.safetensors"
    p.write_bytes(struct.pack("<Q", len(header)) + header + b"\0" * 16)
    with pytest.raises(SafetensorsError):
        SafetensorsFile(str(p))


def test_storage_types():
    from swifttransformer_amd.weights import storage_dtype
    assert storage_dtype("matrix", torch.bfloat16) == torch.bfloat16
    assert storage_dtype("vector", torch.bfloat16) == torch.float32     # 32-bit vectors stay 32-bit
    assert storage_dtype("int", torch.bfloat16) == torch.int32
    assert storage_dtype("table", torch.float32) == torch.float32


def test_sharded_model_folder(tmp_path):
    """model.safetensors.index.json naming several shard files."""
    import json as _json
    d = tiny.write_model("A", str(tmp_path))
    files = ModelFiles(d)
    names = sorted(files.keys())
    half = len(names) // 2
    shards = {"model-00001-of-00002.safetensors": names[:half], "model-00002-of-00002.safetensors": names[half:]}
    weight_map = {}
    for fname, ks in shards.items():
        save_safetensors(os.path.join(d, fname), {k: files.tensor(k).clone() for k in ks})
        weight_map.update({k: fname for k in ks})
    expect = {k: files.tensor(k).clone() for k in names}
    del files
    os.remove(os.path.join(d, "model.safetensors"))
    with open(os.path.join(d, "model.safetensors.index.json"), "w") as f:
        _json.dump({"metadata": {}, "weight_map": weight_map}, f)
    sharded = ModelFiles(d)
    assert sorted(sharded.keys()) == names
    for k in names:
        assert torch.equal(sharded.tensor(k), expect[k])
    match_specs(_specs("A"), {k: sharded.shape(k) for k in sharded.keys()})
    os.remove(os.path.join(d, "model.safetensors.index.json"))
    with pytest.raises(FileNotFoundError):
        ModelFiles(d)


def test_float16_and_float32_files_load_as_declared(tmp_path):
    from swifttransformer_amd.weights import load_tensors
    for file_dtype in (torch.float16, torch.float32):
        d = tiny.write_model("A", str(tmp_path / str(file_dtype)), file_dtype=file_dtype)
        t = load_tensors(d, _specs("A"), torch.bfloat16, "cpu")
        assert t["model.decoder.layers.0.fc1.weight"].dtype == torch.bfloat16       # matrices: engine dtype
        assert t["model.decoder.layers.0.fc1.bias"].dtype == torch.float32          # vectors: 32-bit
        t32 = load_tensors(d, _specs("A"), torch.float32, "cpu")
        assert all(v.dtype == torch.float32 for v in t32.values())


def test_named_sizes():
    """The family's sizes by the reference's names (src/examples/lib/common_gpt_hyper_params.h:105-116)."""
    from swifttransformer_amd.config import preset, preset_names
    assert preset_names() == ["opt_125m", "opt_1.3b", "opt_2.7b", "opt_6.7b", "opt_13b", "opt_30b"]
    hp = preset("opt_1.3b")
    assert (hp.hidden_size, hp.num_hidden_layers, hp.num_attention_heads, hp.head_dim, hp.ffn_dim,
            hp.vocab_size, hp.max_position_embeddings) == (2048, 24, 32, 64, 8192, 50272, 2048)
    assert preset("opt_2.7b").head_dim == 80 and preset("opt_30b").num_attention_heads == 56
    assert preset("opt_125m", num_hidden_layers=2).num_hidden_layers == 2
    with pytest.raises(KeyError, match="valid names"):
        preset("opt_350m")


def test_random_values_depend_on_seed_name_and_index_only():
    """Random weights are a function of (seed, tensor name, element index): independent of the
    order of generation and of the chunking, normal to the table's accuracy."""
    from swifttransformer_amd.weights import TensorSpec, random_tensor, random_tensors
    from swifttransformer_amd.weights import random_init
    a = TensorSpec("layer.w", (300, 70))
    one = random_tensor(a, 5)
    assert torch.equal(one, random_tensor(a, 5)) and not torch.equal(one, random_tensor(a, 6))
    assert not torch.equal(one, random_tensor(TensorSpec("layer.v", (300, 70)), 5))
    # a longer tensor of the same name starts with the same values; small chunks give the same values
    longer = random_tensor(TensorSpec("layer.w", (600, 70)), 5)
    assert torch.equal(longer[:300], one)
    chunk = dict(random_init._CHUNK)
    random_init._CHUNK["cpu"] = 1000
    try:
        assert torch.equal(random_tensor(a, 5), one)
    finally:
        random_init._CHUNK.update(chunk)
    x = (random_tensor(TensorSpec("big", (400000,)), 1).double() / random_init.WEIGHT_STD)
    assert abs(x.mean()) < 0.01 and abs(x.std() - 1) < 0.01 and abs((x ** 4).mean() - 3) < 0.1
    assert abs((x[1:] * x[:-1]).mean()) < 0.01
    gain = random_tensor(TensorSpec("g", (50000,), "vector", init="gain"), 1).double()
    assert abs(gain.mean() - 1) < 0.005 and abs(gain.std() - random_init.GAIN_STD) < 0.005
    # in memory: what a bfloat16 folder would hold, in the loader's storage types
    t = random_tensors([a, TensorSpec("b", (70,), "vector")], 5, torch.float32, "cpu")
    assert torch.equal(t["layer.w"], one.to(torch.bfloat16).float()) and t["b"].dtype == torch.float32


def test_model_in_memory_equals_its_folder(tmp_path):
    """``random_model`` (what the benchmarks run) and ``write_random_model`` + ``load_model`` (what
    the tests and the command lines run) hold the same tensors for a seed, in both engine types."""
    from swifttransformer_amd.models import load_model, random_model
    hp = tiny.hyper("B")
    d = tiny.write_model("B", str(tmp_path), seed=11)
    for dtype in (torch.bfloat16, torch.float32):
        mem, disk = random_model(hp, dtype, seed=11, device="cpu"), load_model(d, dtype, "cpu")
        compared = 0
        for pm, pd in zip(mem.all_parts(), disk.all_parts()):
            for n, tm in vars(pm).items():
                if torch.is_tensor(tm):
                    td = getattr(pd, n)
                    assert tm.dtype == td.dtype and torch.equal(tm, td), f"{type(pm).__name__}.{n}"
                    compared += 1
        assert compared > 20


def test_named_sizes_go_through_the_registry():
    from swifttransformer_amd.config.registry import hyper_param_by_name, register_architecture

    class Hp:
        architecture = "NamedToyForCausalLM"

    register_architecture("NamedToyForCausalLM", Hp, lambda hp: None, short_name="namedtoy",
                          presets=lambda name, **kw: (name, kw))
    assert hyper_param_by_name("opt_2.7b").hidden_size == 2560
    assert hyper_param_by_name("OPT-1.3B", num_hidden_layers=3).num_hidden_layers == 3
    assert hyper_param_by_name("namedtoy_small", depth=2) == ("namedtoy_small", {"depth": 2})
    with pytest.raises(KeyError, match="families"):
        hyper_param_by_name("llama_7b")
    with pytest.raises(KeyError, match="valid names"):
        hyper_param_by_name("opt_350m")
