"""Configuration, registry, safetensors reading and the loader's one clear error."""
import json
import os
import struct

import pytest
import torch

from emulated_ops import EmulatedOps
from tiny_configs import TINY_A, TINY_B, TINY_C, make_model_dir


def test_qwen2_config_reads_its_keys():
    from machserve_amd.config import Qwen2Config, config_from_dict
    c = config_from_dict(dict(TINY_B))
    assert isinstance(c, Qwen2Config)
    assert (c.hidden_size, c.num_hidden_layers, c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (192, 3, 6, 1, 32)
    assert (c.intermediate_size, c.vocab_size, c.rms_norm_eps, c.rope_theta) == (320, 1000, 1e-5, 1e6)
    assert c.tie_word_embeddings is False and c.layer_window(2) is None
    c = config_from_dict(dict(TINY_C))
    assert c.head_dim == 48 and [c.layer_window(i) for i in range(4)] == [None, None, 40, 40]
    spec = c.to_spec()
    assert [l.mixer.window for l in spec.layers] == [None, None, 40, 40] and list(spec.order) == [0, 1, 2, 3]
    # nested text_config, num_key_value_heads defaulting to the heads, rope_parameters
    raw = {"architectures": ["Qwen2ForCausalLM"], "text_config": {
        "hidden_size": 32, "num_hidden_layers": 1, "num_attention_heads": 2, "intermediate_size": 64, "vocab_size": 10,
        "max_position_embeddings": 77, "rms_norm_eps": 2e-6, "rope_parameters": {"rope_theta": 123.0}}}
    c = config_from_dict(raw)
    assert c.num_key_value_heads == 2 and c.head_dim == 16 and c.rope_theta == 123.0 and c.tie_word_embeddings is None
    assert c.max_position_embeddings == 77 and c.rms_norm_eps == 2e-6


def test_yarn_rope_scaling_is_read_with_the_reference_s_keys_and_defaults():
    """crates/mach-server/src/startup.rs:172-199: type yarn, factor, original_max_position_embeddings, beta_fast 32,
    beta_slow 1, mscale 1, mscale_all_dim 0; the scores' scale takes mscale_all_dim's square only when it is set."""
    import math
    from machserve_amd.config import YarnSpec, config_from_dict
    raw = dict(TINY_A, rope_scaling={"type": "yarn", "factor": 4.0, "original_max_position_embeddings": 64})
    c = config_from_dict(raw)
    assert c.rope_scaling == YarnSpec(4.0, 64, 32.0, 1.0, 1.0, 0.0) and c.attention_scale() is None
    spec = c.to_spec()
    assert all(l.mixer.position.yarn == c.rope_scaling and l.mixer.scale is None for l in spec.layers)
    assert config_from_dict(c.to_dict()) == c
    c2 = config_from_dict(dict(TINY_A, rope_scaling={"rope_type": "yarn", "factor": 40.0, "original_max_position_embeddings": 4096,
                                                      "beta_fast": 16, "beta_slow": 2, "mscale": 0.9, "mscale_all_dim": 0.707}))
    assert c2.rope_scaling == YarnSpec(40.0, 4096, 16.0, 2.0, 0.9, 0.707)
    m = 0.1 * 0.707 * math.log(40.0) + 1
    assert abs(c2.attention_scale() - m * m / 4.0) < 1e-12      # head size 16
    assert config_from_dict(dict(TINY_A, rope_scaling=None)).rope_scaling is None
    assert config_from_dict(dict(TINY_A, rope_scaling={"type": "default"})).rope_scaling is None


@pytest.mark.parametrize("change,match", [
    ({"hidden_size": None}, "missing key 'hidden_size'"),
    ({"num_hidden_layers": 0}, "num_hidden_layers"),
    ({"num_key_value_heads": 3}, "not a multiple"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"type": "yarn"}}, "factor > 1"),
    ({"rope_scaling": {"type": "yarn", "factor": 4.0}}, "original_max_position_embeddings"),
    ({"rope_scaling": {"type": "linear", "factor": 2.0}}, "only yarn"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0}}, "only yarn"),
    ({"use_sliding_window": True}, "sliding_window"),
    ({"architectures": ["LlamaForCausalLM"]}, "not supported"),
    ({"hidden_size": 66}, "head_dim"),
    # constants that change every logit (or cap every request) are not guessed either
    ({"max_position_embeddings": None}, "missing key 'max_position_embeddings'"),
    ({"rms_norm_eps": None}, "missing key 'rms_norm_eps'"),
    ({"rope_theta": None}, "missing key 'rope_theta'"),
    ({"rope_theta": -1.0}, "rope_theta"),
])
def test_config_errors_name_the_key(change, match):
    from machserve_amd.config import ConfigError, config_from_dict
    raw = dict(TINY_A)
    raw.update(change)
    with pytest.raises(ConfigError, match=match):
        config_from_dict(raw)


def test_registry_lists_architectures_and_takes_new_ones():
    from machserve_amd.config import ConfigError, architectures, config_from_dict, register_architecture
    assert "Qwen2ForCausalLM" in architectures()
    with pytest.raises(ConfigError, match="Qwen2ForCausalLM"):
        config_from_dict({"architectures": ["Nope"]})
    assert config_from_dict({k: v for k, v in TINY_A.items() if k != "architectures"}).hidden_size == 64  # by model_type

    class Other:
        @classmethod
        def from_dict(cls, raw):
            return "other"
    register_architecture("OtherForCausalLM", Other)
    assert config_from_dict({"architectures": ["OtherForCausalLM"]}) == "other"


def test_random_model_folder_round_trip(tmp_path):
    """Written by our writer, read back by our reader and by the safetensors package."""
    from safetensors.torch import load_file
    from machserve_amd.config import load_config
    from machserve_amd.weights import Checkpoint, random_tensor_dict
    d = make_model_dir(tmp_path, "B")
    cfg = load_config(d)
    ck = Checkpoint(d)
    theirs = load_file(os.path.join(d, "model.safetensors"))
    ours = random_tensor_dict(cfg, 1)
    assert sorted(ck.names()) == sorted(theirs) == sorted(ours)
    for n in ck.names():
        assert torch.equal(ck.tensor(n), theirs[n]) and torch.equal(ours[n], theirs[n])
    w = theirs["model.layers.0.mlp.gate_proj.weight"]
    assert abs(w.std().item() - 0.02) < 2e-3 and abs(w.mean().item()) < 1e-3
    assert abs(theirs["model.norm.weight"].mean().item() - 1.0) < 1e-2
    assert "model.layers.2.self_attn.k_proj.bias" in theirs and "lm_head.weight" in theirs
    assert "lm_head.weight" not in load_file(os.path.join(make_model_dir(tmp_path, "A"), "model.safetensors"))
    assert not any("bias" in n for n in load_file(os.path.join(make_model_dir(tmp_path, "C"), "model.safetensors")))
    # another seed, other numbers; bfloat16 storage
    assert not torch.equal(random_tensor_dict(cfg, 2)["model.norm.weight"], ours["model.norm.weight"])
    d16 = make_model_dir(tmp_path / "bf16", "A", torch.bfloat16)
    assert Checkpoint(d16).meta("model.norm.weight")[0] == torch.bfloat16


def _load(d, **kw):
    from machserve_amd.engine import load_model
    return load_model(d, dtype="float32", device="cpu", page_size=16, num_pages=4, ops=EmulatedOps(), **kw)


def _rewrite(d, edit):
    from safetensors.torch import load_file, save_file
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    edit(t)
    save_file(t, path)


def test_loader_lists_missing_unexpected_and_wrong_shapes_in_one_error(tmp_path):
    from machserve_amd.weights import WeightsError
    d = make_model_dir(tmp_path, "A")

    def edit(t):
        del t["model.layers.1.mlp.up_proj.weight"]
        del t["model.norm.weight"]
        t["model.layers.0.extra.weight"] = torch.zeros(3)
        t["model.layers.0.self_attn.o_proj.weight"] = t["model.layers.0.self_attn.o_proj.weight"].t().contiguous()[:, :32].contiguous()
        t["model.layers.0.mlp.down_proj.weight"] = t["model.layers.0.mlp.down_proj.weight"].t().contiguous()
    _rewrite(d, edit)
    with pytest.raises(WeightsError) as e:
        _load(d)
    msg = str(e.value)
    assert e.value.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.value.unexpected == ["model.layers.0.extra.weight"]
    assert len(e.value.shapes) == 2
    for part in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (2)", "model.layers.0.mlp.down_proj.weight: checkpoint [160, 64], model [64, 160]"):
        assert part in msg
    # a transposed tensor of the same element count is a wrong shape here
    # (the reference compares element counts only, crates/mach-model/src/loader.rs:1016-1033)


def test_bias_presence_decides_and_head_rule(tmp_path):
    from machserve_amd.weights import WeightsError
    d = make_model_dir(tmp_path, "A")
    _rewrite(d, lambda t: [t.pop(k) for k in list(t) if k.endswith("proj.bias")])
    lm = _load(d)
    assert all(b.mixer.b_qkv is None for b in lm.model.blocks)
    # one of the three biases alone is accepted, the others count as zero
    d2 = make_model_dir(tmp_path / "x", "A")
    _rewrite(d2, lambda t: [t.pop(k) for k in list(t) if k.endswith("k_proj.bias") or k.endswith("v_proj.bias")])
    lm = _load(d2)
    assert lm.model.blocks[0].mixer.b_qkv[64:].abs().max() == 0 and lm.model.blocks[0].mixer.b_qkv[:64].abs().max() > 0
    # untied model without its head: missing
    d3 = make_model_dir(tmp_path / "y", "B")
    _rewrite(d3, lambda t: t.pop("lm_head.weight"))
    with pytest.raises(WeightsError, match="lm_head.weight"):
        _load(d3)
    # tie_word_embeddings absent: the head tensor decides (crates/mach-model/src/loader.rs:1025-1033)
    cfg = json.load(open(os.path.join(d3, "config.json")))
    del cfg["tie_word_embeddings"]
    json.dump(cfg, open(os.path.join(d3, "config.json"), "w"))
    lm = _load(d3)
    assert lm.model.head.weight is None
    # tied model that also stores a head: accepted, the table is used
    d4 = make_model_dir(tmp_path / "z", "A")
    _rewrite(d4, lambda t: t.__setitem__("lm_head.weight", torch.zeros(512, 64)))
    assert _load(d4).model.head.weight is None


def test_dtype_roles(tmp_path):
    """Matrices take the element type of the run; vectors stay 32-bit."""
    d = make_model_dir(tmp_path, "A", torch.bfloat16)
    from machserve_amd.engine import load_model
    lm = load_model(d, dtype="bfloat16", device="cpu", page_size=16, num_pages=4, ops=EmulatedOps(torch.bfloat16))
    assert lm.model.embedding.weight.dtype == torch.bfloat16
    assert lm.model.blocks[0].mixer.w_qkv.dtype == torch.bfloat16
    assert lm.model.final_norm.weight.dtype == torch.float32
    assert lm.model.blocks[0].mixer.b_qkv.dtype == torch.float32
    lm32 = _load(d)
    assert lm32.model.embedding.weight.dtype == torch.float32


def _write_raw(path, header: bytes, data: bytes = b""):
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(header)) + header + data)


def test_safetensors_corruption_is_an_error_not_a_crash(tmp_path):
    """crates/mach-model/tests/load_safetensors.rs:620-731."""
    from machserve_amd.weights import SafetensorsError, SafetensorsFile
    p = str(tmp_path / "m.safetensors")
    open(p, "wb").write(b"\x01\x02")
    with pytest.raises(SafetensorsError, match="truncated"):
        SafetensorsFile(p)
    open(p, "wb").write(struct.pack("<Q", 1 << 40))
    with pytest.raises(SafetensorsError, match="cap"):
        SafetensorsFile(p)
    open(p, "wb").write(struct.pack("<Q", 100) + b"{}")
    with pytest.raises(SafetensorsError, match="truncated header"):
        SafetensorsFile(p)
    _write_raw(p, b"{not json")
    with pytest.raises(SafetensorsError, match="JSON"):
        SafetensorsFile(p)
    _write_raw(p, b'{"a":{"dtype":"F32","shape":[2],"data_offsets":[0,8]},"a":{"dtype":"F32","shape":[2],"data_offsets":[0,8]}}', b"\0" * 8)
    with pytest.raises(SafetensorsError, match="duplicate"):
        SafetensorsFile(p)
    _write_raw(p, b'{"a":{"dtype":"F32","shape":[4],"data_offsets":[0,16]}}', b"\0" * 8)
    with pytest.raises(SafetensorsError, match="outside"):
        SafetensorsFile(p)
    _write_raw(p, b'{"a":{"dtype":"F32","shape":[3],"data_offsets":[0,8]}}', b"\0" * 8)
    with pytest.raises(SafetensorsError, match="bytes for shape"):
        SafetensorsFile(p)
    _write_raw(p, b'{"a":{"dtype":"F8_E4M3","shape":[8],"data_offsets":[0,8]}}', b"\0" * 8)
    with pytest.raises(SafetensorsError, match="unsupported dtype"):
        SafetensorsFile(p)
    _write_raw(p, b'{"__metadata__":{"format":"pt"},"a":{"dtype":"I64","shape":[1],"data_offsets":[0,8]}}', struct.pack("<q", 7))
    assert SafetensorsFile(p).tensor("a").item() == 7


def test_shards_equal_single_file_and_renaming(tmp_path):
    """crates/mach-model/tests/load_safetensors.rs:554; prefix rule loader.rs:52-57."""
    from safetensors.torch import load_file, save_file
    from machserve_amd.weights import Checkpoint, SafetensorsError
    d = make_model_dir(tmp_path, "A")
    whole = load_file(os.path.join(d, "model.safetensors"))
    names = sorted(whole)
    sh = tmp_path / "shards"
    sh.mkdir()
    save_file({n: whole[n] for n in names[::2]}, str(sh / "model-00001-of-00002.safetensors"))
    save_file({n.replace("model.", "model.language_model.", 1): whole[n] for n in names[1::2]},
              str(sh / "model-00002-of-00002.safetensors"))
    ck = Checkpoint(str(sh))
    assert sorted(ck.names()) == names and all(torch.equal(ck.tensor(n), whole[n]) for n in names)
    save_file({names[0]: whole[names[0]]}, str(sh / "model-00003.safetensors"))
    with pytest.raises(SafetensorsError, match="appears in"):
        Checkpoint(str(sh))


def test_the_folders_index_is_checked_against_its_files(tmp_path):
    """crates/mach-model/src/loader.rs:327-502: a right index passes; every disagreement between
    ``model.safetensors.index.json`` and the shards is reported, all in one message."""
    from safetensors.torch import load_file, save_file
    from machserve_amd.engine import load_model
    from machserve_amd.weights import Checkpoint, SafetensorsError
    d = make_model_dir(tmp_path, "A")
    whole = load_file(os.path.join(d, "model.safetensors"))
    names = sorted(whole)
    sh = tmp_path / "indexed"
    sh.mkdir()
    files = ["model-00001-of-00002.safetensors", "model-00002-of-00002.safetensors"]
    save_file({n: whole[n] for n in names[::2]}, str(sh / files[0]))
    save_file({n: whole[n] for n in names[1::2]}, str(sh / files[1]))
    total = sum(t.numel() * t.element_size() for t in whole.values())
    weight_map = {n: files[i % 2] for i, n in enumerate(names)}

    def write(wm, total_size=total):
        (sh / "model.safetensors.index.json").write_text(json.dumps({"metadata": {"total_size": total_size}, "weight_map": wm}))

    write(weight_map)
    ck = Checkpoint(str(sh))
    assert sorted(ck.names()) == names
    (sh / "config.json").write_text(open(os.path.join(d, "config.json")).read())
    load_model(str(sh), dtype="float32", device="cpu", page_size=16, num_pages=2, ops=EmulatedOps())   # and the model loads from it
    # several disagreements at once: a tensor the index does not list, one listed in the other shard, one that
    # no shard holds, and a wrong total
    wm = dict(weight_map)
    del wm[names[0]]
    wm[names[1]] = files[0]
    wm["model.layers.9.ghost.weight"] = files[1]
    write(wm, total + 4)
    with pytest.raises(SafetensorsError) as e:
        Checkpoint(str(sh))
    msg = str(e.value)
    assert f"{names[0]!r} of {files[0]} is absent from the index" in msg
    assert f"{names[1]!r} lies in {files[1]}, the index lists it in {files[0]}" in msg
    assert "'model.layers.9.ghost.weight' is listed in" in msg and "no shard holds it" in msg
    assert f"total_size = {total + 4}" in msg and f"describe {total} bytes" in msg
    # a shard that is missing, a file that is not indexed
    write({**weight_map, "x": "model-00003-of-00002.safetensors"})
    with pytest.raises(SafetensorsError, match="named by the index but missing"):
        Checkpoint(str(sh))
    write({n: files[0] for n in names[::2]})
    with pytest.raises(SafetensorsError, match="'model-00002-of-00002.safetensors' is not named by the index"):
        Checkpoint(str(sh))
    # a shard named by a path, and a broken index
    write({**weight_map, "y": "../elsewhere.safetensors"})
    with pytest.raises(SafetensorsError, match="beside the index"):
        Checkpoint(str(sh))
    (sh / "model.safetensors.index.json").write_text("{\"weight_map\": 3}")
    with pytest.raises(SafetensorsError, match="weight_map"):
        Checkpoint(str(sh))
    # a single file is read on its own, whatever index lies beside it
    assert sorted(Checkpoint(str(sh / files[0])).names()) == names[::2]


def test_random_weights_command(tmp_path):
    from safetensors.torch import load_file
    from machserve_amd.cli import main
    from machserve_amd.weights import random_tensor_dict
    from machserve_amd.config import config_from_dict
    cfg = tmp_path / "c.json"
    cfg.write_text(json.dumps(TINY_B))
    assert main(["random-weights", "--config", str(cfg), "--seed", "5", "--out", str(tmp_path / "m"), "--dtype", "bf16"]) == 0
    got = load_file(str(tmp_path / "m" / "model.safetensors"))
    want = random_tensor_dict(config_from_dict(dict(TINY_B)), 5, torch.bfloat16)
    assert sorted(got) == sorted(want) and all(torch.equal(got[k], want[k]) for k in got)
    assert json.load(open(tmp_path / "m" / "config.json"))["torch_dtype"] == "bfloat16"
