"""Weights: the safetensors container, the check against a model's declared tensors, the
random-weights mode (no GPU)."""
import json
import os
import struct

import numpy as np
import pytest
import torch

import tiny
from picolm_amd import LlamaConfig, write_random_model
from picolm_amd.engine import build_from_config_dict, tensor_specs_for
from picolm_amd.weights import (Checkpoint, SafetensorsError, SafetensorsFile, TensorDict, WeightFetcher, WeightsError, stored_dtype,
                                check_specs, random_tensors, write_safetensors)


def test_container_round_trip_with_the_safetensors_package(tmp_path):
    from safetensors.torch import load_file, save_file
    g = torch.Generator().manual_seed(0)
    tensors = {"a.weight": torch.randn(3, 5, generator=g).to(torch.bfloat16), "b": torch.randn(7, generator=g),
               "ids": torch.arange(6, dtype=torch.int32).reshape(2, 3)}
    ours = str(tmp_path / "ours.safetensors")
    write_safetensors(ours, tensors, metadata={"format": "pt"})
    theirs = load_file(ours)                                    # their reader takes our file
    for k, v in tensors.items():
        assert torch.equal(theirs[k], v)
    their_file = str(tmp_path / "theirs.safetensors")
    save_file(tensors, their_file)
    sf = SafetensorsFile(their_file)                            # our reader takes their file
    assert sorted(sf.names()) == sorted(tensors)
    for k, v in tensors.items():
        assert sf.info(k) == (v.dtype, tuple(v.shape))
        assert torch.equal(sf.tensor(k), v)


def test_container_faults_are_reported(tmp_path):
    p = str(tmp_path / "x.safetensors")
    with pytest.raises(SafetensorsError, match="no such file"):
        SafetensorsFile(p)
    open(p, "wb").write(b"abc")
    with pytest.raises(SafetensorsError, match="too short"):
        SafetensorsFile(p)
    open(p, "wb").write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(p)
    hdr = json.dumps({"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}).encode()
    open(p, "wb").write(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)      # data too short
    with pytest.raises(SafetensorsError, match="offsets"):
        SafetensorsFile(p)
    hdr = json.dumps({"t": {"dtype": "F32", "shape": [3], "data_offsets": [0, 16]}}).encode()
    open(p, "wb").write(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 16)     # size does not match the shape
    with pytest.raises(SafetensorsError, match="needs 12 bytes"):
        SafetensorsFile(p)
    hdr = json.dumps({"t": {"dtype": "Q4", "shape": [3], "data_offsets": [0, 3]}}).encode()
    open(p, "wb").write(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 3)
    with pytest.raises(SafetensorsError, match="Q4"):
        SafetensorsFile(p)


def test_random_model_folder(tmp_path):
    for which in "AB":
        d = tiny.make_model_dir(tmp_path, which)
        cfg = LlamaConfig.from_json_file(d)
        assert cfg == LlamaConfig.from_dict(dict(tiny.CONFIGS[which][0], torch_dtype="bfloat16"))
        ck = Checkpoint(d)
        check_specs(ck, tensor_specs_for(cfg))                    # the folder holds exactly what the model declares
        assert ("lm_head.weight" in ck.names()) == (not cfg.tie_word_embeddings)
        w = tiny.read_weights_f64(d)
        std, sigma = tiny.CONFIGS[which][1]["std"], tiny.CONFIGS[which][1]["norm_sigma"]
        q = w["model.layers.0.self_attn.q_proj.weight"]
        assert ck.info("model.layers.0.self_attn.q_proj.weight")[0] == torch.bfloat16
        assert abs(q.std() - std) < 0.15 * std and abs(q.mean()) < 0.2 * std
        n = w["model.layers.1.input_layernorm.weight"]
        assert (np.all(n == 1.0) if sigma == 0 else abs((n - 1).std() - sigma) < 0.5 * sigma)
    # the same seed gives the same bytes, another seed does not; a tensor does not depend on the others
    cfg = LlamaConfig.from_dict(tiny.TINY_A)
    a = dict(random_tensors(tensor_specs_for(cfg), 5))
    b = dict(random_tensors(tensor_specs_for(cfg), 5))
    c = dict(random_tensors(tensor_specs_for(cfg), 6))
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    cfg1 = LlamaConfig.from_dict(dict(tiny.TINY_A, num_hidden_layers=1))
    a1 = dict(random_tensors(tensor_specs_for(cfg1), 5))
    assert torch.equal(a1["model.layers.0.mlp.up_proj.weight"], a["model.layers.0.mlp.up_proj.weight"])


def test_one_error_lists_missing_unexpected_and_misshaped():
    cfg = LlamaConfig.from_dict(tiny.TINY_B)
    specs = tensor_specs_for(cfg)
    t = dict(random_tensors(specs, 0))
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.9.extra.weight"] = torch.zeros(2)
    t["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(5, 96, dtype=torch.bfloat16)
    t["model.layers.2.input_layernorm.weight"] = torch.zeros(96, dtype=torch.int64)
    with pytest.raises(WeightsError) as e:
        check_specs(TensorDict(t, "broken"), specs)
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"] or \
        sorted(err.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.9.extra.weight"]
    assert err.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (96, 96), (5, 96))]
    assert err.wrong_dtype == [("model.layers.2.input_layernorm.weight", "int64")]
    msg = str(err)
    for word in ("broken", "missing (2)", "unexpected (1)", "wrong shape (1)", "expected [96, 96] found [5, 96]", "int64"):
        assert word in msg


def test_head_is_optional_and_ties_to_the_embedding():
    cfg = LlamaConfig.from_dict(tiny.TINY_B)                     # untied by configuration
    specs = tensor_specs_for(cfg)
    t = dict(random_tensors(specs, 0))
    del t["lm_head.weight"]                                      # picolm ties when the tensor is absent
    check_specs(TensorDict(t), specs)
    tied = LlamaConfig.from_dict(tiny.TINY_A)
    t = dict(random_tensors(tensor_specs_for(tied), 0))
    assert "lm_head.weight" not in t
    t["lm_head.weight"] = torch.zeros(256, 64)                   # a stray copy in a tied model is accepted
    check_specs(TensorDict(t), tensor_specs_for(tied))


def test_storage_policy_and_aliases(tmp_path):
    t = {"model.language_model.a": torch.ones(2, dtype=torch.float16), "model.b": torch.ones(2, dtype=torch.float32),
         "model.c": torch.ones(2, dtype=torch.bfloat16), "model.idx": torch.arange(3, dtype=torch.int64)}
    os.makedirs(tmp_path / "m")
    write_safetensors(str(tmp_path / "m" / "model.safetensors"), t)
    ck = Checkpoint(str(tmp_path / "m"))
    assert sorted(ck.names()) == ["model.a", "model.b", "model.c", "model.idx"]        # safetensors.c:170-183
    f = WeightFetcher(ck, "cpu")
    assert f.get("model.a").dtype == torch.bfloat16              # float16 is rounded to bfloat16
    assert f.get("model.b").dtype == torch.float32               # stored in 32-bit, stays so
    assert f.get("model.c").dtype == torch.bfloat16
    assert f.get("model.idx", kind="int").dtype == torch.int32
    # the 32-bit runtime widens float16 exactly instead (picolm keeps float16 as it is,
    # safetensors.c:163-164); everything else is kept as above
    third = torch.tensor([1 / 3, 0.1], dtype=torch.float16)
    write_safetensors(str(tmp_path / "m" / "model.safetensors"), dict(t, **{"model.language_model.a": third}))
    f32 = WeightFetcher(Checkpoint(str(tmp_path / "m")), "cpu", torch.float32)
    assert f32.get("model.a").dtype == torch.float32 and torch.equal(f32.get("model.a"), third.float())
    assert f32.get("model.c").dtype == torch.bfloat16 and f32.get("model.b").dtype == torch.float32
    bf = WeightFetcher(Checkpoint(str(tmp_path / "m")), "cpu", torch.bfloat16)
    assert bf.get("model.a").dtype == torch.bfloat16 and not torch.equal(bf.get("model.a").float(), third.float())
    assert stored_dtype(torch.float16, "float", torch.float32) == torch.float32
    assert stored_dtype(torch.float16, "float", torch.bfloat16) == torch.bfloat16 == stored_dtype(torch.float16)


def test_buffers_that_are_no_parameters_are_ignored():
    cfg = LlamaConfig.from_dict(tiny.TINY_A)
    specs = tensor_specs_for(cfg)
    t = dict(random_tensors(specs, 0))
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(8)      # older checkpoints carry these
    check_specs(TensorDict(t), specs)
    t["model.layers.0.self_attn.rotary_emb.other"] = torch.ones(8)
    with pytest.raises(WeightsError) as e:
        check_specs(TensorDict(t), specs)
    assert e.value.unexpected == ["model.layers.0.self_attn.rotary_emb.other"]


def test_sharded_folder(tmp_path):
    cfg = LlamaConfig.from_dict(tiny.TINY_A)
    specs = tensor_specs_for(cfg)
    t = dict(random_tensors(specs, 3))
    names = sorted(t)
    d = tmp_path / "sharded"
    os.makedirs(d)
    halves = {"model-00001-of-00002.safetensors": names[:7], "model-00002-of-00002.safetensors": names[7:]}
    wm = {}
    for fn, ns in halves.items():
        write_safetensors(str(d / fn), {n: t[n] for n in ns})
        wm.update({n: fn for n in ns})
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": wm}))
    ck = Checkpoint(str(d))
    check_specs(ck, specs)
    assert torch.equal(ck.tensor(names[9]), t[names[9]])
    with pytest.raises(SafetensorsError, match="no model.safetensors"):
        Checkpoint(str(tmp_path))


def test_list_kv_prints_the_folders_metadata(tmp_path, capsys):
    """picolm's --list-kv (picolm/picolm.c:187): here config.json's entries and the safetensors metadata."""
    from picolm_amd import LlamaConfig, cli, write_random_model
    d = write_random_model(LlamaConfig.from_dict(tiny.TINY_A), str(tmp_path / "m"), seed=1)
    assert cli.main([d, "--list-kv"]) == 0
    out = capsys.readouterr().out.splitlines()
    assert f"config.hidden_size = {tiny.TINY_A['hidden_size']}" in out
    assert 'config.architectures = ["LlamaForCausalLM"]' in out
    assert out == sorted(out, key=lambda l: (not l.startswith("config."), l))

