"""Configuration and registry (no GPU)."""
import json
import os

import pytest

from picolm_amd.config import (ConfigError, LlamaConfig, known_architectures, read_config_json, register_architecture,
                               resolve, unregister_architecture)
import picolm_amd.engine.llama  # noqa: F401  registers LlamaForCausalLM
import tiny


def test_reads_every_key_of_both_tiny_configs():
    a = LlamaConfig.from_dict(tiny.TINY_A)
    b = LlamaConfig.from_dict(tiny.TINY_B)
    assert (a.hidden_size, a.intermediate_size, a.num_attention_heads, a.num_key_value_heads) == (64, 176, 4, 2)
    assert (a.num_hidden_layers, a.vocab_size, a.head_dim, a.rms_norm_eps, a.rope_theta) == (2, 256, 16, 1e-5, 10000.0)
    assert a.rope_scaling is None and a.tie_word_embeddings and a.max_position_embeddings == 128
    assert a.eos_token_ids == (2,) and a.rope_style == "pairwise"
    assert b.rope_scaling.factor == 8.0 and b.rope_scaling.original_max_position_embeddings == 64
    assert b.eos_token_ids == (3, 7) and not b.tie_word_embeddings and b.rope_style == "half"
    for k in ("hidden_size", "intermediate_size", "num_attention_heads", "num_hidden_layers", "vocab_size",
              "rms_norm_eps", "rope_theta", "max_position_embeddings"):
        assert getattr(a, k) != getattr(b, k), k


def test_defaults_follow_picolm():
    d = dict(architectures=["LlamaForCausalLM"], hidden_size=64, intermediate_size=96, num_attention_heads=4,
             num_hidden_layers=1, vocab_size=50)
    c = LlamaConfig.from_dict(d)
    assert c.num_key_value_heads == 4            # absent -> as many as heads
    assert c.head_dim == 16                      # hidden / heads   (safetensors.c:76)
    assert c.rms_norm_eps == 1e-6                # safetensors.c:78
    assert c.rope_theta == 10000.0               # safetensors.c:102
    assert c.bos_token_id == 1 and c.eos_token_ids == (2,)     # safetensors.c:309-310
    assert c.max_position_embeddings == 4096     # safetensors.c:495
    c2 = LlamaConfig.from_dict(dict(d, rms_norm_eps=0, rope_theta=-1.0, head_dim=0))
    assert c2.rms_norm_eps == 1e-6 and c2.rope_theta == 10000.0 and c2.head_dim == 16


def test_text_config_is_preferred():
    inner = dict(tiny.TINY_A)
    c = LlamaConfig.from_dict({"architectures": ["LlamaForCausalLM"], "text_config": inner, "hidden_size": 999})
    assert c.hidden_size == 64


def test_round_trip():
    for cfg in (tiny.TINY_A, tiny.TINY_B, tiny.TINY_C):
        c = LlamaConfig.from_dict(cfg)
        assert LlamaConfig.from_dict(json.loads(json.dumps(c.to_dict()))) == c


@pytest.mark.parametrize("change,word", [
    (dict(num_key_value_heads=3), "num_key_value_heads"),
    (dict(head_dim=15), "head_dim"),
    (dict(vocab_size=0), "vocab_size"),
    (dict(num_hidden_layers=-1), "num_hidden_layers"),
    (dict(hidden_size="wide"), "hidden_size"),
    (dict(rope_scaling={"rope_type": "yarn", "factor": 2}), "rope_scaling"),
    (dict(rope_scaling={"rope_type": "llama3", "factor": 8}), "low_freq_factor"),
    (dict(rope_scaling={"rope_type": "llama3", "factor": 8, "low_freq_factor": 4, "high_freq_factor": 1,
                        "original_max_position_embeddings": 64}), "high_freq_factor"),
    (dict(rope_style="spiral"), "rope_style"),
    (dict(eos_token_id=100000), "eos_token_id"),
    (dict(torch_dtype="int8"), "torch_dtype"),
])
def test_each_fault_names_its_key(change, word):
    with pytest.raises(ConfigError) as e:
        LlamaConfig.from_dict(dict(tiny.TINY_A, **change))
    assert word in str(e.value)


def test_missing_key_is_named():
    d = dict(tiny.TINY_A)
    del d["intermediate_size"]
    with pytest.raises(ConfigError, match="intermediate_size"):
        LlamaConfig.from_dict(d)


def test_registry_resolves_by_architecture_name(tmp_path):
    assert "LlamaForCausalLM" in known_architectures()
    arch = resolve(tiny.TINY_A)
    assert arch.parse_config(tiny.TINY_A).hidden_size == 64
    with pytest.raises(ConfigError, match="MambaForCausalLM.*LlamaForCausalLM"):
        resolve(dict(tiny.TINY_A, architectures=["MambaForCausalLM"]))
    with pytest.raises(ConfigError, match="architectures"):
        resolve({k: v for k, v in tiny.TINY_A.items() if k != "architectures"})
    register_architecture("ToyForTests", lambda d: d, lambda c: c)
    try:
        assert resolve({"architectures": ["ToyForTests"]}).name == "ToyForTests"
        with pytest.raises(ConfigError, match="already registered"):
            register_architecture("ToyForTests", None, None)
    finally:
        unregister_architecture("ToyForTests")
    with pytest.raises(ConfigError, match="no config.json"):
        read_config_json(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not JSON"):
        read_config_json(str(tmp_path))


def test_model_structure_comes_from_the_configuration():
    from picolm_amd.engine import build_from_config_dict
    for cfg in (tiny.TINY_A, tiny.TINY_B, tiny.TINY_C):
        m = build_from_config_dict(cfg)
        c = m.config
        assert len(m.blocks) == c.num_hidden_layers
        att = m.blocks[0].mixer
        assert (att.H, att.G, att.d) == (c.num_attention_heads, c.num_key_value_heads, c.head_dim)
        assert m.blocks[0].mixer_norm.eps == c.rms_norm_eps and m.blocks[0].ffn.F == c.intermediate_size
        assert att.position.theta == c.rope_theta and att.position.style == c.rope_style
        specs = {s.name: s for s in m.tensor_specs()}
        assert specs["model.embed_tokens.weight"].shape == (c.vocab_size, c.hidden_size)
        assert specs[f"model.layers.{c.num_hidden_layers - 1}.mlp.down_proj.weight"].shape == (c.hidden_size, c.intermediate_size)
        g = m.cache_spec.kv_groups
        assert len(g) == 1 and g[0].n_entries == c.num_hidden_layers and g[0].n_kv_heads == c.num_key_value_heads
        written = [s for s in specs.values() if s.init is not None]
        assert len(written) == 2 + 9 * c.num_hidden_layers + (0 if c.tie_word_embeddings else 1)


def test_head_size_limits_are_named_when_the_configuration_is_read():
    d = dict(architectures=["LlamaForCausalLM"], hidden_size=100, intermediate_size=96, num_attention_heads=6,
             num_hidden_layers=1, vocab_size=50)
    with pytest.raises(ConfigError, match="hidden_size.*not divisible.*num_attention_heads"):
        LlamaConfig.from_dict(d)                                   # picolm would floor to 16 silently
    assert LlamaConfig.from_dict(dict(d, head_dim=20)).head_dim == 20     # given: no division takes place
    assert LlamaConfig.from_dict(dict(d, num_attention_heads=5)).head_dim == 20      # any even size, not only 16s
    with pytest.raises(ConfigError, match="head_dim.*1024"):
        LlamaConfig.from_dict(dict(d, head_dim=1026))
    assert LlamaConfig.from_dict(dict(d, head_dim=1024)).head_dim == 1024
    assert LlamaConfig.from_dict(dict(d, head_dim=320)).head_dim == 320              # four times picolm's own bound


def test_modules_named_in_the_environment_register_their_architectures(tmp_path, monkeypatch):
    """An architecture outside the package: its module is named in PICOLM_ARCHITECTURES and
    imported before the first name is looked up; one that cannot be imported is an error that
    names it."""
    import subprocess
    import sys
    from picolm_amd.config import import_architecture_modules
    (tmp_path / "my_arch.py").write_text(
        "from picolm_amd.config import register_architecture, LlamaConfig\n"
        "register_architecture('MyLM', LlamaConfig.from_dict, lambda cfg: None)\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, PYTHONPATH=os.pathsep.join([str(tmp_path), root]), PICOLM_ARCHITECTURES=" my_arch ,")
    out = subprocess.run([sys.executable, "-c", "from picolm_amd import known_architectures; print(known_architectures())"],
                         env=env, capture_output=True, text=True)
    assert out.returncode == 0 and "'LlamaForCausalLM', 'MyLM'" in out.stdout, out.stderr
    out = subprocess.run([sys.executable, "-c", "from picolm_amd import known_architectures; print(known_architectures())"],
                         env=dict(env, PICOLM_ARCHITECTURES="no_such_module_here"), capture_output=True, text=True)
    assert out.returncode != 0 and "PICOLM_ARCHITECTURES: cannot import 'no_such_module_here'" in out.stderr
    assert import_architecture_modules("") == [] and import_architecture_modules(" , ") == []
    with pytest.raises(ConfigError, match="cannot import 'no_such_module_here'"):
        import_architecture_modules("no_such_module_here")


def test_options_that_the_layers_do_not_have_are_refused():
    """Bias tensors and other activations than silu: picolm ignores the keys and has neither; a
    config.json that asks for them is refused by name, not computed without them."""
    d = dict(tiny.TINY_A)
    assert LlamaConfig.from_dict(dict(d, attention_bias=False, mlp_bias=False, hidden_act="silu")).hidden_size == 64
    for key, value, word in (("attention_bias", True, "attention_bias"), ("mlp_bias", True, "mlp_bias"), ("hidden_act", "gelu", "hidden_act")):
        with pytest.raises(ConfigError, match=word):
            LlamaConfig.from_dict(dict(d, **{key: value}))
