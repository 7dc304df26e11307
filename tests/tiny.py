"""The tiny configurations the tests use, their random model folders, and helpers that run
the plain implementation on them.  The two configurations differ in every size and option:
head counts and grouping, widths that are no power of two, layers, vocabulary, eps, rope
base and scaling, pairing style, tied or separate head, weight spread."""
from __future__ import annotations

import json
import os

import numpy as np

TINY_A = dict(
    architectures=["LlamaForCausalLM"], hidden_size=64, intermediate_size=176, num_attention_heads=4,
    num_key_value_heads=2, num_hidden_layers=2, vocab_size=256, head_dim=16, rms_norm_eps=1e-5,
    rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=True, max_position_embeddings=128,
    eos_token_id=2, rope_style="pairwise")
TINY_A_WEIGHTS = dict(seed=0, std=0.02, norm_sigma=0.0)

TINY_B = dict(
    architectures=["LlamaForCausalLM"], hidden_size=96, intermediate_size=256, num_attention_heads=6,
    num_key_value_heads=6, num_hidden_layers=3, vocab_size=384, head_dim=16, rms_norm_eps=1e-6,
    rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=64),
    tie_word_embeddings=False, max_position_embeddings=256, eos_token_id=[3, 7], rope_style="half")
TINY_B_WEIGHTS = dict(seed=1, std=0.05, norm_sigma=0.1)

# a third one for the sizes the other two share: head size 32 (48 heads*dim != hidden), GQA 3:1,
# odd layer count, a vocabulary that is no multiple of anything
TINY_C = dict(
    architectures=["LlamaForCausalLM"], hidden_size=80, intermediate_size=112, num_attention_heads=3,
    num_key_value_heads=1, num_hidden_layers=1, vocab_size=131, head_dim=32, rms_norm_eps=1e-4,
    rope_theta=1000.0, rope_scaling=None, tie_word_embeddings=False, max_position_embeddings=512,
    eos_token_id=5, rope_style="pairwise")
TINY_C_WEIGHTS = dict(seed=2, std=0.08, norm_sigma=0.2)

# a fourth whose widths are multiples of 128 and 64, as real checkpoints' are: the kernels that
# want such widths (the product with the norm inside, tiles loaded straight into LDS, split K,
# matrix-core attention at head size 64) run in the engine only with this one
TINY_D = dict(
    architectures=["LlamaForCausalLM"], hidden_size=256, intermediate_size=320, num_attention_heads=4,
    num_key_value_heads=2, num_hidden_layers=2, vocab_size=515, head_dim=64, rms_norm_eps=1e-5,
    rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=False, max_position_embeddings=512,
    eos_token_id=1, rope_style="half")
TINY_D_WEIGHTS = dict(seed=3, std=0.04, norm_sigma=0.3)

# a fifth with the head size and grouping of the large checkpoints (128, four query heads a KV
# head) and a width of 1024: the kernels at the sizes they have there, and the norm that decode
# batches of 17 to 64 rows split between the products around it
TINY_E = dict(
    architectures=["LlamaForCausalLM"], hidden_size=1024, intermediate_size=1536, num_attention_heads=8,
    num_key_value_heads=2, num_hidden_layers=2, vocab_size=1031, head_dim=128, rms_norm_eps=1e-5,
    rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=128),
    tie_word_embeddings=False, max_position_embeddings=1024, eos_token_id=2, rope_style="half")
TINY_E_WEIGHTS = dict(seed=4, std=0.03, norm_sigma=0.2)

# a sixth whose head size is given by hidden / heads and is no multiple of 16 (20), with an odd
# vocabulary below 100: the vector-ALU attention with a partly filled column group in both
# precisions, next to products on the matrix cores (the widths are multiples of 8)
TINY_F = dict(
    architectures=["LlamaForCausalLM"], hidden_size=120, intermediate_size=200, num_attention_heads=6,
    num_key_value_heads=3, num_hidden_layers=2, vocab_size=97, rms_norm_eps=1e-5,
    rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=False, max_position_embeddings=512,
    eos_token_id=2, rope_style="half")
TINY_F_WEIGHTS = dict(seed=5, std=0.06, norm_sigma=0.1)

# a seventh with a head wider than the 256 columns that the attention kernel holds in LDS at a
# time (picolm's own bound, picolm/model_attention.c:163): keys, values and the merge of a split
# context go through in pieces
TINY_G = dict(
    architectures=["LlamaForCausalLM"], hidden_size=144, intermediate_size=208, num_attention_heads=3,
    num_key_value_heads=1, num_hidden_layers=2, vocab_size=203, head_dim=328, rms_norm_eps=1e-6,
    rope_theta=100000.0, rope_scaling=None, tie_word_embeddings=True, max_position_embeddings=1024,
    eos_token_id=4, rope_style="pairwise")
TINY_G_WEIGHTS = dict(seed=6, std=0.05, norm_sigma=0.1)

CONFIGS = {"A": (TINY_A, TINY_A_WEIGHTS), "B": (TINY_B, TINY_B_WEIGHTS), "C": (TINY_C, TINY_C_WEIGHTS),
           "D": (TINY_D, TINY_D_WEIGHTS), "E": (TINY_E, TINY_E_WEIGHTS), "F": (TINY_F, TINY_F_WEIGHTS),
           "G": (TINY_G, TINY_G_WEIGHTS)}


def make_model_dir(tmp_path, which: str, dtype: str = "bfloat16") -> str:
    from picolm_amd import LlamaConfig, write_random_model
    cfg_dict, w = CONFIGS[which]
    cfg = LlamaConfig.from_dict(cfg_dict)
    out = os.path.join(str(tmp_path), f"tiny_{which}_{dtype}")
    if not os.path.exists(os.path.join(out, "model.safetensors")):
        write_random_model(cfg, out, dtype=dtype, **w)
    return out


def read_weights_f64(model_dir: str) -> dict:
    """The folder's tensors as float64 arrays, read with the safetensors package (not with
    the engine's own reader)."""
    import torch
    from safetensors import safe_open
    out = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for k in f.keys():
            out[k] = f.get_tensor(k).to(torch.float64).numpy()
    return out


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def plain_logits(model_dir: str, tokens) -> np.ndarray:
    from plain import llama_plain as P
    return P.forward(read_weights_f64(model_dir), read_config(model_dir), tokens)


def random_tokens(rng: np.random.Generator, n: int, vocab: int) -> list[int]:
    return [int(t) for t in rng.integers(0, vocab, size=n)]


def spread(hidden_size: int, std: float) -> float:
    """hidden_size * std^2: the variance of a projected value (a query's or key's element, an
    attention score) when the weights are N(0, std^2) and the rows have unit RMS.  The engine's
    distance from the plain implementation grows with its square root in both precisions (measured
    at widths of 256 to 2,048 and std of 0.01 to 0.08: in bfloat16 from 0.3 % of the largest logit
    at a spread of 0.03 to 4.6 % at 13, in 32-bit from 6e-7 to 2e-5 of it), as rounding errors of
    values that large do; the tiny configurations all lie below 1."""
    return hidden_size * std * std


def spread_of(which: str) -> float:
    cfg, w = CONFIGS[which]
    return spread(cfg["hidden_size"], w["std"])


def tolerance(dtype: str, ref, weight_spread: float = 0.0, layers: int = 1) -> float:
    """The largest distance of a logit from the plain implementation's that the tests accept:
    2e-5 (32-bit) or 2e-2 (bfloat16) of the largest logit in absolute value (of 1 if that is
    smaller), times the square root of the weights' spread where that exceeds 1 (see `spread`),
    times `depth_factor(layers)`."""
    scale = max(1.0, float(np.abs(ref).max()))
    return (2e-5 if dtype == "float32" else 2e-2) * scale * max(1.0, float(np.sqrt(weight_spread))) * depth_factor(layers)


def depth_factor(layers: int) -> float:
    """What depth adds to the bound: sqrt(layers / 4) beyond four layers.  Every layer's roundings
    are independent of the others' and add in quadrature: at the Llama-3.1-8B layer sizes the
    bfloat16 engine's largest distance from the 32-bit engine is 0.43 to 0.49 of the depth-less
    bound at one layer, 0.71 at 4, 1.02 at 8, 1.44 at 16 and 2.2 at 32 (0.36 sqrt(layers) from four
    layers on), and the 32-bit engine's distance from the plain implementation 0.29 of its bound
    at 4 layers and 0.80 at 32.  Every tiny configuration has at most four layers."""
    return max(1.0, float(np.sqrt(layers / 4.0)))
