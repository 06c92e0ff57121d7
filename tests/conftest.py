import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


# Tiny Llama configurations that differ in every size and option.  A and B are the two the
# baseline names (B's head size 24 is not a multiple of 16: only the plain attention kernel
# takes it); C has a width, a vocabulary and an intermediate size that are no powers of two and
# a head size of 48.
TINY_A = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=256, hidden_size=64,
    intermediate_size=176, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
    head_dim=16, rms_norm_eps=1e-5, rope_theta=10000.0, max_position_embeddings=512,
    tie_word_embeddings=True, hidden_act="silu", torch_dtype="bfloat16", eos_token_id=255,
)
TINY_B = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=384, hidden_size=96,
    intermediate_size=256, num_hidden_layers=3, num_attention_heads=4, num_key_value_heads=1,
    head_dim=24, rms_norm_eps=1e-6, rope_theta=500000.0, max_position_embeddings=256,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=64),
    tie_word_embeddings=False, hidden_act="silu", torch_dtype="bfloat16", eos_token_id=[382, 383],
)
TINY_C = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=389, hidden_size=120,
    intermediate_size=250, num_hidden_layers=4, num_attention_heads=6, num_key_value_heads=3,
    head_dim=48, rms_norm_eps=3e-6, rope_theta=20000.0, max_position_embeddings=1024,
    rope_scaling=dict(rope_type="llama3", factor=4.0, low_freq_factor=1.0, high_freq_factor=2.0,
                      original_max_position_embeddings=128),
    tie_word_embeddings=False, hidden_act="silu", torch_dtype="bfloat16",
)
# head size 32: the sizes at which the product epilogues and the workgroup attention kernel that
# need multiples of 32 take part (the other three have 16, 24 and 48)
TINY_D = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=301, hidden_size=160,
    intermediate_size=208, num_hidden_layers=2, num_attention_heads=5, num_key_value_heads=1,
    head_dim=32, rms_norm_eps=2e-5, rope_theta=300000.0, max_position_embeddings=512,
    rope_scaling=dict(rope_type="llama3", factor=16.0, low_freq_factor=1.0, high_freq_factor=8.0,
                      original_max_position_embeddings=256),
    tie_word_embeddings=True, hidden_act="silu", torch_dtype="bfloat16",
)
# Two layers at the head sizes and with widths of the order of the served models (64 as in the 1B
# shape, 128 as in the 3B and 8B shapes): here the matrix-core attention kernels, the few-rows
# products with their fused epilogues and the vendor products are the ones that run.
MID_E = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=2003, hidden_size=512,
    intermediate_size=1536, num_hidden_layers=2, num_attention_heads=8, num_key_value_heads=2,
    head_dim=64, rms_norm_eps=1e-5, rope_theta=500000.0, max_position_embeddings=2048,
    rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=512),
    tie_word_embeddings=True, hidden_act="silu", torch_dtype="bfloat16",
)
MID_F = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=1501, hidden_size=640,
    intermediate_size=1056, num_hidden_layers=2, num_attention_heads=6, num_key_value_heads=2,
    head_dim=128, rms_norm_eps=1e-6, rope_theta=500000.0, max_position_embeddings=2048,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=1024),
    tie_word_embeddings=False, hidden_act="silu", torch_dtype="bfloat16",
)
TINY = {"A": (TINY_A, 11), "B": (TINY_B, 23), "C": (TINY_C, 37), "D": (TINY_D, 41),
        "E": (MID_E, 53), "F": (MID_F, 59)}


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders of the test configurations, written by the random-weights mode."""
    from kv_cache_optimization_for_llm_amd.weights.random_init import write_random_model
    base = tmp_path_factory.mktemp("models")
    out = {}
    for name, (cfg, seed) in TINY.items():
        out[name] = write_random_model(str(base / name), cfg, seed)
    return out


@pytest.fixture(scope="session")
def sharp_model_dirs(tmp_path_factory):
    """The same configurations with matrices N(0, 1 / sqrt(in)) instead of N(0, 0.02).  With the
    small weights every attention row is nearly uniform and a tied model's best next token is its
    input token: generated tokens would come out the same with attention switched off.  With
    these, scores spread over several units, the picks depend on the keys, and an engine that
    drops or misplaces one picks other tokens than the plain implementation."""
    from kv_cache_optimization_for_llm_amd.weights.random_init import write_random_model
    base = tmp_path_factory.mktemp("sharp_models")
    return {name: write_random_model(str(base / name), cfg, seed, gain=1.0) for name, (cfg, seed) in TINY.items()}


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("a test marked gpu ran without a GPU; run GPU tests with -m gpu on an MI355X")
    return torch.device("cuda:0")
