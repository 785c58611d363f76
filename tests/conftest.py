import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


# Two tiny GPT-2 configurations that differ in every size and option.
TINY_A = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, n_embd=64, n_head=4,
              n_inner=None, vocab_size=512, n_positions=128, layer_norm_epsilon=1e-5,
              activation_function="gelu_new", eos_token_id=511, bos_token_id=511)
TINY_B = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=3, n_embd=96, n_head=3,
              n_inner=320, vocab_size=1000, n_positions=256, layer_norm_epsilon=1e-6,
              activation_function="gelu", eos_token_id=999, bos_token_id=999)
TINY = {"a": (TINY_A, 0, 4), "b": (TINY_B, 1, 8)}     # config, seed, page size


# The layer sizes of GPT-2 small and GPT-2 XL (width, heads, inner width, vocabulary, positions as in the
# real models; two layers): the sizes the benchmarks run, where other kernels and tile shapes are chosen
# than at the tiny sizes.
REAL_SMALL = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, n_embd=768, n_head=12,
                  n_inner=3072, vocab_size=50257, n_positions=1024, layer_norm_epsilon=1e-5,
                  activation_function="gelu_new", eos_token_id=50256, bos_token_id=50256)
REAL_XL = dict(REAL_SMALL, n_embd=1600, n_head=25, n_inner=6400)
REAL = {"small2": (REAL_SMALL, 2, 16), "xl2": (REAL_XL, 4, 16)}
CONFIGS = {**TINY, **REAL}


@pytest.fixture(scope="session")
def real_model_dirs(tmp_path_factory):
    """Model folders at GPT-2 small and XL layer sizes (two layers each), random weights."""
    from mini_llm_amd import write_random_model
    out = {}
    for name, (cfg, seed, _) in REAL.items():
        d = tmp_path_factory.mktemp(f"real_{name}")
        write_random_model(dict(cfg), str(d), seed)
        out[name] = str(d)
    return out


@pytest.fixture(scope="session")
def tiny_model_dirs(tmp_path_factory):
    """Model folders of the two tiny configurations, random weights, made once per session."""
    from mini_llm_amd import write_random_model
    out = {}
    for name, (cfg, seed, _) in TINY.items():
        d = tmp_path_factory.mktemp(f"tiny_{name}")
        write_random_model(dict(cfg), str(d), seed)
        out[name] = str(d)
    return out
