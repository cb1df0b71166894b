import os
import sys

import pytest

# The vendor library's algorithm for a new shape is otherwise chosen by timing (in an engine's
# warm-up step and before a graph is recorded), which can differ from run to run and with it the
# last bits of bfloat16 results; tests want the same bits every time.
os.environ.setdefault("LYAPUNOV_AMD_GEMM_TUNE", "0")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
TESTS = os.path.dirname(os.path.abspath(__file__))
if TESTS not in sys.path:
    sys.path.insert(0, TESTS)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; runs the HIP kernels")


# Two tiny configurations that differ in every size and option: layers, width,
# heads and groups (grouped vs one shared key/value head), head size, a
# feed-forward width that is no multiple of 8, vocabulary, rope base, frequency
# scaling, tied vs separate head, eps, norm weights, page size.
TINY_A = dict(
    architectures=["LlamaForCausalLM"], vocab_size=256, hidden_size=64, intermediate_size=172, num_hidden_layers=2,
    num_attention_heads=4, num_key_value_heads=2, head_dim=16, max_position_embeddings=256, rms_norm_eps=1e-5,
    rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=True,
)
TINY_B = dict(
    architectures=["LlamaForCausalLM"], vocab_size=515, hidden_size=96, intermediate_size=256, num_hidden_layers=3,
    num_attention_heads=3, num_key_value_heads=1, head_dim=32, max_position_embeddings=512, rms_norm_eps=1e-6,
    rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=64),
    tie_word_embeddings=False,
)
# A third one whose sizes are multiples of 64, as a real model's are: only then do the steps with
# few rows take the kernels that a large model takes (the weight-streaming products with their
# fused epilogues and the norm folded into them).
TINY_C = dict(
    architectures=["LlamaForCausalLM"], vocab_size=320, hidden_size=128, intermediate_size=192, num_hidden_layers=2,
    num_attention_heads=4, num_key_value_heads=2, head_dim=32, max_position_embeddings=512, rms_norm_eps=1e-5,
    rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=True,
)
# init_std is chosen large enough that attention is peaked: with the usual 0.02
# every score is near 0, the softmax is flat, and a wrong key or a wrong
# position barely moves the logits.
TINY = {"A": (TINY_A, dict(seed=0, init_std=0.15, norm_init_std=0.0, block_size=4)),
        "B": (TINY_B, dict(seed=2, init_std=0.1, norm_init_std=0.1, block_size=16)),
        "C": (TINY_C, dict(seed=5, init_std=0.1, norm_init_std=0.1, block_size=16))}


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """name -> dtype -> folder with config.json and model.safetensors (random
    weights, written by the package's random-weights mode)."""
    from lyapunov_engine_amd.weights import write_random_model

    out = {}
    for name, (cfg, opt) in TINY.items():
        out[name] = {}
        for dtype in ("float32", "bfloat16"):
            d = tmp_path_factory.mktemp(f"tiny{name}_{dtype}")
            write_random_model(dict(cfg), str(d), opt["seed"], dtype, init_std=opt["init_std"],
                               norm_init_std=opt["norm_init_std"])
            out[name][dtype] = str(d)
    return out
