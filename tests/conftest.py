import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))
if str(ROOT / "tests") not in sys.path:
    sys.path.insert(0, str(ROOT / "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


# Two tiny configurations of the architecture that differ in every size and option:
# layers, width, heads, groups, head size (heads * head size equal to / different from
# the width), intermediate size, vocabulary (one not a power of two), theta, eps,
# tied / untied head, page size.  A third has the head size and page size (64) of the
# kernels that only serve such sizes (prompt attention with tiles shared through LDS),
# one kv head for all q heads and room for 512 positions.
TINY_A = dict(vocab_size=256, hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
              num_key_value_heads=2, head_dim=16, max_position_embeddings=128, rms_norm_eps=1e-6, rope_theta=1e4,
              tie_word_embeddings=True)
TINY_B = dict(vocab_size=503, hidden_size=96, intermediate_size=224, num_hidden_layers=3, num_attention_heads=8,
              num_key_value_heads=2, head_dim=32, max_position_embeddings=256, rms_norm_eps=1e-5, rope_theta=1e6,
              tie_word_embeddings=False)
TINY_C = dict(vocab_size=300, hidden_size=128, intermediate_size=160, num_hidden_layers=2, num_attention_heads=4,
              num_key_value_heads=1, head_dim=64, max_position_embeddings=512, rms_norm_eps=1e-6, rope_theta=5e5,
              tie_word_embeddings=False)
TINY = {"A": (TINY_A, 16, 0), "B": (TINY_B, 8, 1), "C": (TINY_C, 64, 2)}   # name -> (config, page size, weight seed)


@pytest.fixture(scope="session")
def tiny_dirs(tmp_path_factory):
    """Model folders (config.json, model.safetensors) of the tiny configurations, written once per session."""
    import torch
    from vosti_amd.config import Qwen3Config
    from vosti_amd.weights import write_random_model
    out = {}
    for name, (cfg, page, seed) in TINY.items():
        d = tmp_path_factory.mktemp(f"tiny_{name}")
        write_random_model(Qwen3Config(**cfg), seed, d, dtype=torch.bfloat16)
        out[name] = d
    return out
