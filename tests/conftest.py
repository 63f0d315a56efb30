import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def _has_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# Two tiny configurations of the architecture that differ in every size and option.
TINY = {
    "a": dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
              intermediate_size=192, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-5,
              sliding_window=None, max_position_embeddings=4096, tie_word_embeddings=False),
    "b": dict(num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=3, head_dim=32,
              intermediate_size=320, vocab_size=384, rope_theta=1e6, rms_norm_eps=1e-6,
              sliding_window=8, max_position_embeddings=4096, tie_word_embeddings=False),
    # odd sizes: width and vocabulary that are no power of two nor a multiple of 8, one kv
    # head, tied head, adjacent pairing, windowed and full layers mixed
    "c": dict(num_hidden_layers=4, hidden_size=100, num_attention_heads=5, num_key_value_heads=1, head_dim=48,
              intermediate_size=172, vocab_size=301, rope_theta=500000.0, rms_norm_eps=3e-6,
              sliding_window=70, max_position_embeddings=2048, tie_word_embeddings=True,
              rope_pairing="adjacent",
              layer_types=["sliding_attention", "full_attention", "sliding_attention", "full_attention"]),
}


@pytest.fixture(scope="session")
def tiny_folders(tmp_path_factory):
    """name -> (folder, plain config dict, plain float32 weights)."""
    import braidinfer_amd as B
    import plain_mistral as P
    out = {}
    for name, d in TINY.items():
        cfg = B.MistralConfig.from_dict(d)
        folder = str(tmp_path_factory.mktemp(f"tiny_{name}"))
        # std well above the 0.02 of the benchmark shapes so that attention and the
        # feed-forward move the logits; norm weights jittered so a skipped weight shows
        B.Engine.write_random_folder(folder, cfg, seed=11 + ord(name), std=0.08, vector_jitter=0.3)
        pc, pw = P.read_folder(folder)
        out[name] = (folder, pc, pw)
    return out


@pytest.fixture(scope="session")
def engines(tiny_folders):
    """Engines are made once per (config, dtype) and shared, so slots are used again
    across tests as they would be in a long-running process."""
    import braidinfer_amd as B
    cache = {}

    def get(name, dtype, max_tokens=4096):
        key = (name, dtype, max_tokens)
        if key not in cache:
            cache[key] = B.Engine.from_folder(tiny_folders[name][0], dtype=dtype, max_tokens=max_tokens)
        return cache[key]
    return get
