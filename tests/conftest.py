import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders of the tiny configurations, written once per session into
    a temporary folder."""
    from imparo_amd import write_random_model
    from tiny_configs import CONFIGS, C_KEEP_F32
    out = {}
    for name, (cfg, seed) in CONFIGS.items():
        d = str(tmp_path_factory.mktemp(f"tiny_{name}"))
        write_random_model(cfg, seed, d, keep_float32=C_KEEP_F32 if name == "C" else ())
        out[name] = d
    return out


@pytest.fixture(scope="session")
def plain_models(model_dirs):
    from plain_lfm2 import PlainLfm2
    return {name: PlainLfm2(d) for name, d in model_dirs.items()}


@pytest.fixture(scope="session")
def loud_model_dirs(tmp_path_factory):
    """Tiny A and B with the layers' matrices drawn 8 times wider. With the
    stated spreads the layers add little to the embedding and a greedy
    continuation is one token repeated, which a dropped token or a stale state
    would not change; these models' continuations move with every token."""
    from imparo_amd import write_random_model
    from tiny_configs import CONFIGS
    out = {}
    for name in ("A", "B"):
        cfg, seed = CONFIGS[name]
        d = str(tmp_path_factory.mktemp(f"loud_{name}"))
        write_random_model(cfg, seed, d, layer_gain=8.0)
        out[name] = d
    return out


@pytest.fixture(scope="session")
def loud_plain_models(loud_model_dirs):
    from plain_lfm2 import PlainLfm2
    return {name: PlainLfm2(d) for name, d in loud_model_dirs.items()}


def assert_varied(sequences):
    """A test of generation must be able to fail: its expected tokens are no
    repeated token."""
    for seq in sequences:
        assert len(set(seq)) > len(seq) // 2, f"the expected continuation {seq} hardly moves"


def prompt_tokens(vocab, n, seed):
    import torch
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
