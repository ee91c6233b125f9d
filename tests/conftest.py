import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run on an MI355X box)")


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """Model folders (config.json + model.safetensors, bf16 values) of the tiny configurations, made once."""
    import tiny
    from jllm_serve_amd.weights import write_random_model
    out = {}
    for name, (cfg, seed, page) in tiny.CONFIGS.items():
        d = str(tmp_path_factory.mktemp("model_" + name))
        write_random_model(d, cfg, seed)
        out[name] = d
    return out


@pytest.fixture(scope="session")
def plain_logits(model_folders):
    """name -> function(tokens) -> float64 logits of the plain implementation, cached per token list."""
    import tiny
    cache = {}

    def get(name, tokens):
        key = (name, tuple(tokens))
        if key not in cache:
            cache[key] = tiny.plain_forward(model_folders[name], tokens)
        return cache[key]
    return get
