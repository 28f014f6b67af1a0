import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    config.addinivalue_line("markers", "slow: full-size (7B/13B) case that takes minutes")


@pytest.fixture(scope="session")
def lva():
    """the llama-vulkan_amd package (hyphenated directory name, hence importlib)"""
    return importlib.import_module("llama-vulkan_amd")


@pytest.fixture(scope="session")
def orc():
    import oracle
    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def ctx(lva):
    c = lva.Context(0)
    yield c
    c.close()


@pytest.fixture(scope="session")
def tiny_models(lva, tmp_path_factory):
    """tiny seeded GGJT files shared by the tests: name -> path"""
    d = tmp_path_factory.mktemp("models")
    out = {}
    for name, wtype, seed, shape in [
        ("tiny_q4", lva.LV_Q4_0, 5, dict(vocab=512, dim=256, heads=4, layers=2, ff=704)),      # head size 64
        ("tiny_q8", lva.LV_Q8_0, 6, dict(vocab=512, dim=256, heads=2, layers=2, ff=704)),      # head size 128
        ("small_q4", lva.LV_Q4_0, 7, dict(vocab=1024, dim=512, heads=16, layers=3, ff=1376)),  # head size 32
        # feed-forward widths that 128 divides: a prompt batch takes gate and up as one paired GEMM with SwiGLU in its epilogue
        ("pair_q4", lva.LV_Q4_0, 8, dict(vocab=512, dim=256, heads=2, layers=2, ff=640)),
        ("pair_q8", lva.LV_Q8_0, 9, dict(vocab=512, dim=512, heads=4, layers=2, ff=768)),
    ]:
        p = str(d / f"{name}.ggml")
        lva.write_model(p, wtype=wtype, seed=seed, **shape)
        out[name] = p
    return out
