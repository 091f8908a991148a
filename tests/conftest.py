import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders of the tiny configurations, written once per session."""
    from helpers import TINY_CONFIGS, make_model_dir
    base = tmp_path_factory.mktemp("models")
    return {name: make_model_dir(str(base / name), cfg, seed) for name, (cfg, seed) in TINY_CONFIGS.items()}


@pytest.fixture(autouse=True)
def _seeded():
    """Every test draws the same random inputs in every run."""
    import torch
    torch.manual_seed(1234)
    yield


def pytest_terminal_summary(terminalreporter):
    from helpers import WORST, _TOL
    if WORST:
        terminalreporter.write_line("worst error against the plain implementation / tolerance, per configuration:")
        for (dtype, name), err in sorted(WORST.items()):
            t = _TOL.get(dtype, {}).get(name)
            if dtype == "kernels":
                import test_kernels_gpu
                t = test_kernels_gpu.ATTN_TOL
            terminalreporter.write_line(f"  {dtype:9s} {name:6s} {err:.2e}" + (f" / {t:.1e}" if t else ""))
