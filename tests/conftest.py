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


@pytest.fixture(scope="session")
def disunex_dirs(tmp_path_factory):
    """Model folders of the tiny Disunex configurations (sharpened weights), once per session."""
    from disunex_models import DISUNEX_CONFIGS, make_disunex_dir
    base = tmp_path_factory.mktemp("disunex")
    return {name: make_disunex_dir(str(base / name), cfg, seed) for name, (cfg, seed) in DISUNEX_CONFIGS.items()}


@pytest.fixture(scope="session")
def netovik_dirs(tmp_path_factory):
    """Model folders of the tiny Netovik configurations (sharpened weights), once per session."""
    from netovik_models import NETOVIK_CONFIGS, make_netovik_dir
    base = tmp_path_factory.mktemp("netovik")
    return {name: make_netovik_dir(str(base / name), cfg, seed) for name, (cfg, seed) in NETOVIK_CONFIGS.items()}


@pytest.fixture(scope="session")
def sipilorn_dirs(tmp_path_factory):
    """Model folders of the tiny Sipilorn configurations (sharpened weights), once per session."""
    from sipilorn_models import SIPILORN_CONFIGS, make_sipilorn_dir
    base = tmp_path_factory.mktemp("sipilorn")
    return {name: make_sipilorn_dir(str(base / name), cfg, seed) for name, (cfg, seed) in SIPILORN_CONFIGS.items()}


@pytest.fixture(scope="session")
def rutevik_dirs(tmp_path_factory):
    """Model folders of the tiny Rutevik configurations (sharpened weights), once per session."""
    from rutevik_models import RUTEVIK_CONFIGS, make_rutevik_dir
    base = tmp_path_factory.mktemp("rutevik")
    return {name: make_rutevik_dir(str(base / name), cfg, seed) for name, (cfg, seed) in RUTEVIK_CONFIGS.items()}


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
