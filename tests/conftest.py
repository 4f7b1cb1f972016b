import importlib.util
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "lichtfeld-studio_amd")
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def load_package():
    """Import lichtfeld-studio_amd/ (not a valid identifier) as `lichtfeld_studio_amd`."""
    name = "lichtfeld_studio_amd"
    if name in sys.modules:
        return sys.modules[name]
    spec = importlib.util.spec_from_file_location(name, os.path.join(PKG_DIR, "__init__.py"),
                                                  submodule_search_locations=[PKG_DIR])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gsx():
    return load_package()


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle
    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    load_package()._lib.lib()  # fail loudly if libgsx.so is missing
    return torch.device("cuda:0")


@pytest.fixture(scope="session")
def cpp():
    """gsx_torch_ext: the pybind11 module over the C++ host layer (csrc/host/gsplat_ops.cpp), built in-tree by
    build_ext.py.  Missing build = failure, not skip."""
    import torch  # noqa: F401  (libtorch must be loaded first)
    if PKG_DIR not in sys.path:
        sys.path.insert(0, PKG_DIR)
    import gsx_torch_ext
    return gsx_torch_ext


def pytest_terminal_summary(terminalreporter):
    """the measured gradient / Adam miss fractions of the GPU parity tests (oracle/checks.py), printed whether or not
    output capture is on"""
    try:
        from oracle import checks
    except Exception:
        return
    if checks.REPORT:
        terminalreporter.write_sep("-", "measured parity: fraction of elements outside 1e-3 relative, needed multipliers")
        for line in checks.REPORT:
            terminalreporter.write_line(line)
        if checks.PLAIN:
            worst = max(checks.PLAIN, key=lambda x: x[1])
            terminalreporter.write_line(
                f"plain form over {len(checks.PLAIN)} tensors: |gpu - fp32 checker| <= {checks.PLAIN_RTOL:g} |fp32| + "
                f"{checks.PLAIN_ATOL_RMS:g} rms(fp32) holds everywhere; largest atol needed {max(worst[1], 0.0):.2e} rms "
                f"({worst[0].strip()})")
