"""pytest configuration: import paths, the ``gpu`` marker, shared helpers."""
import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
PKG = ROOT / "flash-linear-attention-npu_amd"
for p in (str(ROOT), str(PKG)):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    import fla_hip

    fla_hip.load_library()  # fail loudly if the HIP library is missing
    return torch.device("cuda:0")


def pytest_sessionfinish(session, exitstatus):
    """After a GPU run: the measured error of every assert_close, largest share of its tolerance first."""
    import json

    import util

    if not util.RECORDS:
        return
    out = ROOT / "gpurun_out"
    try:
        out.mkdir(exist_ok=True)
        rows = sorted(util.RECORDS, key=lambda r: -(r["max_abs"] / (r["tol"] * (1.0 + r["max_ref"]))))
        (out / "parity_errors.json").write_text(json.dumps(rows, indent=0))
    except OSError:
        pass
