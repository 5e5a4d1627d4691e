import os
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

os.environ.setdefault("HSA_ENABLE_IPC_MODE_LEGACY", "0")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (MI355X); run with -m gpu")
    config.addinivalue_line("markers", "slow: larger parity cases")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip_gpu = pytest.mark.skip(reason="no ROCm GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip_gpu)


@pytest.fixture(scope="session")
def golden_dir():
    return ROOT / "tests" / "golden"


def pytest_terminal_summary(terminalreporter):
    """16-bit parity figures of the run: the raw max-abs error beside the magnitude-scaled one the assertions use."""
    try:
        from tests import gpu_util
    except Exception:  # noqa: BLE001
        return
    rec = gpu_util.RAW_16BIT
    if not rec:
        return
    worst_raw = max(rec, key=lambda r: r[0])
    worst_small = max(rec, key=lambda r: r[1])
    worst_scaled = max(rec, key=lambda r: r[2])
    terminalreporter.write_line(
        f"16-bit comparisons: {len(rec)}; worst raw max-abs {worst_raw[0]:.3e} (where max |want| = {worst_raw[3]:.2f}); "
        f"worst raw max-abs over entries with |want| <= 2: {worst_small[1]:.3e}; worst magnitude-scaled: "
        f"{worst_scaled[2]:.3e}")
