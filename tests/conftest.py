import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(Path(__file__).resolve().parent))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _has_gpu() -> bool:
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    import oracle_lib
    return oracle_lib.load()


@pytest.fixture(scope="session")
def rotation_fixture():
    import numpy as np
    raw = np.fromfile(ROOT / "tests" / "golden" / "rotation_seed42.f16", dtype=np.float16)
    assert raw.size == 128 * 128
    return raw.reshape(128, 128)


def pytest_terminal_summary(terminalreporter, exitstatus, config):
    """How much of the attention tolerance the GPU parity tests used: one line (shown with -q too) and the table of
    every test's largest relative error as a JSON file in the run's output folder."""
    import json
    import parity_log
    if not parity_log.WORST:
        return
    worst = sorted(parity_log.WORST.items(), key=lambda kv: -kv[1])
    by_file = {}
    for test, err in worst:
        f = test.split("::", 1)[0]
        if f not in by_file:
            by_file[f] = (err, test)
    try:
        out = ROOT / "gpurun_out"
        out.mkdir(exist_ok=True)
        (out / "parity_rel_err.json").write_text(json.dumps(dict(worst), indent=1))
    except OSError:
        pass
    terminalreporter.write_line(
        f"parity: largest attention rel err {worst[0][1]:.2e} of 2e-3 allowed ({worst[0][0]}); "
        f"{len(worst)} tests compared outputs; per file: " +
        "; ".join(f"{f} {e:.2e}" for f, (e, _) in sorted(by_file.items())))
