import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda", 0)


def pytest_terminal_summary(terminalreporter, exitstatus, config):
    """The measured numbers of every image comparison against the oracle, worst per label (pytest -q swallows the
    lines check_images prints): threshold-adjacent pixel count, largest error on the other ("solid") pixels and on
    all pixels, pixels beyond 1e-4, lowest PSNR."""
    from tests import helpers

    if not helpers.IMAGE_REPORT:
        return
    import re
    tr = terminalreporter
    tr.write_line("image parity vs oracle (worst per label; solid = pixels without a threshold-adjacent decision)")
    merged = {}  # the many small parametrised frames share one line per family ("tiny (64, 48) deg 2" -> "tiny")
    for label, slot in helpers.IMAGE_REPORT.items():
        key = re.sub(r"\s*\(\d+, \d+\) deg \d+", "", label)
        if key not in merged:
            merged[key] = slot
            continue
        m = merged[key]
        m["frames"] += slot["frames"]
        m["fragile"], m["pixels"] = max(m["fragile"], slot["fragile"]), max(m["pixels"], slot["pixels"])
        for name in ("image", "depth", "alpha"):
            if name in slot and name in m:
                a, b = m[name], slot[name]
                a["solid"], a["all"] = max(a["solid"], b["solid"]), max(a["all"], b["all"])
                a["over_tol"], a["psnr"] = max(a["over_tol"], b["over_tol"]), min(a["psnr"], b["psnr"])
    for label, slot in merged.items():
        parts = []
        for name in ("image", "depth", "alpha"):
            if name in slot:
                w = slot[name]
                parts.append("%s solid %.2g all %.2g >1e-4: %d psnr %.0f" % (name, w["solid"], w["all"], w["over_tol"],
                                                                            min(w["psnr"], 999.0)))
        tr.write_line("  %s [%d frame(s), %d/%d adjacent]: %s" % (label[:60], slot["frames"], slot["fragile"],
                                                                  slot["pixels"], "; ".join(parts)))
