import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _have_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_sessionfinish(session, exitstatus):
    """After a GPU session: the achieved parity figures (worst |err| / sum|x||w| and worst
    relative error per comparison label), so that they can be quoted next to the tolerances."""
    try:
        import json
        import util
        if not util.PARITY_LOG:
            return
        out = os.path.join(ROOT, "gpurun_out")
        os.makedirs(out, exist_ok=True)
        rows = {k: dict(normwise=v[0], relative=v[1], rtol=v[2]) for k, v in util.PARITY_LOG.items()}
        fp32 = [v for v in util.PARITY_LOG.values() if v[2] <= 1e-4]
        fp16 = [v for v in util.PARITY_LOG.values() if v[2] > 1e-4]
        summary = dict(
            fp32_worst_normwise=max([v[0] for v in fp32], default=0.0),
            fp32_worst_relative=max([v[1] for v in fp32], default=0.0),
            fp16_worst_normwise=max([v[0] for v in fp16], default=0.0),
            fp16_worst_relative=max([v[1] for v in fp16], default=0.0), comparisons=len(rows))
        with open(os.path.join(out, "parity_achieved.json"), "w") as f:
            json.dump(dict(summary=summary, rows=rows), f, indent=1, sort_keys=True)
    except Exception:
        pass
