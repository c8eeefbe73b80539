import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


def pytest_sessionfinish(session, exitstatus):
    """Writes the raw error figures of every attention comparison of this run (tests/helpers.py: PARITY_LOG) to
    parity_errors.json in the run's output folder, worst case per (test function, tensor): the asserted figures are measured
    above the bf16 rounding floor, and this file is where the raw ones can be audited."""
    try:
        import json
        import torch
        import helpers
        if not helpers.PARITY_LOG or not torch.cuda.is_available():
            return   # (a session without a GPU only holds the helper's own tests: it must not replace a GPU run's report)
        worst = {}
        for test_id, what, e in helpers.PARITY_LOG:
            name = test_id.split("::")[-1].split("[")[0]
            tensor = what.split(" ")[0]
            w = worst.setdefault((name, tensor), dict(cases=0, max_abs=0.0, mre=0.0, floor=0.0, max_abs_scaled=0.0, mre_excess=-1.0,
                                                       ref_absmax=0.0))
            w["cases"] += 1
            for key in ("max_abs", "mre", "max_abs_scaled", "mre_excess", "ref_absmax"):
                w[key] = max(w[key], e[key])
            if e["mre"] >= w["mre"]:
                w["floor"] = e["floor"]
        out_dir = os.path.join(ROOT, "gpurun_out")
        os.makedirs(out_dir, exist_ok=True)
        rows = [dict(test=k[0], tensor=k[1], **v) for k, v in sorted(worst.items())]
        with open(os.path.join(out_dir, "parity_errors.json"), "w") as f:
            json.dump(rows, f, indent=1)
    except Exception as exc:  # a report only: never the reason a run fails
        print(f"parity report not written: {exc}")
