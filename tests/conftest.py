import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run with -m gpu on an MI355X)")


@pytest.fixture(scope="session")
def hip_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    return torch.device("cuda:0")


def pytest_terminal_summary(terminalreporter):
    """The fp32 fixtures are compared with a stated floor; what they measure with no floor at all is
    printed here, so that a regression in it is visible in the log of every run."""
    try:
        import golden_util as G
    except Exception:
        return
    if not G.FP32_WORST:
        return
    tr = terminalreporter
    tr.write_sep("-", "fp32 results against the reference's fixtures, no floor: worst |a-b|/max(|a|,|b|) (fp32 ulps, abs) at")
    for opt in sorted(G.FP32_WORST):
        for kind in ("param", "state"):
            if kind in G.FP32_WORST[opt]:
                rel, ulps, absd, where = G.FP32_WORST[opt][kind]
                tr.write_line(f"  {opt:12s} {kind:5s} {rel:9.3e}  ({ulps:5.1f} ulp, abs {absd:8.2e})  {where}")
