import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    from oracle import pyoracle

    pyoracle.lib()
    return pyoracle


@pytest.fixture(scope="session")
def boundary_indices(orc):
    """Origin, first / quarter / middle / last index of every class, and the
    neighbours of every class boundary — the fixture of
    llvq-search/tests/fastdec.rs:28-51 and g3_index.rs (class_boundaries_roundtrip)."""
    out = [0, 1, orc.N12 - 1, orc.N12, orc.N12 + 1, orc.N13 - 1, orc.N13]
    for ci in range(orc.lib().orc_n_classes()):
        info = orc.class_info(ci)
        lo, hi = info["lo"], info["hi"]
        card = hi - lo + 1
        out += [lo, lo + 1 if card > 1 else lo, lo + card // 4, lo + card // 2, lo + 3 * card // 4, hi - 1 if card > 1 else hi, hi]
    return np.unique(np.array(out, dtype=np.uint64))


@pytest.fixture(scope="session")
def gpu_rt():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import llvq_amd

    rt = llvq_amd.FusedRuntime(device=0)
    yield rt
    rt.close()
