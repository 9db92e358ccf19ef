import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 (MI355X) device")


@pytest.fixture(scope="session")
def oracle():
    from oracle.binding import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def reference():
    """The real NiuTensor CPU implementation; only where oracle/_ref has been built."""
    from oracle.binding import Reference
    if not Reference.available():
        pytest.skip("oracle/_ref/libnts_ref.so has not been built (needs the reference tree)")
    return Reference()


@pytest.fixture(scope="session")
def known_answers():
    with open(os.path.join(GOLDEN, "reference_known_answers.json")) as f:
        return json.load(f)["cases"]


class Generated:
    """tests/golden/ref_generated.npz: outputs of the compiled reference (see make_fixtures.py)."""

    def __init__(self, file="ref_generated.npz"):
        self.z = np.load(os.path.join(GOLDEN, file), allow_pickle=False)
        self.names = [str(n) for n in self.z["index"]]

    def case(self, name):
        pre = name + "/"
        return {k[len(pre):]: self.z[k] for k in self.z.files if k.startswith(pre)}

    def of_kind(self, kind):
        return [n for n in self.names if str(self.z[n + "/kind"]) == kind]


@pytest.fixture(scope="session")
def generated():
    return Generated()


@pytest.fixture(scope="session")
def generated_backward():
    """tests/golden/ref_generated_backward.npz: gradients left by the compiled reference's autograd step."""
    return Generated("ref_generated_backward.npz")


@pytest.fixture(scope="session")
def generated_attention():
    """tests/golden/ref_generated_attention.npz: the compiled reference's softmax and attention chain."""
    return Generated("ref_generated_attention.npz")


@pytest.fixture(scope="session")
def gpu():
    """cuda:0 with the HIP library loaded. No fallback: a missing library is an error."""
    import torch
    import niutensor_amd as nt
    assert torch.cuda.is_available(), "a GPU test was selected but no GPU is visible"
    nt.load()
    rc = nt.load().ntsamd_init(0)
    assert rc == 0, nt.load().ntsamd_last_error().decode()
    return torch.device("cuda:0")
