import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def cfg1():
    """Golden vectors from the unmodified reference CPU build (tests/golden/make_cfg1_fixture.py)."""
    import numpy as np

    z = np.load(os.path.join(ROOT, "tests", "golden", "cfg1_reference.npz"))
    n_head, n_kv, d, n_prefill, n_decode, out_base, n_embd = (int(x) for x in z["meta"])
    return dict(q=z["q"], k=z["k"], v=z["v"], logits_a=z["logits_a"], logits_b=z["logits_b"],
                n_head=n_head, n_kv=n_kv, d=d, n_prefill=n_prefill, n_decode=n_decode,
                out_base=out_base, n_embd=n_embd)
