import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (os.path.join(ROOT, "flash-colsum_amd"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    import numpy as np

    path = os.path.join(ROOT, "tests", "golden", "colsum_golden.npz")
    blob = np.load(path, allow_pickle=False)
    names = sorted({key.split("/")[0] for key in blob.files})
    cases = {}
    for n in names:
        causal, cls_len = (int(v) for v in blob[n + "/meta"])
        scale = float(blob[n + "/scale"][0])
        cases[n] = dict(q=blob[n + "/q"], k=blob[n + "/k"], out=blob[n + "/out"], causal=bool(causal),
                        cls_len=None if cls_len < 0 else cls_len, scale=None if scale != scale else scale)
    return cases


@pytest.fixture(scope="session")
def golden_ext():
    """Brute-force vectors for the shapes beyond the reference operator's domain (make_golden_ext.py)."""
    import numpy as np

    blob = np.load(os.path.join(ROOT, "tests", "golden", "colsum_ext_golden.npz"), allow_pickle=False)
    cases = {}
    for n in sorted({key.split("/")[0] for key in blob.files}):
        causal, cls_len, k_past = (int(v) for v in blob[n + "/meta"])
        scale = float(blob[n + "/scale"][0])
        cases[n] = dict(q=blob[n + "/q"], k=blob[n + "/k"], out=blob[n + "/out"], causal=bool(causal),
                        cls_len=None if cls_len < 0 else cls_len, k_past=None if k_past < 0 else k_past,
                        scale=None if scale != scale else scale)
    return cases
