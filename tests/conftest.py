import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def load_golden(name):
    """Load one committed fixture as a dict of torch tensors (numpy .npz, no pickles)."""
    with np.load(os.path.join(GOLDEN_DIR, name + ".npz"), allow_pickle=False) as z:
        blob = {k: z[k] for k in z.files}
    meta = blob.pop("meta", None)
    out = {k: torch.from_numpy(np.ascontiguousarray(v)) for k, v in blob.items()}
    if meta is not None:
        batch, N, E, C, n, L, seed, xa_zero = (int(v) for v in meta)
        out["meta"] = dict(batch=batch, N=N, E=E, C=C, n=n, L=L, seed=seed, xa_zero=bool(xa_zero))
        out["alpha"] = float(out["alpha"])
    return out


def load_npz(name):
    """A committed fixture as a dict of numpy arrays, untouched (for fixtures with their own layout)."""
    with np.load(os.path.join(GOLDEN_DIR, name + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


GOLDEN_CASES = ["cfg1_n2_L8", "small_n4_L3", "bench_like_n8_L5", "odd_n3_L3"]


@pytest.fixture(params=GOLDEN_CASES)
def golden_case(request):
    return request.param, load_golden(request.param)


def has_gpu():
    return torch.cuda.is_available()


def record_errors(kind, **values):
    """Appends one line of measured errors to the file $NCN_ERROR_REPORT names, if any: the figures that the tolerances of
    the tests that call it are set from (a margin over the worst case measured)."""
    path = os.environ.get("NCN_ERROR_REPORT")
    if path:
        import json
        with open(path, "a") as fh:
            fh.write(json.dumps({"kind": kind, **values}) + "\n")
