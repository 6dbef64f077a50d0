import glob
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")

# tolerances of the filter outputs, on data normalised to [0, 1]
MAX_ABS_TOL = 1e-3
REL_L2_TOL = 1e-4


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def golden_lattice_cases(f64=False):
    """Names of the lattice cases computed with T = float (default) or T = double (*_f64)."""
    names = sorted(os.path.basename(p)[len("lattice_"):-len(".npz")]
                   for p in glob.glob(os.path.join(GOLDEN, "lattice_*.npz")))
    return [n for n in names if n.endswith("_f64") == f64]


def load_golden(name):
    return dict(np.load(os.path.join(GOLDEN, name + ".npz")))


def bits(a):
    """Bit patterns: of doubles for a float64 array, of floats for anything else."""
    a = np.asarray(a)
    if a.dtype == np.float64:
        return np.ascontiguousarray(a).view(np.uint64)
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def sorted_keys(keys):
    """Rows of an [M, pd] int16 key array in lexicographic order."""
    keys = np.asarray(keys)
    order = np.lexsort(keys.T[::-1])
    return keys[order], order


def rel_l2(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


@pytest.fixture(scope="session")
def oracle_mod():
    import oracle
    return oracle
