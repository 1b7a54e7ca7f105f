import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _ensure_cpu_libs():
    """The CPU suite needs the oracle and the workload generator; build them if absent."""
    from library_amd import build
    if not os.path.exists(os.path.join(ROOT, "oracle", "liboracle.so")):
        build.build_oracle()
    if not os.path.exists(build.WORKLOADS):
        build.build_workloads()


@pytest.fixture(scope="session")
def oracle():
    _ensure_cpu_libs()
    from oracle.bindings import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def ref():
    """The reference's own CPU path; only where oracle/_ref has been built."""
    from oracle.bindings import Ref
    if not Ref.available():
        pytest.skip("oracle/_ref not built here (needs the reference sources)")
    return Ref()


@pytest.fixture(scope="session")
def golden():
    def load(name):
        return np.load(os.path.join(GOLDEN, name), allow_pickle=False)
    return load


def csr_from_lengths(lengths, ncols, seed, dtype):
    lengths = np.asarray(lengths, dtype=np.int64)
    row_ptr = np.zeros(lengths.size + 1, dtype=np.int32)
    row_ptr[1:] = np.cumsum(lengths)
    rng = np.random.default_rng(seed)
    col = np.empty(int(row_ptr[-1]), dtype=np.int32)
    for r, ln in enumerate(lengths):
        col[row_ptr[r]:row_ptr[r + 1]] = np.sort(rng.choice(ncols, size=int(ln), replace=False))
    val = rng.uniform(-1, 1, size=col.size).astype(dtype)
    return row_ptr, col, val


def row_ptr_from_lengths(lengths):
    lengths = np.asarray(lengths, dtype=np.int64)
    row_ptr = np.zeros(lengths.size + 1, dtype=np.int32)
    row_ptr[1:] = np.cumsum(lengths)
    return row_ptr


# row-length shapes used by both the CPU and the GPU analysis tests
def analysis_shapes():
    rng = np.random.default_rng(1234)
    return {
        "uniform7": np.full(300, 7),
        "giant_first": np.r_[9000, rng.integers(0, 5, 400)],
        "giant_last": np.r_[rng.integers(0, 5, 400), 9000],
        "giant_mid": np.r_[rng.integers(0, 5, 200), 20000, rng.integers(0, 5, 200)],
        "empties": np.r_[np.zeros(70, int), rng.integers(0, 3, 60), np.zeros(3000, int), 5, np.zeros(9, int)],
        "leading_empty": np.r_[np.zeros(5, int), 4096, 4096, 1],
        "all_empty": np.zeros(50, int),
        "one_row": np.array([37]),
        "two": np.array([3, 1]),
        "exact_tiles": np.full(512, 8),
        "zipf": np.minimum(rng.zipf(2.0, 6000), 5000),
        "stencil_like": np.r_[3, np.full(2000, 5), 3],
    }
