"""MatrixMarket reader (host code of the library, no GPU): checked against scipy.io.mmread, an
independent implementation of the format, and against the expansion rule of the reference's reader
(hip/test/io.hip:180-330: the mirror image follows its entry and carries the same value)."""
import io
import os

import numpy as np
import pytest
import scipy.io
import scipy.sparse as sp

from library_amd import capi


def _write(path, header, size, body):
    with open(path, "w") as f:
        f.write(header + "\n% a comment\n%\n" + size + "\n" + "\n".join(body) + "\n")


def _dense(m, n, r, c, v):
    a = np.zeros((m, n))
    np.add.at(a, (r, c), v)
    return a


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_general_real_matches_scipy(tmp_path, dtype):
    rng = np.random.default_rng(5)
    A = sp.random(37, 53, density=0.1, random_state=7, format="coo", dtype=np.float64)
    p = tmp_path / "g.mtx"
    scipy.io.mmwrite(str(p), A, precision=17)
    m, n, r, c, v = capi.mtx_read(p, dtype)
    B = scipy.io.mmread(str(p)).tocoo()
    assert (m, n) == B.shape and v.dtype == dtype
    assert np.array_equal(r, B.row) and np.array_equal(c, B.col)  # file order kept
    assert np.array_equal(v, B.data.astype(dtype))


def test_symmetric_integer_pattern_and_complex(tmp_path):
    # symmetric real: equals scipy's expansion; mirror follows its entry
    p = tmp_path / "s.mtx"
    _write(p, "%%MatrixMarket matrix coordinate real symmetric", "4 4 5",
           ["1 1 2.5", "2 1 -1.25", "3 3 4", "4 2 1e-3", "4 4 7"])
    m, n, r, c, v = capi.mtx_read(p, np.float64)
    assert (m, n) == (4, 4)
    assert r.tolist() == [0, 1, 0, 2, 3, 1, 3] and c.tolist() == [0, 0, 1, 2, 1, 3, 3]
    assert v.tolist() == [2.5, -1.25, -1.25, 4.0, 1e-3, 1e-3, 7.0]
    assert np.array_equal(_dense(m, n, r, c, v), scipy.io.mmread(str(p)).toarray())
    # integer general
    p = tmp_path / "i.mtx"
    _write(p, "%%MatrixMarket matrix coordinate integer general", "3 5 3", ["1 5 7", "3 1 -2", "2 2 9"])
    m, n, r, c, v = capi.mtx_read(p, np.float32)
    assert np.array_equal(_dense(m, n, r, c, v), scipy.io.mmread(str(p)).toarray())
    # pattern symmetric: ones
    p = tmp_path / "p.mtx"
    _write(p, "%%MatrixMarket matrix coordinate pattern symmetric", "3 3 3", ["1 1", "3 1", "3 2"])
    m, n, r, c, v = capi.mtx_read(p, np.float64)
    assert np.array_equal(_dense(m, n, r, c, v), scipy.io.mmread(str(p)).toarray())
    # skew-symmetric: the reference mirrors with the SAME value (scipy negates it)
    p = tmp_path / "k.mtx"
    _write(p, "%%MatrixMarket matrix coordinate real skew-symmetric", "3 3 2", ["2 1 3.0", "3 2 -4.0"])
    m, n, r, c, v = capi.mtx_read(p, np.float64)
    assert np.array_equal(_dense(m, n, r, c, v), np.abs(scipy.io.mmread(str(p)).toarray()) * np.array(
        [[0, 1, 0], [1, 0, -1], [0, -1, 0]]))
    # complex Hermitian (the kind of file the reference ships, matrix_test/mhd1280b.mtx): real parts
    p = tmp_path / "h.mtx"
    _write(p, "%%MatrixMarket matrix coordinate complex Hermitian", "3 3 3", ["1 1 2 0", "2 1 .25 -1.5", "3 3 1e1 0"])
    m, n, r, c, v = capi.mtx_read(p, np.float64)
    assert np.array_equal(_dense(m, n, r, c, v), scipy.io.mmread(str(p)).toarray().real)


def test_errors(tmp_path):
    with pytest.raises(RuntimeError):
        capi.mtx_read(tmp_path / "missing.mtx", np.float64)
    p = tmp_path / "a.mtx"
    _write(p, "%%MatrixMarket matrix array real general", "2 2", ["1", "2", "3", "4"])
    with pytest.raises(RuntimeError):
        capi.mtx_read(p, np.float64)
    p = tmp_path / "t.mtx"  # fewer entries than promised
    _write(p, "%%MatrixMarket matrix coordinate real general", "2 2 3", ["1 1 1.0"])
    with pytest.raises(RuntimeError):
        capi.mtx_read(p, np.float64)
    p = tmp_path / "o.mtx"  # index outside the matrix
    _write(p, "%%MatrixMarket matrix coordinate real general", "2 2 1", ["3 1 1.0"])
    with pytest.raises(RuntimeError):
        capi.mtx_read(p, np.float64)
    p = tmp_path / "e.mtx"  # empty matrix is fine
    _write(p, "%%MatrixMarket matrix coordinate real general", "4 6 0", [])
    m, n, r, c, v = capi.mtx_read(p, np.float32)
    assert (m, n, r.size) == (4, 6, 0)


def test_reference_sample_file():
    """tests/golden/reference_test_matrix.mtx is the reference's own matrix_test/test.mtx (a data
    file): declared complex Hermitian, but with one value per entry and both triangles stored.  The
    reference's reader (hip/test/io.hip:180-250) takes the first value and mirrors every
    off-diagonal entry right after it, whatever else the file holds: 16 entries from 8 lines."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_test_matrix.mtx")
    m, n, r, c, v = capi.mtx_read(path, np.float32)
    assert (m, n) == (4, 4)
    lines = [(1, 3, 1), (1, 4, 2), (2, 3, 3), (2, 4, 4), (3, 1, 5), (3, 2, 6), (4, 1, 7), (4, 2, 8)]
    want = []
    for i, j, a in lines:
        want += [(i - 1, j - 1, float(a)), (j - 1, i - 1, float(a))]
    assert list(zip(r.tolist(), c.tolist(), v.tolist())) == want


def test_mhd1280b_matches_scipy():
    """The SuiteSparse matrix the reference ships (matrix_test/mhd1280b.mtx, complex Hermitian):
    real parts, Hermitian expansion, against scipy.io.mmread."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mhd1280b.mtx")
    m, n, r, c, v = capi.mtx_read(path, np.float64)
    A = scipy.io.mmread(path).tocsr()
    assert (m, n) == A.shape == (1280, 1280) and r.size == 22778
    B = sp.coo_matrix((v, (r, c)), shape=(m, n)).tocsr()
    assert abs(B - A.real).max() == 0.0


def test_reader_survives_garbage(tmp_path):
    """Truncations and byte flips of a valid file must end in an error status or a consistent
    result, never in a crash or an index outside the matrix."""
    rng = np.random.default_rng(9)
    good = ("%%MatrixMarket matrix coordinate real symmetric\n% c\n6 6 7\n"
            "1 1 1.5\n2 1 -2\n3 3 4e0\n4 2 .5\n5 5 1\n6 1 2\n6 6 3\n").encode()
    p = tmp_path / "f.mtx"
    for case in range(300):
        b = bytearray(good)
        if case % 3 == 0:
            b = b[:int(rng.integers(0, len(b)))]
        else:
            for _ in range(int(rng.integers(1, 6))):
                b[int(rng.integers(0, len(b)))] = int(rng.integers(0, 256))
        p.write_bytes(bytes(b))
        try:
            m, n, r, c, v = capi.mtx_read(p, np.float64)
        except RuntimeError:
            continue
        assert r.size == c.size == v.size
        if r.size:
            assert 0 <= r.min() and r.max() < m and 0 <= c.min() and c.max() < n
