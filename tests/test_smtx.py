"""The DLMC ``.smtx`` pattern format and its MatrixMarket companion (reference benchmark/utils.py:11-44).
Index work: everything is compared bit for bit.  Witnesses that do not share code with the module
under test: scipy's MatrixMarket reader and scipy's CSR construction."""
import numpy as np
import pytest

from intrasm_engine_amd import smtx
from intrasm_engine_amd import workloads as W


def _write(tmp_path, text, name="a.smtx"):
    p = tmp_path / name
    p.write_text(text)
    return str(p)


def test_reads_the_three_line_format(tmp_path):
    # the 3 x 4 matrix [[1,0,2,0],[0,0,0,0],[0,3,0,4]] as a pattern
    path = _write(tmp_path, "3, 4, 4\n0 2 2 4\n0 2 1 3\n")
    m, k, ro, ci = smtx.read_smtx(path)
    assert (m, k) == (3, 4)
    assert ro.dtype == np.int32 and ci.dtype == np.int32
    assert ro.tolist() == [0, 2, 2, 4] and ci.tolist() == [0, 2, 1, 3]
    # lenient about blanks, as the reference's parser is (it skips empty tokens)
    path = _write(tmp_path, "3,4,4\n 0  2 2   4 \n0 2  1 3  \n\n", "b.smtx")
    m2, k2, ro2, ci2 = smtx.read_smtx(path)
    assert (m2, k2) == (3, 4) and np.array_equal(ro2, ro) and np.array_equal(ci2, ci)


def test_empty_matrix_and_empty_rows(tmp_path):
    m, k, ro, ci = smtx.read_smtx(_write(tmp_path, "2, 5, 0\n0 0 0\n\n"))
    assert (m, k) == (2, 5) and ro.tolist() == [0, 0, 0] and ci.shape == (0,)
    m, k, ro, ci = smtx.read_smtx(_write(tmp_path, "2, 5, 0\n0 0 0", "nolast.smtx"))
    assert ci.shape == (0,)


@pytest.mark.parametrize("text, message", [
    ("3, 4\n0 2 2 4\n0 2 1 3\n", "header must be"),
    ("3, 4, x\n0 2 2 4\n0 2 1 3\n", "three integers"),
    ("3, 4, 4\n0 2 2\n0 2 1 3\n", "row_ptrs has 3 entries"),
    ("3, 4, 5\n0 2 2 4\n0 2 1 3\n", "col_idxs has 4 entries"),
    ("3, 4, 4\n0 2 1 4\n0 2 1 3\n", "row_ptrs decrease"),
    ("3, 4, 4\n1 2 2 4\n0 2 1 3\n", "must start at 0"),
    ("3, 4, 4\n0 2 2 3\n0 2 1 3\n", "end at the number of nonzeros"),
    ("3, 4, 4\n0 2 2 4\n0 4 1 3\n", "column index outside"),
    ("3, 4, 4\n0 2 2 4\n2 0 1 3\n", "row 0 are not strictly ascending"),
    ("3, 4, 4\n0 2 2 4\n0 2 3 3\n", "row 2 are not strictly ascending"),
    ("3, 4, 4\n0 2 2 4\n0 2 1 z\n", "not an integer"),
    ("3, 4, 4\n0 2 2 4\n0 2 1 3\n7\n", "unexpected line"),
])
def test_malformed_files_are_refused(tmp_path, text, message):
    with pytest.raises(smtx.SmtxError, match=message):
        smtx.read_smtx(_write(tmp_path, text))


def test_round_trip_and_scipy_witness(tmp_path):
    scipy_sparse = pytest.importorskip("scipy.sparse")
    scipy_io = pytest.importorskip("scipy.io")
    a = W.config2_matrix(0.95, m=300, k=257, seed=5)
    path = str(tmp_path / "m.smtx")
    smtx.write_smtx(path, a.m, a.k, a.row_offsets, a.column_indices)
    m, k, ro, ci = smtx.read_smtx(path)
    assert (m, k) == (a.m, a.k)
    assert np.array_equal(ro, a.row_offsets) and np.array_equal(ci, a.column_indices)

    # a decreasing pair that straddles a row boundary is legal (last column of a row above the
    # first column of the next): the writer must not refuse it
    smtx.write_smtx(str(tmp_path / "s.smtx"), 2, 4, [0, 1, 2], [3, 0])
    with pytest.raises(smtx.SmtxError):
        smtx.write_smtx(str(tmp_path / "bad.smtx"), 2, 4, [0, 2, 2], [3, 0])

    # .mtx companion: scipy reads back the same pattern, 1-based on disk, values in [0, 1)
    out = smtx.generate_mtx_from_smtx(path, seed=3)
    assert out.endswith("m.mtx")
    with open(out) as f:
        assert f.readline() == "%%MatrixMarket matrix coordinate real general\n"
        assert f.readline() == f"{a.m} {a.k} {a.nnz}\n"
        r, c, v = f.readline().split()
        assert (int(r), int(c)) == (int(np.searchsorted(a.row_offsets, 0, side="right")), int(a.column_indices[0]) + 1)
    back = scipy_sparse.csr_matrix(scipy_io.mmread(out))
    back.sort_indices()
    assert back.shape == (a.m, a.k)
    assert np.array_equal(back.indptr, a.row_offsets) and np.array_equal(back.indices, a.column_indices)
    assert back.data.min() >= 0.0 and back.data.max() < 1.0
    assert np.array_equal(back.data, np.random.default_rng(3).random(a.nnz))     # row-major order, full precision

    csr = smtx.smtx_to_csr(path, seed=9)
    assert csr.nnz == a.nnz and np.array_equal(csr.row_indices, W.swizzle_from_offsets(a.row_offsets))
    assert csr.values.dtype == np.float32 and not np.any(csr.values.astype(np.float16) == 0)
    assert np.array_equal(csr.values, smtx.smtx_to_csr(path, seed=9).values)
    assert smtx.find_smtx(str(tmp_path)) == sorted([path, str(tmp_path / "s.smtx")])
