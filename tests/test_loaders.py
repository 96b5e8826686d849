"""Host-side input adapters of the library (getMatrixFromCSV / getMatrixFromMTX, tool.cu:282-366)."""
import numpy as np
import pytest


def test_csv_dense_rows(tmp_path):
    import cuspamm_amd as sp
    rng = np.random.default_rng(0)
    M = rng.normal(size=(5, 7)).astype(np.float32)
    path = tmp_path / "m.csv"
    path.write_text("\n".join(",".join(repr(float(x)) for x in row) for row in M) + "\n")
    got = sp.load_csv(str(path), 5, 7)
    assert np.array_equal(got, M)
    # padded destination (dims rounded up to a tile multiple, main.h:54-56): pad region is zero
    got = sp.load_csv(str(path), 32, 7, ld=32)
    assert np.array_equal(got[:5, :7], M) and np.all(got[5:] == 0) and np.all(got[:, 7:] == 0)
    # extra lines beyond `rows` are ignored (tool.cu:361); short lines leave zeros
    path.write_text("1,2,3\n4\n5,6,7\n8,9,10\n")
    got = sp.load_csv(str(path), 3, 3)
    assert got.tolist() == [[1, 2, 3], [4, 0, 0], [5, 6, 7]]


def test_mtx_triples(tmp_path):
    import cuspamm_amd as sp
    path = tmp_path / "m.mtx"
    path.write_text("4 4 3\n1 1 2.5\n4 2 -1e-3\n2 3 7\n")      # first line is skipped (tool.cu:288-291)
    got = sp.load_mtx(str(path), 4, 4)
    want = np.zeros((4, 4), dtype=np.float32)
    want[0, 0], want[3, 1], want[1, 2] = 2.5, -1e-3, 7
    assert np.array_equal(got, want)
    path.write_text("hdr\n5 1 1.0\n")
    with pytest.raises(sp.SpammError):
        sp.load_mtx(str(path), 4, 4)                            # index outside the matrix


def test_missing_file():
    import cuspamm_amd as sp
    with pytest.raises(sp.SpammError):
        sp.load_csv("/nonexistent/file.csv", 2, 2)
