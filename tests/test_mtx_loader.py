"""Matrix Market loader: oracle and library against hand-written expected CSR (tests/golden/mtx)."""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
MTX = os.path.join(HERE, "golden", "mtx")
with open(os.path.join(MTX, "expected.json")) as f:
    EXPECTED = {k: v for k, v in json.load(f).items() if not k.startswith("_")}


def _check(got, exp):
    assert got["M"] == exp["M"] and got["K"] == exp["K"]
    assert got["symmetric"] == exp["symmetric"]
    assert got["row_ptr"].tolist() == exp["row_ptr"]
    assert got["col_idx"].tolist() == exp["col_idx"]
    assert [format(int(v), "04x") for v in got["val"]] == exp["val_hex"]


@pytest.mark.parametrize("name", sorted(EXPECTED))
def test_oracle_loader(oracle, name):
    got = oracle.mtx_read(os.path.join(MTX, name))
    assert got["rc"] == 0
    _check(got, EXPECTED[name])


@pytest.mark.parametrize("name", sorted(EXPECTED))
def test_library_loader(smat, name):
    _check(smat.mtx_read(os.path.join(MTX, name)), EXPECTED[name])


def test_error_codes(oracle, smat, tmp_path):
    assert oracle.mtx_read(os.path.join(MTX, "does_not_exist.mtx"))["rc"] == -1
    assert oracle.mtx_read(os.path.join(MTX, "bad_banner.mtx"))["rc"] == -2
    with pytest.raises(smat.SmatError) as e:
        smat.mtx_read(os.path.join(MTX, "does_not_exist.mtx"))
    assert e.value.code == -4
    with pytest.raises(smat.SmatError):
        smat.mtx_read(os.path.join(MTX, "bad_banner.mtx"))
    # the library range-checks indices against the padded shape, where the reference would write out of bounds
    bad = tmp_path / "oob.mtx"
    bad.write_text("%%MatrixMarket matrix coordinate real general\n3 3 1\n17 1 1.0\n")
    with pytest.raises(smat.SmatError):
        smat.mtx_read(bad)
    short = tmp_path / "short.mtx"
    short.write_text("%%MatrixMarket matrix coordinate real general\n3 3 2\n1 1 1.0\n")
    with pytest.raises(smat.SmatError):
        smat.mtx_read(short)


def test_band_file_like_the_reference_generator(oracle, smat, tmp_path):
    # src/generate_matrices.py writes "i j 1" lines for max(0,i-b) <= j < min(N,i+b+1)
    n, b = 100, 3
    lines = [f"{i + 1} {j + 1} 1" for i in range(n) for j in range(max(0, i - b), min(n, i + b + 1))]
    path = tmp_path / "band.mtx"
    path.write_text("%%MatrixMarket matrix coordinate real general\n" + f"{n} {n} {len(lines)}\n" + "\n".join(lines) + "\n")
    a, o = smat.mtx_read(path), oracle.mtx_read(path)
    assert a["M"] == 112 and a["nnz"] == n * (2 * b + 1) - b * (b + 1)
    for key in ("row_ptr", "col_idx", "val"):
        assert np.array_equal(a[key], o[key])


def test_garbled_size_line_is_an_error_not_an_abort(smat, tmp_path):
    """An entry count the file cannot hold (or one that would need terabytes) comes back as an I/O error."""
    for sizes in ("4 4 4000000000000", "4 4 99", "99999999999 4 1"):
        p = tmp_path / "bad.mtx"
        p.write_text(f"%%MatrixMarket matrix coordinate real general\n{sizes}\n1 1 1.0\n")
        with pytest.raises(smat.SmatError, match="size line"):
            smat.mtx_read(p)
