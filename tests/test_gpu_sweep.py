"""The sweep driver end to end on a small tree of .smtx files (the DLMC layout of the reference's runs)."""
import csv
import os

import pytest

from vectorsparse_amd import benchmark_common as bc
from vectorsparse_amd import colvec_csr as cv
from vectorsparse_amd import sweep

pytestmark = pytest.mark.gpu


def _tree(tmp_path):
    root = tmp_path / "dlmc"
    names = ["rn50/random_pruning/0.8/layer_a", "rn50/random_pruning/0.95/layer_b", "rn50/random_pruning/0.9/layer_c"]
    for i, (name, s) in enumerate(zip(names, (0.8, 0.95, 0.9))):
        path = root / (name + ".smtx")
        path.parent.mkdir(parents=True, exist_ok=True)
        pat = cv.uniform_pattern(32, 256, s, seed=i, vec_length=1)
        cv.write_smtx(str(path), pat.m_vec, pat.n, pat.row_offsets, pat.column_indices)
    listing = tmp_path / "rn50_matrices.txt"
    listing.write_text("".join(n + ".smtx\n" for n in names))
    return root, listing, names


@pytest.mark.parametrize("op", ["spmm", "sddmm"])
def test_sweep_over_a_matrix_list(gpu, tmp_path, op):
    root, listing, names = _tree(tmp_path)
    out = tmp_path / "result.csv"
    csv_dir = tmp_path / "csv"
    rc = sweep.main(["--op", op, "--smtx-dir", str(root), "--matrix-list", str(listing), "--start", "0", "--end", "2",
                     "--dimK", "64,128", "--dimV", "2,8", "--iters", "5", "--out", str(out), "--csv-dir", str(csv_dir)])
    assert rc == 0
    with open(out) as f:
        rows = list(csv.DictReader(f))
    # 2 benchmarks x 2 widths x 2 vector lengths x 2 kernels
    assert len(rows) == 16
    assert {r["bm"] for r in rows} == set(names[:2])
    assert {float(r["sparsity"]) for r in rows} == {0.8, 0.95}
    assert all(float(r["us"]) > 0 and float(r["speedup"]) > 0 for r in rows)
    assert all(r["verified"] == "1" and float(r["max_rel_err"]) <= 1e-2 for r in rows), "every point is checked"
    for r in rows:
        k = int(r["N"] if op == "spmm" else r["K"])
        for kernel in (r["kernel"], "dense"):
            path = bc.duration_csv_path(str(csv_dir), r["bm"], k, int(r["V"]), kernel, op)
            assert os.path.exists(path), path
    if op == "spmm":
        assert {(int(r["M"]), int(r["K"])) for r in rows} == {(64, 256), (256, 256)}    # M = 32 rows x V
