"""Reference-faithful generator of the package vs the oracle / libstdc++ fixture; CLI argument handling."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from oracle import c_oracle as co
from vectorsparse_amd import colvec_csr as cv
from vectorsparse_amd import refgen

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")


def test_refgen_matches_fixture_and_oracle():
    with open(os.path.join(GOLDEN, "minstd_uniform.json")) as f:
        gold = json.load(f)
    head = np.array(gold["head_f32_bits"], dtype=np.uint32)
    got32 = refgen.make_dense_matrix(1, gold["total"], dtype=np.float32).reshape(-1)
    bits = got32.view(np.uint32)
    assert np.array_equal(bits[:head.size], head)
    assert int(np.bitwise_xor.reduce(bits)) == gold["xor_f32_bits"]
    assert int(bits[-1]) == gold["last_f32_bits"]
    n = 3 * (1 << 14) + 17      # crosses block boundaries of the jump-ahead
    assert np.array_equal(refgen.make_dense_matrix(1, n).view(np.uint16).reshape(-1),
                          co.make_dense_matrix_f16(n).view(np.uint16))


def test_refgen_calls_restart_the_sequence():
    # the reference passes its engine by value: rhs and values share a prefix
    rhs = refgen.make_dense_matrix(8, 16)
    values = refgen.make_dense_matrix(1, 40)
    assert np.array_equal(rhs.reshape(-1)[:40], values.reshape(-1))


def test_cli_help_and_argument_count():
    for mod in ("vectorsparse_amd.spmm_benchmark", "vectorsparse_amd.sddmm_benchmark"):
        r = subprocess.run([sys.executable, "-m", mod, "--help"], cwd=ROOT, capture_output=True, text=True)
        assert r.returncode == 0 and "positional" in r.stdout
        r = subprocess.run([sys.executable, "-m", mod, "a", "b"], cwd=ROOT, capture_output=True, text=True)
        assert r.returncode == 2


@pytest.mark.gpu
def test_cli_end_to_end(gpu, tmp_path):
    pat = cv.binomial_pattern(32, 256, 0.8, seed=3)
    path = str(tmp_path / "m.smtx")
    cv.write_smtx(path, pat.m_vec, pat.n, pat.row_offsets, pat.column_indices)
    from vectorsparse_amd import sddmm_benchmark, spmm_benchmark
    for kernel in (0, 1):
        assert spmm_benchmark.main([path, "128", "8", str(kernel), "1", "1", "1", "1"]) == 0
        assert sddmm_benchmark.main([path, "64", "4", str(kernel), "1", "0", "1", "1", "1"]) == 0
    assert spmm_benchmark.main(["synthetic:256,512,0.9,1", "64", "4", "0", "0", "1", "1", "1"]) == 0
    assert spmm_benchmark.main([path, "128", "8", "0", "2", "1", "1", "1"]) == 0       # rows in parts (nothing to split)
    lengths = np.array([1500] + [20] * 63)                                             # a row that is split
    ro = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    ci = np.concatenate([np.sort(np.random.default_rng(i).choice(2048, n, replace=False)) for i, n in enumerate(lengths)])
    skew = str(tmp_path / "skew.smtx")
    cv.write_smtx(skew, 64, 2048, ro, ci.astype(np.int32))
    assert spmm_benchmark.main([skew, "128", "8", "0", "2", "1", "1", "1"]) == 0
    assert spmm_benchmark.main([skew, "128", "8", "1", "2", "1", "1", "1"]) == 1       # only on the MFMA path
    assert sddmm_benchmark.main([skew, "64", "8", "0", "1", "2", "1", "1", "1"]) == 0   # SDDMM, rows in parts
    assert sddmm_benchmark.main([skew, "60", "8", "0", "1", "2", "1", "1", "1"]) == 1   # needs k % 8 == 0
    assert spmm_benchmark.main([skew, "128", "8", "0", "3", "1", "1", "1"]) == 1
    assert spmm_benchmark.main([path, "128", "8", "0", "0", "1", "0", "1"]) == 0       # dense baseline
    assert sddmm_benchmark.main([path, "64", "8", "0", "0", "0", "1", "0", "1"]) == 0   # dense baseline
    assert spmm_benchmark.main([path, "128", "8", "2", "0", "0", "1", "1"]) == 1       # Sputnik: unsupported
    assert spmm_benchmark.main([path, "128", "3", "0", "0", "0", "1", "1"]) == 1       # bad vector length
    assert spmm_benchmark.main([path, "128", "8", "0", "0", "0", "1", "0"]) == 1       # fp32: unsupported
