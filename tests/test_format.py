"""Column-vector CSR container, .smtx I/O and the synthetic generators (CPU only)."""
import numpy as np
import pytest

from vectorsparse_amd import colvec_csr as cv


def test_smtx_round_trip_and_v_expansion(tmp_path):
    pat = cv.binomial_pattern(13, 57, 0.8, seed=3)
    path = tmp_path / "a.smtx"
    cv.write_smtx(str(path), pat.m_vec, pat.n, pat.row_offsets, pat.column_indices)
    text = path.read_text().splitlines()
    assert text[0] == "13, 57, %d" % pat.nnz_vec
    assert len(text) == 3
    for V in (1, 2, 4, 8):
        back = cv.read_smtx(str(path), V)
        assert back.m == 13 * V and back.nnz == pat.nnz_vec * V and back.n == 57
        assert np.array_equal(back.row_offsets, pat.row_offsets)
        assert np.array_equal(back.column_indices, pat.column_indices)
        assert back.row_offsets.dtype == np.int32 and back.column_indices.dtype == np.int32


def test_smtx_rejects_inconsistent_files(tmp_path):
    path = tmp_path / "bad.smtx"
    path.write_text("2, 4, 3\n0 1 3\n0 1\n")
    with pytest.raises(ValueError):
        cv.read_smtx(str(path), 4)
    path.write_text("2, 4, 3\n0 1 3\n0 1 7\n")
    with pytest.raises(ValueError):
        cv.read_smtx(str(path), 4)


def test_value_layout_matches_reference_indexing():
    # element (i*V + v, col_j) is values[j*V + v]
    pat = cv.ColVecCSR(2, 3, 2, np.array([0, 1, 3], np.int32), np.array([2, 0, 1], np.int32))
    vals = np.arange(1, 7, dtype=np.float16).reshape(3, 2)
    dense = pat.with_values(vals).to_dense()
    expect = np.array([[0, 0, 1], [0, 0, 2], [3, 5, 0], [4, 6, 0]], dtype=np.float64)
    assert np.array_equal(dense, expect)


def test_uniform_pattern_counts():
    pat = cv.uniform_pattern(64, 256, 0.9, seed=0, vec_length=4).validate()
    assert np.all(pat.row_lengths() == 26)
    for i in range(pat.m_vec):
        row = pat.column_indices[pat.row_offsets[i]:pat.row_offsets[i + 1]]
        assert np.all(np.diff(row) > 0)
    assert cv.uniform_pattern(64, 256, 0.9, seed=0).column_indices.tolist() == pat.column_indices.tolist()


def test_binomial_pattern_is_skewed_and_seeded():
    pat = cv.binomial_pattern(64, 4608, 0.9, seed=1, vec_length=8).validate()
    L = pat.row_lengths()
    assert abs(L.mean() - 460.8) < 10 and L.std() > 5
    again = cv.binomial_pattern(64, 4608, 0.9, seed=1, vec_length=8)
    assert np.array_equal(again.column_indices, pat.column_indices)


def test_band_strided_pattern():
    pat = cv.band_strided_pattern(1024, 8, band_half_width=128, stride=128).validate()
    assert pat.m_vec == 128 and pat.n == 1024
    row = pat.column_indices[pat.row_offsets[40]:pat.row_offsets[41]]
    centre = 40 * 8 + 4
    assert set(range(centre - 128, centre + 129)) <= set(row.tolist())
    assert set(range(127, 1024, 128)) <= set(row.tolist())
    assert np.all(np.diff(row) > 0)


def test_validate_catches_bad_patterns():
    with pytest.raises(ValueError):
        cv.ColVecCSR(2, 4, 3, np.array([0, 1, 2], np.int32), np.array([0, 1], np.int32)).validate()
    with pytest.raises(ValueError):
        cv.ColVecCSR(2, 4, 2, np.array([0, 2, 1], np.int32), np.array([0, 1], np.int32)).validate()
    with pytest.raises(ValueError):
        cv.ColVecCSR(2, 4, 2, np.array([0, 1, 2], np.int32), np.array([0, 4], np.int32)).validate()
    with pytest.raises(ValueError):
        cv.ColVecCSR(2, 4, 2, np.array([0, 1, 2], np.int64), np.array([0, 1], np.int32)).validate()


def test_host_swizzle_mirror():
    ro = np.array([0, 3, 3, 10, 12, 19], np.int32)
    assert cv.identity_row_swizzle(5).tolist() == [0, 1, 2, 3, 4]
    assert cv.sorted_row_swizzle(ro).tolist() == [2, 4, 0, 3, 1]


def test_duration_files_follow_the_plot_scripts_layout(tmp_path):
    """Names as file_name_server.py:6-45 builds them; records as its reader (:57-81) sums them: for every row
    whose fourth field from the end contains "Duration", the next-to-last field in the unit before it."""
    import csv
    from vectorsparse_amd import benchmark_common as bc

    root = str(tmp_path)
    bm = "dlmc/rn50/random_pruning/0.8/bottleneck_1_block_group1_1_1.smtx"
    stem = "dlmc/rn50/random_pruning/0.8/bottleneck_1_block_group1_1_1"
    assert bc.duration_csv_path(root, bm, 256, 8, "wmma", "spmm") == \
        "%s/spmm/%s_wmma_half_sort_k256_v8.csv" % (root, stem)
    assert bc.duration_csv_path(root, bm, 64, 4, "dense", "spmm", sort=False) == \
        "%s/spmm/%s_dense_half_k64_v4.csv" % (root, stem)
    assert bc.duration_csv_path(root, bm, 128, 2, "wmma", "sddmm", sddmm_alg=2) == \
        "%s/sddmm/%s_wmma_half_sort_mma_shfl_k128_v2.csv" % (root, stem)
    assert bc.duration_csv_path(root, bm, 128, 2, "cuda", "sddmm", precision="single") == \
        "%s/sddmm/%s_cuda_single_sort_k128_v2.csv" % (root, stem)
    with pytest.raises(ValueError):
        bc.duration_csv_path(root, bm, 128, 2, "sputnik", "spmm")

    path = bc.duration_csv_path(root, bm, 256, 8, "wmma", "spmm")
    bc.write_duration_csv(path, "spmm_mfma_kernel", 3.84)
    total_ms = 0.0
    with open(path) as f:
        for row in csv.reader(f):
            if len(row) >= 4 and "Duration" in row[-4]:
                assert row[-3] == "nsecond"
                total_ms += float(row[-2]) / 1e6
    assert total_ms == pytest.approx(3.84e-3)
