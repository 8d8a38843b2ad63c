"""Host-side choices of the Python layer that need no GPU: they only read the mask and ask the library's
host-only capacity query."""
import numpy as np
import pytest

from oracle import c_oracle as co
from vectorsparse_amd import colvec_csr as cv
from vectorsparse_amd import _lib, ops, sweep
from util import retired_variants_built


def _largest_union(mask, rows):
    ro, ci = mask.row_offsets, mask.column_indices
    return max(int(np.unique(ci[ro[f]:ro[min(f + rows, mask.m_vec)]]).size) for f in range(0, mask.m_vec, rows))


def test_attention_launch_shape_follows_the_mask():
    rows_for = ops.SparseAttention._union_rows
    # band + strided columns: eight waves per workgroup
    band = cv.band_strided_pattern(4096, 8, band_half_width=128, stride=128)
    assert rows_for(band, 64, 64) == 16
    # a 513-wide window: unions of more than 512 columns, which eight waves stream through LDS
    window = cv.band_strided_pattern(4096, 8, band_half_width=256, stride=4096)
    assert 512 < _largest_union(window, 16) <= 2048
    assert rows_for(window, 64, 64) == 16
    assert rows_for(band, 128, 128) == 16
    # every vector length fills its waves with 16 scalar rows
    for V in (1, 2, 4):
        assert rows_for(cv.band_strided_pattern(2048, V, band_half_width=128, stride=128), 64, 64) == 128 // V
    # a narrow band: the tile over the union is mostly masked out, yet the union is short
    assert rows_for(cv.band_strided_pattern(4096, 8, band_half_width=4, stride=4096), 64, 64) == 16
    # scattered columns: unions beyond the capacity -> the two launches
    scattered = cv.uniform_pattern(512, 4096, 0.9, seed=3, vec_length=8)
    assert _largest_union(scattered, 16) > 2048
    assert rows_for(scattered, 64, 64) == 1
    # head widths the union kernel does not take
    assert rows_for(band, 64, 36) == 1
    # empty masks
    empty = cv.ColVecCSR(4, 64, 8, np.zeros(5, np.int32), np.zeros(0, np.int32))
    assert rows_for(empty, 64, 64) == 1


def test_attention_launch_shape_weighs_union_columns_against_nonzeros():
    """The streamed kernel pays per union column, the two launches per nonzero (measured on MI355X, 16 heads x
    4096: V = 8 uniform random masks switch between 99.5 % and 99.8 % sparsity, V = 1 takes the single launch
    whenever 128 rows' columns fit), and a launch of few workgroups is as long as its longest workgroup."""
    rows_for = ops.SparseAttention._union_rows
    for sparsity, want in ((0.98, 1), (0.99, 1), (0.998, 16)):
        mask = cv.uniform_pattern(512, 4096, sparsity, seed=7, vec_length=8)
        assert _largest_union(mask, 16) <= 2048
        assert rows_for(mask, 64, 64) == want, sparsity
    sparse_v1 = cv.uniform_pattern(4096, 4096, 0.998, seed=7, vec_length=1)
    assert _largest_union(sparse_v1, 128) <= 2048 and rows_for(sparse_v1, 64, 64) == 128
    # the same mask with 16 heads and with 2: 32 workgroups of 900 columns each lose to the two launches
    small = cv.uniform_pattern(2048, 2048, 0.995, seed=7, vec_length=1)
    assert rows_for(small, 64, 64, heads=64) == 128
    assert rows_for(small, 64, 64, heads=2) == 1
    # wider heads run one workgroup per CU: the switch comes earlier
    mask = cv.uniform_pattern(512, 4096, 0.995, seed=7, vec_length=8)
    assert rows_for(mask, 128, 128) == 1


def test_device_problem_reads_the_row_statistics():
    """Row statistics that steer the schedules (no launch: operands stay in host memory here)."""
    rng = np.random.default_rng(0)
    lengths = np.minimum((rng.pareto(1.5, 1024) + 0.3) * 150, 4608).astype(np.int64)
    lengths[5] = 4608
    ro, ci = cv._pattern_from_lengths(rng, 1024, 4608, lengths)
    heavy = ops.DeviceProblem(cv.ColVecCSR(1024, 4608, 8, ro, ci), sort=True, device="cpu")
    assert heavy.longest_row_vec == 4608 and heavy.nnz_vec == int(lengths.sum())
    assert heavy.skewed                                    # SDDMM takes rows in parts by default (the nonzero-range schedule where that entry does not apply)
    swz = heavy.row_indices.numpy()
    assert sorted(swz.tolist()) == list(range(1024)) and np.all(np.diff(lengths[swz]) <= 0)
    even = ops.DeviceProblem(cv.uniform_pattern(1024, 4608, 0.9, seed=1, vec_length=8), device="cpu")
    assert not even.skewed and even.longest_row_vec == 461
    assert even.row_indices.numpy().tolist() == list(range(1024))
    tiny = ops.DeviceProblem(cv.ColVecCSR(2, 8, 2, np.array([0, 0, 0], np.int32), np.zeros(0, np.int32)), device="cpu")
    assert tiny.longest_row_vec == 0 and not tiny.skewed


def test_split_row_choice_follows_the_row_lengths():
    """Where the split-row schedule is ahead of the row-length hints, on the row-length shapes it was measured on."""
    pays = ops.split_rows_pays
    # one dense row among rows of a hundred vectors: pays up to 1024 rows
    for m_vec in (64, 256, 1024):
        assert pays(m_vec, 4608 + 100 * (m_vec - 1), 4608)
    assert not pays(2048, 4608 + 100 * 2047, 4608)
    # uniform lengths: never
    for m_vec in (64, 1024):
        assert not pays(m_vec, 461 * m_vec, 461)
    # longest row at 15 mean lengths (Pareto): the hinted row-per-workgroup schedule is ahead at every size
    assert not pays(128, 128 * 300, 4500) and not pays(1024, 1024 * 300, 4500)
    # too small to matter, and degenerate shapes
    assert not pays(8, 400, 300) and not pays(0, 0, 0)


def test_spmm_launch_shape_choice():
    """The host-side shape choice of the MFMA SpMM: what it picks on the named configurations, and that every
    choice respects what the kernel variants assume (their launch bounds and the grid arithmetic)."""
    shape = ops.spmm_launch_shape
    # headline shape (512 x 4608 x 256, V = 8): narrow tiles so that 64 rows give 256 workgroups, two steps in
    # flight, eight waves per row of about fifteen steps
    headline = shape(64, 8, 256, 4608)
    assert (headline["cols_per_lane"], headline["steps_in_flight"], headline["waves"]) == (4, 2, 8)
    assert headline["team_slots"] == -1 and not headline["ragged"] and not headline["dma"]
    # largest sweep point: wide tiles (128-bit row segments), two steps in flight and waves that pipeline the blocks
    # they walk; four steps in flight only where that walk is switched off and the row lengths are known
    largest = shape(256, 8, 256, 4608)
    assert (largest["cols_per_lane"], largest["steps_in_flight"], largest["pipelined"]) == (8, 2, 1)
    hinted = shape(256, 8, 256, 4608, nonzeros_vec=256 * 461, longest_row_vec=470)
    assert (hinted["steps_in_flight"], hinted["pipelined"]) == (2, 1)
    with _lib.thread_options(spmm_pipe=1):
        # (four steps in flight are compiled only into a library built with VS_RETIRED_VARIANTS=1)
        assert shape(256, 8, 256, 4608, nonzeros_vec=256 * 461, longest_row_vec=470)["steps_in_flight"] == (
            4 if retired_variants_built() else 2)
        assert shape(256, 8, 256, 4608)["pipelined"] == 0
    # rows known to hold one or two blocks on a grid of 4096 workgroups: the plain walk
    assert shape(2048, 8, 256, 4608, nonzeros_vec=2048 * 60, longest_row_vec=100)["pipelined"] == 0
    assert shape(2048, 8, 256, 4608)["pipelined"] == 1
    # one 64-column tile for narrow dense operands, the half-by-half variant for widths off a multiple of 4
    assert shape(512, 8, 64, 4096)["cols_per_lane"] == 4
    assert shape(64, 8, 147, 4608)["ragged"] == 1 and shape(64, 8, 148, 4608)["ragged"] == 0
    # rows of under one step: one wave, one step
    short = shape(4096, 8, 256, 64, nonzeros_vec=4096 * 6, longest_row_vec=6)
    assert (short["steps_in_flight"], short["waves"]) == (1, 1)
    # unhinted launch on a grid that fills the chip keeps guard waves for a row far longer than expected ...
    guarded = shape(1024, 8, 256, 4608)
    assert guarded["waves"] >= 2 and guarded["blocks_per_wave"] >= 2
    # ... and drops them with the lengths known
    assert shape(1024, 8, 256, 4608, nonzeros_vec=1024 * 461, longest_row_vec=470)["blocks_per_wave"] >= 1
    # skewed rows, ordered by length, the count of long rows known: teams for those rows only
    # (on grids of sixteen workgroups per CU or more whose average row is short)
    teams = shape(2048, 8, 256, 4608, nonzeros_vec=2048 * 100 + 4508, longest_row_vec=4608, long_rows=1)
    assert teams["team_slots"] == 1 and teams["steps_in_flight"] == 2 and 4 <= teams["waves"] <= 8
    assert shape(512, 8, 256, 4608, nonzeros_vec=512 * 100 + 4508, longest_row_vec=4608, long_rows=1)["team_slots"] == -1
    assert shape(2048, 8, 256, 4608, nonzeros_vec=2048 * 300 + 4308, longest_row_vec=4608, long_rows=1)["team_slots"] == -1
    with _lib.thread_options(spmm_teams=1):
        assert shape(2048, 8, 256, 4608, nonzeros_vec=2048 * 100 + 4508, longest_row_vec=4608,
                     long_rows=1)["team_slots"] == -1
    # an override is taken as given
    with _lib.thread_options(spmm_waves=2, spmm_steps=1, spmm_cols_per_lane=8):
        forced = shape(64, 8, 256, 4608)
        assert (forced["cols_per_lane"], forced["steps_in_flight"], forced["waves"]) == (8, 1, 2)
    # invariants over random problems, hinted and not
    rng = np.random.default_rng(11)
    for _ in range(3000):
        m_vec = int(rng.integers(1, 9000))
        k = int(rng.integers(1, 1100))
        n = int(rng.integers(1, 9000))
        batch = int(rng.choice([1, 1, 1, 4, 16]))
        hints = {}
        if rng.random() < 0.6:
            longest = int(rng.integers(0, n + 1))
            mean = int(rng.integers(0, longest + 1))
            hints = dict(nonzeros_vec=min(mean * m_vec, 2**31 - 1), longest_row_vec=longest)
            if rng.random() < 0.5:
                hints["long_rows"] = int(rng.integers(0, m_vec + 1))
        got = shape(m_vec, int(rng.choice([1, 2, 4, 8])), k, n, batch=batch, **hints)
        case = (m_vec, k, n, batch, hints, got)
        assert got["cols_per_lane"] in (4, 8) and got["steps_in_flight"] in (1, 2, 4), case
        assert got["waves"] in (1, 2, 4, 8, 16), case
        # the launch bounds of the variants with 64 / 128 registers of row segments in flight
        assert got["waves"] * 64 <= (256 if got["steps_in_flight"] * got["cols_per_lane"] >= 32 else
                                     512 if got["steps_in_flight"] * got["cols_per_lane"] >= 16 else 1024), case
        assert got["blocks_per_wave"] >= 1 and got["blocks_per_wave"] & (got["blocks_per_wave"] - 1) == 0, case
        assert -1 <= got["team_slots"] <= m_vec, case
        if got["team_slots"] >= 0:
            assert got["steps_in_flight"] == 2 and got["blocks_per_wave"] == 1, case
        if got["pipelined"]:
            assert got["steps_in_flight"] == 2 and not got["ragged"] and not got["dma"], case
        assert bool(got["ragged"]) == (k % 4 != 0), case
        if got["ragged"]:
            assert got["cols_per_lane"] == 4 and got["steps_in_flight"] == 1 and got["waves"] <= 8, case
        if got["cols_per_lane"] == 8:
            assert k % 8 == 0, case
    for bad in (dict(m_vec=0), dict(k=0), dict(vec_length=3), dict(batch=0)):
        args = dict(m_vec=64, vec_length=8, k=256, n=4608)
        args.update(bad)
        with pytest.raises(_lib.VSparseError):
            shape(**args)


def test_attention_parts_route_respects_the_workspace_limit():
    """The automatic three-operator route on row parts is taken only while the SpMM's partial tiles stay below the
    2 GiB the entry point accepts; beyond that the layer falls back to its other routes instead of failing."""
    import types
    layer = ops.SparseAttention.__new__(ops.SparseAttention)
    few = types.SimpleNamespace(n_split=8, parts_max=9)
    many = types.SimpleNamespace(n_split=1000, parts_max=100)
    layer.prob = types.SimpleNamespace(vec_length=8, row_parts=lambda limit: [few])
    assert layer._parts_route_fits(64, 16)
    layer.prob = types.SimpleNamespace(vec_length=8, row_parts=lambda limit: [many])
    assert ops.spmm_row_parts_workspace_bytes(8, 64, many.n_split, many.parts_max, batch=16) >= 2 ** 31
    assert not layer._parts_route_fits(64, 16)
    assert layer._parts_route_fits(64, 1)


def test_thread_option_blocks_nest():
    """Leaving an inner `thread_options` block restores the enclosing block's overrides (not the process-wide ones),
    and a rejected value leaves them untouched."""
    shape = ops.spmm_launch_shape
    auto = shape(64, 8, 256, 4608)
    with _lib.thread_options(spmm_waves=2):
        assert shape(64, 8, 256, 4608)["waves"] == 2
        with _lib.thread_options(spmm_cols_per_lane=8):
            inner = shape(64, 8, 256, 4608)
            assert (inner["waves"], inner["cols_per_lane"]) == (2, 8)
        after = shape(64, 8, 256, 4608)
        assert (after["waves"], after["cols_per_lane"]) == (2, auto["cols_per_lane"])
        with pytest.raises(_lib.VSparseError):
            with _lib.thread_options(spmm_waves=99):
                pass
        assert shape(64, 8, 256, 4608)["waves"] == 2
    assert shape(64, 8, 256, 4608) == auto


def test_sweep_benchmark_selection(tmp_path):
    """The sweep driver's file handling (job_launcher.py:25-50): list files, ranges, layer widths, buckets."""
    from vectorsparse_amd import sweep

    root = tmp_path / "dlmc"
    names = ["rn50/random_pruning/0.8/layer_a", "rn50/random_pruning/0.95/layer_b", "rn50/magnitude_pruning/0.9/layer_c"]
    for i, name in enumerate(names):
        path = root / (name + ".smtx")
        path.parent.mkdir(parents=True, exist_ok=True)
        pat = cv.uniform_pattern(8, 64, 0.5, seed=i, vec_length=1)
        cv.write_smtx(str(path), pat.m_vec, pat.n, pat.row_offsets, pat.column_indices)
    listing = tmp_path / "rn50_matrices.txt"
    listing.write_text("".join(n + ".smtx\n" for n in names))
    widths = tmp_path / "rn50_batchsizes.txt"
    widths.write_text("layer_a,196\nlayer_b,49\nlayer_c,3136\n")

    everything = sweep.file_benchmarks(str(root))
    assert sorted(n for n, _ in everything) == sorted(names)
    picked = sweep.file_benchmarks(str(root), str(listing), 1, 3)
    assert [n for n, _ in picked] == names[1:3]
    assert all(p.endswith(".smtx") and cv.read_smtx(p, 2).m_vec == 8 for _, p in picked)

    table = sweep.layer_widths(str(widths))
    assert table == {"layer_a": 196, "layer_b": 49, "layer_c": 3136}
    assert sweep.widths_for(names[0], (64, 256), 1, table) == [64, 256]
    assert sweep.widths_for(names[1], (-1,), 2, table) == [98]          # the layer's own width, scaled
    assert sweep.int_list("1,2, 8") == (1, 2, 8)

    assert sweep.sparsity_bucket(names[0], 0.79) == 0.8
    assert sweep.sparsity_bucket(names[1], 0.5) == 0.95                 # the directory decides, not the file
    assert sweep.sparsity_bucket(names[2], 0.5) == 0.9
    assert sweep.sparsity_bucket("synthetic/m64", 0.8765) == 0.88


def test_plot_reads_the_sweep_result_file(tmp_path):
    """Geometric means per (path, V, k, sparsity bucket) from the rows the sweep writes."""
    import csv
    from vectorsparse_amd import plot

    rows = []
    for V in (2, 8):
        for k in (64, 256):
            for s, ups in ((0.7, (1.0, 4.0)), (0.9, (2.0, 8.0))):
                for kernel, scale in (("wmma", 1.0), ("cuda", 0.5)):
                    for up in ups:
                        rows.append({"op": "spmm", "bm": "x", "k": k, "M": 64, "K": 128, "N": k, "sparsity": s, "V": V,
                                     "kernel": kernel, "nnz_vec": 1, "us": 1.0, "dense_us": up, "speedup": up * scale,
                                     "tflops": 1.0, "gbs": 1.0})
    result = tmp_path / "result.csv"
    with open(result, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=list(rows[0].keys()))
        w.writeheader()
        w.writerows(rows)
    geo = tmp_path / "geo.csv"
    assert plot.main(["--csv", str(result), "--geo", str(geo)]) == 0
    with open(geo) as f:
        table = list(csv.reader(f))
    assert table[0] == ["path", "V", "k", "0.7", "0.9"]
    means = {(r[0], int(r[1]), int(r[2])): (float(r[3]), float(r[4])) for r in table[1:]}
    assert len(means) == 8
    assert means[("mma", 8, 256)] == pytest.approx((2.0, 4.0))      # sqrt(1 * 4), sqrt(2 * 8)
    assert means[("fpu", 2, 64)] == pytest.approx((1.0, 2.0))


def test_the_sweep_check_catches_a_wrong_result():
    """The driver's verification must fail on a result that is wrong in one sampled row."""
    pat = sweep.spmm_grid_pattern(64, 256, 0.9, 8)
    B = cv.dense_uniform(256, 64, seed=1)
    ref = co.spmm_host_ref_f32(pat.m_vec, 8, 64, 256, pat.row_offsets, pat.column_indices, pat.values, B)
    assert sweep.verify_spmm(pat, B, ref.astype(np.float16))[0]
    bad = ref.astype(np.float16).copy()
    bad[0, 5] += np.float16(1.0)
    assert not sweep.verify_spmm(pat, B, bad)[0]
    A = cv.dense_normal(64, 32, seed=2)
    R = cv.dense_normal(256, 32, seed=3)
    good = co.sddmm_host_ref_f32(pat.m_vec, 32, 8, pat.row_offsets, pat.column_indices, A, R)
    assert sweep.verify_sddmm(pat, A, R, good.astype(np.float16))[0]
    worse = good.astype(np.float16).copy()
    worse[3] = -worse[3] + np.float16(2.0)
    assert not sweep.verify_sddmm(pat, A, R, worse)[0]


def test_row_parts_dispatch_list():
    """vs_spmm_row_parts (host): every nonzero in exactly one slot, the parts of a split row in ascending order and
    whole 64-vector blocks except the last, the list longest first, the counts as promised."""
    import ctypes
    rng = np.random.default_rng(12)
    for trial in range(40):
        m_vec = int(rng.integers(0, 200))
        lengths = np.minimum((rng.pareto(1.2, m_vec) + 0.1) * rng.integers(1, 300), 5000).astype(np.int64)
        lengths[rng.random(m_vec) < 0.1] = 0
        ro = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
        limit = int(rng.choice([0, 1, 64, 100, 512, 1000, 4096]))
        parts = ops.RowParts(m_vec, ro, limit)
        default = max(1152, 4 * (int(ro[-1]) // m_vec)) if m_vec else 1152
        step = ((default if limit == 0 else limit) + 63) // 64 * 64
        assert parts.slots.shape == (parts.n_slots + parts.n_split, 4)
        s = parts.slots[:parts.n_slots]
        tail = parts.slots[parts.n_slots:]   # behind the list: {row, parts} of every split row, by its number
        for number, (row, count, _, _) in enumerate(tail):
            mine = s[(s[:, 3] != 0) & ((s[:, 3] >> 16) == number)]
            assert len(mine) == count and (mine[:, 0] == row).all()
        seg = s[:, 2] - s[:, 1]
        assert (seg >= 0).all() and (seg <= step).all()
        assert (np.diff(seg) <= 0).all(), "longest first"
        assert parts.longest_part_vec == (int(seg.max()) if len(seg) else 0)
        covered = np.zeros(int(ro[-1]), dtype=np.int32)
        seen_rows = set()
        split_ids = set()
        for row in range(m_vec):
            mine = s[s[:, 0] == row]
            assert len(mine) >= 1, "every row, the empty ones included, has a slot"
            seen_rows.add(row)
            if len(mine) == 1:
                assert mine[0, 3] == 0 and mine[0, 1] == ro[row] and mine[0, 2] == ro[row + 1]
                assert ro[row + 1] - ro[row] <= step
            else:
                info = mine[:, 3]
                assert ((info & 255) == len(mine)).all() and len(mine) <= parts.parts_max
                assert np.array_equal((info >> 8) & 255, np.arange(len(mine))), "parts in ascending order in the list"
                assert len(set(info >> 16)) == 1
                split_ids.add(int(info[0] >> 16))
                assert mine[0, 1] == ro[row] and mine[-1, 2] == ro[row + 1]
                assert np.array_equal(mine[1:, 1], mine[:-1, 2]), "parts follow each other without gaps"
                assert ((mine[:-1, 2] - mine[:-1, 1]) % 64 == 0).all()
            for b, e in mine[:, 1:3]:
                covered[b:e] += 1
        assert (covered == 1).all()
        assert split_ids == set(range(parts.n_split))
        assert parts.parts_max == (max((s[:, 3] & 255)) if parts.n_split else 0)
    # more rows beyond the limit than a split row's number can count: the first 32767 are split, the others whole
    m_vec = 33000
    ro = (np.arange(m_vec + 1, dtype=np.int64) * 128).astype(np.int32)
    parts = ops.RowParts(m_vec, ro, 64)
    assert parts.n_split == 32767 and parts.parts_max == 2 and parts.n_slots == m_vec + 32767
    assert parts.longest_part_vec == 128
    s = parts.slots[:parts.n_slots]
    whole = s[s[:, 3] == 0]
    assert np.array_equal(np.sort(whole[:, 0]), np.arange(32767, m_vec)) and (whole[:, 2] - whole[:, 1] == 128).all()
    halves = s[s[:, 3] != 0]
    assert (halves[:, 2] - halves[:, 1] == 64).all() and np.array_equal(np.sort(halves[:, 3] >> 16),
                                                                        np.repeat(np.arange(32767), 2))
    covered = np.zeros(int(ro[-1]), dtype=np.int32)
    np.add.at(covered, (s[:, 1][:, None] + np.arange(64)[None, :]).reshape(-1), 1)
    np.add.at(covered, (whole[:, 1][:, None] + 64 + np.arange(64)[None, :]).reshape(-1), 1)
    assert (covered == 1).all()
    # too little room: the counts say what the list needs
    ro = np.array([0, 2000, 2010], dtype=np.int32)
    slots = np.zeros((2, 4), dtype=np.int32)
    c = [ctypes.c_int(0) for _ in range(4)]
    st = _lib.lib().vs_spmm_row_parts(2, ro.ctypes.data, 512, slots.ctypes.data, 2, *[ctypes.addressof(x) for x in c])
    assert st == 801 and c[0].value == 5 and c[1].value == 1 and c[2].value == 4
    assert _lib.lib().vs_spmm_row_parts(2, ro.ctypes.data, -1, slots.ctypes.data, 2, *[ctypes.addressof(x) for x in c]) == 1
    assert _lib.lib().vs_wmma_spmm_row_parts_workspace_bytes(1, 8, 256, 0, 0) == 0
    assert _lib.lib().vs_wmma_spmm_row_parts_workspace_bytes(1, 8, 256, 3, 4) > 3 * 4 * 8 * 256 * 4
    assert _lib.lib().vs_wmma_spmm_row_parts_workspace_bytes(5, 8, 256, 3, 4) > 5 * 3 * 4 * 8 * 256 * 4
