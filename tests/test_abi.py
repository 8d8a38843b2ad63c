"""The C-ABI library loads, exports what include/vsparse.h declares, and validates arguments.

No kernel is launched here: every call either is a host helper or is rejected (or is a no-op)
before any device work.
"""
import ctypes
import os
import re

import numpy as np
import pytest

from oracle import c_oracle as co
from vectorsparse_amd import _lib, ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "vsparse.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vs_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    names = _declared()
    assert len(names) >= 13
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert hasattr(raw, name), "libvsparse.so does not export %s" % name
    assert sorted(_lib.SIGNATURES) == names


def test_version_and_status_text():
    L = _lib.lib()
    assert L.vs_version() >= 100
    assert b"success" in L.vs_status_string(0)
    assert b"invalid" in L.vs_status_string(1)
    assert b"not supported" in L.vs_status_string(801)


def test_swizzles_match_oracle():
    rng = np.random.default_rng(1)
    lengths = rng.integers(0, 9, 300)
    ro = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    assert np.array_equal(ops.IdentityRowSwizzle(300), co.identity_row_swizzle(300))
    assert np.array_equal(ops.SortedRowSwizzle(300, ro), co.sorted_row_swizzle(300, ro))
    assert ops.SortedRowSwizzle(0, np.zeros(1, np.int32)).size == 0


def test_argument_validation_without_launch():
    L = _lib.lib()
    p = 0x1000  # never dereferenced: all calls below return before any device work
    INVALID, OK = 1, 0
    # unsupported vector length (the reference prints "Unsupported Vector Length!" and launches nothing)
    assert L.vs_wmma_spmm_f16(4, 3, 64, 64, p, p, p, p, p, p, None) == INVALID
    assert L.vs_cuda_spmm_f16(4, 16, 64, 64, p, p, p, p, p, p, None) == INVALID
    assert L.vs_wmma_sddmm_f16(4, 64, 64, 10, p, p, p, p, p, p, 5, None, 1) == INVALID
    assert L.vs_cuda_sddmm_f16(4, 64, 64, 10, p, p, p, p, p, p, 0, None) == INVALID
    # negative sizes, null pointers, misaligned operands
    assert L.vs_wmma_spmm_f16(-1, 8, 64, 64, p, p, p, p, p, p, None) == INVALID
    assert L.vs_wmma_spmm_f16(4, 8, 64, 64, None, p, p, p, p, p, None) == INVALID
    assert L.vs_wmma_spmm_f16(4, 8, 64, 64, p, p, p, p, p, None, None) == INVALID
    assert L.vs_wmma_spmm_f16(4, 8, 64, 64, p, p, p, p + 2, p, p, None) == INVALID
    assert L.vs_wmma_spmm_f16(4, 8, 64, 64, p, p, p, p, p + 8, p, None) == INVALID
    assert L.vs_cuda_sddmm_f16(4, 64, 64, 10, p, p, p, None, p, p, 8, None) == INVALID
    assert L.vs_wmma_sddmm_f16(4, 64, 64, 10, p, p, p, p, p, p + 2, 8, None, 1) == INVALID
    # algorithm 3 is the reference's timing-only hardware simulation; unknown algorithms launch nothing
    assert L.vs_wmma_sddmm_f16(4, 64, 64, 10, p, p, p, p, p, p, 8, None, 3) == INVALID
    assert L.vs_wmma_sddmm_f16(4, 64, 64, 10, p, p, p, p, p, p, 8, None, -1) == INVALID
    # shapes a path cannot take
    # (the reference-shaped entry points take any dense width / contraction length; the split-row schedule needs
    # k % 4 == 0)
    assert L.vs_wmma_spmm_f16_ws(4, 8, 66, 64, 10, p, p, p, p, p, p, None, 0, None) == 801
    assert L.vs_wmma_spmm_f16_noalloc(4, 8, 66, 64, 10, p, p, p, p, p, p, None) == 801
    assert L.vs_wmma_spmm_f16_noalloc(4, 8, 4224, 64, 10, p, p, p, p, p, p, None) == 801   # beyond the scratch
    # empty problems succeed without touching the device
    assert L.vs_wmma_spmm_f16(0, 8, 64, 64, None, None, None, None, None, None, None) == OK
    assert L.vs_cuda_spmm_f16(4, 8, 0, 64, None, None, None, None, None, None, None) == OK
    assert L.vs_wmma_sddmm_f16(4, 64, 64, 0, None, None, None, None, None, None, 8, None, 1) == OK
    assert L.vs_cuda_sddmm_f16(0, 64, 64, 0, None, None, None, None, None, None, 8, None) == OK


def test_attention_planning_helpers_are_consistent():
    """Host-only planning helpers of the union attention kernel: capacity, row rounding, plan size."""
    L = _lib.lib()
    used = ctypes.c_int(0)
    for V in (1, 2, 4, 8):
        per_wave = 16 // V
        for request in (2, per_wave, 3 * per_wave + 1, 8 * per_wave, 128):
            built = L.vs_sparse_attention_union_capacity(V, 4096, 64, 64, request, 0, None)
            cap = L.vs_sparse_attention_union_capacity(V, 4096, 64, 64, request, 1, ctypes.addressof(used))
            assert used.value % per_wave == 0 and used.value <= 8 * per_wave      # whole waves, at most 8
            assert used.value >= min(request, 8 * per_wave)
            blocks = -(-512 // used.value)
            size = L.vs_sparse_attention_plan_bytes(512, V, 4096, 64, 64, request)
            if used.value == 8 * per_wave:
                # eight waves stream the union: 16 rounds of 128 ranks, 4 mask words per row and round
                assert 0 < built <= 512 and cap == 2048
                assert size == 4 * (16 + blocks * (4 + 16 * (used.value * 4 + 128)))
            else:
                # smaller workgroups hold it at once; a plan frees LDS for more columns
                assert cap % 32 == 0 and 0 < built <= cap <= 512
                mask_words = (used.value * 16 + 3) // 4 * 4
                assert size == 4 * (16 + blocks * (4 + mask_words + cap))
    wide = L.vs_sparse_attention_union_capacity(8, 4096, 128, 128, 16, 0, None)
    narrow = L.vs_sparse_attention_union_capacity(8, 4096, 32, 32, 16, 0, None)
    assert 0 < narrow <= 512 and 0 < wide <= 512               # wide heads: one workgroup per CU with all of its LDS
    assert L.vs_sparse_attention_union_capacity(8, 4096, 64, 36, 16, 0, None) == 0    # d_v % 8 != 0: per-row path only
    assert L.vs_sparse_attention_union_capacity(8, 4096, 256, 64, 16, 0, None) == 0   # d_qk > 128
    for with_plan in (0, 1):
        assert L.vs_sparse_attention_union_capacity(8, 1 << 22, 64, 64, 16, with_plan, None) == 0  # column bitmap too large for LDS
    # the bitmap of 400k columns fits the plan kernel's LDS but not beside the K / V rows
    assert L.vs_sparse_attention_union_capacity(8, 400000, 64, 64, 16, 0, None) == 0
    assert L.vs_sparse_attention_union_capacity(8, 400000, 64, 64, 16, 1, None) > 0
    assert L.vs_sparse_attention_union_capacity(3, 4096, 64, 64, 16, 0, None) == 0
    assert L.vs_sparse_attention_plan_bytes(512, 8, 4096, 64, 64, 1) == 0
    # a plan buffer that is too small, null or misaligned is rejected before any launch
    assert L.vs_sparse_attention_plan(512, 8, 4096, 64, 64, 16, 64, 64, 256, 16, None) == 1
    assert L.vs_sparse_attention_plan(512, 8, 4096, 64, 64, 16, 64, 64, None, 1 << 20, None) == 1
    assert L.vs_sparse_attention_plan(512, 8, 4096, 64, 64, 16, 64, 64, 264, 1 << 20, None) == 1


def test_options():
    _lib.set_option("spmm_waves", 4)
    _lib.set_option("spmm_waves", 0)
    with pytest.raises(_lib.VSparseError):
        _lib.set_option("spmm_waves", 17)
    with pytest.raises(_lib.VSparseError):
        _lib.set_option("no_such_option", 1)
    with pytest.raises(_lib.VSparseError):
        _lib.set_option("spmm_cols_per_lane", 3)
    # every documented name is known, takes 0 (automatic) and rejects a value outside its range
    ranges = {"spmm_waves": 17, "spmm_cols_per_lane": 5, "spmm_steps": 3, "spmm_guard_waves": 17, "spmm_teams": 3, "spmm_pipe": 3, "spmm_blocks_per_wave": 3, "spmm_gather": 3,
              "spmm_flat_launches": 3, "spmm_flat_waves": 17, "spmm_flat_shared": 3, "spmm_parts_launches": 3, "sddmm_group": 3,
              "sddmm_block_waves": 17, "sddmm_flat_supers": 17, "attention_waves": 9}
    for name, bad in ranges.items():
        _lib.set_option(name, 0)
        with pytest.raises(_lib.VSparseError):
            _lib.set_option(name, bad)
    for name in ("spmm_flat_piece", "sddmm_slots", "attention_chunk"):
        _lib.set_option(name, 0)
    with _lib.thread_options(spmm_steps=2, spmm_guard_waves=2):
        pass
    # the two retired variants: accepted by a library built with them, 801 (not 1) otherwise
    for name, value in (("spmm_steps", 4), ("spmm_gather", 2)):
        assert _lib.lib().vs_set_option(name.encode(), value) in (0, 801)
        _lib.set_option(name, 0)


def test_header_is_plain_c_and_cxx(tmp_path):
    """include/vsparse.h compiles as C99 and as C++ with nothing but itself."""
    import subprocess
    src_c = tmp_path / "use.c"
    src_c.write_text('#include "vsparse.h"\nint main(void) { return vs_version() > 0 ? 0 : 1; }\n')
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-fsyntax-only",
                           "-I", os.path.join(ROOT, "include"), str(src_c)])
    src_cpp = tmp_path / "use.cpp"
    src_cpp.write_text('#include "vsparse.h"\nint main() { return vs_version() > 0 ? 0 : 1; }\n')
    subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Werror", "-fsyntax-only",
                           "-I", os.path.join(ROOT, "include"), str(src_cpp)])


def test_reference_side_shim_compiles(tmp_path):
    """The header-only C++ shim carries the reference's overload sets (include/wmma_spmm.cuh:7-29,
    include/cuda_spmm.cuh:7-29, include/wmma_sddmm.cuh:7-33, include/cuda_sddmm.cuh:7-32): a caller written
    like the reference's benchmarks (spmm_benchmark.cpp:127,131; sddmm_benchmark.cpp:257,262) compiles
    against it with every operand type combination the reference declares."""
    import subprocess
    hipcc = "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not installed")
    src = tmp_path / "caller.cpp"
    src.write_text("""
#include "vsparse_shim.hpp"
template <typename In, typename Out> hipError_t call_all(const int* i, const In* a, Out* c, hipStream_t s) {
  hipError_t e = spmm::wmmaSpmm(1, 8, 64, 64, i, i, i, a, a, c);
  if (e == hipSuccess) e = spmm::cudaSpmm(1, 8, 64, 64, i, i, i, a, a, c);
  if (e == hipSuccess) e = sddmm::wmmaSddmm(1, 64, 64, 1, i, i, i, a, a, c, 8, s, 0);
  if (e == hipSuccess) e = sddmm::cudaSddmm(1, 64, 64, 1, i, i, i, a, a, c, 8, s);
  return e;
}
template hipError_t call_all<half, half>(const int*, const half*, half*, hipStream_t);
template hipError_t call_all<half, float>(const int*, const half*, float*, hipStream_t);
template hipError_t call_all<float, float>(const int*, const float*, float*, hipStream_t);
""")
    subprocess.check_call([hipcc, "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-Wall", "-Werror",
                           "-Wno-unused-command-line-argument", "-fsyntax-only",
                           "-I", os.path.join(ROOT, "include"), str(src)])
