"""ctypes binding of libvsparse.so.  Raises if the library is missing: there is no fallback path."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libvsparse.so")

_vp = ctypes.c_void_p
_int = ctypes.c_int
_ll = ctypes.c_longlong

# name -> argtypes, exactly the declarations of include/vsparse.h
SIGNATURES = {
    "vs_version": ([], _int),
    "vs_status_string": ([_int], ctypes.c_char_p),
    "vs_wmma_spmm_f16": ([_int] * 4 + [_vp] * 7, _int),
    "vs_wmma_spmm_f16_f32out": ([_int] * 4 + [_vp] * 7, _int),
    "vs_wmma_spmm_workspace_bytes": ([_int] * 5, _ll),
    "vs_wmma_spmm_f16_ws": ([_int] * 5 + [_vp] * 7 + [_ll, _vp], _int),
    "vs_wmma_spmm_f16_f32out_ws": ([_int] * 5 + [_vp] * 7 + [_ll, _vp], _int),
    "vs_wmma_spmm_noalloc_scratch_bytes": ([], _ll),
    "vs_wmma_spmm_noalloc_reset": ([_vp], _int),
    "vs_wmma_spmm_f16_noalloc": ([_int] * 5 + [_vp] * 6 + [_vp], _int),
    "vs_wmma_spmm_slab_workspace_bytes": ([_int] * 4, _ll),
    "vs_wmma_spmm_f16_slab": ([_int] * 4 + [_vp] * 7 + [_ll, _vp], _int),
    "vs_cuda_spmm_f16": ([_int] * 4 + [_vp] * 7, _int),
    "vs_cuda_spmm_f16_f32out": ([_int] * 4 + [_vp] * 7, _int),
    "vs_wmma_sddmm_f16": ([_int] * 4 + [_vp] * 6 + [_int, _vp, _int], _int),
    "vs_wmma_sddmm_f16_f32out": ([_int] * 4 + [_vp] * 6 + [_int, _vp, _int], _int),
    "vs_cuda_sddmm_f16": ([_int] * 4 + [_vp] * 6 + [_int, _vp], _int),
    "vs_cuda_sddmm_f16_f32out": ([_int] * 4 + [_vp] * 6 + [_int, _vp], _int),
    "vs_wmma_spmm_f16_batched": ([_int] * 7 + [_vp] * 3 + [_vp, _ll, _vp, _ll, _vp, _ll, _vp], _int),
    "vs_wmma_spmm_f16_batched_sorted": ([_int] * 8 + [_vp] * 3 + [_vp, _ll, _vp, _ll, _vp, _ll, _vp], _int),
    "vs_wmma_spmm_launch_shape": ([_int] * 8 + [_vp], _int),
    "vs_cuda_spmm_f16_batched": ([_int] * 7 + [_vp] * 3 + [_vp, _ll, _vp, _ll, _vp, _ll, _vp], _int),
    "vs_wmma_sddmm_f16_batched": ([_int] * 5 + [_vp] * 3 + [_vp, _ll, _vp, _ll, _vp, _ll, _int, _vp, _int], _int),
    "vs_cuda_sddmm_f16_batched": ([_int] * 5 + [_vp] * 3 + [_vp, _ll, _vp, _ll, _vp, _ll, _int, _vp], _int),
    "vs_wmma_spmm_softmax_f16_batched": ([_int] * 7 + [_vp] * 3 + [_vp, _ll, _vp, _ll, _vp, _ll, ctypes.c_float, _vp],
                                         _int),
    "vs_sparse_attention_f16": ([_int] * 6 + [_vp] * 3 + [_vp, _ll, _vp, _ll, _vp, _ll, _vp, _ll, ctypes.c_float, _int,
                                 _vp, _ll, _vp],
                                _int),
    "vs_sparse_attention_union_capacity": ([_int] * 6 + [_vp], _int),
    "vs_sparse_attention_plan_bytes": ([_int] * 6, _ll),
    "vs_sparse_attention_plan": ([_int] * 6 + [_vp] * 3 + [_ll, _vp], _int),
    "vs_sparse_softmax_f16": ([_int] * 3 + [_vp] * 2 + [_vp, _ll, _vp, _ll, ctypes.c_float, _vp], _int),
    "vs_sparse_softmax_row_parts_workspace_bytes": ([_int] * 4, _ll),
    "vs_sparse_softmax_f16_row_parts": ([_int] * 3 + [_vp, _int, _int] + [_vp, _ll, _vp, _ll, ctypes.c_float, _vp, _ll, _vp],
                                        _int),
    "vs_identity_row_swizzle": ([_int, _vp], None),
    "vs_sorted_row_swizzle": ([_int, _vp, _vp], None),
    "vs_spmm_row_parts": ([_int, _vp, _int, _vp, _int, _vp, _vp, _vp, _vp], _int),
    "vs_wmma_spmm_row_parts_workspace_bytes": ([_int] * 5, _ll),
    "vs_wmma_spmm_f16_row_parts": ([_int] * 5 + [_vp] + [_int] * 4 + [_vp] + [_vp, _ll, _vp, _ll, _vp, _ll] + [_vp, _ll, _vp],
                                   _int),
    "vs_wmma_sddmm_f16_row_parts": ([_int] * 4 + [_vp, _int, _vp] + [_vp, _ll, _vp, _ll, _vp, _ll] + [_int, _vp], _int),
    "vs_set_option": ([ctypes.c_char_p, _int], _int),
    "vs_set_thread_option": ([ctypes.c_char_p, _int], _int),
    "vs_clear_thread_options": ([], None),
}

_lib = None


class VSparseError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        msg = lib().vs_status_string(status)
        super().__init__("%s failed with status %d: %s" % (where, status, msg.decode() if msg else "?"))


def lib():
    """Load the library once; a missing file is an error, never a silent fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s not found: build it with `python -m vectorsparse_amd.build` "
                "(hipcc --offload-arch=gfx950)" % LIB_PATH)
        # PyTorch ships a HIP runtime of its own.  Whichever copy a process loads first is the one that sees the
        # GPU; a second copy loaded later reports "no ROCm-capable device".  The tensors this package works on are
        # torch's, so torch goes first and the library binds to the runtime that is already there.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = ctypes.CDLL(LIB_PATH)
        for name, (argtypes, restype) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = L
    return _lib


def check(status, where):
    if status != 0:
        raise VSparseError(status, where)


def set_option(name, value):
    """Process-wide launch-shape override (0 = automatic)."""
    check(lib().vs_set_option(name.encode(), int(value)), "vs_set_option(%s)" % name)


class thread_options:
    """Launch-shape overrides for the calls the current thread makes inside the `with` block, e.g.
    `with thread_options(spmm_waves=4): prob.spmm(...)`.  Other threads are not affected.  Blocks nest: leaving an
    inner block puts back what the enclosing block had set."""

    _stack = __import__("threading").local()

    def __init__(self, **values):
        self.values = values

    def __enter__(self):
        frames = getattr(self._stack, "frames", None)
        if frames is None:
            frames = self._stack.frames = []
        frames.append(self.values)
        try:
            self._apply(frames)
        except Exception:
            frames.pop()            # a rejected value: the enclosing blocks' options stay in force
            self._apply(frames)
            raise
        return self

    def __exit__(self, *exc):
        frames = self._stack.frames
        frames.pop()
        self._apply(frames)
        return False

    @staticmethod
    def _apply(frames):
        """The thread's options = the process-wide ones overridden by every open block, outermost first."""
        lib().vs_clear_thread_options()
        for values in frames:
            for name, value in values.items():
                check(lib().vs_set_thread_option(name.encode(), int(value)), "vs_set_thread_option(%s)" % name)
