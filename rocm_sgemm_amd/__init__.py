"""Python binding of the MI355X SGEMM library (librocm_sgemm.so, hand-written gfx950 HIP kernels).

A thin ctypes layer over the C ABI in include/rocm_sgemm.h.  `gemm` mirrors the reference entry
point rocm_sgemm::gemm<layout_C, layout_A, layout_B>(C, A, B, M, N, K, stream)
(reference rocm_sgemm/include/rocm_sgemm/gemm.hpp:51-52): same argument order, layouts named
row_major / col_major, raw device buffers, stream-ordered and non-blocking.

There is no CPU fallback: if the shared library is missing the import of the native handle raises.
PyTorch is used by callers only to own device memory and streams; this module accepts anything with
a `data_ptr()` method or a plain integer device address.
"""

import ctypes
import os

__all__ = [
    "ROW_MAJOR", "COL_MAJOR", "Config", "SgemmError", "NoKernelError", "lib", "lib_path", "gemm",
    "gemm_no_alloc", "gemm_with_config", "gemm_strided_batched", "find_config", "nearest_config", "predict_us", "table", "family", "config_supported", "map_workgroup",
    "release_workspaces", "version", "CXX_SYMBOLS", "C_SYMBOLS",
]

ROW_MAJOR = 0
COL_MAJOR = 1
_LAYOUT_NAMES = {"row_major": ROW_MAJOR, "col_major": COL_MAJOR, "r": ROW_MAJOR, "c": COL_MAJOR,
                 ROW_MAJOR: ROW_MAJOR, COL_MAJOR: COL_MAJOR}

(STATUS_OK, STATUS_INVALID_ARG, STATUS_NO_KERNEL, STATUS_LAUNCH_FAILED, STATUS_BAD_CONFIG,
 STATUS_WORKSPACE_TOO_LARGE) = range(6)
NO_ALLOC_SCRATCH_BYTES = 128 * 1024 * 1024

# Every extern "C" symbol declared in include/rocm_sgemm.h.
C_SYMBOLS = (
    "rocm_sgemm_f32", "rocm_sgemm_f32_no_alloc", "rocm_sgemm_workspace_bytes", "rocm_sgemm_f32_with_config",
    "rocm_sgemm_f32_strided_batched",
    "rocm_sgemm_f32_strided_batched_with_config", "rocm_sgemm_nearest_config", "rocm_sgemm_find_config",
    "rocm_sgemm_find_config_batched", "rocm_sgemm_predict_us",
    "rocm_sgemm_table_size", "rocm_sgemm_table_entry", "rocm_sgemm_family_size",
    "rocm_sgemm_family_entry", "rocm_sgemm_config_supported", "rocm_sgemm_map_workgroup",
    "rocm_sgemm_release_workspaces", "rocm_sgemm_last_error", "rocm_sgemm_version",
)


def cxx_symbol(layout_c, layout_a, layout_b):
    """Itanium-mangled name of rocm_sgemm::gemm<(m_layout)c, (m_layout)a, (m_layout)b, float>."""
    return (f"_ZN10rocm_sgemm4gemmILNS_8m_layoutE{layout_c}ELS1_{layout_a}ELS1_{layout_b}EfEEv"
            "PT2_S3_S3_mmmRP12ihipStream_t")


# The eight symbols a program compiled against the reference header leaves undefined.
CXX_SYMBOLS = tuple(cxx_symbol(c, a, b) for c in (0, 1) for a in (0, 1) for b in (0, 1))


class Config(ctypes.Structure):
    """struct rocm_sgemm_config."""
    _fields_ = [(n, ctypes.c_int) for n in
                ("macro_m", "macro_n", "k_tile", "waves_m", "waves_n", "mfma", "stages", "split_k",
                 "group_m", "wave_slots", "waves_k", "partial_sums")]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}

    _DEFAULTS = {"mfma": 32, "stages": 0, "split_k": 1, "group_m": 4, "wave_slots": 0, "waves_k": 1,
                 "partial_sums": 0}

    @classmethod
    def from_dict(cls, d):
        return cls(*(int(d[n] if n in d else cls._DEFAULTS[n]) for n, _ in cls._fields_))

    def __repr__(self):
        return "Config(" + ", ".join(f"{k}={v}" for k, v in self.as_dict().items()) + ")"


class SgemmError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"rocm_sgemm status {status}: {message}")
        self.status = status


class NoKernelError(SgemmError):
    """Counterpart of the std::runtime_error the reference throws for an empty kernel-table slot."""


def lib_path():
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "librocm_sgemm.so")


_lib = None


def lib():
    """Loads librocm_sgemm.so once.  Raises if it has not been built - there is no fallback."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `python -m rocm_sgemm_amd.build` "
            "(the library has no CPU or PyTorch fallback)")
    try:
        # If PyTorch is going to be used in this process its bundled HIP runtime must be the one
        # the library binds to, so import it first when available.
        import torch  # noqa: F401
    except ImportError:
        pass
    handle = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
    c_int, c_size_t, c_void_p = ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p
    cfg_p = ctypes.POINTER(Config)
    handle.rocm_sgemm_f32.argtypes = [c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_size_t,
                                      c_size_t, c_size_t, c_void_p]
    handle.rocm_sgemm_f32_with_config.argtypes = [cfg_p] + handle.rocm_sgemm_f32.argtypes
    handle.rocm_sgemm_f32_no_alloc.argtypes = handle.rocm_sgemm_f32.argtypes
    handle.rocm_sgemm_workspace_bytes.argtypes = [c_int, c_int, c_int, c_size_t, c_size_t, c_size_t,
                                                  ctypes.POINTER(c_size_t)]
    c_float, c_ll = ctypes.c_float, ctypes.c_longlong
    handle.rocm_sgemm_f32_strided_batched.argtypes = [
        c_int, c_int, c_int, c_float, c_void_p, c_size_t, c_ll, c_void_p, c_size_t, c_ll, c_float,
        c_void_p, c_size_t, c_ll, c_size_t, c_size_t, c_size_t, c_size_t, c_void_p]
    handle.rocm_sgemm_f32_strided_batched_with_config.argtypes = \
        [cfg_p] + handle.rocm_sgemm_f32_strided_batched.argtypes
    handle.rocm_sgemm_find_config.argtypes = [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, cfg_p]
    handle.rocm_sgemm_nearest_config.argtypes = [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, cfg_p]
    handle.rocm_sgemm_table_entry.argtypes = [c_int] + [ctypes.POINTER(c_size_t)] * 3 \
        + [ctypes.POINTER(c_int)] * 3 + [cfg_p]
    handle.rocm_sgemm_family_entry.argtypes = [c_int, cfg_p]
    handle.rocm_sgemm_config_supported.argtypes = [cfg_p, c_int, c_int, c_int]
    handle.rocm_sgemm_map_workgroup.argtypes = [c_int] * 4 + [ctypes.POINTER(c_int)] * 2
    handle.rocm_sgemm_last_error.restype = ctypes.c_char_p
    handle.rocm_sgemm_version.restype = ctypes.c_char_p
    handle.rocm_sgemm_release_workspaces.restype = None
    handle.rocm_sgemm_predict_us.argtypes = [cfg_p, c_size_t, c_size_t, c_size_t, c_size_t]
    handle.rocm_sgemm_find_config_batched.argtypes = [c_size_t, c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, cfg_p]
    handle.rocm_sgemm_predict_us.restype = ctypes.c_double
    for name in C_SYMBOLS:
        if getattr(handle, name).restype not in (ctypes.c_char_p, ctypes.c_double, None):
            getattr(handle, name).restype = c_int
    _lib = handle
    return _lib


def _layout(v):
    try:
        return _LAYOUT_NAMES[v]
    except KeyError:
        raise ValueError(f"layout must be 'row_major' or 'col_major', got {v!r}") from None


def _ptr(buf):
    if buf is None:
        return None
    if isinstance(buf, int):
        return ctypes.c_void_p(buf)
    return ctypes.c_void_p(buf.data_ptr())


def _stream(stream):
    if stream is None:
        return None
    if isinstance(stream, int):
        return ctypes.c_void_p(stream)
    return ctypes.c_void_p(stream.cuda_stream)  # torch.cuda.Stream


def _check(status):
    if status == STATUS_OK:
        return
    msg = lib().rocm_sgemm_last_error().decode()
    if status == STATUS_NO_KERNEL:
        raise NoKernelError(status, msg)
    raise SgemmError(status, msg)


def gemm(C, A, B, M, N, K, layout_c="row_major", layout_a="row_major", layout_b="row_major",
         stream=None):
    """C (M x N) <- A (M x K) @ B (K x N) on `stream`; buffers are dense, packed device memory."""
    _check(lib().rocm_sgemm_f32(_layout(layout_c), _layout(layout_a), _layout(layout_b),
                                _ptr(C), _ptr(A), _ptr(B), M, N, K, _stream(stream)))


def gemm_no_alloc(C, A, B, M, N, K, layout_c="row_major", layout_a="row_major", layout_b="row_major",
                  stream=None):
    """The same product as `gemm` without any device allocation: partial products of a split-K or
    stream-K-tail config live in the library's fixed scratch array (NO_ALLOC_SCRATCH_BYTES per
    GPU, shared by all calls on it); a problem that needs more raises SgemmError with
    STATUS_WORKSPACE_TOO_LARGE."""
    _check(lib().rocm_sgemm_f32_no_alloc(_layout(layout_c), _layout(layout_a), _layout(layout_b),
                                         _ptr(C), _ptr(A), _ptr(B), M, N, K, _stream(stream)))


def workspace_bytes(M, N, K, layout_a="row_major", layout_b="row_major", layout_c="row_major"):
    """Bytes of workspace `gemm` would use for the partial products of this problem under the config
    it plans (0 = none); what `gemm_no_alloc` holds against NO_ALLOC_SCRATCH_BYTES.  Host only."""
    out = ctypes.c_size_t()
    _check(lib().rocm_sgemm_workspace_bytes(_layout(layout_c), _layout(layout_a), _layout(layout_b), M, N, K,
                                            ctypes.byref(out)))
    return out.value


def gemm_with_config(config, C, A, B, M, N, K, layout_c="row_major", layout_a="row_major",
                     layout_b="row_major", stream=None):
    """Same product with an explicit Config (what a tuner trial calls)."""
    if isinstance(config, dict):
        config = Config.from_dict(config)
    _check(lib().rocm_sgemm_f32_with_config(ctypes.byref(config), _layout(layout_c),
                                            _layout(layout_a), _layout(layout_b), _ptr(C), _ptr(A),
                                            _ptr(B), M, N, K, _stream(stream)))


def gemm_strided_batched(C, A, B, M, N, K, batch_count=1, alpha=1.0, beta=0.0, lda=0, ldb=0, ldc=0,
                         stride_a=0, stride_b=0, stride_c=0, layout_c="row_major",
                         layout_a="row_major", layout_b="row_major", stream=None, config=None):
    """For b < batch_count: C_b <- alpha * A_b @ B_b + beta * C_b with Z_b = Z + b * stride_z
    elements and leading dimensions lda / ldb / ldc (0 = packed)."""
    if isinstance(config, dict):
        config = Config.from_dict(config)
    args = (_layout(layout_c), _layout(layout_a), _layout(layout_b), alpha, _ptr(A), lda, stride_a,
            _ptr(B), ldb, stride_b, beta, _ptr(C), ldc, stride_c, M, N, K, batch_count, _stream(stream))
    if config is None:
        _check(lib().rocm_sgemm_f32_strided_batched(*args))
    else:
        _check(lib().rocm_sgemm_f32_strided_batched_with_config(ctypes.byref(config), *args))


def find_config(M, N, K, layout_a="row_major", layout_b="row_major", layout_c="row_major", batch_count=1):
    """Config the library would use for this problem, or for `batch_count` such products launched
    together (host-only; argument order A, B, C as in the reference's find_best_config)."""
    out = Config()
    if batch_count == 1:
        _check(lib().rocm_sgemm_find_config(M, N, K, _layout(layout_a), _layout(layout_b),
                                            _layout(layout_c), ctypes.byref(out)))
    else:
        _check(lib().rocm_sgemm_find_config_batched(M, N, K, batch_count, _layout(layout_a), _layout(layout_b),
                                                    _layout(layout_c), ctypes.byref(out)))
    return out


def nearest_config(M, N, K, layout_a="row_major", layout_b="row_major", layout_c="row_major"):
    """The table lookup alone (the reference's find_best_config rule), before any planning."""
    out = Config()
    _check(lib().rocm_sgemm_nearest_config(M, N, K, _layout(layout_a), _layout(layout_b),
                                           _layout(layout_c), ctypes.byref(out)))
    return out


def predict_us(config, M, N, K, batch_count=1):
    """The library's cost model: rough microseconds of `batch_count` M x N x K products launched
    together under `config`."""
    if isinstance(config, dict):
        config = Config.from_dict(config)
    return lib().rocm_sgemm_predict_us(ctypes.byref(config), M, N, K, batch_count)


def table():
    """The tuned table as a list of ((M, N, K, layout_a, layout_b, layout_c), Config)."""
    out = []
    L = lib()
    for i in range(L.rocm_sgemm_table_size()):
        m, n, k = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
        a, b, c = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        cfg = Config()
        _check(L.rocm_sgemm_table_entry(i, ctypes.byref(m), ctypes.byref(n), ctypes.byref(k),
                                        ctypes.byref(a), ctypes.byref(b), ctypes.byref(c),
                                        ctypes.byref(cfg)))
        out.append(((m.value, n.value, k.value, a.value, b.value, c.value), cfg))
    return out


def family():
    """Tile shapes compiled into the library (the tuner's search space)."""
    out = []
    L = lib()
    for i in range(L.rocm_sgemm_family_size()):
        cfg = Config()
        _check(L.rocm_sgemm_family_entry(i, ctypes.byref(cfg)))
        out.append(cfg)
    return out


def config_supported(config, layout_c="row_major", layout_a="row_major", layout_b="row_major"):
    if isinstance(config, dict):
        config = Config.from_dict(config)
    return bool(lib().rocm_sgemm_config_supported(ctypes.byref(config), _layout(layout_c),
                                                  _layout(layout_a), _layout(layout_b)))


def map_workgroup(workgroup, grid_m, grid_n, group_m):
    tm, tn = ctypes.c_int(), ctypes.c_int()
    _check(lib().rocm_sgemm_map_workgroup(workgroup, grid_m, grid_n, group_m, ctypes.byref(tm),
                                          ctypes.byref(tn)))
    return tm.value, tn.value


def release_workspaces():
    """Frees the per-stream workspace buffers the library holds (waits for the device)."""
    lib().rocm_sgemm_release_workspaces()


def version():
    return lib().rocm_sgemm_version().decode()
