"""ctypes binding of tuna_amd/libtuna_amd.so (the C ABI declared in include/tuna_amd.h) and of its
diagnostic build tuna_amd/libtuna_amd_bench.so (include/tuna_amd_bench.h on top of the same ABI).

Both are built in-tree by ``make -C tuna_amd/csrc`` (see build()) from the same object files; the
diagnostic build adds timing loops, yardstick kernels and process-wide switches between kernels that
compute identical results.  ``lib()`` is the library the ops call: the product library unless
``diagnostic_build()`` is active (bench.py, the tuner, A/B tests).  There is no fallback
implementation: if a shared object is missing or does not load, every op raises.
"""
import contextlib
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtuna_amd.so")
BENCH_LIB_PATH = os.path.join(_HERE, "libtuna_amd_bench.so")
CSRC = os.path.join(_HERE, "csrc")

OK = 0
ERR_INVALID_ARG = 1
ERR_UNSUPPORTED = 2
ERR_HIP = 3
ERR_NO_DEVICE = 4
ERR_WORKSPACE = 5

DECODE_GEMM = 1
DECODE_DEQUANT = 2
EPILOGUE_NONE, EPILOGUE_RESIDUAL, EPILOGUE_SILU_MUL = 0, 1, 2


class GemmConfig(ctypes.Structure):
    """Mirror of ``tuna_gemm_config`` (include/tuna_amd.h)."""

    _fields_ = [
        ("rows_per_wave", ctypes.c_int32),
        ("waves_m", ctypes.c_int32),
        ("waves_k", ctypes.c_int32),
        ("split_k", ctypes.c_int32),
        ("prefetch", ctypes.c_int32),
        ("x_chunk", ctypes.c_int32),
        ("token_tiles", ctypes.c_int32),
        ("xcd_swizzle", ctypes.c_int32),
        ("k_stagger", ctypes.c_int32),
        ("lds_tile_rows", ctypes.c_int32),
    ]

    FIELDS = tuple(f for f, _ in _fields_)

    def to_dict(self):
        return {f: int(getattr(self, f)) for f in self.FIELDS}

    @classmethod
    def from_dict(cls, d):
        return cls(**{f: int(d.get(f, 0) if f in ("k_stagger", "lds_tile_rows") else d[f]) for f in cls.FIELDS})


class GemmProblem(ctypes.Structure):
    """Mirror of ``tuna_gemm_problem`` (include/tuna_amd.h)."""

    _fields_ = [("q", ctypes.c_void_p), ("x", ctypes.c_void_p), ("code", ctypes.c_void_p), ("absmax", ctypes.c_void_p),
                ("out", ctypes.c_void_p), ("m", ctypes.c_int32), ("n", ctypes.c_int32), ("k", ctypes.c_int32)]


# name -> (restype, argtypes); also the list of symbols the header declares
_vp, _i, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
_cfgp = ctypes.POINTER(GemmConfig)
_ip = ctypes.POINTER(ctypes.c_int)
_fp = ctypes.POINTER(ctypes.c_float)
_vpp = ctypes.POINTER(ctypes.c_void_p)
# the product ABI (include/tuna_amd.h): every symbol libtuna_amd.so exports, and nothing else
SIGNATURES = {
    "tuna_version": (_i, []),
    "tuna_status_string": (ctypes.c_char_p, [_i]),
    "tuna_last_error": (ctypes.c_char_p, []),
    "tuna_matmul": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "tuna_matmul_ex": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _cfgp, _i, _vp]),
    "tuna_init": (_i, []),
    "tuna_matmul_static": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _cfgp, _i, _vp]),
    "tuna_matmul_fused": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _cfgp, _i, _i, _vp, _vp]),
    "tuna_matmul_multi": (_i, [ctypes.POINTER(GemmProblem), _i, _vp]),
    "tuna_matmul_multi_fused": (_i, [ctypes.POINTER(GemmProblem), ctypes.POINTER(ctypes.c_int32), _vpp, _i, _vp]),
    "tuna_matmul_multi_blockwise": (_i, [ctypes.POINTER(GemmProblem), _i, _i, _vp]),
    "tuna_matmul_grouped": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _ip, _cfgp, _i, _vp]),
    "tuna_dequant": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp]),
    "tuna_quantize": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp]),
    "tuna_quantize_blockwise": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "tuna_dequant_blockwise": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "tuna_matmul_blockwise": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "tuna_matmul_blockwise_ex": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _cfgp, _vp]),
    "tuna_select_config_blockwise": (_i, [_i, _i, _i, _i, _cfgp, _ip]),
    "tuna_validate_config_blockwise": (_i, [_i, _i, _i, _i, _cfgp]),
    "tuna_blockwise_table_size": (_i, []),
    "tuna_blockwise_table_entry": (_i, [_i, _ip, _ip, _ip, _ip, _ip, _cfgp]),
    "tuna_dequant_ex": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "tuna_select_config": (_i, [_i, _i, _i, _cfgp, _ip]),
    "tuna_select_config_ex": (_i, [_i, _i, _i, _i, _cfgp, _ip]),
    "tuna_derive_config": (_i, [_i, _i, _i, _cfgp]),
    "tuna_select_config_grouped": (_i, [_i, _i, _i, _i, _i, _cfgp]),
    "tuna_validate_config": (_i, [_i, _i, _i, _cfgp]),
    "tuna_validate_config_ex": (_i, [_i, _i, _i, _cfgp, _i]),
    "tuna_config_footprint": (_i, [_i, _i, _i, _cfgp, ctypes.POINTER(_sz), ctypes.POINTER(_sz)]),
    "tuna_config_segments": (_i, [_i, _i, _i, _cfgp, _i, _i, _ip, _i, _ip]),
    "tuna_config_contributors": (_i, [_i, _i, _i, _cfgp, _i, _i, _ip, _ip, _ip]),
    "tuna_config_table_size": (_i, []),
    "tuna_config_table_entry": (_i, [_i, _ip, _ip, _ip, _ip, _cfgp]),
    "tuna_config_table_next_from": (_i, [_i]),
    "tuna_config_table_derived_range": (_i, [_i, _ip, _ip]),
    "tuna_describe_launch": (_i, [_i, _i, _i, _cfgp, _i, ctypes.c_char_p, _sz]),
    "tuna_release_workspaces": (_i, []),
}
# what the diagnostic build exports on top of it (include/tuna_amd_bench.h)
BENCH_SIGNATURES = {
    "tuna_set_blockwise_scales_lds": (_i, [_i]),
    "tuna_time_matmul": (_i, [_vpp, _vpp, _i, _vp, _vp, _vp, _i, _i, _i, _cfgp, _i, _i, _i, _i, _vp, _fp]),
    "tuna_time_matmul_streams": (_i, [_vpp, _vpp, _i, _vp, _vp, _vpp, _i, _i, _i, _i, _cfgp, _i, _i, _i, _i, _fp]),
    "tuna_time_empty_launches": (_i, [_vp, _i, _i, _i, _i, _i, _i, _fp]),
    "tuna_measure_handover": (_i, [_i, _i, _i, _i, _i, _i, _vp, ctypes.POINTER(ctypes.c_double)]),
    "tuna_time_matmul_multi": (_i, [ctypes.POINTER(GemmProblem), _i, _i, _i, _i, _i, _vp, _fp]),
    "tuna_time_matmul_grouped": (_i, [_vpp, _vpp, _i, _vp, _vp, _vp, _i, _i, _i, _ip, _cfgp, _i, _i, _i, _i, _vp, _fp]),
    "tuna_time_dequant": (_i, [_vpp, _vpp, _i, _vp, _vp, _i, _i, _i, _i, _vp, _fp]),
    "tuna_time_copy": (_i, [_vp, _vp, _sz, _i, _i, _vp, _fp]),
    "tuna_time_read": (_i, [_vp, _vp, _sz, _i, _i, _i, _i, _vp, _fp]),
    "tuna_time_unit_rate": (_i, [_i, _vp, _i, _i, _vp, _fp, ctypes.POINTER(ctypes.c_double)]),
    "tuna_selftest_quantizer_division": (_i, [_vp, _vp]),
    "tuna_set_multi_shape": (_i, [_i, _i]),
    "tuna_set_multi_min_batch": (_i, [_i]),
    "tuna_time_matmul_blockwise": (_i, [_vpp, _vpp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _cfgp, _i, _i, _i, _vp, _fp]),
    "tuna_blockwise_launches": (ctypes.c_ulonglong, [_i]),
    "tuna_multi_launches": (ctypes.c_ulonglong, []),
    "tuna_set_lean_kernels": (_i, [_i]),
    "tuna_set_weight_path": (_i, [_i]),
    "tuna_set_multi_weight_path": (_i, [_i]),
    "tuna_lean_launches": (ctypes.c_ulonglong, []),
}


def build(force: bool = True) -> str:
    """Compile the HIP sources for gfx950 into libtuna_amd.so (hipcc, in-tree)."""
    if force:
        subprocess.run(["make", "-C", CSRC, "clean"], check=True, capture_output=True)
    r = subprocess.run(["make", "-C", CSRC, "-j8"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building libtuna_amd.so failed:\n" + r.stdout[-4000:] + r.stderr[-4000:])
    return LIB_PATH


_libs = {}
_active = "product"


def _load(which: str):
    if which not in _libs:
        path = LIB_PATH if which == "product" else BENCH_LIB_PATH
        if not os.path.exists(path):
            raise RuntimeError(
                f"{path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C tuna_amd/csrc`; tuna_amd has no non-HIP fallback")
        # The HIP runtime must be the one PyTorch-ROCm already uses in this process (torch
        # bundles its own libamdhip64): load torch first so that this library binds to it.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = ctypes.CDLL(path)
        sigs = dict(SIGNATURES)
        if which != "product":
            sigs.update(BENCH_SIGNATURES)
        for name, (res, args) in sigs.items():
            fn = getattr(L, name)  # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _libs[which] = L
    return _libs[which]


def lib():
    """The library the ops call: libtuna_amd.so, or the diagnostic build while diagnostic_build() is active.
    Raises if it is not built (no fallback path exists)."""
    return _load(_active)


def bench_lib():
    """libtuna_amd_bench.so: the product's object files plus timing loops, yardsticks and routing switches."""
    return _load("bench")


@contextlib.contextmanager
def diagnostic_build():
    """While active, every op of this package runs in libtuna_amd_bench.so, so that its process-wide switches
    (tuna_set_*) and launch counters apply to the calls made.  Yields that library."""
    global _active
    prev, _active = _active, "bench"
    try:
        yield bench_lib()
    finally:
        _active = prev


def use_diagnostic_build() -> None:
    """For a whole process (bench.py, the tuner): route every op through libtuna_amd_bench.so from now on."""
    global _active
    _active = "bench"
    bench_lib()


class TunaError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"tuna_amd status {status}: {message}")
        self.status = status


def check(status: int, L=None) -> None:
    """Raises TunaError with the library's message unless `status` is OK (`L`: the library that returned it,
    default the active one)."""
    if status != OK:
        L = L or lib()
        msg = L.tuna_last_error().decode() or L.tuna_status_string(status).decode()
        raise TunaError(status, msg)
