"""tuna_amd: MI355X (gfx950) FP16-activation x 4-bit-codebook-weight GEMM.

Public surface (mirrors the reference's `tuna` extension, extension.cpp:51-55):
    matmul(x, q, s, c, o, m, n, k)         dequant(q, absmax, codebook, o, m, k)
plus the host-side helpers around it (config table, quantizer/packer, synthetic
inputs, tuner).  torch is imported lazily so that the config tooling works without it.
"""
__version__ = "0.1.0"


def __getattr__(name):
    if name in ("matmul", "dequant", "select_config", "validate_config", "config_footprint", "config_table",
                "time_matmul", "time_dequant", "time_copy", "GemmConfig", "TunaError"):
        from . import ops
        return getattr(ops, name)
    raise AttributeError(name)
