"""The two ops of the reference's extension, on PyTorch-ROCm tensors.

Mirror of extension.cpp:26-55: ``matmul(x, q, s, c, o, m, n, k)`` and
``dequant(q, absmax, codebook, o, m, k)``, both returning None and writing into the
caller's ``o`` on the current stream of the tensors' device.  Unlike the reference,
which performs no checks at all (extension.cpp:26-38), wrong dtypes, shapes, devices
or non-contiguous tensors raise instead of invoking undefined behaviour, and shapes
outside the tuned table run on a derived config instead of silently doing nothing
(kernel.cu:3018-3156).

PyTorch is only the carrier of device memory and streams here; the work happens in
libtuna_amd.so behind the C ABI of include/tuna_amd.h.
"""
import ctypes

import torch

from . import _lib
from ._lib import GemmConfig, TunaError  # noqa: F401  (re-exported)


def _require(t: torch.Tensor, name: str, dtype: torch.dtype, numel: int) -> None:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if t.device.type != "cuda":
        raise ValueError(f"{name} must live on a HIP device (got {t.device})")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype} (got {t.dtype})")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if t.numel() != numel:
        raise ValueError(f"{name} has {t.numel()} elements, expected {numel}")


def _stream(dev: torch.device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def matmul(x, q, s, c, o, m: int, n: int, k: int, config: GemmConfig = None,
           decode_mode: int = _lib.DECODE_GEMM) -> None:
    """o[n, m] = x[n, k] @ decode(q, c, s)[m, k]^T  (extension.cpp:26-38).

    x fp16 [n, k]; q uint8 [m/8, k/8, 32]; s fp32 [m] (absmax per weight row);
    c fp32 [16] (codebook); o fp16 [n, m], overwritten.
    """
    m, n, k = int(m), int(n), int(k)
    if m <= 0 or n <= 0 or k <= 0 or m % 8 or k % 8:
        raise ValueError(f"m and k must be positive multiples of 8 and n positive (m={m}, n={n}, k={k})")
    _require(x, "x", torch.float16, n * k)
    _require(q, "q", torch.uint8, m * k // 2)
    _require(s, "s", torch.float32, m)
    _require(c, "c", torch.float32, 16)
    _require(o, "o", torch.float16, n * m)
    for name, t in (("q", q), ("s", s), ("c", c), ("o", o)):
        if t.device != x.device:
            raise ValueError(f"{name} is on {t.device}, x on {x.device}")
    L = _lib.lib()
    with torch.cuda.device(x.device):
        if config is None and decode_mode == _lib.DECODE_GEMM:
            rc = L.tuna_matmul(q.data_ptr(), x.data_ptr(), c.data_ptr(), s.data_ptr(), o.data_ptr(), m, n, k,
                               _stream(x.device))
        else:
            rc = L.tuna_matmul_ex(q.data_ptr(), x.data_ptr(), c.data_ptr(), s.data_ptr(), o.data_ptr(), m, n, k,
                                  ctypes.byref(config) if config is not None else None, int(decode_mode),
                                  _stream(x.device))
    _lib.check(rc)


def matmul_static(x, q, s, c, o, m: int, n: int, k: int, config: GemmConfig = None,
                  decode_mode: int = _lib.DECODE_GEMM) -> None:
    """matmul through tuna_matmul_static: same result, but the split-K partial sums live in a fixed
    array of the loaded library instead of an allocated workspace (for callers that cannot
    allocate).  Raises TunaError (ERR_WORKSPACE) if the launch needs more than that array holds."""
    m, n, k = int(m), int(n), int(k)
    _require(x, "x", torch.float16, n * k)
    _require(q, "q", torch.uint8, m * k // 2)
    _require(s, "s", torch.float32, m)
    _require(c, "c", torch.float32, 16)
    _require(o, "o", torch.float16, n * m)
    with torch.cuda.device(x.device):
        rc = _lib.lib().tuna_matmul_static(q.data_ptr(), x.data_ptr(), c.data_ptr(), s.data_ptr(), o.data_ptr(), m, n, k,
                                           ctypes.byref(config) if config is not None else None, int(decode_mode),
                                           _stream(x.device))
    _lib.check(rc)


def matmul_fused(x, q, s, c, o, m: int, n: int, k: int, epilogue: int, residual=None, config: GemmConfig = None,
                 decode_mode: int = _lib.DECODE_GEMM) -> None:
    """matmul with a fused epilogue (tuna_matmul_fused).

    EPILOGUE_RESIDUAL: o[n, m] = fp16(x @ W^T + residual), residual fp16 [n, m] (may be o).
    EPILOGUE_SILU_MUL: weight rows interleaved (2i: gate_i, 2i+1: up_i); o[n, m/2] =
    fp16(silu(gate) * up)."""
    m, n, k = int(m), int(n), int(k)
    _require(x, "x", torch.float16, n * k)
    _require(q, "q", torch.uint8, m * k // 2)
    _require(s, "s", torch.float32, m)
    _require(c, "c", torch.float32, 16)
    _require(o, "o", torch.float16, n * (m // 2 if epilogue == _lib.EPILOGUE_SILU_MUL else m))
    rp = None
    if epilogue == _lib.EPILOGUE_RESIDUAL:
        if residual is None:
            raise ValueError("EPILOGUE_RESIDUAL needs a residual tensor")
        _require(residual, "residual", torch.float16, n * m)
        rp = residual.data_ptr()
    with torch.cuda.device(x.device):
        rc = _lib.lib().tuna_matmul_fused(q.data_ptr(), x.data_ptr(), c.data_ptr(), s.data_ptr(), o.data_ptr(), m, n, k,
                                          ctypes.byref(config) if config is not None else None, int(decode_mode),
                                          int(epilogue), rp, _stream(x.device))
    _lib.check(rc)


def problem_array(problems, block_size: int = None, epilogues=None):
    """ctypes array of GemmProblem for matmul_multi / time_matmul_multi from (x, q, s, c, o, m, n, k) tuples
    (block_size: s is [m, k / block_size]; epilogues: per problem, EPILOGUE_SILU_MUL makes o [n, m/2])."""
    arr = (_lib.GemmProblem * len(problems))()
    for i, (x, q, s, c, o, m, n, k) in enumerate(problems):
        m, n, k = int(m), int(n), int(k)
        _require(x, "x", torch.float16, n * k)
        _require(q, "q", torch.uint8, m * k // 2)
        _require(s, "s", torch.float32, m if block_size is None else m * (k // int(block_size)))
        _require(c, "c", torch.float32, 16)
        _require(o, "o", torch.float16, n * m // 2 if epilogues is not None and epilogues[i] == _lib.EPILOGUE_SILU_MUL else n * m)
        arr[i] = _lib.GemmProblem(q.data_ptr(), x.data_ptr(), c.data_ptr(), s.data_ptr(), o.data_ptr(), m, n, k)
    return arr


def matmul_multi(problems, block_size: int = None, epilogues=None, residuals=None) -> None:
    """Several independent GEMMs in one call (tuna_matmul_multi): `problems` is a list of
    (x, q, s, c, o, m, n, k) tuples, each with the meaning of matmul's arguments.  With block_size every s is
    [m, k / block_size], one scale per block of a row (tuna_matmul_multi_blockwise).  With epilogues (one
    EPILOGUE_* per problem) and residuals (a tensor or None per problem) the stores are fused as in matmul_fused
    (tuna_matmul_multi_fused)."""
    if not problems:
        return
    if block_size is not None and (int(block_size) <= 0 or any(int(p[7]) % int(block_size) for p in problems)):
        raise ValueError(f"block_size={block_size} must divide every k")
    if epilogues is not None and (block_size is not None or len(epilogues) != len(problems)):
        raise ValueError("epilogues: one per problem, per-row scales only")
    arr = problem_array(problems, block_size, epilogues)
    dev = problems[0][0].device
    with torch.cuda.device(dev):
        if epilogues is not None:
            eps = (ctypes.c_int32 * len(problems))(*[int(e) for e in epilogues])
            res = (ctypes.c_void_p * len(problems))()
            for i, (ep, (x, q, s, c, o, m, n, k)) in enumerate(zip(epilogues, problems)):
                if ep == _lib.EPILOGUE_RESIDUAL:
                    if residuals is None or residuals[i] is None:
                        raise ValueError(f"problem {i}: EPILOGUE_RESIDUAL needs a residual tensor")
                    _require(residuals[i], "residual", torch.float16, int(n) * int(m))
                    res[i] = residuals[i].data_ptr()
            rc = _lib.lib().tuna_matmul_multi_fused(arr, eps, ctypes.cast(res, ctypes.POINTER(ctypes.c_void_p)), len(problems),
                                                    _stream(dev))
        elif block_size is None:
            rc = _lib.lib().tuna_matmul_multi(arr, len(problems), _stream(dev))
        else:
            rc = _lib.lib().tuna_matmul_multi_blockwise(arr, len(problems), int(block_size), _stream(dev))
    _lib.check(rc)


def matmul_grouped(x, q, s, c, o, m_group: int, n_groups: int, k: int, token_offsets, config: GemmConfig = None,
                   decode_mode: int = _lib.DECODE_GEMM) -> None:
    """Grouped GEMM (mixture of experts): o[t, :] = x[t, :] @ decode(W_e)^T for the tokens t of
    group e, token_offsets[e] <= t < token_offsets[e+1] (tuna_matmul_grouped).

    x fp16 [n_total, k], rows sorted by group; q uint8 [n_groups*m_group/8, k/8, 32] and s fp32
    [n_groups*m_group]: the groups' weights stacked along m; o fp16 [n_total, m_group];
    token_offsets: n_groups+1 non-decreasing host ints.  Groups without tokens cost nothing; without a config a
    group of more than 64 tokens runs as a dense GEMM of its own (same bits as `matmul` on its slices).
    """
    m_group, n_groups, k = int(m_group), int(n_groups), int(k)
    offs = [int(v) for v in token_offsets]
    if len(offs) != n_groups + 1:
        raise ValueError(f"token_offsets needs {n_groups + 1} entries, got {len(offs)}")
    n_total = offs[-1]
    m = m_group * n_groups
    _require(x, "x", torch.float16, n_total * k)
    _require(q, "q", torch.uint8, m * k // 2)
    _require(s, "s", torch.float32, m)
    _require(c, "c", torch.float32, 16)
    _require(o, "o", torch.float16, n_total * m_group)
    for name, t in (("q", q), ("s", s), ("c", c), ("o", o)):
        if t.device != x.device:
            raise ValueError(f"{name} is on {t.device}, x on {x.device}")
    arr = (ctypes.c_int * (n_groups + 1))(*offs)
    with torch.cuda.device(x.device):
        rc = _lib.lib().tuna_matmul_grouped(q.data_ptr(), x.data_ptr(), c.data_ptr(), s.data_ptr(), o.data_ptr(), m_group,
                                            n_groups, k, arr, ctypes.byref(config) if config is not None else None,
                                            int(decode_mode), _stream(x.device))
    _lib.check(rc)


def dequant(q, absmax, codebook, o, m: int, k: int, decode_mode: int = _lib.DECODE_DEQUANT, block_size: int = None) -> None:
    """o[m, k] = decode(q, codebook, absmax) as fp16  (extension.cpp:40-49).  block_size: weights per
    scale along a row, absmax [m, k/block_size] (the quantizer's layout for block_size < k,
    test.py:15-17); None = one scale per row."""
    m, k = int(m), int(k)
    if m <= 0 or k <= 0 or m % 8 or k % 8:
        raise ValueError(f"m and k must be positive multiples of 8 (m={m}, k={k})")
    bs = k if block_size is None else int(block_size)
    if bs <= 0 or k % bs:
        raise ValueError(f"block_size={bs} must divide k={k}")
    _require(q, "q", torch.uint8, m * k // 2)
    _require(absmax, "absmax", torch.float32, m * (k // bs))
    _require(codebook, "codebook", torch.float32, 16)
    _require(o, "o", torch.float16, m * k)
    for name, t in (("absmax", absmax), ("codebook", codebook), ("o", o)):
        if t.device != q.device:
            raise ValueError(f"{name} is on {t.device}, q on {q.device}")
    L = _lib.lib()
    with torch.cuda.device(q.device):
        if bs != k:
            rc = L.tuna_dequant_blockwise(q.data_ptr(), absmax.data_ptr(), codebook.data_ptr(), o.data_ptr(), m, k, bs,
                                          int(decode_mode), _stream(q.device))
        elif decode_mode == _lib.DECODE_DEQUANT:
            rc = L.tuna_dequant(q.data_ptr(), absmax.data_ptr(), codebook.data_ptr(), o.data_ptr(), m, k,
                                _stream(q.device))
        else:
            rc = L.tuna_dequant_ex(q.data_ptr(), absmax.data_ptr(), codebook.data_ptr(), o.data_ptr(), m, k,
                                   int(decode_mode), _stream(q.device))
    _lib.check(rc)


def matmul_blockwise(x, q, s, c, o, m: int, n: int, k: int, block_size: int, config: GemmConfig = None) -> None:
    """matmul with one scale per block_size consecutive weights of a row: s fp32 [m, k/block_size]
    (tuna_matmul_blockwise_ex; config None = the library's choice: its blockwise table, else a derived config)."""
    m, n, k, bs = int(m), int(n), int(k), int(block_size)
    if bs <= 0 or k % bs:
        raise ValueError(f"block_size={bs} must divide k={k}")
    _require(x, "x", torch.float16, n * k)
    _require(q, "q", torch.uint8, m * k // 2)
    _require(s, "s", torch.float32, m * (k // bs))
    _require(c, "c", torch.float32, 16)
    _require(o, "o", torch.float16, n * m)
    with torch.cuda.device(x.device):
        rc = _lib.lib().tuna_matmul_blockwise_ex(q.data_ptr(), x.data_ptr(), c.data_ptr(), s.data_ptr(), o.data_ptr(), m, n, k, bs,
                                                 ctypes.byref(config) if config is not None else None, _stream(x.device))
    _lib.check(rc)


def select_config_blockwise(m: int, n: int, k: int, block_size: int):
    """(config, from_table) tuna_matmul_blockwise runs for the shape (tuna_select_config_blockwise).  Host only."""
    cfg = GemmConfig()
    hit = ctypes.c_int(0)
    _lib.check(_lib.lib().tuna_select_config_blockwise(int(m), int(n), int(k), int(block_size), ctypes.byref(cfg), ctypes.byref(hit)))
    return cfg, bool(hit.value)


def validate_config_blockwise(m: int, n: int, k: int, block_size: int, config: GemmConfig) -> None:
    """Raises TunaError unless `config` can run the blockwise GEMM (tuna_validate_config_blockwise).  Host only."""
    _lib.check(_lib.lib().tuna_validate_config_blockwise(int(m), int(n), int(k), int(block_size), ctypes.byref(config)))


BLOCKWISE_FAMILIES = ("narrow", "batched", "many-token", "streaming")


def blockwise_family(config: GemmConfig) -> str:
    """The kernel a blockwise config names (the rule of tuna_matmul_blockwise_ex)."""
    from .make_configs import blockwise_family as fam

    return fam(config.to_dict())


def quantize(w, codebook=None, block_size: int = None):
    """fp16 weights [m, k] on a HIP device -> (q uint8 [m/8, k/8, 32], absmax fp32 [m] - or
    [m, k/block_size] - and codebook fp32 [16]): the reference harness's quantizer + packer
    (test.py:7-68) as one kernel (tuna_quantize / tuna_quantize_blockwise).  `codebook` defaults to
    the NF4 constants, block_size to k (one scale per row, what the GEMM of the reference runs)."""
    from .quantize import nf4_codebook

    if w.dim() != 2:
        raise ValueError("w must be [m, k]")
    m, k = w.shape
    if m % 8 or k % 8:
        raise ValueError("m and k must be multiples of 8")
    bs = k if block_size is None else int(block_size)
    if bs <= 0 or k % bs:
        raise ValueError(f"block_size={bs} must divide k={k}")
    _require(w, "w", torch.float16, m * k)
    code = nf4_codebook(w.device) if codebook is None else codebook
    _require(code, "codebook", torch.float32, 16)
    q = torch.empty((m // 8, k // 8, 32), dtype=torch.uint8, device=w.device)
    absmax = torch.empty((m,) if block_size is None else (m, k // bs), dtype=torch.float32, device=w.device)
    with torch.cuda.device(w.device):
        rc = _lib.lib().tuna_quantize_blockwise(w.data_ptr(), code.data_ptr(), q.data_ptr(), absmax.data_ptr(), int(m), int(k),
                                                bs, _stream(w.device))
    _lib.check(rc)
    return q, absmax, code


def select_config(m: int, n: int, k: int, decode_mode: int = _lib.DECODE_GEMM):
    """(GemmConfig, from_table) the library would use for shape (m, n, k).  Host only."""
    cfg = GemmConfig()
    hit = ctypes.c_int(0)
    _lib.check(_lib.lib().tuna_select_config_ex(int(m), int(n), int(k), int(decode_mode), ctypes.byref(cfg),
                                                ctypes.byref(hit)))
    return cfg, bool(hit.value)


def derive_config(m: int, n: int, k: int):
    """GemmConfig the library derives for shape (m, n, k) when the table has no entry (also for shapes that have
    one: the tuner's seed, and what an entry has to beat).  Host only."""
    cfg = GemmConfig()
    _lib.check(_lib.lib().tuna_derive_config(int(m), int(n), int(k), ctypes.byref(cfg)))
    return cfg


def select_config_grouped(m_group: int, n_active: int, max_tokens: int, k: int, decode_mode: int = _lib.DECODE_GEMM):
    """GemmConfig matmul_grouped(config=None) runs for n_active groups with tokens.  Host only."""
    cfg = GemmConfig()
    _lib.check(_lib.lib().tuna_select_config_grouped(int(m_group), int(n_active), int(max_tokens), int(k),
                                                     int(decode_mode), ctypes.byref(cfg)))
    return cfg


def validate_config(m: int, n: int, k: int, cfg: GemmConfig, decode_mode: int = _lib.DECODE_GEMM) -> None:
    """Raises TunaError unless `cfg` can run shape (m, n, k).  Host only."""
    _lib.check(_lib.lib().tuna_validate_config_ex(int(m), int(n), int(k), ctypes.byref(cfg), int(decode_mode)))


def config_footprint(m: int, n: int, k: int, cfg: GemmConfig):
    """(dynamic LDS bytes, split-K workspace bytes) of a launch.  Host only."""
    lds, ws = ctypes.c_size_t(0), ctypes.c_size_t(0)
    _lib.check(_lib.lib().tuna_config_footprint(int(m), int(n), int(k), ctypes.byref(cfg), ctypes.byref(lds),
                                                ctypes.byref(ws)))
    return lds.value, ws.value


def config_segments(m: int, n: int, k: int, cfg: GemmConfig, n_workgroups: int = 0, workgroup: int = 0):
    """Segments (row tile, first k-step, k-steps, partial-sum slot or -1) that workgroup
    `workgroup` of `n_workgroups` walks in a launch of `cfg`.  Host only."""
    L = _lib.lib()
    cnt = ctypes.c_int(0)
    _lib.check(L.tuna_config_segments(int(m), int(n), int(k), ctypes.byref(cfg), int(n_workgroups), int(workgroup),
                                      None, 0, ctypes.byref(cnt)))
    buf = (ctypes.c_int * (4 * max(cnt.value, 1)))()
    _lib.check(L.tuna_config_segments(int(m), int(n), int(k), ctypes.byref(cfg), int(n_workgroups), int(workgroup),
                                      buf, cnt.value, ctypes.byref(cnt)))
    return [tuple(buf[4 * i:4 * i + 4]) for i in range(cnt.value)]


def config_contributors(m: int, n: int, k: int, cfg: GemmConfig, n_workgroups: int, row_tile: int):
    """(first workgroup, count, slot of the first) of the partial sums of a row tile under a
    balanced split; (-1, split_k, 0) under a fixed split.  Host only."""
    a, b, c = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    _lib.check(_lib.lib().tuna_config_contributors(int(m), int(n), int(k), ctypes.byref(cfg), int(n_workgroups),
                                                   int(row_tile), ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)))
    return a.value, b.value, c.value


def config_table():
    """The built-in tuned table as a list of (m, n_lo, n_hi, k, GemmConfig)."""
    L = _lib.lib()
    out = []
    for i in range(L.tuna_config_table_size()):
        m, lo, hi, k = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        cfg = GemmConfig()
        _lib.check(L.tuna_config_table_entry(i, ctypes.byref(m), ctypes.byref(lo), ctypes.byref(hi), ctypes.byref(k),
                                             ctypes.byref(cfg)))
        out.append((m.value, lo.value, hi.value, k.value, cfg))
    return out


def config_table_next_from():
    """Per entry of config_table(): the token count from which select_config hands out the next bucket's entry
    (n_hi + 1: never)."""
    L = _lib.lib()
    return [L.tuna_config_table_next_from(i) for i in range(L.tuna_config_table_size())]


def config_table_derived_ranges():
    """Per entry of config_table(): (from, to) - select_config hands out the derived config for token counts in
    [from, to) of the entry's range ((0, 0): for none)."""
    L = _lib.lib()
    out = []
    for i in range(L.tuna_config_table_size()):
        a, b = ctypes.c_int(), ctypes.c_int()
        _lib.check(L.tuna_config_table_derived_range(i, ctypes.byref(a), ctypes.byref(b)))
        out.append((a.value, b.value))
    return out


def _ptr_array(tensors):
    arr = (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])
    return ctypes.cast(arr, ctypes.POINTER(ctypes.c_void_p)), arr


def time_matmul(q_list, absmax_list, x, c, o, m, n, k, config=None, decode_mode=_lib.DECODE_GEMM, warmup=10,
                iters=100, use_graph=False) -> float:
    """Milliseconds for `iters` GEMMs rotating over the weight sets, measured with HIP
    events on the current stream (tuna_time_matmul).  Synchronises."""
    assert len(q_list) == len(absmax_list) and len(q_list) > 0
    qp, _qk = _ptr_array(q_list)
    ap, _ak = _ptr_array(absmax_list)
    ms = ctypes.c_float(0)
    L = _lib.bench_lib()
    with torch.cuda.device(x.device):
        rc = L.tuna_time_matmul(qp, ap, len(q_list), x.data_ptr(), c.data_ptr(), o.data_ptr(), int(m), int(n), int(k),
                                ctypes.byref(config) if config is not None else None, int(decode_mode), int(warmup),
                                int(iters), int(bool(use_graph)), _stream(x.device), ctypes.byref(ms))
    _lib.check(rc, _lib.bench_lib())
    return ms.value



def time_matmul_streams(q_list, absmax_list, x, c, outs, m, n, k, config=None, decode_mode=_lib.DECODE_GEMM, warmup=10,
                        iters=100, use_graph=False) -> float:
    """Milliseconds for `iters` GEMMs dealt round-robin to len(outs) streams (tuna_time_matmul_streams): launch i
    writes outs[i % len(outs)] on stream i % len(outs).  Synchronises."""
    assert len(q_list) == len(absmax_list) and len(q_list) > 0 and len(outs) > 0
    qp, _qk = _ptr_array(q_list)
    ap, _ak = _ptr_array(absmax_list)
    op, _ok = _ptr_array(outs)
    ms = ctypes.c_float(0)
    L = _lib.bench_lib()
    with torch.cuda.device(x.device):
        rc = L.tuna_time_matmul_streams(qp, ap, len(q_list), x.data_ptr(), c.data_ptr(), op, len(outs), int(m), int(n), int(k),
                                        ctypes.byref(config) if config is not None else None, int(decode_mode),
                                        int(bool(use_graph)), int(warmup), int(iters), ctypes.byref(ms))
    _lib.check(rc, L)
    return ms.value


def time_empty_launches(device, blocks=192, threads=512, n_streams=1, use_graph=False, warmup=100, iters=1000) -> float:
    """Milliseconds for `iters` launches of a kernel that does nothing (tuna_time_empty_launches)."""
    sink = torch.zeros(4, dtype=torch.int32, device=device)
    ms = ctypes.c_float(0)
    L = _lib.bench_lib()
    with torch.cuda.device(device):
        rc = L.tuna_time_empty_launches(sink.data_ptr(), int(blocks), int(threads), int(n_streams), int(bool(use_graph)),
                                        int(warmup), int(iters), ctypes.byref(ms))
    _lib.check(rc, L)
    return ms.value


def measure_handover(device, same_xcd: bool, store_sc1: bool, load_sc1: bool, reuse: bool, pairs=16, iters=200) -> dict:
    """The hand-over yardstick (tuna_measure_handover): latencies of one producer -> consumer step in nanoseconds."""
    out = (ctypes.c_double * 6)()
    L = _lib.bench_lib()
    with torch.cuda.device(device):
        rc = L.tuna_measure_handover(int(same_xcd), int(store_sc1), int(load_sc1), int(reuse), int(pairs), int(iters),
                                     _stream(device), out)
    _lib.check(rc, L)
    return {"store_ack_ns": round(out[0], 1), "atomic_round_trip_ns": round(out[1], 1), "load_ns": round(out[2], 1),
            "mismatches": int(out[3]), "timeouts": int(out[4]), "pairs_on_one_xcd": int(out[5]), "pairs": int(pairs)}


def time_matmul_blockwise(q_list, absmax_list, x, c, o, m, n, k, block_size, config=None, warmup=10, iters=100,
                          use_graph=False) -> float:
    """Milliseconds for `iters` blockwise GEMMs rotating over the weight sets (tuna_time_matmul_blockwise)."""
    assert len(q_list) == len(absmax_list) and len(q_list) > 0
    qp, _qk = _ptr_array(q_list)
    ap, _ak = _ptr_array(absmax_list)
    ms = ctypes.c_float(0)
    L = _lib.bench_lib()
    with torch.cuda.device(x.device):
        rc = L.tuna_time_matmul_blockwise(qp, ap, len(q_list), x.data_ptr(), c.data_ptr(), o.data_ptr(), int(m), int(n), int(k),
                                          int(block_size), ctypes.byref(config) if config is not None else None, int(warmup),
                                          int(iters), int(bool(use_graph)), _stream(x.device), ctypes.byref(ms))
    _lib.check(rc, L)
    return ms.value


def time_matmul_grouped(q_list, absmax_list, x, c, o, m_group, n_groups, k, token_offsets, config=None,
                        decode_mode=_lib.DECODE_GEMM, warmup=10, iters=100, use_graph=False) -> float:
    """Milliseconds for `iters` grouped GEMMs rotating over the weight sets
    (tuna_time_matmul_grouped).  Synchronises."""
    assert len(q_list) == len(absmax_list) and len(q_list) > 0
    qp, _qk = _ptr_array(q_list)
    ap, _ak = _ptr_array(absmax_list)
    arr = (ctypes.c_int * (int(n_groups) + 1))(*[int(v) for v in token_offsets])
    ms = ctypes.c_float(0)
    with torch.cuda.device(x.device):
        rc = _lib.bench_lib().tuna_time_matmul_grouped(qp, ap, len(q_list), x.data_ptr(), c.data_ptr(), o.data_ptr(), int(m_group),
                                                 int(n_groups), int(k), arr,
                                                 ctypes.byref(config) if config is not None else None, int(decode_mode),
                                                 int(warmup), int(iters), int(bool(use_graph)), _stream(x.device),
                                                 ctypes.byref(ms))
    _lib.check(rc, _lib.bench_lib())
    return ms.value

def time_matmul_multi(batches, warmup=10, iters=100, use_graph=False) -> float:
    """Milliseconds for `iters` matmul_multi calls rotating over `batches` (equally long lists of
    (x, q, s, c, o, m, n, k) problems), HIP events on the current stream (tuna_time_matmul_multi)."""
    count = len(batches[0])
    assert count > 0 and all(len(b) == count for b in batches)
    arr = problem_array([p for b in batches for p in b])
    dev = batches[0][0][0].device
    ms = ctypes.c_float(0)
    with torch.cuda.device(dev):
        rc = _lib.bench_lib().tuna_time_matmul_multi(arr, len(batches), count, int(warmup), int(iters), int(bool(use_graph)),
                                               _stream(dev), ctypes.byref(ms))
    _lib.check(rc, _lib.bench_lib())
    return ms.value


def time_dequant(q_list, absmax_list, c, o, m, k, warmup=5, iters=20) -> float:
    qp, _qk = _ptr_array(q_list)
    ap, _ak = _ptr_array(absmax_list)
    ms = ctypes.c_float(0)
    L = _lib.bench_lib()
    with torch.cuda.device(o.device):
        rc = L.tuna_time_dequant(qp, ap, len(q_list), c.data_ptr(), o.data_ptr(), int(m), int(k), int(warmup),
                                 int(iters), _stream(o.device), ctypes.byref(ms))
    _lib.check(rc, _lib.bench_lib())
    return ms.value


def time_copy(src, dst, warmup=5, iters=20) -> float:
    nbytes = src.numel() * src.element_size()
    assert dst.numel() * dst.element_size() >= nbytes
    ms = ctypes.c_float(0)
    L = _lib.bench_lib()
    with torch.cuda.device(src.device):
        rc = L.tuna_time_copy(src.data_ptr(), dst.data_ptr(), nbytes, int(warmup), int(iters), _stream(src.device),
                              ctypes.byref(ms))
    _lib.check(rc, _lib.bench_lib())
    return ms.value


def time_read(src, blocks=0, variant=0, warmup=5, iters=20) -> float:
    """Milliseconds for `iters` read-only passes over `src` (tuna_time_read)."""
    nbytes = src.numel() * src.element_size()
    sink = torch.zeros(4, dtype=torch.int32, device=src.device)
    ms = ctypes.c_float(0)
    L = _lib.bench_lib()
    with torch.cuda.device(src.device):
        rc = L.tuna_time_read(src.data_ptr(), sink.data_ptr(), nbytes, int(blocks), int(variant), int(warmup), int(iters),
                              _stream(src.device), ctypes.byref(ms))
    _lib.check(rc, _lib.bench_lib())
    return ms.value


def time_unit_rate(unit: int, device, warmup=2, iters=5):
    """(milliseconds for `iters` launches, flops or LDS bytes per launch) of one of the matrix-core / LDS
    yardstick kernels (tuna_time_unit_rate)."""
    sink = torch.zeros(4, dtype=torch.int32, device=device)
    ms = ctypes.c_float(0)
    work = ctypes.c_double(0)
    with torch.cuda.device(device):
        rc = _lib.bench_lib().tuna_time_unit_rate(int(unit), sink.data_ptr(), int(warmup), int(iters), _stream(device),
                                            ctypes.byref(ms), ctypes.byref(work))
    _lib.check(rc, _lib.bench_lib())
    return ms.value, work.value


def describe_launch(m: int, n: int, k: int, config: GemmConfig = None, decode_mode: int = _lib.DECODE_GEMM) -> str:
    """Name and template arguments of the kernel a GEMM launch would start (tuna_describe_launch)."""
    buf = ctypes.create_string_buffer(256)
    _lib.check(_lib.lib().tuna_describe_launch(int(m), int(n), int(k), ctypes.byref(config) if config is not None else None,
                                               int(decode_mode), buf, 256))
    return buf.value.decode()


def set_lean_kernels(enabled: bool) -> bool:
    """Diagnostic switch (tuna_set_lean_kernels) of the diagnostic build: whether qualifying small launches use the
    stripped-down kernel.  Results are bit-identical either way.  Returns the previous setting.  It applies to ops
    called while _lib.diagnostic_build() is active; the product library has no such switch."""
    return bool(_lib.bench_lib().tuna_set_lean_kernels(int(bool(enabled))))


def set_weight_path(through_lds: bool) -> bool:
    """Diagnostic switch (tuna_set_weight_path): unsplit 16-wave launches of up to 16 tokens stage the
    packed weights through LDS instead of registers.  Bit-identical results.  Returns the previous setting."""
    return bool(_lib.bench_lib().tuna_set_weight_path(int(bool(through_lds))))


def lean_launches() -> int:
    """Diagnostic (tuna_lean_launches): GEMM launches of this process that took the stripped-down kernel."""
    return int(_lib.bench_lib().tuna_lean_launches())
