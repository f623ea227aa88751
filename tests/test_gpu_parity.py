"""GPU parity tests: the HIP path (through the C ABI) against the CPU oracle.

Bit-exact for the decode (dequant op, and the GEMM's in-register decode read out through
one-hot activations); GEMM outputs within REL_TOL of the oracle's float64 contraction.
"""
import ctypes

import numpy as np
import pytest

from helpers import (O, REL_FLOOR_D2, REL_TOL, f16_bits_to_f64, make_inputs_np, rel_err, run_dequant, run_gemm, to_dev,
                     ulp_diff_f16)

pytestmark = pytest.mark.gpu


def cfg(**kw):
    from tuna_amd.ops import GemmConfig

    base = dict(rows_per_wave=64, waves_m=2, waves_k=4, split_k=1, prefetch=4, x_chunk=512, token_tiles=1,
                xcd_swizzle=0)
    base.update(kw)
    return GemmConfig.from_dict(base)


# ----------------------------------------------------------------------------- dequant

@pytest.mark.parametrize("m,k", [(8, 8), (8, 256), (64, 64), (72, 40), (136, 1032), (4096, 4096)])
@pytest.mark.parametrize("mode", [O.D2, O.D1])
def test_dequant_bit_exact(m, k, mode):
    print(f"dequant m={m} k={k} mode={mode}", flush=True)
    q, _, code, absmax = make_inputs_np(m, 1, k, seed=m * 31 + k)
    got = run_dequant(q, code, absmax, m, k, decode_mode=mode)
    want = O.dequant(q, absmax, code, m, k, mode=mode)
    assert np.array_equal(got, want)


def test_dequant_arbitrary_codebook_and_scales():
    """Random (non-NF4) codebook, scales over many binades, incl. results that are fp16 subnormals."""
    m, k = 256, 512
    rng = np.random.default_rng(5)
    q = rng.integers(0, 256, size=(m // 8, k // 8, 32), dtype=np.uint8)
    code = rng.standard_normal(16).astype(np.float32)
    absmax = (2.0 ** rng.uniform(-20, 3, size=m)).astype(np.float32)
    for mode in (O.D2, O.D1):
        got = run_dequant(q, code, absmax, m, k, decode_mode=mode)
        want = O.dequant(q, absmax, code, m, k, mode=mode)
        assert np.array_equal(got, want), mode


# ----------------------------------------------------------------------------- GEMM decode read-out

@pytest.mark.parametrize("m,k", [(64, 64), (128, 512), (200, 1032), (1024, 4096)])
def test_gemm_decode_readout_bit_exact(m, k):
    """One-hot activations turn the GEMM into a read-out of its in-register decode:
    out[t, r] = 1.0 * W[r, k_t] exactly, so it must equal the oracle's D1 image bit for bit."""
    print(f"readout m={m} k={k}", flush=True)
    q, _, code, absmax = make_inputs_np(m, 16, k, seed=k)
    want_img = O.dequant(q, absmax, code, m, k, mode=O.D1)
    rng = np.random.default_rng(1)
    for rep in range(3):
        cols = rng.choice(k, size=16, replace=False)
        x = np.zeros((16, k), np.float16)
        x[np.arange(16), cols] = 1.0
        got = run_gemm(q, x, code, absmax, m, 16, k)
        want = want_img[:, cols].T
        # +0 and -0 compare equal as values; the sum 0 + (-0) of the accumulator is +0
        assert np.array_equal(f16_bits_to_f64(got), f16_bits_to_f64(want))
        nz = (want & 0x7fff) != 0
        assert np.array_equal(got[nz], want[nz])


def test_gemm_decode_readout_dequant_rounding_mode():
    """decode_mode=TUNA_DECODE_DEQUANT makes the GEMM multiply with the D2 image."""
    m, k = 128, 512
    q, _, code, absmax = make_inputs_np(m, 16, k, seed=3)
    want_img = O.dequant(q, absmax, code, m, k, mode=O.D2)
    cols = np.arange(16) * 7 + 3
    x = np.zeros((16, k), np.float16)
    x[np.arange(16), cols] = 1.0
    got = run_gemm(q, x, code, absmax, m, 16, k, decode_mode=O.D2)
    assert np.array_equal(f16_bits_to_f64(got), f16_bits_to_f64(want_img[:, cols].T))


# ----------------------------------------------------------------------------- GEMM vs oracle

@pytest.mark.parametrize("n", [1, 16])
@pytest.mark.parametrize("name", ["mistral_attn_out", "mistral_qkv"])
def test_gemm_with_dequant_rounding_through_the_dispatcher_on_benchmark_configs(name, n):
    """tuna_matmul_ex(cfg=NULL, TUNA_DECODE_DEQUANT) on benchmark configurations 0 and 1: the GEMM
    over the dequant op's weights (fp32 product, one rounding), against the oracle's float64 sums
    over D2 weights; the one-hot read-out pins the decode itself bit for bit."""
    from tuna_amd.synth import SHAPES

    m, k = SHAPES[name]
    print(f"D2 dispatch {name} m={m} k={k} n={n}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=3)
    got = run_gemm(q, x, code, absmax, m, n, k, config=None, decode_mode=O.D2, prefill=float("nan"))
    rng = np.random.default_rng(n)
    rows = np.sort(rng.choice(m, size=512, replace=False)).astype(np.int32)
    ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D2, rows=rows)
    assert not np.isnan(f16_bits_to_f64(got)).any()
    e = rel_err(f16_bits_to_f64(got[:, rows]), ref)
    print(f"  rel_err={e:.3e}", flush=True)
    assert e <= REL_TOL
    cols = rng.choice(k, size=n, replace=False)
    xh = np.zeros((n, k), np.float16)
    xh[np.arange(n), cols] = 1.0
    got_h = run_gemm(q, xh, code, absmax, m, n, k, config=None, decode_mode=O.D2)
    img = O.dequant(q, absmax, code, m, k, mode=O.D2)
    assert np.array_equal(got_h, img[:, cols].T)


def _random_shapes(count, seed, m_step, k_step):
    """Seeded shapes no table entry has: m and k multiples of the given steps, a token count from every bucket."""
    rng = np.random.default_rng(seed)
    tokens = [1, 2, 3, 5, 8, 11, 13, 16, 17, 24, 31, 32, 40, 63, 64, 65, 100, 128, 130, 200, 256, 300, 511, 512, 700, 1030]
    out = []
    for i in range(count):
        # about a third each: small, one-pass sized (8 .. 60 MB packed) and long-k shapes
        kind = i % 3
        if kind == 0:
            m, k = int(rng.integers(1, 40)) * m_step, int(rng.integers(1, 24)) * k_step
        elif kind == 1:
            m, k = int(rng.integers(2048 // m_step, 12288 // m_step)) * m_step, int(rng.integers(2048 // k_step, 6144 // k_step)) * k_step
        else:
            m, k = int(rng.integers(1024 // m_step, 4096 // m_step)) * m_step, int(rng.integers(8192 // k_step, 20480 // k_step)) * k_step
        n = tokens[int(rng.integers(0, len(tokens)))]
        if m * n > 6_000_000:     # keeps the output and the oracle's sample small
            n = tokens[int(rng.integers(0, 12))]
        out.append((m, n, k))
    return out


@pytest.mark.parametrize("m,n,k", _random_shapes(36, 20240607, 8, 8) + _random_shapes(24, 77, 64, 256))
def test_gemm_through_the_dispatcher_on_random_shapes(m, n, k):
    """tuna_matmul without a config on seeded random shapes (multiples of 8, and multiples of 64 x 256 that the
    streaming kernels' derived configs take): whatever kernel the dispatcher picks, every output is written, a
    row sample matches the oracle's float64 sums, and one-hot activations read the decoded weights out exactly."""
    print(f"random shape m={m} n={n} k={k}", flush=True)
    from tuna_amd import ops

    print("  " + ops.describe_launch(m, n, k, None), flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=m + 3 * n + 7 * k)
    got = run_gemm(q, x, code, absmax, m, n, k, prefill=float("nan"))
    assert not np.isnan(f16_bits_to_f64(got)).any()
    rng = np.random.default_rng(m + n)
    rows = np.sort(rng.choice(m, size=min(m, 96), replace=False)).astype(np.int32)
    ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1, rows=rows)
    e = rel_err(f16_bits_to_f64(got[:, rows]), ref)
    assert e <= REL_TOL, e
    nh = min(n, k)
    cols = rng.choice(k, size=nh, replace=False)
    xh = np.zeros((n, k), np.float16)
    xh[np.arange(nh), cols] = 1.0
    got_h = run_gemm(q, xh, code, absmax, m, n, k)
    img = O.dequant(q, absmax, code, m, k, mode=O.D1)
    assert np.array_equal(got_h[:nh], img[:, cols].T)
    assert not got_h[nh:].any() or np.array_equal(got_h[nh:] & 0x7fff, np.zeros_like(got_h[nh:]))


@pytest.mark.parametrize("m,n,k", _random_shapes(30, 4242, 16, 256))
def test_blockwise_gemm_through_the_dispatcher_on_random_shapes(m, n, k):
    """tuna_matmul_blockwise (a scale per 64 or 128 weights) on seeded random shapes, routed by the library
    between the narrow-row, batched streaming and many-token kernels: complete output, oracle on a row sample,
    exact read-out of the decoded weights."""
    import torch

    from tuna_amd import ops

    bs = 64 if (m // 16) % 2 else 128
    print(f"random blockwise shape m={m} n={n} k={k} block={bs}", flush=True)
    rng = np.random.default_rng(m + n + k)
    q, x, code, _ = make_inputs_np(m, n, k, seed=m + 5 * n + k)
    absmax = rng.uniform(0.005, 0.02, size=(m, k // bs)).astype(np.float16).astype(np.float32)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_blockwise(dx, dq, da, dc, out, m, n, k, bs)
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(np.uint16)
    assert not np.isnan(got.view(np.float16)).any()
    rows = np.sort(rng.choice(m, size=min(m, 96), replace=False)).astype(np.int32)
    ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1, rows=rows, block_size=bs)
    e = rel_err(f16_bits_to_f64(got[:, rows]), ref)
    assert e <= REL_TOL, e
    nh = min(n, k)
    cols = rng.choice(k, size=nh, replace=False)
    xh = np.zeros((n, k), np.float16)
    xh[np.arange(nh), cols] = 1.0
    dxh, = to_dev(xh)
    ops.matmul_blockwise(dxh, dq, da, dc, out, m, n, k, bs)
    torch.cuda.synchronize()
    img = O.dequant(q, absmax, code, m, k, mode=O.D1, block_size=bs)
    assert np.array_equal(out.cpu().numpy().view(np.uint16)[:nh], img[:, cols].T)


@pytest.mark.parametrize("m,n,k,bs", [(2048, 100, 2048, 64), (1024, 256, 4096, 64), (1536, 130, 6144, 128), (1024, 72, 8192, 64),
                                      (3072, 130, 3072, 64), (1024, 500, 1024, 64)])
def test_blockwise_gemm_on_small_shapes_from_65_to_512_tokens_runs_a_round_of_narrow_row_workgroups(m, n, k, bs):
    """Small shapes at 65..512 tokens: the library's blockwise config is one round of narrow-row workgroups with the token
    passes (one or two token tiles each) side by side; complete output, oracle on a row sample, exact read-out of the
    decoded weights through one-hot activations."""
    import torch

    from tuna_amd import ops

    c, hit = ops.select_config_blockwise(m, n, k, bs)
    print(f"blockwise narrow round m={m} n={n} k={k} block={bs}: {c.to_dict()}", flush=True)
    assert not hit and ops.blockwise_family(c) == "narrow" and c.token_tiles in (1, 2) and c.split_k == 1
    assert 64 <= (m // c.rows_per_wave) * -(-n // (16 * c.token_tiles)) <= 256
    rng = np.random.default_rng(m + n + k + bs)
    q, x, code, _ = make_inputs_np(m, n, k, seed=m + 3 * n + k)
    absmax = rng.uniform(0.005, 0.02, size=(m, k // bs)).astype(np.float16).astype(np.float32)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_blockwise(dx, dq, da, dc, out, m, n, k, bs)
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(np.uint16)
    assert not np.isnan(got.view(np.float16)).any()
    rows = np.sort(rng.choice(m, size=96, replace=False)).astype(np.int32)
    ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1, rows=rows, block_size=bs)
    e = rel_err(f16_bits_to_f64(got[:, rows]), ref)
    assert e <= REL_TOL, e
    nh = min(n, k)
    cols = rng.choice(k, size=nh, replace=False)
    xh = np.zeros((n, k), np.float16)
    xh[np.arange(nh), cols] = 1.0
    dxh, = to_dev(xh)
    ops.matmul_blockwise(dxh, dq, da, dc, out, m, n, k, bs)
    torch.cuda.synchronize()
    img = O.dequant(q, absmax, code, m, k, mode=O.D1, block_size=bs)
    assert np.array_equal(out.cpu().numpy().view(np.uint16)[:nh], img[:, cols].T)


SMALL = [
    # m, n, k
    (8, 1, 8), (8, 16, 8), (64, 16, 64), (72, 3, 40), (136, 16, 1032), (256, 16, 128),
    (512, 16, 4096), (4096, 1, 4096), (1024, 17, 2048), (1024, 33, 1024), (512, 64, 2048), (256, 100, 512),
]


@pytest.mark.parametrize("m,n,k", SMALL)
def test_gemm_matches_oracle_small(m, n, k):
    print(f"gemm m={m} n={n} k={k}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=m + n + k)
    got = run_gemm(q, x, code, absmax, m, n, k, prefill=float("nan"))
    ref = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
    assert np.isfinite(f16_bits_to_f64(got)).all()
    e = rel_err(f16_bits_to_f64(got), ref)
    assert e <= REL_TOL, e
    # against the correctly rounded fp16 result the GPU may differ by fp32-accumulation noise only
    want = O.gemm(q, x, code, absmax, m, n, k, mode=O.D1)
    assert rel_err(f16_bits_to_f64(got), f16_bits_to_f64(want)) <= REL_TOL
    # and the reference's dequantize-then-matmul (D2 weights, 1 fp16 ulp away from the GEMM's
    # D1 weights on ~20 % of the entries) is within the same tolerance, under the floor that
    # comparison across the two decodes allows (see helpers.py), once the sum is long enough
    # that single-weight roundings average out
    if k >= 1024:
        ref2 = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D2)
        assert rel_err(f16_bits_to_f64(got), ref2, REL_FLOOR_D2) <= REL_TOL


@pytest.mark.parametrize("name", ["mistral_attn_out", "mistral_qkv"])
def test_gemm_matches_oracle_full_config(name):
    """Benchmark configurations 0 and 1 in full (all rows), seed 0."""
    from tuna_amd.synth import SHAPES

    m, k = SHAPES[name]
    n = 16
    print(f"gemm full {name} m={m} k={k}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=0)
    got = run_gemm(q, x, code, absmax, m, n, k)
    ref = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
    e = rel_err(f16_bits_to_f64(got), ref)
    print(f"  rel_err={e:.3e}", flush=True)
    assert e <= REL_TOL
    ref2 = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D2)
    e2 = rel_err(f16_bits_to_f64(got), ref2, REL_FLOOR_D2)
    print(f"  vs dequantize-then-matmul rel_err={e2:.3e}", flush=True)
    assert e2 <= REL_TOL


CONFIGS = [
    dict(),
    dict(split_k=2),
    dict(split_k=8, x_chunk=512),
    dict(waves_m=1, waves_k=8, prefetch=2, x_chunk=512, split_k=3),
    dict(waves_m=4, waves_k=2, prefetch=8, x_chunk=512),
    dict(rows_per_wave=128, waves_m=2, waves_k=4, prefetch=4, x_chunk=1024, split_k=2),
    dict(rows_per_wave=128, waves_m=2, waves_k=2, prefetch=2, x_chunk=128),
    dict(rows_per_wave=128, waves_m=1, waves_k=1, prefetch=2, x_chunk=64, split_k=4, xcd_swizzle=1),
    dict(waves_m=4, waves_k=4, prefetch=2, x_chunk=512, split_k=2, xcd_swizzle=1),  # 16 waves
    dict(rows_per_wave=64, waves_m=1, waves_k=16, prefetch=2, x_chunk=2048),        # 16 waves along k
    dict(token_tiles=2, split_k=2, prefetch=2, x_chunk=256),
    dict(token_tiles=4, waves_m=2, waves_k=2, prefetch=2, x_chunk=128, split_k=5),
    dict(waves_m=1, waves_k=4, prefetch=4, x_chunk=512, split_k=7),                 # 4-wave workgroups
    dict(waves_m=8, waves_k=1, prefetch=2, x_chunk=64),                             # no k split: store from registers
    dict(waves_m=16, waves_k=1, prefetch=2, x_chunk=64, xcd_swizzle=1),
    dict(rows_per_wave=128, waves_m=4, waves_k=1, prefetch=2, x_chunk=64),
    dict(token_tiles=2, waves_m=4, waves_k=1, prefetch=4, x_chunk=128),
    dict(waves_m=2, waves_k=2, prefetch=2, x_chunk=128, split_k=1),                 # many x chunks per workgroup
    # workgroups of 3, 5, 7 ... waves along the rows (row tiles that are not a power of two)
    dict(waves_m=7, waves_k=1, prefetch=2, x_chunk=64),
    dict(waves_m=3, waves_k=4, prefetch=2, x_chunk=256, split_k=2),
    dict(waves_m=7, waves_k=2, prefetch=2, x_chunk=256, xcd_swizzle=1),
    dict(waves_m=5, waves_k=2, prefetch=4, x_chunk=256, split_k=0),
    # staggered start of the k walk per row tile (wraps around inside the segment)
    dict(k_stagger=1),
    dict(k_stagger=3, split_k=2, prefetch=2, x_chunk=256),
    dict(k_stagger=5, waves_m=1, waves_k=8, prefetch=2, x_chunk=512, split_k=3, xcd_swizzle=1),
    dict(k_stagger=1, waves_m=8, waves_k=1, prefetch=2, x_chunk=64),
    dict(k_stagger=7, waves_m=7, waves_k=2, prefetch=4, x_chunk=256),
    dict(k_stagger=2, token_tiles=2, waves_m=4, waves_k=1, prefetch=4, x_chunk=128),
    dict(k_stagger=9, split_k=0, waves_m=2, waves_k=4, prefetch=2, x_chunk=256),
    dict(k_stagger=4096, rows_per_wave=128, waves_m=2, waves_k=2, prefetch=2, x_chunk=128),
    # balanced split (split_k = 0): k ranges of all row tiles divided evenly over the workgroups
    dict(split_k=0),
    dict(split_k=0, waves_m=1, waves_k=8, prefetch=2, x_chunk=512, xcd_swizzle=1),
    dict(split_k=0, waves_m=8, waves_k=1, prefetch=2, x_chunk=64, xcd_swizzle=1),
    dict(split_k=0, waves_m=4, waves_k=4, prefetch=2, x_chunk=512),                 # 16 waves
    dict(split_k=0, token_tiles=2, waves_m=2, waves_k=4, prefetch=4, x_chunk=512),
    dict(split_k=0, rows_per_wave=128, waves_m=2, waves_k=2, prefetch=2, x_chunk=128),
]


@pytest.mark.parametrize("ci", range(len(CONFIGS)))
@pytest.mark.parametrize("m,n,k", [(1024, 16, 2048), (520, 37, 1096)])
def test_gemm_every_config_family(ci, m, n, k):
    """Every tile-config family gives the oracle's result, including ragged m, n, k."""
    c = cfg(**CONFIGS[ci])
    print(f"gemm cfg#{ci} {c.to_dict()} m={m} n={n} k={k}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=ci)
    got = run_gemm(q, x, code, absmax, m, n, k, config=c, prefill=float("nan"))
    ref = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
    e = rel_err(f16_bits_to_f64(got), ref)
    assert e <= REL_TOL, e


@pytest.mark.parametrize("ckw", [
    dict(split_k=0, waves_m=1, waves_k=2, prefetch=2, x_chunk=128),     # 2400 units: ~4.7 per workgroup
    dict(split_k=0, waves_m=2, waves_k=1, prefetch=2, x_chunk=64, xcd_swizzle=1),
    dict(split_k=0, waves_m=1, waves_k=4, prefetch=4, x_chunk=512),     # one unit per row tile: whole tiles only
])
def test_balanced_split_walks_whole_and_partial_row_tiles(ckw):
    """More row tiles than workgroups: a workgroup's share is a tail of one row tile, whole
    row tiles and a head of another.  Full comparison with the oracle, and the same bits on
    a second launch (workspace slots and arrival counters are left reusable)."""
    m, n, k = 38400, 16, 512
    c = cfg(**ckw)
    print(f"balanced {c.to_dict()} m={m} n={n} k={k}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=21)
    got = run_gemm(q, x, code, absmax, m, n, k, config=c, prefill=float("nan"))
    ref = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
    e = rel_err(f16_bits_to_f64(got), ref)
    assert e <= REL_TOL, e
    again = run_gemm(q, x, code, absmax, m, n, k, config=c, prefill=float("nan"))
    assert np.array_equal(got, again)


def test_split_k_is_deterministic_and_order_independent():
    """Same launch twice: identical bits (no atomics).  Different split counts: only fp32
    re-association noise, i.e. at most 1 fp16 ulp apart after the final rounding."""
    m, n, k = 2048, 16, 4096
    q, x, code, absmax = make_inputs_np(m, n, k, seed=11)
    outs = {}
    for s in (1, 2, 4, 8, 16, 0):
        c = cfg(split_k=s, x_chunk=512)
        a = run_gemm(q, x, code, absmax, m, n, k, config=c)
        for _ in range(3):
            b = run_gemm(q, x, code, absmax, m, n, k, config=c, prefill=float("nan"))
            assert np.array_equal(a, b), s
        outs[s] = a
    for s in (2, 4, 8, 16, 0):
        assert ulp_diff_f16(outs[1], outs[s]) <= 1, s


def test_gemm_linearity_and_zero():
    m, n, k = 1024, 16, 1024
    q, x, code, absmax = make_inputs_np(m, n, k, seed=2)
    zero = run_gemm(q, np.zeros_like(x), code, absmax, m, n, k, prefill=float("nan"))
    assert not (zero & 0x7fff).any()
    y1 = f16_bits_to_f64(run_gemm(q, x, code, absmax, m, n, k))
    y2 = f16_bits_to_f64(run_gemm(q, (x * np.float16(2)).astype(np.float16), code, absmax, m, n, k))
    # scaling by 2 is exact in fp16 and fp32, so the outputs scale exactly wherever the
    # smaller one is a normal fp16 number (subnormal outputs round on a coarser grid)
    normal = np.abs(y1) >= 2.0 ** -14
    assert normal.mean() > 0.99
    assert np.array_equal(y2[normal], 2 * y1[normal])


# ----------------------------------------------------------------------------- full benchmark sizes

@pytest.mark.parametrize("name", list(__import__("tuna_amd.synth", fromlist=["SHAPES"]).SHAPES))
def test_baseline_shapes_row_subset_and_readout(name):
    """Full-size 16-token shapes with device-generated weights.
    (1) 64 random 8-row blocks are copied back and checked against the oracle;
    (2) size-independent property over ALL rows: with one-hot activations the GEMM must
        reproduce columns of the dequant kernel's D1 image exactly (the dequant kernel
        itself is checked against the oracle on the same row subset)."""
    import torch

    from tuna_amd import ops
    from tuna_amd.quantize import nf4_codebook
    from tuna_amd.synth import SHAPES, make_weights_torch, make_x_torch

    m, k = SHAPES[name]
    n = 16
    print(f"baseline shape {name} m={m} k={k}", flush=True)
    dev = torch.device("cuda")
    q, absmax = make_weights_torch(m, k, seed=1234, device=dev)
    x = make_x_torch(n, k, seed=0, device=dev)
    code = nf4_codebook(dev)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device=dev)
    ops.matmul(x, q, absmax, code, out, m, n, k)
    torch.cuda.synchronize()

    rng = np.random.default_rng(7)
    mbs = np.sort(rng.choice(m // 8, size=64, replace=False))
    rows = (mbs[:, None] * 8 + np.arange(8)[None, :]).ravel()
    q_sub = q[torch.from_numpy(mbs).to(dev)].cpu().numpy()          # [64, k/8, 32] = packed 512 x k
    a_sub = absmax.cpu().numpy()[rows]
    x_np = x.cpu().numpy().view(np.uint16)
    code_np = code.cpu().numpy()
    ref = O.gemm_f64(q_sub, x_np, code_np, a_sub, len(rows), n, k, mode=O.D1)
    got = out.cpu().numpy().view(np.uint16)[:, rows]
    e = rel_err(f16_bits_to_f64(got), ref)
    print(f"  subset rel_err={e:.3e}", flush=True)
    assert e <= REL_TOL

    img = torch.empty((m, k), dtype=torch.float16, device=dev)
    ops.dequant(q, absmax, code, img, m, k, decode_mode=O.D1)
    torch.cuda.synchronize()
    img_sub = img[torch.from_numpy(rows).to(dev)].cpu().numpy().view(np.uint16)
    assert np.array_equal(img_sub, O.dequant(q_sub, a_sub, code_np, len(rows), k, mode=O.D1))

    cols = torch.from_numpy(rng.choice(k, size=n, replace=False)).to(dev)
    xh = torch.zeros((n, k), dtype=torch.float16, device=dev)
    xh[torch.arange(n, device=dev), cols] = 1.0
    ops.matmul(xh, q, absmax, code, out, m, n, k)
    torch.cuda.synchronize()
    assert torch.equal(out.float(), img[:, cols].t().float())


@pytest.mark.parametrize("n", [1, 13, 64, 256, 1024])
@pytest.mark.parametrize("name", ["llama70b_qkv", "llama70b_attn_out", "llama70b_gate_up", "llama70b_down"])
def test_token_sweep_llama70b_layer_set(name, n):
    """The M sweep of benchmark configuration 3 ({1, 16, 64, 256}, plus the 1024 the bench also times and 13,
    which the dispatcher serves with the 16-token entry)
    on all four Llama-70B shapes with the tuned table's entries - narrow-row, lean, streaming and
    many-token kernels at their real sizes - checked on a row subset (16 tokens is covered above)."""
    import torch

    from tuna_amd import ops
    from tuna_amd.quantize import nf4_codebook
    from tuna_amd.synth import SHAPES, make_weights_torch, make_x_torch

    m, k = SHAPES[name]
    used, hit = ops.select_config(m, n, k)
    assert hit
    print(f"token sweep {name} m={m} k={k} n={n} cfg={used.to_dict()}", flush=True)
    dev = torch.device("cuda")
    q, absmax = make_weights_torch(m, k, seed=n, device=dev)
    x = make_x_torch(n, k, seed=n, device=dev)
    code = nf4_codebook(dev)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device=dev)
    ops.matmul(x, q, absmax, code, out, m, n, k)
    torch.cuda.synchronize()
    assert not torch.isnan(out).any()                       # every output was written
    rng = np.random.default_rng(n)
    mbs = np.sort(rng.choice(m // 8, size=16 if n >= 256 else 32, replace=False))
    rows = (mbs[:, None] * 8 + np.arange(8)[None, :]).ravel()
    q_sub = q[torch.from_numpy(mbs).to(dev)].cpu().numpy()
    ref = O.gemm_f64(q_sub, x.cpu().numpy().view(np.uint16), code.cpu().numpy(), absmax.cpu().numpy()[rows],
                     len(rows), n, k, mode=O.D1)
    got = out[:, torch.from_numpy(rows).to(dev)].cpu().numpy().view(np.uint16)
    e = rel_err(f16_bits_to_f64(got), ref)
    print(f"  rel_err={e:.3e}", flush=True)
    assert e <= REL_TOL


def _entries_for_keys_inside_buckets():
    import json
    import os

    from tuna_amd import make_configs

    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "tuna_amd", "configs", "param_map.json")
    with open(path) as f:
        return sorted(key for key in json.load(f) if int(key.split("_")[1]) in make_configs.SUB_KEYS)


@pytest.mark.parametrize("key", _entries_for_keys_inside_buckets())
def test_every_entry_for_the_upper_part_of_a_bucket_matches_the_oracle(key):
    """Table entries whose key lies inside a token bucket (24, 48, 96, 192, 384: they cover the bucket from that count
    up): the lookup hands out the entry at its lower edge, and the launch is checked against the oracle on a row
    subset there, one token below (the bucket's own entry) and at the bucket's last count."""
    import torch

    from tuna_amd import make_configs, ops
    from tuna_amd.quantize import nf4_codebook
    from tuna_amd.synth import make_weights_torch, make_x_torch

    m, n_key, k = (int(t) for t in key.split("_"))
    dev = torch.device("cuda")
    q, absmax = make_weights_torch(m, k, seed=n_key, device=dev)
    code = nf4_codebook(dev)
    rng = np.random.default_rng(m + n_key)
    mbs = np.sort(rng.choice(m // 8, size=8, replace=False))
    rows = (mbs[:, None] * 8 + np.arange(8)[None, :]).ravel()
    q_sub = q[torch.from_numpy(mbs).to(dev)].cpu().numpy()
    a_sub = absmax.cpu().numpy()[rows]
    entry = [cfg for (m_, lo, hi, k_, cfg) in ops.config_table() if (m_, lo, k_) == (m, n_key, k)]
    assert len(entry) == 1
    for n in (n_key, n_key - 1, make_configs.N_BUCKETS[make_configs.SUB_KEYS[n_key]][1]):
        used, hit = ops.select_config(m, n, k)
        assert hit and (n != n_key or used.to_dict() == entry[0].to_dict())
        print(f"entry {key} at n={n}: {ops.describe_launch(m, n, k, used)}", flush=True)
        x = make_x_torch(n, k, seed=n, device=dev)
        out = torch.full((n, m), float("nan"), dtype=torch.float16, device=dev)
        ops.matmul(x, q, absmax, code, out, m, n, k)
        torch.cuda.synchronize()
        assert not torch.isnan(out).any()
        ref = O.gemm_f64(q_sub, x.cpu().numpy().view(np.uint16), code.cpu().numpy(), a_sub, len(rows), n, k, mode=O.D1)
        got = out[:, torch.from_numpy(rows).to(dev)].cpu().numpy().view(np.uint16)
        e = rel_err(f16_bits_to_f64(got), ref)
        print(f"  rel_err={e:.3e}", flush=True)
        assert e <= REL_TOL


@pytest.mark.parametrize("name,n,kernel", [("mistral_qkv", 1200, "128 rows x 256 tokens"), ("llama70b_qkv", 1536, "gemm_wide_kernel"),
                                           ("mistral_attn_out", 700, "128 rows x 256 tokens> split_k=2"), ("llama70b_attn_out", 600, "128 rows x 256 tokens"),
                                           ("mistral_down", 1000, "split_k=2"),
                                           ("mistral_qkv", 300, "TT=2"), ("mistral_qkv", 72, "TT=1"), ("llama70b_attn_out", 270, "gemm_")])
def test_table_shapes_between_the_counts_their_upper_entries_are_tuned_at(name, n, kernel):
    """Above 512 tokens the table's entries are tuned at 512, 1024 and 2048 tokens; at other counts a shape of fewer than
    24576 rows runs what the derivation's cost model picks (its entry at counts with as many 128-token tiles as the
    tuning count: mistral_down), through the plain entry point.  The last three cases lie in the stretch of a bucket
    below 512 tokens where the tuner timed the derived config ahead of the entry.  Row-subset check against the oracle."""
    import torch

    from tuna_amd import ops
    from tuna_amd.quantize import nf4_codebook
    from tuna_amd.synth import SHAPES, make_weights_torch, make_x_torch

    m, k = SHAPES[name]
    used, hit = ops.select_config(m, n, k)
    desc = ops.describe_launch(m, n, k, None)
    print(f"table shape {name} m={m} k={k} n={n}: {desc}", flush=True)
    assert hit and kernel in desc
    if name != "mistral_down":
        assert used.to_dict() == ops.derive_config(m, n, k).to_dict()
    dev = torch.device("cuda")
    q, absmax = make_weights_torch(m, k, seed=n, device=dev)
    x = make_x_torch(n, k, seed=n + 1, device=dev)
    code = nf4_codebook(dev)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device=dev)
    ops.matmul(x, q, absmax, code, out, m, n, k)
    torch.cuda.synchronize()
    assert not torch.isnan(out).any()
    rng = np.random.default_rng(n)
    mbs = np.sort(rng.choice(m // 8, size=4, replace=False))
    rows = (mbs[:, None] * 8 + np.arange(8)[None, :]).ravel()
    q_sub = q[torch.from_numpy(mbs).to(dev)].cpu().numpy()
    ref = O.gemm_f64(q_sub, x.cpu().numpy().view(np.uint16), code.cpu().numpy(), absmax.cpu().numpy()[rows],
                     len(rows), n, k, mode=O.D1)
    got = out[:, torch.from_numpy(rows).to(dev)].cpu().numpy().view(np.uint16)
    e = rel_err(f16_bits_to_f64(got), ref)
    print(f"  rel_err={e:.3e}", flush=True)
    assert e <= REL_TOL


@pytest.mark.parametrize("name,n", [("mistral_attn_out", 3072), ("mistral_down", 3100), ("llama70b_qkv", 4096), ("llama70b_qkv", 2560)])
def test_token_counts_far_into_the_last_bucket_take_the_256_x_256_tile(name, n):
    """The last bucket of the table is open-ended and tuned at 2048 tokens; away from that count a shape of fewer than
    24576 rows takes the pick of the derivation's cost model, which far into the bucket is the 256 x 256 many-token
    tile, through the plain entry point.  Row-subset check against the oracle."""
    import torch

    from tuna_amd import ops
    from tuna_amd.quantize import nf4_codebook
    from tuna_amd.synth import SHAPES, make_weights_torch, make_x_torch

    m, k = SHAPES[name]
    used, hit = ops.select_config(m, n, k)
    assert hit and (used.lds_tile_rows, used.token_tiles) == (256, 16)
    assert "gemm_wide_kernel" in ops.describe_launch(m, n, k, None)
    print(f"last bucket {name} m={m} k={k} n={n}", flush=True)
    dev = torch.device("cuda")
    q, absmax = make_weights_torch(m, k, seed=n, device=dev)
    x = make_x_torch(n, k, seed=n + 1, device=dev)
    code = nf4_codebook(dev)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device=dev)
    ops.matmul(x, q, absmax, code, out, m, n, k)
    torch.cuda.synchronize()
    assert not torch.isnan(out).any()                       # every output was written
    rng = np.random.default_rng(n)
    mbs = np.sort(rng.choice(m // 8, size=4, replace=False))
    rows = (mbs[:, None] * 8 + np.arange(8)[None, :]).ravel()
    q_sub = q[torch.from_numpy(mbs).to(dev)].cpu().numpy()
    ref = O.gemm_f64(q_sub, x.cpu().numpy().view(np.uint16), code.cpu().numpy(), absmax.cpu().numpy()[rows],
                     len(rows), n, k, mode=O.D1)
    got = out[:, torch.from_numpy(rows).to(dev)].cpu().numpy().view(np.uint16)
    e = rel_err(f16_bits_to_f64(got), ref)
    print(f"  rel_err={e:.3e}", flush=True)
    assert e <= REL_TOL                                      # max relative error 1e-2


@pytest.mark.parametrize("n", [1, 16, 40, 100, 200, 300, 600, 1000, 1500])
@pytest.mark.parametrize("m,k", [(2560, 2560), (2560, 10240), (7680, 2560), (10240, 2560)])
def test_reference_table_2560_wide_shapes_every_bucket(m, k, n):
    """The four 2560-wide shapes of the reference's table (param_map.json keys 2560_*_2560,
    2560_*_10240, 7680_*_2560, 10240_*_2560; dispatched at kernel.cu:3022-3155) with the tuned
    entry of every token bucket, checked against the oracle on a random subset of 8-row blocks."""
    import torch

    from tuna_amd import ops
    from tuna_amd.quantize import nf4_codebook
    from tuna_amd.synth import make_weights_torch, make_x_torch

    _, hit = ops.select_config(m, n, k)
    assert hit, "no tuned table entry"
    print(f"2560-wide shape m={m} k={k} n={n}", flush=True)
    dev = torch.device("cuda")
    q, absmax = make_weights_torch(m, k, seed=m + n, device=dev)
    x = make_x_torch(n, k, seed=k + n, device=dev)
    code = nf4_codebook(dev)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device=dev)
    ops.matmul(x, q, absmax, code, out, m, n, k)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    rng = np.random.default_rng(m * 31 + k + n)
    mbs = np.sort(rng.choice(m // 8, size=8, replace=False))
    rows = (mbs[:, None] * 8 + np.arange(8)[None, :]).ravel()
    q_sub = q[torch.from_numpy(mbs).to(dev)].cpu().numpy()
    ref = O.gemm_f64(q_sub, x.cpu().numpy().view(np.uint16), code.cpu().numpy(), absmax.cpu().numpy()[rows],
                     len(rows), n, k, mode=O.D1)
    got = out.cpu().numpy().view(np.uint16)[:, rows]
    e = rel_err(f16_bits_to_f64(got), ref)
    print(f"  rel_err={e:.3e}", flush=True)
    assert e <= REL_TOL


@pytest.mark.parametrize("m,k,n,kernel", [(5120, 5120, 16, "gemm_narrow_kernel"), (2048, 2048, 3, "gemm_narrow_kernel"),
                                           (11008, 4096, 9, "gemm_narrow_kernel"), (3072, 8192, 16, "gemm_lean_kernel"),
                                           (20480, 5120, 1, "gemm_lean_kernel"), (22016, 4096, 16, "weights through LDS"),
                                           (37888, 3584, 12, "weights through LDS"), (4096, 11008, 16, "gemm_kernel"),
                                           (1024, 1024, 16, "gemm_narrow_kernel<LW=1"), (2560, 5120, 4, "gemm_narrow_kernel<LW=1"), (1024, 4096, 1, "gemm_narrow_kernel<LW=1")])
def test_derived_configs_for_untuned_shapes_up_to_16_tokens(m, k, n, kernel):
    _check_derived(m, k, n, kernel)


@pytest.mark.parametrize("m,k,n,kernel", [(8192, 3072, 64, "gemm_narrow_kernel"), (5120, 5120, 20, "gemm_narrow_kernel"),
                                           (4096, 12288, 32, "gemm_lean_kernel"), (12288, 4096, 64, "weights through LDS"),
                                           (37888, 3584, 40, "weights through LDS"), (3072, 8192, 128, "gemm_narrow_kernel"), (1024, 8192, 64, "gemm_narrow_kernel<LW=1,WK=8,U=4,PERM=1,TT=1>"), (2048, 12288, 48, "gemm_lean_kernel"),
                                           (1536, 6144, 40, "gemm_narrow_kernel<LW=2,WK=8,U=4,PERM=1,TT=1>"), (2048, 8192, 20, "gemm_narrow_kernel<LW=1"), (4096, 11008, 48, "64 rows x 128 tokens> split_k=4"), (6144, 24576, 48, "weights through LDS> x_chunk=256 split_k=4"), (1024, 8192, 256, "gemm_narrow_kernel<LW=4,WK=8,U=4,PERM=1,TT=1>"), (1536, 12288, 160, "gemm_narrow_kernel"), (1024, 4096, 512, "gemm_narrow_kernel<LW=4,WK=8,U=4,PERM=1,TT=2>"),
                                           (5120, 5120, 200, "128 rows x 128 tokens> split_k=3"), (12288, 4096, 300, "TT=4"),
                                           (3072, 8192, 512, "128 rows x 256 tokens> split_k=4"), (20480, 5120, 64, "TT=2"),
                                           (18432, 6144, 256, "256 rows x 256 tokens> split_k=3"), (2048, 2048, 384, "TT=2"),
                                           (20480, 5120, 384, "TT=8"), (16384, 8192, 640, "gemm_wide_kernel"),
                                           (2560, 6912, 300, "128 rows x 128 tokens> split_k=4"), (4096, 11008, 100, "64 rows x 128 tokens> split_k=4"), (5120, 13824, 1000, "256 rows x 256 tokens> split_k=3"), (22016, 4096, 704, "128 rows x 256 tokens")])
def test_derived_configs_for_untuned_shapes_from_17_to_512_tokens(m, k, n, kernel):
    """The same for 17 tokens and more: narrow-row (up to 512 tokens on small shapes) and lean workgroups with the token passes side by side in the grid,
    the streaming kernel with 16, 32 or 64 tokens per pass, and from 256 tokens the tile that a cost model of the
    grid picks (chunks of 32 ... 128 tokens of the streaming kernel side by side, or a many-token tile)."""
    _check_derived(m, k, n, kernel)


def _check_derived(m, k, n, kernel):
    """Shapes outside the table at up to 16 tokens: one round of narrow-row workgroups where a tile height gives one,
    the streaming kernel with the weights through LDS for many rows, the lean split-K kernel where k divides in
    powers of two, the general kernel otherwise - each through the plain entry point, on a random subset of rows."""
    import torch

    from tuna_amd import ops
    from tuna_amd.quantize import nf4_codebook
    from tuna_amd.synth import make_weights_torch, make_x_torch

    cfg, hit = ops.select_config(m, n, k)
    assert not hit
    desc = ops.describe_launch(m, n, k, None)
    print(f"derived config m={m} n={n} k={k}: {desc}", flush=True)
    assert kernel in desc
    dev = torch.device("cuda")
    q, absmax = make_weights_torch(m, k, seed=m + n, device=dev)
    x = make_x_torch(n, k, seed=k + n, device=dev)
    code = nf4_codebook(dev)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device=dev)
    ops.matmul(x, q, absmax, code, out, m, n, k)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    rng = np.random.default_rng(m + k + n)
    mbs = np.sort(rng.choice(m // 8, size=32, replace=False))
    rows = (mbs[:, None] * 8 + np.arange(8)[None, :]).ravel()
    q_sub = q[torch.from_numpy(mbs).to(dev)].cpu().numpy()
    ref = O.gemm_f64(q_sub, x.cpu().numpy().view(np.uint16), code.cpu().numpy(), absmax.cpu().numpy()[rows],
                     len(rows), n, k, mode=O.D1)
    got = out.cpu().numpy().view(np.uint16)[:, rows]
    e = rel_err(f16_bits_to_f64(got), ref)
    print(f"  rel_err={e:.3e}", flush=True)
    assert e <= REL_TOL                                      # max relative error 1e-2


@pytest.mark.parametrize("m,k,n,split", [(12288, 1024, 1000, 1), (16384, 8192, 1000, 1), (5120, 8192, 1300, None), (5120, 4096, 1300, None)])
def test_derived_config_for_an_untuned_shape_with_very_many_tokens(m, k, n, split):
    """A shape outside the table with very many tokens gets the 256 x 256 many-token tile when its tiles fill the
    device in one round (192 and 256 tiles), not when smaller tiles make a fuller round (120 tiles of 256 x 256
    against 240 of 128 x 256), through the plain entry point; checked on a random subset of rows."""
    import torch

    from tuna_amd import ops
    from tuna_amd.quantize import nf4_codebook
    from tuna_amd.synth import make_weights_torch, make_x_torch

    cfg, hit = ops.select_config(m, n, k)
    assert not hit
    if split is None:
        assert (cfg.lds_tile_rows, cfg.token_tiles) != (256, 16)
    else:
        assert (cfg.lds_tile_rows, cfg.token_tiles, cfg.split_k) == (256, 16, split)
        assert "gemm_wide_kernel" in ops.describe_launch(m, n, k, None)
    print(f"derived config m={m} n={n} k={k} {cfg.to_dict()}", flush=True)
    dev = torch.device("cuda")
    q, absmax = make_weights_torch(m, k, seed=7, device=dev)
    x = make_x_torch(n, k, seed=8, device=dev)
    code = nf4_codebook(dev)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device=dev)
    ops.matmul(x, q, absmax, code, out, m, n, k)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    rng = np.random.default_rng(13)
    mbs = np.sort(rng.choice(m // 8, size=16, replace=False))
    rows = (mbs[:, None] * 8 + np.arange(8)[None, :]).ravel()
    q_sub = q[torch.from_numpy(mbs).to(dev)].cpu().numpy()
    ref = O.gemm_f64(q_sub, x.cpu().numpy().view(np.uint16), code.cpu().numpy(), absmax.cpu().numpy()[rows],
                     len(rows), n, k, mode=O.D1)
    got = out.cpu().numpy().view(np.uint16)[:, rows]
    e = rel_err(f16_bits_to_f64(got), ref)
    print(f"  rel_err={e:.3e}", flush=True)
    assert e <= REL_TOL                                      # max relative error 1e-2


@pytest.mark.parametrize("m,k,n,tiles", [(66560, 1024, 50, 4), (66560, 1024, 100, 8), (66560, 1024, 300, 8),
                                         (16384, 2048, 100, 2)])
def test_derived_config_for_a_large_untuned_shape_with_many_tokens(m, k, n, tiles):
    """A shape outside the table with many rows and more than 32 tokens gets the streaming kernel
    with four or eight token tiles (one pass of 64 or 128 tokens, or three passes of 128 side by
    side); checked on a random subset of rows."""
    import torch

    from tuna_amd import ops
    from tuna_amd.quantize import nf4_codebook
    from tuna_amd.synth import make_weights_torch, make_x_torch

    cfg, hit = ops.select_config(m, n, k)
    assert not hit and cfg.token_tiles == tiles and cfg.lds_tile_rows in (0, -1)   # (-1: the packed weights through LDS)
    print(f"derived config m={m} n={n} k={k} {cfg.to_dict()}", flush=True)
    dev = torch.device("cuda")
    q, absmax = make_weights_torch(m, k, seed=5, device=dev)
    x = make_x_torch(n, k, seed=6, device=dev)
    code = nf4_codebook(dev)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device=dev)
    ops.matmul(x, q, absmax, code, out, m, n, k)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    rng = np.random.default_rng(11)
    mbs = np.sort(rng.choice(m // 8, size=32, replace=False))
    rows = (mbs[:, None] * 8 + np.arange(8)[None, :]).ravel()
    q_sub = q[torch.from_numpy(mbs).to(dev)].cpu().numpy()
    ref = O.gemm_f64(q_sub, x.cpu().numpy().view(np.uint16), code.cpu().numpy(), absmax.cpu().numpy()[rows],
                     len(rows), n, k, mode=O.D1)
    got = out.cpu().numpy().view(np.uint16)[:, rows]
    e = rel_err(f16_bits_to_f64(got), ref)
    print(f"  rel_err={e:.3e}", flush=True)
    assert e <= REL_TOL


# ----------------------------------------------------------------------------- error behaviour

def test_errors_raise_instead_of_silent_noop():
    import torch

    from tuna_amd import ops

    dev = "cuda"
    m, n, k = 64, 16, 64
    q = torch.zeros((m // 8, k // 8, 32), dtype=torch.uint8, device=dev)
    x = torch.zeros((n, k), dtype=torch.float16, device=dev)
    s = torch.ones(m, dtype=torch.float32, device=dev)
    c = torch.zeros(16, dtype=torch.float32, device=dev)
    o = torch.zeros((n, m), dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        ops.matmul(x, q, s, c, o, 60, n, k)          # m not a multiple of 8
    with pytest.raises(TypeError):
        ops.matmul(x.float(), q, s, c, o, m, n, k)   # wrong dtype
    with pytest.raises(ValueError):
        ops.matmul(x, q, s, c, o[:, :32], m, n, k)   # wrong size / non-contiguous
    with pytest.raises(ops.TunaError):
        ops.matmul(x, q, s, c, o, m, n, k, config=cfg(prefetch=3))
    with pytest.raises(ops.TunaError):
        ops.matmul(x, q, s, c, o, m, n, k, config=cfg(x_chunk=1 << 20))  # exceeds LDS
    ops.matmul(x, q, s, c, o, m, n, k)               # and the valid call still works
    torch.cuda.synchronize()


# ----------------------------------------------------------------------------- grouped GEMM (per-expert token lists)
def _run_grouped(q, x, code, absmax, m_group, n_groups, k, offsets, config=None, decode_mode=1):
    import torch

    from tuna_amd import ops

    dq, dx, dc, da = to_dev(q, x, code, absmax)
    n_total = offsets[-1]
    out = torch.full((max(n_total, 1), m_group), float("nan"), dtype=torch.float16, device="cuda")[:n_total]
    ops.matmul_grouped(dx, dq, da, dc, out, m_group, n_groups, k, offsets, config=config, decode_mode=decode_mode)
    torch.cuda.synchronize()
    return out.cpu().numpy().view(np.uint16)


def _grouped_reference(q, x, code, absmax, m_group, n_groups, k, offsets, mode=O.D1):
    """Per expert: the oracle's dense GEMM on that expert's packed rows and tokens."""
    n_total = offsets[-1]
    ref = np.zeros((n_total, m_group), dtype=np.float64)
    qb = q.reshape(n_groups, m_group // 8, k // 8, 32)
    for e in range(n_groups):
        lo, hi = offsets[e], offsets[e + 1]
        if hi > lo:
            ref[lo:hi] = O.gemm_f64(np.ascontiguousarray(qb[e]), np.ascontiguousarray(x[lo:hi]), code,
                                    np.ascontiguousarray(absmax[e * m_group:(e + 1) * m_group]), m_group, hi - lo, k, mode=mode)
    return ref


@pytest.mark.parametrize("m_group,n_groups,k,counts,ckw", [
    (256, 8, 1024, [4, 4, 4, 4, 4, 4, 4, 4], None),
    (256, 8, 1024, [0, 7, 0, 16, 1, 0, 3, 5], None),                       # empty experts are skipped
    (512, 4, 2048, [16, 0, 0, 16], dict(split_k=2, x_chunk=512)),
    (512, 4, 2048, [3, 20, 0, 9], dict(token_tiles=2, split_k=2, prefetch=2, x_chunk=256)),   # 20 tokens: two token tiles
    (384, 5, 1096, [2, 0, 33, 1, 6], dict(waves_m=3, waves_k=2, prefetch=2, x_chunk=128)),     # ragged k, 3 token chunks
    (1024, 3, 512, [5, 5, 5], dict(waves_m=8, waves_k=1, prefetch=2, x_chunk=64)),            # register-store epilogue
    (256, 6, 2048, [1, 0, 2, 0, 0, 9], dict(split_k=0, waves_m=1, waves_k=4, prefetch=2, x_chunk=256)),  # balanced split
    (128, 64, 256, [i % 3 for i in range(64)], None),                      # 64 experts
    (512, 4, 2048, [40, 64, 33, 7], None),                                 # 33..64 tokens: four token tiles, one pass
    (1024, 3, 4096, [48, 0, 64], None),
])
def test_grouped_gemm_matches_per_expert_oracle(m_group, n_groups, k, counts, ckw):
    offsets = [0]
    for c in counts:
        offsets.append(offsets[-1] + c)
    n_total = offsets[-1]
    m = m_group * n_groups
    config = cfg(**ckw) if ckw else None
    print(f"grouped m_group={m_group} n_groups={n_groups} k={k} counts={counts} cfg={ckw}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n_total, k, seed=77)
    got = _run_grouped(q, x, code, absmax, m_group, n_groups, k, offsets, config)
    ref = _grouped_reference(q, x, code, absmax, m_group, n_groups, k, offsets)
    assert not np.isnan(f16_bits_to_f64(got)).any()          # every output row was written
    e = rel_err(f16_bits_to_f64(got), ref)
    assert e <= REL_TOL, e


@pytest.mark.parametrize("m_group,n_groups,k,counts", [
    (256, 4, 1024, [65, 3, 0, 130]),        # two groups as dense GEMMs, one through the grouped kernel, one empty
    (512, 3, 512, [200, 96, 257]),          # every group a dense GEMM (nothing left for the grouped kernel)
    (256, 5, 2048, [64, 65, 1, 0, 300]),    # 64 tokens still fit one pass of the grouped kernel, 65 do not
])
def test_grouped_gemm_with_groups_of_many_tokens_matches_per_expert_oracle(m_group, n_groups, k, counts):
    """Groups of more than 64 tokens run as dense GEMMs of their own (the library's config for their token count),
    the others in one grouped launch: every row against the oracle, and the rows of a large group bit-identical to
    the dense call on that group's slices."""
    offsets = [0]
    for c in counts:
        offsets.append(offsets[-1] + c)
    n_total = offsets[-1]
    m = m_group * n_groups
    print(f"grouped, many tokens: m_group={m_group} n_groups={n_groups} k={k} counts={counts}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n_total, k, seed=78)
    got = _run_grouped(q, x, code, absmax, m_group, n_groups, k, offsets, None)
    ref = _grouped_reference(q, x, code, absmax, m_group, n_groups, k, offsets)
    assert not np.isnan(f16_bits_to_f64(got)).any()          # every output row was written
    e = rel_err(f16_bits_to_f64(got), ref)
    assert e <= REL_TOL, e
    qb = q.reshape(n_groups, m_group // 8, k // 8, 32)
    for g, c in enumerate(counts):
        if c > 64:
            lo, hi = offsets[g], offsets[g + 1]
            dense = run_gemm(np.ascontiguousarray(qb[g]), np.ascontiguousarray(x[lo:hi]), code,
                             np.ascontiguousarray(absmax[g * m_group:(g + 1) * m_group]), m_group, c, k)
            assert np.array_equal(dense, got[lo:hi]), g


def test_grouped_gemm_with_a_large_group_and_the_dequantizers_rounding():
    """decode_mode D2 (fp32 multiply, then round) reaches the dense launches of the large groups too."""
    m_group, n_groups, k, counts = 256, 3, 512, [7, 150, 0]
    offsets = [0, 7, 157, 157]
    q, x, code, absmax = make_inputs_np(m_group * n_groups, offsets[-1], k, seed=79)
    got = _run_grouped(q, x, code, absmax, m_group, n_groups, k, offsets, None, decode_mode=O.D2)
    ref = _grouped_reference(q, x, code, absmax, m_group, n_groups, k, offsets, mode=O.D2)
    assert not np.isnan(f16_bits_to_f64(got)).any()
    assert rel_err(f16_bits_to_f64(got), ref) <= REL_TOL
    qb = q.reshape(n_groups, m_group // 8, k // 8, 32)
    dense = run_gemm(np.ascontiguousarray(qb[1]), np.ascontiguousarray(x[7:157]), code, np.ascontiguousarray(absmax[256:512]),
                     m_group, 150, k, decode_mode=O.D2)
    assert np.array_equal(dense, got[7:157])


def test_grouped_gemm_with_one_group_equals_dense_bits():
    """One group owning every token is the dense GEMM: identical bits."""
    m, n, k = 1024, 16, 2048
    q, x, code, absmax = make_inputs_np(m, n, k, seed=5)
    c = cfg(split_k=2)
    dense = run_gemm(q, x, code, absmax, m, n, k, config=c)
    grouped = _run_grouped(q, x, code, absmax, m, 1, k, [0, n], c)
    assert np.array_equal(dense, grouped)


def test_grouped_gemm_rejects_bad_arguments():
    import torch

    from tuna_amd import ops

    q, x, code, absmax = make_inputs_np(512, 8, 256, seed=1)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    out = torch.empty((8, 256), dtype=torch.float16, device="cuda")
    with pytest.raises(ops.TunaError):
        ops.matmul_grouped(dx, dq, da, dc, out, 256, 2, 256, [0, 9, 8])         # decreasing offsets
    with pytest.raises(ops.TunaError):
        ops.matmul_grouped(dx, dq, da, dc, out, 256, 2, 256, [0, 4, 8], config=cfg(waves_m=8, waves_k=1, prefetch=2, x_chunk=64))  # 512-row tiles straddle groups


# ----------------------------------------------------------------------------- many-token kernel (weights decoded once into LDS)
TILED = [(256, 8), (256, 4), (128, 16), (128, 8), (64, 16), (64, 8)]   # (lds_tile_rows, token_tiles)


@pytest.mark.parametrize("tile", TILED)
@pytest.mark.parametrize("m,n,k,split", [(512, 256, 512, 1), (520, 300, 1096, 1), (256, 70, 2048, 4), (1024, 129, 200, 3),
                                         (256, 40, 64, 1), (264, 130, 192, 1), (512, 64, 320, 1), (256, 200, 576, 1),
                                         (128, 260, 1088, 1), (256, 33, 1408, 2)])
def test_many_token_kernel_matches_oracle(tile, m, n, k, split):
    """Every tile shape of the many-token kernel, ragged m / n / k and split-K, against the
    oracle's float64 contraction of the same fp16 weights; k ranges of 1, 2, 3, 5, 9, 11, 17 and 18 steps per
    workgroup (the loop is unrolled by the four or eight register sets: every length of its tail, a split that
    gets no step at all)."""
    rows, tt = tile
    c = cfg(lds_tile_rows=rows, token_tiles=tt, split_k=split)
    print(f"many-token tile {rows}x{16 * tt} m={m} n={n} k={k} split={split}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=rows + tt + split)
    got = run_gemm(q, x, code, absmax, m, n, k, config=c, prefill=float("nan"))
    ref = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
    e = rel_err(f16_bits_to_f64(got), ref)
    assert e <= REL_TOL, e
    again = run_gemm(q, x, code, absmax, m, n, k, config=c, prefill=float("nan"))
    assert np.array_equal(got, again)


@pytest.mark.parametrize("tile", [t for t in TILED if t != (64, 8)])
@pytest.mark.parametrize("m,n,k,split", [(512, 256, 512, 1), (520, 300, 1096, 1), (256, 70, 2048, 4), (1024, 129, 200, 3)])
def test_many_token_kernel_with_32x32_mfma_tiles_matches_oracle(tile, m, n, k, split):
    """The same tiles multiplied with v_mfma_f32_32x32x16_f16 (rows_per_wave = 32 in a many-token
    config): ragged m / n / k and split-K against the oracle's float64 sums, run-to-run identical,
    and within fp32 summation-order noise of the 16 x 16 x 32 variant."""
    from tuna_amd import ops

    rows, tt = tile
    c32 = cfg(lds_tile_rows=rows, token_tiles=tt, split_k=split, rows_per_wave=32)
    c16 = cfg(lds_tile_rows=rows, token_tiles=tt, split_k=split)
    assert "mfma 32x32x16" in ops.describe_launch(m, n, k, c32) and "mfma" not in ops.describe_launch(m, n, k, c16)
    print(f"many-token tile {rows}x{16 * tt} with 32x32 MFMA tiles, m={m} n={n} k={k} split={split}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=rows + tt + split)
    got = run_gemm(q, x, code, absmax, m, n, k, config=c32, prefill=float("nan"))
    ref = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
    e = rel_err(f16_bits_to_f64(got), ref)
    assert e <= REL_TOL, e                                   # max relative error 1e-2
    again = run_gemm(q, x, code, absmax, m, n, k, config=c32, prefill=float("nan"))
    assert np.array_equal(got, again)
    other = run_gemm(q, x, code, absmax, m, n, k, config=c16, prefill=float("nan"))
    assert rel_err(f16_bits_to_f64(got), f16_bits_to_f64(other)) <= 2e-3   # one fp16 ulp of the larger outputs


@pytest.mark.parametrize("mfma_rows", [64, 32])
@pytest.mark.parametrize("m,n,k,split", [(512, 256, 512, 1), (520, 300, 1088, 1), (256, 70, 2048, 4), (1024, 129, 192, 3),
                                         (256, 40, 64, 1), (264, 130, 192, 1), (512, 600, 320, 1), (768, 513, 576, 2),
                                         (256, 256, 128, 1), (1280, 1024, 256, 1)])
def test_many_token_kernel_with_the_256_x_256_tile_matches_oracle_and_the_smaller_tiles(mfma_rows, m, n, k, split):
    """The 256 x 256 tile (one wave per SIMD, a wave owns 128 x 128) with both MFMA shapes: ragged m and n,
    split-K with a remainder, k ranges of 1 ... 32 steps per workgroup (its loop is unrolled by two: odd and even
    lengths), against the oracle's float64 sums; run-to-run identical; and, unsplit, the bits of the 128 x 128
    tile with the same MFMA shape (the same products added in the same order)."""
    from tuna_amd import ops

    c = cfg(lds_tile_rows=256, token_tiles=16, split_k=split, rows_per_wave=mfma_rows)
    assert "gemm_wide_kernel" in ops.describe_launch(m, n, k, c)
    print(f"many-token tile 256x256 mfma_rows={mfma_rows} m={m} n={n} k={k} split={split}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=m + n + split)
    got = run_gemm(q, x, code, absmax, m, n, k, config=c, prefill=float("nan"))
    ref = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
    e = rel_err(f16_bits_to_f64(got), ref)
    assert e <= REL_TOL, e                                   # max relative error 1e-2
    again = run_gemm(q, x, code, absmax, m, n, k, config=c, prefill=float("nan"))
    assert np.array_equal(got, again)
    if split == 1:
        small = run_gemm(q, x, code, absmax, m, n, k, config=cfg(lds_tile_rows=128, token_tiles=8, rows_per_wave=mfma_rows),
                         prefill=float("nan"))
        assert np.array_equal(got, small)


@pytest.mark.parametrize("mfma_rows", [64, 32])
@pytest.mark.parametrize("m,n,k,split", [(256, 256, 200, 1), (520, 300, 1096, 1), (256, 70, 72, 1), (512, 257, 4104, 3),
                                         (264, 31, 8, 1), (256, 256, 120, 2)])
def test_the_256_x_256_tile_with_k_that_is_not_a_multiple_of_64(m, n, k, split, mfma_rows):
    """The last k-step of the 256 x 256 tile is partly beyond k (its variant for such k stores zeros for the
    activations of those slots): against the oracle, bit-equal to the 128 x 128 tile with the same MFMA shape, which
    masks its k tail the same way, and unchanged when NaNs follow x in memory (what lies beyond a token's k values -
    the next token's row, or whatever follows the last one - never enters a sum)."""
    import torch

    from tuna_amd import ops

    print(f"256 x 256 tile, k tail: m={m} n={n} k={k} split={split} mfma_rows={mfma_rows}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=m + n + k)
    c = cfg(lds_tile_rows=256, token_tiles=16, split_k=split, rows_per_wave=mfma_rows)
    assert "gemm_wide_kernel" in ops.describe_launch(m, n, k, c)
    got = run_gemm(q, x, code, absmax, m, n, k, config=c, prefill=float("nan"))
    ref = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
    assert not np.isnan(f16_bits_to_f64(got)).any()
    assert rel_err(f16_bits_to_f64(got), ref) <= REL_TOL
    if split == 1:
        other = run_gemm(q, x, code, absmax, m, n, k, config=cfg(lds_tile_rows=128, token_tiles=8, rows_per_wave=mfma_rows))
        assert np.array_equal(got, other)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    big_x = torch.full((n * k + 4096,), float("nan"), dtype=torch.float16, device="cuda")
    big_x[:n * k] = dx.reshape(-1)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul(big_x[:n * k].view(n, k), dq, da, dc, out, m, n, k, config=c)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), got)


def test_many_token_kernel_decode_readout_is_bit_exact():
    """One-hot activations turn the GEMM into a readout of the decoded weights: bit-exact D1."""
    m, k = 256, 256
    q, _, code, absmax = make_inputs_np(m, 16, k, seed=9)
    code = (np.random.default_rng(3).standard_normal(16)).astype(np.float32)
    x = np.zeros((k, k), dtype=np.float16)
    x[np.arange(k), np.arange(k)] = 1.0
    got = run_gemm(q, x, code, absmax, m, k, k, config=cfg(lds_tile_rows=128, token_tiles=8), prefill=float("nan"))
    want = O.dequant(q, absmax, code, m, k, mode=O.D1)          # [m, k] fp16 bits
    assert np.array_equal(got.T, want)
    got32 = run_gemm(q, x, code, absmax, m, k, k, config=cfg(lds_tile_rows=128, token_tiles=8, rows_per_wave=32), prefill=float("nan"))
    assert np.array_equal(got32.T, want)                        # 32 x 32 x 16 MFMA tiles: the same read-out
    for mfma_rows in (64, 32):                                  # the 256 x 256 tile, both MFMA shapes
        wide = run_gemm(q, x, code, absmax, m, k, k, config=cfg(lds_tile_rows=256, token_tiles=16, rows_per_wave=mfma_rows),
                        prefill=float("nan"))
        assert np.array_equal(wide.T, want)


# ----------------------------------------------------------------------------- stream capture / graph replay, several streams
def test_graph_replay_matches_eager_for_split_k_and_many_token_configs():
    """The ops are stream-ordered and capturable once their workspace exists: a captured graph
    of five GEMMs (fixed split-K, balanced split, many-token kernels with split-K, the streaming kernel's split twin) is replayed
    with new inputs written in place, with eager work and synchronisations in between, and
    every replay must give the bits of the eager call."""
    import torch

    from tuna_amd import ops

    m, n, k = 1024, 144, 2048
    cfgs = [cfg(split_k=4, x_chunk=512), cfg(split_k=0, waves_m=1, waves_k=8, prefetch=2, x_chunk=512),
            cfg(lds_tile_rows=128, token_tiles=8, split_k=2), cfg(lds_tile_rows=256, token_tiles=16, split_k=2),
            # the streaming kernel's twin with k split across workgroups (two token tiles, five token chunks)
            cfg(waves_m=2, waves_k=4, prefetch=2, x_chunk=256, token_tiles=2, split_k=4)]
    assert "gemm_mid_kernel" in ops.describe_launch(m, n, k, cfgs[-1]) and "split_k=4" in ops.describe_launch(m, n, k, cfgs[-1])
    q, x, code, absmax = make_inputs_np(m, n, k, seed=31)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    outs = [torch.zeros((n, m), dtype=torch.float16, device="cuda") for _ in cfgs]
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for c, o in zip(cfgs, outs):          # first call on this stream allocates the split-K workspace
            ops.matmul(dx, dq, da, dc, o, m, n, k, config=c)
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for c, o in zip(cfgs, outs):
                ops.matmul(dx, dq, da, dc, o, m, n, k, config=c)
    for rep in range(4):
        _, x2, _, _ = make_inputs_np(m, n, k, seed=100 + rep)
        dx.copy_(torch.from_numpy(x2).cuda())
        for o in outs:
            o.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        for c, g in zip(cfgs, got):
            eager = torch.zeros((n, m), dtype=torch.float16, device="cuda")
            ops.matmul(dx, dq, da, dc, eager, m, n, k, config=c)
            torch.cuda.synchronize()
            assert torch.equal(g.view(torch.int16), eager.view(torch.int16)), (rep, c.to_dict())


def test_two_streams_do_not_share_split_k_partial_sums():
    """Split-K GEMMs enqueued on two streams at once (each stream owns its workspace) give the
    same bits as run alone."""
    import torch

    from tuna_amd import ops

    m, n, k = 4096, 16, 4096
    c = cfg(waves_m=1, waves_k=8, prefetch=2, x_chunk=1024, split_k=4, xcd_swizzle=1)
    data = []
    for seed in (41, 42):
        q, x, code, absmax = make_inputs_np(m, n, k, seed=seed)
        data.append(to_dev(q, x, code, absmax))
    alone = []
    for dq, dx, dc, da in data:
        o = torch.zeros((n, m), dtype=torch.float16, device="cuda")
        ops.matmul(dx, dq, da, dc, o, m, n, k, config=c)
        torch.cuda.synchronize()
        alone.append(o)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [torch.zeros((n, m), dtype=torch.float16, device="cuda") for _ in range(2)]
    for _ in range(20):
        for st, (dq, dx, dc, da), o in zip(streams, data, outs):
            with torch.cuda.stream(st):
                ops.matmul(dx, dq, da, dc, o, m, n, k, config=c)
    torch.cuda.synchronize()
    for o, ref in zip(outs, alone):
        assert torch.equal(o.view(torch.int16), ref.view(torch.int16))


# ----------------------------------------------------------------------------- quantizer + packer on the device
@pytest.mark.parametrize("m,k", [(8, 8), (64, 256), (72, 1096), (4096, 4096)])
def test_device_quantizer_is_bit_exact(m, k):
    """tuna_quantize against the oracle's quantizer: packed bytes and scales identical, for the
    NF4 codebook and an arbitrary one, incl. all-zero rows, near-midpoint values, subnormals."""
    import torch

    from tuna_amd import ops

    rng = np.random.default_rng(m + k)
    from tuna_amd.quantize import NF4_CODE

    code = np.array(NF4_CODE, np.float32)
    w = (rng.standard_normal((m, k)) * 0.03).astype(np.float16)
    if m >= 8 and k >= 16:
        w[1] = 0
        w[2] = 0
        w[2, 5] = np.float16(-0.25)
        mids = ((code[:-1] + code[1:]) / 2).astype(np.float32)
        w[3, :15] = (mids * 0.5).astype(np.float16)
        w[3, 15] = np.float16(0.5)
        w[4] = np.float16(6e-8)
        w[4, 0] = np.float16(-1.2e-7)
    print(f"quantize m={m} k={k}", flush=True)
    for cb in (code, rng.standard_normal(16).astype(np.float32)):
        dw, dc = to_dev(w, cb)
        q, absmax, _ = ops.quantize(dw, dc)
        torch.cuda.synchronize()
        q_ref, a_ref = O.quantize(w.view(np.uint16), cb, m, k)
        assert np.array_equal(absmax.cpu().numpy(), a_ref)
        assert np.array_equal(q.cpu().numpy(), q_ref)


def test_quantize_then_matmul_end_to_end():
    """Real fp16 weights -> device quantizer -> GEMM, against the fp32 product of the
    dequantized weights (the reference harness's own flow, test.py:71-106)."""
    import torch

    from tuna_amd import ops

    m, n, k = 1024, 16, 2048
    rng = np.random.default_rng(12)
    w = (rng.standard_normal((m, k)) * 0.02).astype(np.float16)
    x = (rng.standard_normal((n, k)) * 0.1).astype(np.float16)
    dw, dx = to_dev(w, x)
    q, absmax, code = ops.quantize(dw)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul(dx, q, absmax, code, out, m, n, k)
    torch.cuda.synchronize()
    ref = O.gemm_f64(q.cpu().numpy(), x, code.cpu().numpy(), absmax.cpu().numpy(), m, n, k, mode=O.D1)
    e = rel_err(out.cpu().numpy().astype(np.float64), ref)
    assert e <= REL_TOL, e


# ----------------------------------------------------------------------------- fused epilogues
FUSED_CFGS = [
    dict(),                                                              # in-workgroup k split, direct store
    dict(split_k=3, x_chunk=512),                                        # cross-workgroup split: finishing workgroup stores
    dict(waves_m=8, waves_k=1, prefetch=2, x_chunk=64),                  # register-store epilogue
    dict(split_k=0, waves_m=1, waves_k=8, prefetch=2, x_chunk=512),      # balanced split
    dict(lds_tile_rows=128, token_tiles=8, split_k=1),                   # many-token kernel
    dict(lds_tile_rows=64, token_tiles=8, split_k=2),                    # many-token kernel, split-K
    dict(lds_tile_rows=256, token_tiles=16, split_k=1),                  # 256 x 256 tile
    dict(lds_tile_rows=256, token_tiles=16, split_k=2, rows_per_wave=32),  # 256 x 256 tile, 32 x 32 MFMA tiles, split-K
]


@pytest.mark.parametrize("ci", range(len(FUSED_CFGS)))
def test_fused_residual_and_silu_mul_epilogues(ci):
    """out = fp16(sum + residual) (also in place) and out = fp16(silu(gate) * up) on interleaved
    gate/up rows, against the oracle's float64 sums pushed through the same formulas."""
    import torch

    from tuna_amd import _lib, ops

    m, n, k = 1024, 48, 1096
    if FUSED_CFGS[ci].get("lds_tile_rows") == 256:
        k = 1088                                                         # that tile takes k in multiples of 64
    c = cfg(**FUSED_CFGS[ci])
    print(f"fused cfg#{ci} {c.to_dict()}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=60 + ci)
    rng = np.random.default_rng(ci)
    res = (rng.standard_normal((n, m)) * 0.05).astype(np.float16)
    ref = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
    dq, dx, dc, da, dres = to_dev(q, x, code, absmax, res)
    # residual, separate output
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_fused(dx, dq, da, dc, out, m, n, k, _lib.EPILOGUE_RESIDUAL, residual=dres, config=c)
    torch.cuda.synchronize()
    want = ref + res.astype(np.float64)
    assert rel_err(out.cpu().numpy().astype(np.float64), want) <= REL_TOL
    # residual in place: out is the residual
    inplace = dres.clone()
    ops.matmul_fused(dx, dq, da, dc, inplace, m, n, k, _lib.EPILOGUE_RESIDUAL, residual=inplace, config=c)
    torch.cuda.synchronize()
    assert torch.equal(inplace.view(torch.int16), out.view(torch.int16))
    # silu(gate) * up on interleaved rows
    out2 = torch.full((n, m // 2), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_fused(dx, dq, da, dc, out2, m, n, k, _lib.EPILOGUE_SILU_MUL, config=c)
    torch.cuda.synchronize()
    g, u = ref[:, 0::2], ref[:, 1::2]
    want2 = g / (1.0 + np.exp(-g)) * u
    # a product of two sums that are each within tolerance: relative to an output, the error of a
    # near-zero factor is amplified, so the floor of the metric is the wider one (5e-2 of the largest output)
    assert rel_err(out2.cpu().numpy().astype(np.float64), want2, floor=REL_FLOOR_D2) <= REL_TOL


# ----------------------------------------------------------------------------- lean kernel
LEAN_CASES = [
    # m, n, k, config: launches that qualify for the stripped-down kernel
    (1024, 16, 2048, dict(waves_m=2, waves_k=4, split_k=4, prefetch=2, x_chunk=512)),
    (512, 5, 4096, dict(waves_m=1, waves_k=8, split_k=2, prefetch=4, x_chunk=1024)),      # 8 pieces of x per thread
    (256, 16, 1024, dict(waves_m=4, waves_k=1, split_k=1, prefetch=2, x_chunk=64)),        # register-store epilogue
    (256, 40, 512, dict(waves_m=1, waves_k=2, split_k=1, prefetch=2, x_chunk=128)),        # three token chunks, ragged
    (1024, 16, 4096, dict(waves_m=1, waves_k=16, split_k=2, prefetch=2, x_chunk=2048)),    # 16 waves along k
    (512, 16, 8192, dict(waves_m=1, waves_k=8, split_k=8, prefetch=4, x_chunk=1024, xcd_swizzle=1)),
    (448, 1, 1024, dict(waves_m=7, waves_k=1, split_k=2, prefetch=8, x_chunk=256)),        # 7 waves, deepest ring
    (128, 16, 256, dict(waves_m=1, waves_k=4, split_k=1, prefetch=2, x_chunk=256)),        # one ring turn per wave
]


@pytest.mark.usefixtures("diagnostic_build")
@pytest.mark.parametrize("ci", range(len(LEAN_CASES)))
def test_lean_kernel_equals_general_kernel_bit_for_bit(ci):
    """Small aligned launches take a stripped-down kernel; it must give the bits of the general
    kernel with the same config (same decode, same summation order), for the plain store and both
    fused epilogues, and be within tolerance of the oracle."""
    import torch

    from tuna_amd import _lib, ops

    m, n, k, kw = LEAN_CASES[ci]
    c = cfg(**kw)
    print(f"lean case#{ci} {m}x{n}x{k} {c.to_dict()}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=80 + ci)
    res = (np.random.default_rng(ci).standard_normal((n, m)) * 0.05).astype(np.float16)
    dq, dx, dc, da, dres = to_dev(q, x, code, absmax, res)
    outs = {}
    prev = ops.set_lean_kernels(True)
    try:
        for lean in (True, False):
            ops.set_lean_kernels(lean)
            before = ops.lean_launches()
            o_plain = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
            o_res = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
            o_silu = torch.full((n, m // 2), float("nan"), dtype=torch.float16, device="cuda")
            ops.matmul(dx, dq, da, dc, o_plain, m, n, k, config=c)
            ops.matmul_fused(dx, dq, da, dc, o_res, m, n, k, _lib.EPILOGUE_RESIDUAL, residual=dres, config=c)
            ops.matmul_fused(dx, dq, da, dc, o_silu, m, n, k, _lib.EPILOGUE_SILU_MUL, config=c)
            torch.cuda.synchronize()
            assert ops.lean_launches() - before == (3 if lean else 0)   # the case really qualifies
            outs[lean] = (o_plain, o_res, o_silu)
    finally:
        ops.set_lean_kernels(prev)
    for a, b in zip(outs[True], outs[False]):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    ref = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
    assert rel_err(outs[True][0].cpu().numpy().astype(np.float64), ref) <= REL_TOL


# ----------------------------------------------------------------------------- 17..128-token streaming kernel
MID_CASES = [
    # m, n, k, config of the launch, config of the general-kernel launch it is compared with (None: the same)
    (512, 32, 512, dict(waves_m=8, waves_k=1, prefetch=2, token_tiles=2, x_chunk=256), None),
    (1024, 17, 1024, dict(waves_m=8, waves_k=1, prefetch=4, token_tiles=2, x_chunk=512), None),       # ragged second tile
    (2048, 30, 2048, dict(waves_m=8, waves_k=1, prefetch=8, token_tiles=2, x_chunk=512), None),
    (512, 64, 512, dict(waves_m=4, waves_k=1, prefetch=2, token_tiles=4, x_chunk=128), None),
    (1344, 100, 1024, dict(waves_m=7, waves_k=1, prefetch=2, token_tiles=2, x_chunk=256), None),      # 7 waves, 4 token chunks
    # ring depths and workgroup sizes only this kernel has: the general kernel with ring 2 (and 8 waves)
    # adds the same products in the same order
    (1536, 50, 2048, dict(waves_m=8, waves_k=1, prefetch=8, token_tiles=4, x_chunk=256),
     dict(waves_m=8, waves_k=1, prefetch=2, token_tiles=4, x_chunk=256)),
    (4096, 32, 1024, dict(waves_m=16, waves_k=1, prefetch=4, token_tiles=2, x_chunk=512),
     dict(waves_m=8, waves_k=1, prefetch=4, token_tiles=2, x_chunk=512)),
    # staggered k walk per row tile (wraps inside a chunk of x and inside a ring turn)
    (2048, 32, 2048, dict(waves_m=4, waves_k=1, prefetch=2, token_tiles=2, x_chunk=256, k_stagger=3), None),
    (1536, 64, 1024, dict(waves_m=2, waves_k=4, prefetch=2, token_tiles=4, x_chunk=256, k_stagger=5), None),
    (16640, 16, 1024, dict(waves_m=1, waves_k=2, prefetch=4, token_tiles=1, x_chunk=256, k_stagger=2), None),   # 260 tiles
    # one token tile (large shapes at up to 16 tokens; launches the lean kernel does not take: several tiles per CU)
    (33280, 16, 1024, dict(waves_m=2, waves_k=4, prefetch=2, token_tiles=1, x_chunk=1024), None),
    (38400, 9, 512, dict(waves_m=1, waves_k=1, prefetch=8, token_tiles=1, x_chunk=256), None),
    # eight token tiles (128 tokens per pass): a token's sums do not depend on the tile count
    (1024, 128, 1024, dict(waves_m=8, waves_k=1, prefetch=2, token_tiles=8, x_chunk=128),
     dict(waves_m=8, waves_k=1, prefetch=2, token_tiles=4, x_chunk=128)),
    (768, 200, 512, dict(waves_m=4, waves_k=2, prefetch=2, token_tiles=8, x_chunk=128),
     dict(waves_m=4, waves_k=2, prefetch=2, token_tiles=4, x_chunk=128)),                            # two passes, ragged
    # waves along k: summed through LDS in wave order, as in the general kernel
    (1024, 32, 1024, dict(waves_m=4, waves_k=2, prefetch=2, token_tiles=2, x_chunk=256), None),
    (1024, 33, 2048, dict(waves_m=2, waves_k=4, prefetch=2, token_tiles=4, x_chunk=256), None),
    (768, 40, 1024, dict(waves_m=3, waves_k=2, prefetch=4, token_tiles=2, x_chunk=256), None),       # 6 waves, 3 token chunks
    (512, 64, 4096, dict(waves_m=1, waves_k=8, prefetch=2, token_tiles=2, x_chunk=512), None),       # 8 waves along k
    # more row tiles than CUs: the workgroups walk (296 tiles of 256 rows), one chunk of x per tile
    (75776, 33, 256, dict(waves_m=4, waves_k=1, prefetch=2, token_tiles=4, x_chunk=128), None),
    (37888, 20, 512, dict(waves_m=2, waves_k=2, prefetch=2, token_tiles=2, x_chunk=128), None),      # the same with a reduction per tile
    # more (row tiles x token chunks) than CUs: walkers whose token chunks run side by side
    (19200, 40, 256, dict(waves_m=1, waves_k=2, prefetch=2, token_tiles=2, x_chunk=128), None),      # 300 tiles x 2 chunks
    (16640, 150, 256, dict(waves_m=2, waves_k=2, prefetch=2, token_tiles=2, x_chunk=128), None),     # 130 x 5, ragged last chunk
    (2048, 1100, 512, dict(waves_m=1, waves_k=4, prefetch=2, token_tiles=2, x_chunk=256), None),     # 32 x 35: more workgroups than CUs
    (51200, 300, 256, dict(waves_m=8, waves_k=1, prefetch=2, token_tiles=8, x_chunk=128),
     dict(waves_m=8, waves_k=1, prefetch=2, token_tiles=4, x_chunk=128)),                            # 100 x 3, eight token tiles
    # k split across workgroups: the parts of a row tile meet through the workspace, summed in k order
    (1024, 32, 4096, dict(waves_m=4, waves_k=2, prefetch=2, token_tiles=2, x_chunk=256, split_k=2), None),
    (1024, 33, 2048, dict(waves_m=2, waves_k=4, prefetch=2, token_tiles=4, x_chunk=256, split_k=4), None),   # two chunks per part, ragged
    (512, 64, 4096, dict(waves_m=1, waves_k=8, prefetch=2, token_tiles=2, x_chunk=512, split_k=8), None),    # one chunk per part, two token chunks
    (1024, 64, 2048, dict(waves_m=4, waves_k=1, prefetch=2, token_tiles=4, x_chunk=128, split_k=4), None),   # all waves along the rows
    (37888, 20, 512, dict(waves_m=2, waves_k=2, prefetch=2, token_tiles=2, x_chunk=128, split_k=2), None),   # 592 (tile, part) pairs: walkers
    (16640, 150, 256, dict(waves_m=2, waves_k=2, prefetch=2, token_tiles=2, x_chunk=128, split_k=2), None),  # 260 pairs x 5 token chunks side by side
    (2048, 100, 8192, dict(waves_m=2, waves_k=4, prefetch=2, token_tiles=4, x_chunk=256, split_k=16), None), # 16 parts: four round trips of four
]


@pytest.mark.usefixtures("diagnostic_build")
@pytest.mark.parametrize("ci", range(len(MID_CASES)))
def test_mid_token_kernel_equals_general_kernel_bit_for_bit(ci):
    """Dense launches with two, four or eight token tiles, unsplit or with k split into a power of two of
    equal parts, take the 17..128-token streaming kernel; it must give the bits of the general kernel (same
    decode, same summation order), for the plain store and both fused epilogues, and be within tolerance of
    the oracle."""
    import torch

    from tuna_amd import _lib, ops

    m, n, k, kw, kw_general = MID_CASES[ci]
    c, cg = cfg(**kw), cfg(**(kw_general or kw))
    print(f"mid case#{ci} {m}x{n}x{k} {c.to_dict()}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=180 + ci)
    res = (np.random.default_rng(ci).standard_normal((n, m)) * 0.05).astype(np.float16)
    dq, dx, dc, da, dres = to_dev(q, x, code, absmax, res)
    outs = {}
    prev = ops.set_lean_kernels(True)
    try:
        for twin in (True, False):
            ops.set_lean_kernels(twin)
            before = ops.lean_launches()
            o_plain = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
            o_res = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
            o_silu = torch.full((n, m // 2), float("nan"), dtype=torch.float16, device="cuda")
            cc = c if twin else cg
            ops.matmul(dx, dq, da, dc, o_plain, m, n, k, config=cc)
            ops.matmul_fused(dx, dq, da, dc, o_res, m, n, k, _lib.EPILOGUE_RESIDUAL, residual=dres, config=cc)
            ops.matmul_fused(dx, dq, da, dc, o_silu, m, n, k, _lib.EPILOGUE_SILU_MUL, config=cc)
            torch.cuda.synchronize()
            assert ops.lean_launches() - before == (3 if twin else 0)   # the case really qualifies
            outs[twin] = (o_plain, o_res, o_silu)
    finally:
        ops.set_lean_kernels(prev)
    for a, b in zip(outs[True], outs[False]):
        assert not torch.isnan(a.float()).any()
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    ref = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
    assert rel_err(outs[True][0].cpu().numpy().astype(np.float64), ref) <= REL_TOL   # max relative error 1e-2


LDS_PATH_CASES = [
    # m, n, k, waves_m, waves_k, prefetch, x_chunk, k_stagger
    (1024, 16, 4096, 16, 1, 4, 1024, 2),      # all waves along the rows (chunks of 512 k beside the rings)
    (2048, 16, 8192, 4, 4, 2, 1024, 2),       # waves along k: sums through LDS
    (512, 5, 2048, 2, 8, 2, 512, 0),
    (256 * 300, 16, 1024, 4, 4, 2, 1024, 3),  # more row tiles than compute units: workgroups that walk two tiles
    (1024 * 260, 3, 512, 16, 1, 2, 512, 1),
    # two, four and eight token tiles per pass (9th entry), 8 and 16 waves
    (512, 32, 4096, 2, 4, 4, 512, 1, 2),
    (2048, 27, 2048, 4, 4, 2, 512, 0, 2),      # 16 waves, ragged token count
    (1024, 40, 2048, 4, 2, 4, 256, 2, 4),
    (2048, 100, 1024, 8, 1, 2, 128, 0, 8),     # one pass of 128 tokens, 100 present
    (1024, 300, 1024, 4, 2, 2, 128, 3, 8),     # three token chunks
    (512 * 70, 1100, 512, 8, 1, 2, 128, 0, 8), # 70 row tiles x 9 token chunks: chunks of a walker side by side
    # k split across workgroups (10th entry)
    (1024, 64, 4096, 2, 4, 2, 256, 0, 4, 4),
    (2048, 32, 8192, 4, 4, 2, 512, 0, 2, 2),   # 16 waves
    (512 * 70, 40, 1024, 4, 2, 4, 256, 0, 2, 4),  # 140 row tiles x 4 parts: walkers
]


@pytest.mark.usefixtures("diagnostic_build")
@pytest.mark.gpu
@pytest.mark.parametrize("ci", range(len(LDS_PATH_CASES)))
def test_weights_staged_through_lds_equal_the_register_ring_bit_for_bit(ci):
    """The diagnostic switch that stages the packed weights (and x, and the scales) through LDS with
    global -> LDS loads runs the same arithmetic in the same order: equal bits, and the launch
    description says which path ran."""
    import torch

    from tuna_amd import ops

    m, n, k, wm, wk, pf, xc, st = LDS_PATH_CASES[ci][:8]
    tt = LDS_PATH_CASES[ci][8] if len(LDS_PATH_CASES[ci]) > 8 else 1
    split = LDS_PATH_CASES[ci][9] if len(LDS_PATH_CASES[ci]) > 9 else 1
    c = cfg(rows_per_wave=64, waves_m=wm, waves_k=wk, split_k=split, prefetch=pf, x_chunk=xc, k_stagger=st, token_tiles=tt)
    print(f"lds path case#{ci} {m}x{n}x{k} {c.to_dict()}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=700 + ci)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    c_lds = cfg(rows_per_wave=64, waves_m=wm, waves_k=wk, split_k=split, prefetch=pf, x_chunk=xc, k_stagger=st, token_tiles=tt,
                lds_tile_rows=-1)
    outs = {}
    prev = ops.set_weight_path(False)
    try:
        # the register ring, the diagnostic switch, and a config that asks for the LDS path itself
        for mode, (staged, cc) in {"registers": (False, c), "switch": (True, c), "config": (False, c_lds)}.items():
            ops.set_weight_path(staged)
            d = ops.describe_launch(m, n, k, cc)
            assert d.startswith("gemm_mid_kernel") and (("through LDS" in d) == (mode != "registers")), d
            o = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
            ops.matmul(dx, dq, da, dc, o, m, n, k, config=cc)
            ops.matmul(dx, dq, da, dc, o, m, n, k, config=cc)   # twice: the second launch finds LDS-independent state
            torch.cuda.synchronize()
            outs[mode] = o
    finally:
        ops.set_weight_path(prev)
    assert not torch.isnan(outs["switch"].float()).any()
    assert torch.equal(outs["switch"].view(torch.int16), outs["registers"].view(torch.int16))
    assert torch.equal(outs["config"].view(torch.int16), outs["registers"].view(torch.int16))
    outs = {True: outs["config"]}
    rows = np.random.default_rng(ci).choice(m, size=min(m, 256), replace=False).astype(np.int32)
    ref = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1, rows=rows)
    assert rel_err(outs[True].cpu().numpy().astype(np.float64)[:, rows], ref) <= REL_TOL   # max relative error 1e-2


# ----------------------------------------------------------------------------- narrow-row kernel
NARROW_CASES = [
    # m, n, k, rows_per_wave, waves_k, prefetch
    (256, 16, 1024, 16, 4, 2),
    (256, 5, 4096, 32, 16, 8),      # one ring turn per wave, 1024 threads
    (64, 40, 512, 32, 2, 2),        # three token chunks, the last one ragged
    (48, 1, 2048, 16, 8, 4),        # three workgroups of 16 rows, one token
    (512, 16, 8192, 32, 8, 4),
    (128, 16, 64, 16, 1, 2),        # a single wave: two passes over the row pairs
    (128, 33, 256, 32, 1, 2),
    (4096, 16, 4096, 16, 16, 2),    # full-size attention output projection, 256 workgroups
    (256, 16, 2048, 64, 8, 4),      # 64 rows per workgroup (waves_m = 0 selects the kernel)
    (192, 19, 1024, 64, 4, 8),
    (128, 7, 4096, 64, 16, 2),
    (6144, 16, 4096, 24, 8, 4),     # 24 rows per workgroup: a 32-row tile three quarters full, 256 workgroups
    (72, 3, 1024, 24, 8, 2),        # three such workgroups, the last block row of the matrix in the last one
    (240, 11, 2048, 24, 16, 4),
    # two and four 16-token tiles per workgroup (7th entry: token_tiles)
    (256, 32, 1024, 32, 8, 2, 2),
    (128, 50, 2048, 16, 4, 4, 4),   # 64 tokens per chunk, 50 present
    (256, 100, 512, 64, 4, 2, 2),   # four chunks of 32, the last one ragged
    (96, 64, 4096, 32, 8, 4, 4),
]


def narrow_cfg(rows, wk, pf, tt=1):
    return cfg(rows_per_wave=rows, waves_m=0 if rows == 64 else 1, waves_k=wk, split_k=1, prefetch=pf, x_chunk=32 * wk * pf,
               token_tiles=tt)


@pytest.mark.parametrize("ci", range(len(NARROW_CASES)))
def test_narrow_row_kernel_matches_oracle(ci):
    """rows_per_wave 16 / 32 selects the kernel with one workgroup per 16 / 32 weight rows and no
    split across workgroups: plain store and both fused epilogues against the oracle's float64
    sums, the rows outside the result untouched (NaN prefill)."""
    import torch

    from tuna_amd import _lib, ops

    m, n, k, rows, wk, pf = NARROW_CASES[ci][:6]
    c = narrow_cfg(rows, wk, pf, *NARROW_CASES[ci][6:])
    print(f"narrow case#{ci} {m}x{n}x{k} {c.to_dict()}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=90 + ci)
    res = (np.random.default_rng(ci).standard_normal((n, m)) * 0.05).astype(np.float16)
    ref = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
    dq, dx, dc, da, dres = to_dev(q, x, code, absmax, res)
    pad = torch.full((n + 2, m), float("nan"), dtype=torch.float16, device="cuda")   # a guard row on either side
    out = pad[1:n + 1]
    ops.matmul(dx, dq, da, dc, out, m, n, k, config=c)
    o_res = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    o_silu = torch.full((n, m // 2), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_fused(dx, dq, da, dc, o_res, m, n, k, _lib.EPILOGUE_RESIDUAL, residual=dres, config=c)
    ops.matmul_fused(dx, dq, da, dc, o_silu, m, n, k, _lib.EPILOGUE_SILU_MUL, config=c)
    torch.cuda.synchronize()
    assert rel_err(out.cpu().numpy().astype(np.float64), ref) <= REL_TOL
    assert torch.isnan(pad[0]).all() and torch.isnan(pad[n + 1]).all()
    assert rel_err(o_res.cpu().numpy().astype(np.float64), ref + res.astype(np.float64)) <= REL_TOL
    g, u = ref[:, 0::2], ref[:, 1::2]
    assert rel_err(o_silu.cpu().numpy().astype(np.float64), g / (1.0 + np.exp(-g)) * u, floor=REL_FLOOR_D2) <= REL_TOL
    # repeatable bit for bit
    again = torch.empty((n, m), dtype=torch.float16, device="cuda")
    ops.matmul(dx, dq, da, dc, again, m, n, k, config=c)
    torch.cuda.synchronize()
    assert torch.equal(again.view(torch.int16), out.view(torch.int16))


@pytest.mark.parametrize("rows,wk,pf", [(16, 4, 2), (32, 8, 4), (32, 16, 2), (64, 8, 2), (24, 8, 8)])
def test_narrow_row_kernel_decode_readout_is_bit_exact(rows, wk, pf):
    """One-hot activations read the narrow-row kernel's in-register decode out: the oracle's D1 image."""
    m, k = (264 if rows == 24 else 256), 2048
    q, _, code, absmax = make_inputs_np(m, 16, k, seed=rows + wk)
    want_img = O.dequant(q, absmax, code, m, k, mode=O.D1)
    cols = np.random.default_rng(wk).choice(k, size=16, replace=False)
    x = np.zeros((16, k), np.float16)
    x[np.arange(16), cols] = 1.0
    got = run_gemm(q, x, code, absmax, m, 16, k, config=narrow_cfg(rows, wk, pf))
    assert np.array_equal(f16_bits_to_f64(got), f16_bits_to_f64(want_img[:, cols].T))


def test_narrow_row_configs_that_do_not_fit_are_rejected():
    from tuna_amd import ops

    q, x, code, absmax = make_inputs_np(256, 16, 1024, seed=1)
    for m, k, kw in [(264, 1024, dict()),                       # m not a multiple of the rows
                     (256, 1000, dict()),                       # k not a multiple of 32 * waves_k * prefetch
                     (256, 1024, dict(split_k=2)), (256, 1024, dict(waves_m=2)), (256, 1024, dict(token_tiles=3))]:
        c = cfg(**{**dict(rows_per_wave=16, waves_m=1, waves_k=4, split_k=1, prefetch=2, x_chunk=256, token_tiles=1), **kw})
        with pytest.raises(ops.TunaError):
            ops.validate_config(m, 16, k, c)


# ----------------------------------------------------------------------------- golden fixtures on the device
def test_golden_fixtures_through_the_device_path():
    """The committed fixtures (tests/golden/*.npz: packed bytes, scales, activations and the
    expected fp16 bits) through tuna_dequant and tuna_matmul: dequant bit-exact in both
    roundings, the GEMM within one fp16 rounding of the stored D1 result."""
    import os

    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    cb = O.nf4_codebook()
    blk = np.load(os.path.join(golden, "block_64x128.npz"))
    assert np.array_equal(run_dequant(blk["q"], cb, blk["absmax"], 64, 128, decode_mode=O.D1), blk["image_d1"])
    assert np.array_equal(run_dequant(blk["q"], cb, blk["absmax"], 64, 128, decode_mode=O.D2), blk["image_d2"])
    gm = np.load(os.path.join(golden, "gemm_256x16x128.npz"))
    got = run_gemm(gm["q"], gm["x"].view(np.float16), cb, gm["absmax"], 256, 16, 128, prefill=float("nan"))
    # (the fixture is the float64 sum rounded once; fp32 accumulation moves a few results by an ulp)
    assert rel_err(f16_bits_to_f64(got), f16_bits_to_f64(gm["out_d1"])) <= REL_TOL
    assert (got == gm["out_d1"]).mean() > 0.95
    got2 = run_gemm(gm["q"], gm["x"].view(np.float16), cb, gm["absmax"], 256, 16, 128, decode_mode=O.D2, prefill=float("nan"))
    assert rel_err(f16_bits_to_f64(got2), f16_bits_to_f64(gm["out_d2"])) <= REL_TOL
    assert (got2 == gm["out_d2"]).mean() > 0.95


def test_grouped_gemm_on_a_tuned_shape_with_the_librarys_config():
    """Mixtral down projection, all 8 experts active with 4 tokens each, config chosen by the
    library (the tuned entry of the stacked shape is a narrow-row config, which grouped launches
    cannot run: they must fall back instead of patching it)."""
    m_group, n_groups, k = 4096, 8, 14336
    offsets = [4 * e for e in range(n_groups + 1)]
    q, x, code, absmax = make_inputs_np(m_group * n_groups, offsets[-1], k, seed=9)
    got = _run_grouped(q, x, code, absmax, m_group, n_groups, k, offsets, None)
    assert not np.isnan(f16_bits_to_f64(got)).any()
    rng = np.random.default_rng(2)
    rows = np.sort(rng.choice(m_group, size=128, replace=False)).astype(np.int32)
    qb = q.reshape(n_groups, m_group // 8, k // 8, 32)
    for e in range(n_groups):
        ref = O.gemm_f64(np.ascontiguousarray(qb[e]), np.ascontiguousarray(x[4 * e:4 * e + 4]).view(np.uint16), code,
                         np.ascontiguousarray(absmax[e * m_group:(e + 1) * m_group]), m_group, 4, k, mode=O.D1, rows=rows)
        err = rel_err(f16_bits_to_f64(got[4 * e:4 * e + 4][:, rows]), ref)
        assert err <= REL_TOL, (e, err)


def test_captured_graph_survives_growth_of_the_split_k_workspace():
    """A graph captured on a stream keeps the workspace pointers of its split-K launches.  A later,
    larger request on the same stream must not free or move that buffer: the replay after the
    growth gives the bits of the eager call."""
    import torch

    from tuna_amd import ops

    m, n, k = 1024, 16, 2048
    small = cfg(split_k=4, x_chunk=512)
    # balanced split over 129 token chunks: 129 x 64 workgroups x 2 slots x 4 KB = 66 MB of partial sums
    big_n = 16 * 129
    big = cfg(split_k=0, waves_m=1, waves_k=8, prefetch=2, x_chunk=512)
    assert ops.config_footprint(m, big_n, k, big)[1] > 64 << 20 > ops.config_footprint(m, n, k, small)[1] > 0
    q, x, code, absmax = make_inputs_np(m, n, k, seed=61)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    out = torch.zeros((n, m), dtype=torch.float16, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        ops.matmul(dx, dq, da, dc, out, m, n, k, config=small)   # first use on this stream: workspace allocated
        side.synchronize()
        eager = out.clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            ops.matmul(dx, dq, da, dc, out, m, n, k, config=small)
        xb = torch.zeros((big_n, k), dtype=torch.float16, device="cuda")
        xb[:n] = dx
        ob = torch.zeros((big_n, m), dtype=torch.float16, device="cuda")
        ops.matmul(xb, dq, da, dc, ob, m, big_n, k, config=big)  # needs a larger workspace: the old one must stay
        side.synchronize()
    assert torch.equal(ob[:n].view(torch.int16), eager.view(torch.int16)) or rel_err(
        ob[:n].float().cpu().numpy(), eager.float().cpu().numpy()) <= REL_TOL
    for _ in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16))


# ----------------------------------------------------------------------------- several GEMMs in one call
@pytest.mark.parametrize("shapes", [
    [(4096, 16, 4096), (6144, 16, 4096), (4096, 16, 14336), (1024, 5, 2048), (8192, 1, 8192)],   # row tiles of 256, k of 512 ... 14336
    [(10240, 16, 8192), (8192, 16, 8192), (57344, 16, 8192), (8192, 16, 28672)],                   # a Llama-70B layer
    [(128, 16, 1024), (640, 3, 512), (384, 16, 2560)],                                             # 128-row tiles, short k, ragged shares
    [(8192, 16, 28672)],                                                                           # a batch of one
])
@pytest.mark.usefixtures("diagnostic_build")
def test_matmul_multi_with_weights_through_lds_gives_the_register_paths_bits(shapes):
    """The batched kernel's twin that stages packed weights and x through LDS (global -> LDS loads, x
    chunks of 512 k) adds the same products in the same order: equal bits, on batches that exercise
    whole and partial row tiles, segment switches across problems and the deferred hand-over."""
    import torch

    from tuna_amd import _lib

    L = _lib.lib()
    probs, host = _multi_problems(shapes, 900)
    outs = {}
    prev_min = L.tuna_set_multi_min_batch(1)
    prev = L.tuna_set_multi_weight_path(0)
    L.tuna_set_multi_shape(0, 2)              # the LDS twin exists for the ring of two
    try:
        from tuna_amd import ops
        for lds in (0, 1):
            L.tuna_set_multi_weight_path(lds)
            for rep in range(2):
                for p in probs:
                    p[4].fill_(float("nan"))
                before = L.tuna_multi_launches()
                ops.matmul_multi(probs)
                torch.cuda.synchronize()
                assert L.tuna_multi_launches() == before + 1
            outs[lds] = [p[4].clone() for p in probs]
    finally:
        L.tuna_set_multi_weight_path(prev)
        L.tuna_set_multi_min_batch(prev_min)
        L.tuna_set_multi_shape(0, 0)
    for i, (a, b) in enumerate(zip(outs[0], outs[1])):
        assert not torch.isnan(b.float()).any(), i
        assert torch.equal(a.view(torch.int16), b.view(torch.int16)), i
    m, n, k = shapes[0]
    assert _check_against_oracle(host[0], outs[1][0].cpu().numpy().view(np.uint16), m, n, k, seed=1) <= REL_TOL   # max relative error 1e-2


def _multi_problems(shapes, seed0):
    import torch

    probs, host = [], []
    dc = None
    for i, (m, n, k) in enumerate(shapes):
        q, x, code, absmax = make_inputs_np(m, n, k, seed=seed0 + i)
        dq, dx, dc_i, da = to_dev(q, x, code, absmax)
        dc = dc_i if dc is None else dc       # one codebook tensor for the batch (one decode table per launch)
        out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
        probs.append((dx, dq, da, dc, out, m, n, k))
        host.append((q, x, code, absmax))
    return probs, host


def _check_against_oracle(host, got_bits, m, n, k, seed, n_rows=256):
    q, x, code, absmax = host
    rng = np.random.default_rng(seed)
    rows = np.sort(rng.choice(m, size=min(n_rows, m), replace=False)).astype(np.int32)
    ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1, rows=rows)
    return rel_err(f16_bits_to_f64(got_bits[:, rows]), ref)


@pytest.mark.usefixtures("diagnostic_build")
def test_matmul_multi_matches_the_oracle_and_separate_calls():
    """tuna_matmul_multi on a mixed batch: five problems that the batched persistent kernel takes
    in one launch (1..16 tokens, tuned and untuned shapes, k up to 14336), one it cannot take
    (40 tokens, ragged sizes) and one more behind it.  Every output is checked against the oracle
    (row subset), agrees with a separate tuna_matmul call within the same tolerance (the batched
    kernel sums in another order), and a second call gives the same bits again."""
    import torch

    from tuna_amd import _lib, ops

    shapes = [(4096, 16, 4096), (6144, 16, 4096), (4096, 16, 14336), (1024, 5, 2048), (8192, 1, 8192), (520, 40, 1096),
              (10240, 16, 8192)]
    probs, host = _multi_problems(shapes, 300)
    want = []
    for (dx, dq, da, dc, _o, m, n, k) in probs:
        o = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
        ops.matmul(dx, dq, da, dc, o, m, n, k)
        want.append(o)
    torch.cuda.synchronize()
    first = None
    for rep in range(2):
        for p in probs:
            p[4].fill_(float("nan"))
        before = _lib.lib().tuna_multi_launches()
        ops.matmul_multi(probs)
        torch.cuda.synchronize()
        assert _lib.lib().tuna_multi_launches() == before + 1          # problems 0..4 in one launch, the rest one by one
        got = [p[4].cpu().numpy().view(np.uint16).copy() for p in probs]
        for i, ((m, n, k), g, w) in enumerate(zip(shapes, got, want)):
            assert not np.isnan(g.view(np.float16)).any(), (rep, i)
            e = _check_against_oracle(host[i], g, m, n, k, seed=i)
            print(f"  multi problem {i} {m}x{n}x{k}: rel_err={e:.3e}", flush=True)
            assert e <= REL_TOL, (rep, i, e)
            assert rel_err(f16_bits_to_f64(g), w.float().cpu().numpy().astype(np.float64)) <= REL_TOL
        for i in (5, 6):                                               # launched as tuna_matmul would: identical bits
            assert np.array_equal(got[i], want[i].cpu().numpy().view(np.uint16))
        if first is None:
            first = got
        else:
            assert all(np.array_equal(a, b) for a, b in zip(first, got))   # deterministic
    ops.matmul_multi([])                      # an empty batch is a no-op
    ops.matmul_multi(probs[:1])               # a batch of one is a plain call
    torch.cuda.synchronize()
    assert torch.equal(probs[0][4].view(torch.int16), want[0].view(torch.int16))


@pytest.mark.usefixtures("diagnostic_build")
@pytest.mark.parametrize("waves_m,prefetch", [(4, 2), (4, 4), (2, 2), (2, 4), (8, 2), (8, 4), (1, 2), (16, 2)])
def test_matmul_multi_every_workgroup_shape_and_decode_readout(waves_m, prefetch):
    """The batched kernel with every workgroup shape it has (waves along rows x ring depth): oracle
    check on a batch whose shares cut row tiles at many places, and the one-hot read-out of the
    in-register decode (bit-exact whatever the split, since every partial sum but one is zero)."""
    import torch

    from tuna_amd import _lib, ops

    L = _lib.lib()
    shapes = [(2048, 16, 4096), (1024, 7, 8192), (3072, 16, 2048), (1024, 1, 4096)]
    probs, host = _multi_problems(shapes, 330)
    L.tuna_set_multi_shape(waves_m, prefetch)
    try:
        before = L.tuna_multi_launches()
        ops.matmul_multi(probs)
        torch.cuda.synchronize()
        assert L.tuna_multi_launches() == before + 1
        for i, (m, n, k) in enumerate(shapes):
            g = probs[i][4].cpu().numpy().view(np.uint16)
            assert not np.isnan(g.view(np.float16)).any()
            e = _check_against_oracle(host[i], g, m, n, k, seed=i, n_rows=128)
            assert e <= REL_TOL, (i, e)
        # one-hot activations: out[t, r] must be the decoded weight W[r, col_t], bit for bit
        rng = np.random.default_rng(5)
        for i, (m, n, k) in enumerate(shapes):
            cols = rng.choice(k, size=n, replace=False)
            xh = np.zeros((n, k), np.float16)
            xh[np.arange(n), cols] = 1.0
            probs[i][0].copy_(torch.from_numpy(xh).cuda())
            probs[i][4].fill_(float("nan"))
        ops.matmul_multi(probs)
        torch.cuda.synchronize()
        rng = np.random.default_rng(5)
        for i, (m, n, k) in enumerate(shapes):
            cols = rng.choice(k, size=n, replace=False)
            q, _x, code, absmax = host[i]
            img = O.dequant(q, absmax, code, m, k, mode=O.D1)
            assert np.array_equal(probs[i][4].cpu().numpy().view(np.uint16), img[:, cols].T), i
    finally:
        L.tuna_set_multi_shape(0, 0)


def test_matmul_multi_checks_every_problem_before_launching_any():
    import torch

    from tuna_amd import ops

    probs, _ = _multi_problems([(512, 16, 1024), (256, 16, 512)], 310)
    bad = list(probs[1])
    bad[5] = 260                              # m not a multiple of 8: caught by the library, not by the wrapper
    arr = ops.problem_array(probs)
    arr[1].m = 260
    from tuna_amd import _lib

    rc = _lib.lib().tuna_matmul_multi(arr, 2, None)
    assert rc == _lib.ERR_INVALID_ARG
    torch.cuda.synchronize()
    assert torch.isnan(probs[0][4]).all()     # nothing ran


def test_matmul_multi_in_a_captured_graph_replays_correctly():
    """A captured tuna_matmul_multi call replayed several times with fresh activations, eager work
    in between: every replay equals the eager call (the batched kernel's workspace and counters
    are those of the capture stream, allocated by the eager call before the capture)."""
    import torch

    from tuna_amd import ops

    shapes = [(4096, 16, 4096), (1024, 16, 2048), (4096, 16, 14336), (2048, 16, 1024), (8192, 16, 8192)]
    probs, _ = _multi_problems(shapes, 320)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        ops.matmul_multi(probs)               # eager once: the stream's workspace exists afterwards
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            ops.matmul_multi(probs)
    for rep in range(3):
        for i, p in enumerate(probs):
            _, x2, _, _ = make_inputs_np(p[5], p[6], p[7], seed=900 + 10 * rep + i)
            p[0].copy_(torch.from_numpy(x2).cuda())
            p[4].fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [p[4].clone() for p in probs]
        for p in probs:
            p[4].fill_(float("nan"))
        ops.matmul_multi(probs)               # the same batch eagerly: identical bits
        torch.cuda.synchronize()
        for p, g in zip(probs, got):
            assert not torch.isnan(g).any()
            assert torch.equal(g.view(torch.int16), p[4].view(torch.int16)), rep


@pytest.mark.parametrize("m,n,k,ckw", [
    (1024, 16, 2048, dict(waves_m=4, waves_k=4, prefetch=2, x_chunk=512)),
    (2048, 7, 4096, dict(waves_m=4, waves_k=4, prefetch=4, x_chunk=1024)),
    (1024, 16, 8192, dict(waves_m=2, waves_k=8, prefetch=2, x_chunk=512)),
    (4096, 1, 2048, dict(waves_m=8, waves_k=2, prefetch=4, x_chunk=256)),
    (3072, 16, 14336, dict(waves_m=1, waves_k=16, prefetch=2, x_chunk=1024)),
])
@pytest.mark.usefixtures("diagnostic_build")
def test_balanced_split_through_the_batched_kernel_equals_general_kernel_bit_for_bit(m, n, k, ckw):
    """A balanced split over 16-wave workgroups is run by the batched kernel as a batch of one.  It
    walks the segments gemm_kernel's balanced split walks, in the same order, and sums in the same
    order: identical bits (the general kernel is reached with the twins switched off), and both agree
    with the oracle."""
    import torch

    from tuna_amd import _lib, ops

    c = cfg(split_k=0, **ckw)
    assert ops.describe_launch(m, n, k, c).startswith("gemm_multi_kernel")
    q, x, code, absmax = make_inputs_np(m, n, k, seed=m + k)
    before = _lib.lib().tuna_multi_launches()
    got = run_gemm(q, x, code, absmax, m, n, k, config=c, prefill=float("nan"))
    assert _lib.lib().tuna_multi_launches() == before + 1
    prev = ops.set_lean_kernels(False)
    try:
        assert ops.describe_launch(m, n, k, c).startswith("gemm_kernel")
        general = run_gemm(q, x, code, absmax, m, n, k, config=c, prefill=float("nan"))
    finally:
        ops.set_lean_kernels(prev)
    assert np.array_equal(got, general)
    ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1)
    assert rel_err(f16_bits_to_f64(got), ref) <= REL_TOL


# ----------------------------------------------------------------------------- scale blocks finer than a row
@pytest.mark.parametrize("m,k,bs", [(8, 64, 8), (64, 256, 64), (72, 1152, 128), (136, 1032, 24), (4096, 4096, 64), (4096, 4096, 128)])
@pytest.mark.parametrize("mode", [O.D2, O.D1])
def test_blockwise_dequant_bit_exact(m, k, bs, mode):
    import torch

    from tuna_amd import ops

    rng = np.random.default_rng(m + k + bs)
    q = rng.integers(0, 256, size=(m // 8, k // 8, 32), dtype=np.uint8)
    code = O.nf4_codebook()
    absmax = rng.uniform(0.004, 0.03, size=(m, k // bs)).astype(np.float32)
    dq, dc, da = to_dev(q, code, absmax)
    out = torch.full((m, k), float("nan"), dtype=torch.float16, device="cuda")
    ops.dequant(dq, da, dc, out, m, k, decode_mode=mode, block_size=bs)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), O.dequant(q, absmax, code, m, k, mode=mode, block_size=bs))


@pytest.mark.parametrize("m,k,bs", [(8, 64, 8), (64, 256, 64), (72, 1096, None), (72, 1024, 128), (4096, 4096, 64), (4096, 4096, 128),
                                    (4096, 4096, None), (512, 8192, None), (64, 14336, 256), (256, 14336, None)])
def test_device_quantizer_blockwise_and_every_row_length_is_bit_exact(m, k, bs):
    """The rewritten quantizer kernel (rows held in registers up to k = 4096, two passes beyond; block
    maxima by shuffles; binary search for sorted codebooks) against the oracle: packed bytes and
    scales identical, for per-row and per-block scales, incl. zero rows / blocks, near-midpoint
    inputs, fp16 subnormals, and an unsorted codebook (the 16-comparison path)."""
    import torch

    from tuna_amd import ops

    rng = np.random.default_rng(m * 7 + k + (bs or 0))
    w = (rng.standard_normal((m, k)) * 0.03).astype(np.float16)
    code = O.nf4_codebook()
    w[1] = 0
    w[2, :] = 0
    w[2, 5] = np.float16(-0.25)
    mids = ((code[:-1] + code[1:]) / 2).astype(np.float32)
    w[3, :15] = (mids * 0.5).astype(np.float16)
    w[3, 15] = np.float16(0.5)
    w[4] = np.float16(6e-8)
    if bs:
        w[5, bs:2 * bs] = 0
    for cb in (code, rng.standard_normal(16).astype(np.float32), np.sort(rng.standard_normal(16)).astype(np.float32)):
        dw, dc = to_dev(w, cb)
        q, a, _ = ops.quantize(dw, dc, block_size=bs)
        torch.cuda.synchronize()
        q_ref, a_ref = O.quantize(w.view(np.uint16), cb, m, k, block_size=bs)
        assert np.array_equal(a.cpu().numpy(), a_ref)
        assert np.array_equal(q.cpu().numpy(), q_ref)


@pytest.mark.parametrize("m,n,k,bs", [(64, 16, 256, 64), (256, 5, 1024, 128), (1024, 16, 4096, 64), (512, 37, 2048, 256),
                                      (4096, 16, 4096, 128), (2048, 1, 8192, 64)])
def test_blockwise_gemm_matches_oracle_and_reads_out_the_decode(m, n, k, bs):
    """tuna_matmul_blockwise: one scale per `bs` weights of a row.  Against the oracle's float64 sums
    over the blockwise D1 weights, and bit-exact through one-hot activations (out[t, r] = the decoded
    weight W[r, col_t] with its block's scale)."""
    import torch

    from tuna_amd import ops

    rng = np.random.default_rng(m + n + k + bs)
    q, x, code, _ = make_inputs_np(m, n, k, seed=m + bs)
    absmax = rng.uniform(0.005, 0.02, size=(m, k // bs)).astype(np.float16).astype(np.float32)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_blockwise(dx, dq, da, dc, out, m, n, k, bs)
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(np.uint16)
    assert not np.isnan(got.view(np.float16)).any()
    rows = np.sort(rng.choice(m, size=min(m, 256), replace=False)).astype(np.int32)
    ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1, rows=rows, block_size=bs)
    e = rel_err(f16_bits_to_f64(got[:, rows]), ref)
    assert e <= REL_TOL, e
    cols = rng.choice(k, size=n, replace=False)
    xh = np.zeros((n, k), np.float16)
    xh[np.arange(n), cols] = 1.0
    dxh, = to_dev(xh)
    ops.matmul_blockwise(dxh, dq, da, dc, out, m, n, k, bs)
    torch.cuda.synchronize()
    img = O.dequant(q, absmax, code, m, k, mode=O.D1, block_size=bs)
    assert np.array_equal(out.cpu().numpy().view(np.uint16), img[:, cols].T)


def blockwise_cfg(family, m, n, k, bs, shape=None):
    """An explicit config that sends a blockwise launch to one kernel family (the rule of tuna_matmul_blockwise_ex):
    "narrow" with shape = (rows, waves along k, ring) or the first variant that fits, "batched" with the tallest row
    tile the shape allows, "streaming" with four waves by four (eight waves for four token tiles)."""
    from tuna_amd import ops

    tiles = 4 if n > 32 else 2 if n > 16 else 1
    cands = []
    if family == "narrow":
        shapes = [shape] if shape else [(64, 8, 4), (64, 8, 2), (32, 8, 4), (32, 8, 2), (16, 8, 4), (16, 4, 2)]
        for rows, wk, u in shapes:
            for tt in ((2, 1) if n > 16 else (1,)):
                cands.append(cfg(rows_per_wave=rows, waves_m=0 if rows == 64 else 1, waves_k=wk, split_k=1, prefetch=u, x_chunk=512,
                                 token_tiles=tt))
    elif family == "batched":
        for wm in (4, 2, 1):
            cands.append(cfg(rows_per_wave=64, waves_m=wm, waves_k=16 // wm, split_k=0, prefetch=2, x_chunk=512, token_tiles=1))
    elif family == "many-token":
        rows, tok = (128, 16 if n > 128 else 8) if n > 64 else (256, 4)
        tiles_n = -(-m // rows) * -(-n // (16 * tok))
        split = max(1, min(256 // max(1, tiles_n), (k // 64) // 8))
        cands.append(cfg(rows_per_wave=64, waves_m=1, waves_k=1, split_k=split, prefetch=2, x_chunk=64, token_tiles=tok, lds_tile_rows=rows))
    elif family == "streaming":
        wm = 4 if m % 256 == 0 else 2 if m % 128 == 0 else 1
        wk = min(8, (8 if tiles == 4 else 16) // wm)
        cands.append(cfg(rows_per_wave=64, waves_m=wm, waves_k=wk, split_k=1, prefetch=2, x_chunk=256 if tiles == 4 else 512,
                         token_tiles=tiles))
    for c in cands:
        try:
            ops.validate_config_blockwise(m, n, k, bs, c)
            return c
        except ops.TunaError:
            continue
    raise AssertionError(f"no {family} blockwise config for m={m} n={n} k={k} block={bs} shape={shape}")



@pytest.mark.parametrize("m,n,k,bs,shape", [
    (256, 16, 28672, 64, None),          # 16-row tiles, 7168 scales per workgroup: two rounds of the prologue copy
    (1024, 16, 8192, 64, (64, 8, 4)),    # 64-row tiles, 8192 scales: two rounds
    (1024, 5, 4096, 64, (64, 8, 2)),     # exactly one full round
    (512, 37, 2048, 128, (32, 8, 4)),    # three token chunks, ragged last
    (512, 1, 4096, 512, (32, 16, 2)),    # few long blocks
    (256, 16, 1536, 64, (16, 4, 2)),     # k range of three ring turns
    (128, 9, 28672, 64, (64, 8, 4)),     # 64 rows x 449 floats do not fit beside the table: scales stay in memory
    (2560, 16, 10240, 64, None),         # 160 tiles of 16 rows
    (1024, 32, 4096, 64, (64, 8, 4)),    # two token tiles per workgroup, 64 rows
    (512, 23, 2048, 64, (32, 8, 2)),     # two token tiles, the second ragged
    (256, 70, 1024, 128, (16, 4, 2)),    # three passes of two token tiles, the last with one
    (768, 32, 8192, 64, None),           # two token tiles, the library's choice of rows
    (256, 32, 28672, 64, (64, 8, 4)),    # two token tiles, scales in memory (they do not fit in LDS)
])
@pytest.mark.usefixtures("diagnostic_build")
def test_blockwise_narrow_kernel_with_scales_in_lds_and_in_memory(m, n, k, bs, shape):
    """The narrow-row kernel's scale-block variants stage the workgroup's scales in LDS when they fit and read them
    from memory per ring slot when they do not (or when the switch says so): both orders of reading the same scales
    give identical bits, match the oracle's float64 sums, and read the decoded weights out exactly."""
    import torch

    from tuna_amd import _lib, ops

    rng = np.random.default_rng(m + n + k + bs + 2)
    q, x, code, _ = make_inputs_np(m, n, k, seed=m + bs + 2)
    absmax = rng.uniform(0.005, 0.02, size=(m, k // bs)).astype(np.float16).astype(np.float32)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    L = _lib.lib()
    prev_lds = L.tuna_set_blockwise_scales_lds(1)
    c = blockwise_cfg("narrow", m, n, k, bs, shape)
    before = L.tuna_blockwise_launches(0)
    try:
        print(f"blockwise narrow rows m={m} n={n} k={k} block={bs} variant={shape} cfg={c.to_dict()}", flush=True)
        cols = rng.choice(k, size=n, replace=False)
        xh = np.zeros((n, k), np.float16)
        xh[np.arange(n), cols] = 1.0
        dxh, = to_dev(xh)
        img = O.dequant(q, absmax, code, m, k, mode=O.D1, block_size=bs)
        got = {}
        for lds in (1, 0):
            L.tuna_set_blockwise_scales_lds(lds)
            out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
            ops.matmul_blockwise(dx, dq, da, dc, out, m, n, k, bs, config=c)
            torch.cuda.synchronize()
            got[lds] = out.cpu().numpy().view(np.uint16)
            ops.matmul_blockwise(dxh, dq, da, dc, out, m, n, k, bs, config=c)
            torch.cuda.synchronize()
            assert np.array_equal(out.cpu().numpy().view(np.uint16), img[:, cols].T), lds
        assert L.tuna_blockwise_launches(0) == before + 4          # the narrow-row kernel ran all four
        assert not np.isnan(got[1].view(np.float16)).any()
        assert np.array_equal(got[1], got[0])
        rows = np.sort(rng.choice(m, size=min(m, 128), replace=False)).astype(np.int32)
        ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1, rows=rows, block_size=bs)
        e = rel_err(f16_bits_to_f64(got[1][:, rows]), ref)
        assert e <= REL_TOL, e
    finally:
        L.tuna_set_blockwise_scales_lds(prev_lds)


@pytest.mark.usefixtures("diagnostic_build")
@pytest.mark.parametrize("m,n,k,bs", [(256, 16, 1280, 64), (128, 7, 1536, 64), (512, 16, 4096, 128), (1024, 1, 2048, 256),
                                      (256, 16, 2048, 512), (768, 13, 5120, 64), (4096, 16, 4096, 64), (8192, 16, 8192, 64),
                                      (512, 37, 2048, 256), (256, 100, 1024, 64), (256, 530, 512, 64)])
def test_blockwise_gemm_through_the_batched_streaming_kernel(m, n, k, bs):
    """The scale-block variant of the batched streaming kernel (tuna_matmul_blockwise takes it for large aligned shapes; here
    an explicit config sends every shape there): against the oracle's float64 sums over the blockwise D1
    weights on a row sample, bit-exact through one-hot activations (every scale block of every sampled column read
    out), and run-to-run identical.  k ranges that are not whole x chunks, 128-row tiles, blocks longer than a chunk,
    shares that split row tiles (hand-over through the workspace); more than 16 tokens run as the token chunks of a
    batch, 32 chunks to a launch."""
    import torch

    from tuna_amd import _lib, ops

    rng = np.random.default_rng(m + n + k + bs + 1)
    q, x, code, _ = make_inputs_np(m, n, k, seed=m + bs + 1)
    absmax = rng.uniform(0.005, 0.02, size=(m, k // bs)).astype(np.float16).astype(np.float32)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    L = _lib.lib()
    c = blockwise_cfg("batched", m, n, k, bs)
    launches = L.tuna_multi_launches()
    if True:
        print(f"blockwise through the batched kernel m={m} n={n} k={k} block={bs} cfg={c.to_dict()}", flush=True)
        ops.matmul_blockwise(dx, dq, da, dc, out, m, n, k, bs, config=c)
        torch.cuda.synchronize()
        got = out.cpu().numpy().view(np.uint16)
        assert L.tuna_multi_launches() == launches + -(-(-(-n // 16)) // 32)     # the batched kernel ran it
        assert not np.isnan(got.view(np.float16)).any()
        rows = np.sort(rng.choice(m, size=min(m, 192), replace=False)).astype(np.int32)
        ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1, rows=rows, block_size=bs)
        e = rel_err(f16_bits_to_f64(got[:, rows]), ref)
        assert e <= REL_TOL, e
        again = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
        ops.matmul_blockwise(dx, dq, da, dc, again, m, n, k, bs, config=c)
        torch.cuda.synchronize()
        assert np.array_equal(again.cpu().numpy().view(np.uint16), got)
        img = O.dequant(q, absmax, code, m, k, mode=O.D1, block_size=bs)
        for rep in range(2):
            if n > k:
                break
            cols = rng.choice(k, size=n, replace=False)
            xh = np.zeros((n, k), np.float16)
            xh[np.arange(n), cols] = 1.0
            dxh, = to_dev(xh)
            ops.matmul_blockwise(dxh, dq, da, dc, out, m, n, k, bs, config=c)
            torch.cuda.synchronize()
            assert np.array_equal(out.cpu().numpy().view(np.uint16), img[:, cols].T)


@pytest.mark.usefixtures("diagnostic_build")
@pytest.mark.parametrize("m,n,k,bs", [(256, 16, 1024, 64), (512, 7, 2048, 64), (1024, 16, 4096, 128), (2048, 1, 8192, 64),
                                      (256 * 70, 16, 1024, 64), (768, 13, 5120, 64), (512, 16, 8192, 4096), (1024, 16, 2048, 1024),
                                      (4096, 16, 4096, 64), (16384, 16, 4096, 64), (28672, 16, 4096, 64),
                                      (512, 32, 2048, 64), (1024, 23, 4096, 128), (256 * 70, 17, 1024, 64), (28672, 32, 4096, 64),
                                      (512, 64, 2048, 64), (1024, 40, 4096, 128), (256 * 70, 33, 1024, 64), (28672, 64, 4096, 64)])
def test_blockwise_gemm_through_the_streaming_kernel(m, n, k, bs):
    """The scale-block twin of the streaming kernel (tuna_matmul_blockwise takes it for the largest shapes at up to 64
    tokens, two token tiles from 17 and four from 33; here every case goes there, with the library's own config where it names
    this kernel, else four waves by four): oracle on a row sample, exact read-out of the decoded weights with random scales per block (blocks
    shorter and longer than an x chunk, workgroups that walk several row tiles), run-to-run identical."""
    import torch

    from tuna_amd import _lib, ops

    rng = np.random.default_rng(m + n + k + bs + 3)
    q, x, code, _ = make_inputs_np(m, n, k, seed=m + bs + 3)
    absmax = rng.uniform(0.005, 0.02, size=(m, k // bs)).astype(np.float16).astype(np.float32)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    L = _lib.lib()
    c, hit = ops.select_config_blockwise(m, n, k, bs)
    if ops.blockwise_family(c) != "streaming":      # (the library's own choice where that is this kernel already)
        c = blockwise_cfg("streaming", m, n, k, bs)
    before = L.tuna_blockwise_launches(3)
    if True:
        print(f"blockwise through the streaming kernel m={m} n={n} k={k} block={bs} cfg={c.to_dict()}", flush=True)
        out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
        ops.matmul_blockwise(dx, dq, da, dc, out, m, n, k, bs, config=c)
        torch.cuda.synchronize()
        assert L.tuna_blockwise_launches(3) == before + 1     # that kernel ran it
        got = out.cpu().numpy().view(np.uint16)
        assert not np.isnan(got.view(np.float16)).any()
        rows = np.sort(rng.choice(m, size=min(m, 160), replace=False)).astype(np.int32)
        ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1, rows=rows, block_size=bs)
        e = rel_err(f16_bits_to_f64(got[:, rows]), ref)
        assert e <= REL_TOL, e
        again = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
        ops.matmul_blockwise(dx, dq, da, dc, again, m, n, k, bs, config=c)
        torch.cuda.synchronize()
        assert np.array_equal(again.cpu().numpy().view(np.uint16), got)
        img = O.dequant(q, absmax, code, m, k, mode=O.D1, block_size=bs)
        for rep in range(2):
            cols = rng.choice(k, size=n, replace=False)
            xh = np.zeros((n, k), np.float16)
            xh[np.arange(n), cols] = 1.0
            dxh, = to_dev(xh)
            ops.matmul_blockwise(dxh, dq, da, dc, out, m, n, k, bs, config=c)
            torch.cuda.synchronize()
            assert np.array_equal(out.cpu().numpy().view(np.uint16), img[:, cols].T)


@pytest.mark.usefixtures("diagnostic_build")
@pytest.mark.parametrize("m,n,k,bs", [(512, 64, 1024, 64), (528, 130, 2048, 128), (1024, 300, 4096, 64), (256, 1024, 512, 256),
                                      (4096, 33, 4096, 64), (272, 200, 1280, 64), (12288, 1000, 1024, 64)])
def test_blockwise_gemm_with_many_tokens_through_the_many_token_kernel(m, n, k, bs):
    """From 33 tokens tuna_matmul_blockwise decodes a weight tile once per workgroup with the scale of each k-step's block
    (the many-token kernel's scale-block variants): against the oracle's float64 sums over the blockwise D1 weights (row
    sample), bit-exact through one-hot activations, run-to-run identical; ragged m / n, k ranges of 8 to 64 steps; the
    last case is a shape whose per-row config is the 256 x 256 tile, which has no scale-block variant."""
    import torch

    from tuna_amd import _lib, ops

    rng = np.random.default_rng(m + n + k + bs + 2)
    q, x, code, _ = make_inputs_np(m, n, k, seed=m + bs + 2)
    absmax = rng.uniform(0.005, 0.02, size=(m, k // bs)).astype(np.float16).astype(np.float32)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    L = _lib.lib()
    c, _hit = ops.select_config_blockwise(m, n, k, bs)
    if ops.blockwise_family(c) != "many-token":     # (a tuned entry of another kernel family: the tile the derivation would take)
        c = blockwise_cfg("many-token", m, n, k, bs)
    before = L.tuna_blockwise_launches(2)
    print(f"blockwise through the many-token kernel m={m} n={n} k={k} block={bs} cfg={c.to_dict()}", flush=True)
    ops.matmul_blockwise(dx, dq, da, dc, out, m, n, k, bs, config=c)
    torch.cuda.synchronize()
    assert L.tuna_blockwise_launches(2) == before + 1
    got = out.cpu().numpy().view(np.uint16)
    assert not np.isnan(got.view(np.float16)).any()
    rows = np.sort(rng.choice(m, size=min(m, 128), replace=False)).astype(np.int32)
    ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1, rows=rows, block_size=bs)
    e = rel_err(f16_bits_to_f64(got[:, rows]), ref)
    assert e <= REL_TOL, e
    again = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_blockwise(dx, dq, da, dc, again, m, n, k, bs, config=c)
    torch.cuda.synchronize()
    assert np.array_equal(again.cpu().numpy().view(np.uint16), got)
    nh = min(n, k)
    cols = rng.choice(k, size=nh, replace=False)
    xh = np.zeros((n, k), np.float16)
    xh[np.arange(nh), cols] = 1.0
    dxh, = to_dev(xh)
    ops.matmul_blockwise(dxh, dq, da, dc, out, m, n, k, bs, config=c)
    torch.cuda.synchronize()
    img = O.dequant(q, absmax, code, m, k, mode=O.D1, block_size=bs)
    assert np.array_equal(out.cpu().numpy().view(np.uint16)[:nh], img[:, cols].T)


@pytest.mark.usefixtures("diagnostic_build")
def test_matmul_multi_blockwise_matches_the_oracle_and_separate_calls():
    """tuna_matmul_multi_blockwise: four problems with a scale per 64 weights in one launch of the batched kernel, one
    it cannot take (40 tokens) and one more behind it; every output against the oracle's float64 sums over the blockwise
    D1 weights (row sample), within tolerance of a separate tuna_matmul_blockwise call, one-hot read-outs bit-exact, and
    the same bits on a second call."""
    import torch

    from tuna_amd import _lib, ops

    bs = 64
    shapes = [(1024, 16, 2048), (2048, 16, 1024), (512, 3, 4096), (4096, 16, 4096), (256, 40, 1024), (768, 16, 1536)]
    rng = np.random.default_rng(77)
    probs, host = [], []
    dc = None
    for i, (m, n, k) in enumerate(shapes):
        q, x, code, _ = make_inputs_np(m, n, k, seed=500 + i)
        absmax = rng.uniform(0.005, 0.02, size=(m, k // bs)).astype(np.float16).astype(np.float32)
        dq, dx, dc_i, da = to_dev(q, x, code, absmax)
        dc = dc_i if dc is None else dc
        out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
        probs.append((dx, dq, da, dc, out, m, n, k))
        host.append((q, x, code, absmax))
    want = []
    for (dx, dq, da, dcc, _o, m, n, k) in probs:
        o = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
        ops.matmul_blockwise(dx, dq, da, dcc, o, m, n, k, bs)
        want.append(o)
    torch.cuda.synchronize()
    first = None
    for rep in range(2):
        for p in probs:
            p[4].fill_(float("nan"))
        before = _lib.lib().tuna_multi_launches()
        ops.matmul_multi(probs, block_size=bs)
        torch.cuda.synchronize()
        assert _lib.lib().tuna_multi_launches() == before + 1      # problems 0..3 in one launch, the rest one by one
        got = [p[4].cpu().numpy().view(np.uint16).copy() for p in probs]
        for i, ((m, n, k), g, w) in enumerate(zip(shapes, got, want)):
            assert not np.isnan(g.view(np.float16)).any(), (rep, i)
            q, x, code, absmax = host[i]
            rows = np.sort(np.random.default_rng(i).choice(m, size=min(m, 192), replace=False)).astype(np.int32)
            ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1, rows=rows, block_size=bs)
            e = rel_err(f16_bits_to_f64(g[:, rows]), ref)
            assert e <= REL_TOL, (rep, i, e)
            assert rel_err(f16_bits_to_f64(g), w.float().cpu().numpy().astype(np.float64)) <= REL_TOL
        for i in (4, 5):
            assert np.array_equal(got[i], want[i].cpu().numpy().view(np.uint16))
        if first is None:
            first = got
        else:
            assert all(np.array_equal(a, b) for a, b in zip(first, got))
    # one-hot activations read the decode out of the batched launch: every problem's image, its blocks' scales included
    hot = []
    for i, (m, n, k) in enumerate(shapes[:4]):
        cols = rng.choice(k, size=n, replace=False)
        xh = np.zeros((n, k), np.float16)
        xh[np.arange(n), cols] = 1.0
        dxh, = to_dev(xh)
        hot.append((dxh,) + probs[i][1:])
        hot[-1][4].fill_(float("nan"))
        hot[-1] = hot[-1] + (cols,)
    ops.matmul_multi([h[:8] for h in hot], block_size=bs)
    torch.cuda.synchronize()
    for i, h in enumerate(hot):
        q, _, code, absmax = host[i]
        m, n, k = shapes[i]
        img = O.dequant(q, absmax, code, m, k, mode=O.D1, block_size=bs)
        assert np.array_equal(h[4].cpu().numpy().view(np.uint16), img[:, h[8]].T), i
    arr = ops.problem_array(probs[:2], bs)
    assert _lib.lib().tuna_matmul_multi_blockwise(arr, 2, 32, ops._stream(probs[0][0].device)) == _lib.ERR_UNSUPPORTED   # blocks start at 64


def test_blockwise_entry_points_reject_what_they_cannot_run():
    import torch

    from tuna_amd import ops

    q, x, code, _ = make_inputs_np(64, 16, 512, seed=1)
    dq, dx, dc = to_dev(q, x, code)
    da = torch.ones((64, 512 // 32), dtype=torch.float32, device="cuda")
    out = torch.zeros((16, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(ops.TunaError):
        ops.matmul_blockwise(dx, dq, da, dc, out, 64, 16, 512, 32)          # GEMM blocks start at 64
    w = torch.zeros((64, 768), dtype=torch.float16, device="cuda")
    with pytest.raises(ops.TunaError):
        ops.quantize(w, dc, block_size=384)                                 # quantizer blocks: 8..256 (powers of two) or k
    ops.quantize(w, dc, block_size=768)                                     # == k: the per-row op
    torch.cuda.synchronize()


@pytest.mark.usefixtures("diagnostic_build")
def test_quantizer_division_is_the_ieee_division_for_every_quotient_it_can_form():
    """The quantizer divides by a block's maximum with a refined reciprocal and one fused correction.
    Every pair of fp16 values (w, a), a > 0 finite, |w| <= a - 1.0e9 pairs, all there are - gives
    the bits of the IEEE fp32 division."""
    import torch

    from tuna_amd import _lib

    counts = torch.zeros(2, dtype=torch.int64, device="cuda")
    _lib.check(_lib.lib().tuna_selftest_quantizer_division(counts.data_ptr(), None))
    torch.cuda.synchronize()
    n, bad = (int(v) for v in counts.cpu())
    assert n == sum(2 * a + 2 for a in range(1, 0x7c00))      # for magnitude a: the bit patterns 0 .. a with either sign
    assert bad == 0, f"{bad} of {n} quotients differ from the IEEE division"


def test_quantizer_every_fp16_value_against_the_oracle():
    """Rows that hold every fp16 value up to their maximum (k = 65536, per-row scale: the two-pass
    variant) for maxima from the subnormals to 65504, and the same values with one scale per 64
    (different maxima per block): packed bytes and scales identical to the oracle's."""
    import torch

    from tuna_amd import ops

    rng = np.random.default_rng(3)
    allbits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    maxima = np.array([0x3c00, 0x3999, 0x2266, 0x0001, 0x0155, 0x7bff, 0x5640, 0x1c03], np.uint16)   # 1.0, 0.7, 0.0125, ...
    w = np.zeros((8, 65536), np.uint16)
    for r, a in enumerate(maxima):
        row = allbits.copy()
        row[(row & 0x7fff) > a] = 0                       # larger magnitudes, infinities and NaNs out
        w[r] = rng.permutation(row)
    code = O.nf4_codebook()
    dw, dc = to_dev(w.view(np.float16), code)
    for bs in (None, 64, 256):
        q, a, _ = ops.quantize(dw, dc, block_size=bs)
        torch.cuda.synchronize()
        q_ref, a_ref = O.quantize(w, code, 8, 65536, block_size=bs)
        assert np.array_equal(a.cpu().numpy(), a_ref)
        assert np.array_equal(q.cpu().numpy(), q_ref), bs


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k", [(4096, 16, 4096), (6144, 16, 4096), (5120, 16, 5120), (4096, 1, 4096), (8192, 16, 8192),
                                   (28672, 16, 4096), (8192, 16, 28672), (2560, 32, 2560)])
def test_scales_that_are_only_float_aligned_run_through_the_dispatcher(m, n, k):
    """absmax may be any float pointer (the reference's wrapper takes one): a view 4 bytes into a buffer, on shapes
    whose library-chosen kernels read the scales two or four at a time (narrow-row, lean, LDS-staged and batched
    launches), must run - the dispatcher takes a kernel that reads them one by one - and match the oracle."""
    import torch

    from tuna_amd import ops

    print(f"float-aligned scales m={m} n={n} k={k}: aligned launch would be {ops.describe_launch(m, n, k, None)}", flush=True)
    q, x, code, absmax = make_inputs_np(m, n, k, seed=m + n + k)
    dq, dx, dc = to_dev(q, x, code)
    holder = torch.zeros(m + 8, dtype=torch.float32, device="cuda")
    da = holder[1:m + 1]
    da.copy_(torch.from_numpy(absmax))
    assert da.data_ptr() % 16 == 4
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul(dx, dq, da, dc, out, m, n, k)
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(np.uint16)
    assert not np.isnan(f16_bits_to_f64(got)).any()
    rows = np.sort(np.random.default_rng(k).choice(m, size=128, replace=False)).astype(np.int32)
    ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1, rows=rows)
    assert rel_err(f16_bits_to_f64(got[:, rows]), ref) <= REL_TOL


@pytest.mark.gpu
@pytest.mark.usefixtures("diagnostic_build")
@pytest.mark.parametrize("n,dims", [(16, (1024, 512, 2816)), (5, (2048, 1024, 5632)), (16, (512, 256, 1408))])
def test_a_layer_as_one_batched_launch_with_fused_epilogues(n, dims):
    """The four projections of a decoder layer as ONE tuna_matmul_multi_fused call (independent inputs, as the entry
    point requires): QKV plain, attention output + residual, the combined gate+up GEMM with SiLU-mul on interleaved
    rows (output [n, m/2]), down + residual in place.  One launch of the batched kernel's fused-epilogue variant;
    every output against the oracle's float64 sums pushed through the same formulas, and bit for bit against
    tuna_matmul_fused's for the same problems where the two run the same sums (whole row tiles)."""
    import torch

    from tuna_amd import _lib, ops

    hidden, kv, inter = dims
    shapes = [(hidden + 2 * kv, hidden, _lib.EPILOGUE_NONE), (hidden, hidden, _lib.EPILOGUE_RESIDUAL),
              (2 * inter, hidden, _lib.EPILOGUE_SILU_MUL), (hidden, inter, _lib.EPILOGUE_RESIDUAL)]
    print(f"layer as one launch: tokens={n} shapes={[(m, k) for m, k, _ in shapes]}", flush=True)
    rng = np.random.default_rng(n + hidden)
    host, problems, eps, residuals, outs = [], [], [], [], []
    code_dev = None
    for i, (m, k, ep) in enumerate(shapes):
        q, x, code, absmax = make_inputs_np(m, n, k, seed=400 + i + hidden)
        res = (rng.standard_normal((n, m)) * 0.05).astype(np.float16)
        dq, dx, dc, da, dres = to_dev(q, x, code, absmax, res)
        code_dev = code_dev if code_dev is not None else dc          # one codebook pointer: one decode table per launch
        om = m // 2 if ep == _lib.EPILOGUE_SILU_MUL else m
        out = dres.clone() if i == 3 else torch.full((n, om), float("nan"), dtype=torch.float16, device="cuda")
        host.append((q, x, code, absmax, res))
        problems.append((dx, dq, da, code_dev, out, m, n, k))
        eps.append(ep)
        residuals.append(out if i == 3 else dres if ep == _lib.EPILOGUE_RESIDUAL else None)   # down: residual in place
        outs.append(out)
    L = _lib.lib()
    before = L.tuna_multi_launches()
    ops.matmul_multi(problems, epilogues=eps, residuals=residuals)
    torch.cuda.synchronize()
    assert L.tuna_multi_launches() == before + 1                       # all four in one launch
    for i, ((m, k, ep), (q, x, code, absmax, res), out) in enumerate(zip(shapes, host, outs)):
        ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1)
        got = out.cpu().numpy().astype(np.float64)
        assert not np.isnan(got).any(), i
        if ep == _lib.EPILOGUE_RESIDUAL:
            assert rel_err(got, ref + res.astype(np.float64)) <= REL_TOL, i
        elif ep == _lib.EPILOGUE_SILU_MUL:
            g, u = ref[:, 0::2], ref[:, 1::2]
            assert rel_err(got, g / (1.0 + np.exp(-g)) * u, floor=REL_FLOOR_D2) <= REL_TOL, i
        else:
            assert rel_err(got, ref) <= REL_TOL, i
    # without epilogues the same call writes the plain sums: the fused variant changes the stores only
    plain = [torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda") for m, _, _ in shapes]
    ops.matmul_multi([(p[0], p[1], p[2], p[3], o, p[5], p[6], p[7]) for p, o in zip(problems, plain)])
    torch.cuda.synchronize()
    assert torch.equal(plain[0].view(torch.int16), outs[0].view(torch.int16))


@pytest.mark.gpu
def test_batched_launch_with_epilogues_rejects_bad_arguments_and_falls_back_problem_by_problem():
    """A residual epilogue without a residual is an argument error before anything is enqueued; a problem the batched
    kernel cannot take (more than 16 tokens) runs through tuna_matmul_fused with its epilogue."""
    import torch

    from tuna_amd import _lib, ops

    m, n, k = 512, 40, 1024
    q, x, code, absmax = make_inputs_np(m, n, k, seed=77)
    res = (np.random.default_rng(5).standard_normal((n, m)) * 0.05).astype(np.float16)
    dq, dx, dc, da, dres = to_dev(q, x, code, absmax, res)
    out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        ops.matmul_multi([(dx, dq, da, dc, out, m, n, k)], epilogues=[_lib.EPILOGUE_RESIDUAL], residuals=[None])
    arr = ops.problem_array([(dx, dq, da, dc, out, m, n, k)])
    eps = (ctypes.c_int32 * 1)(_lib.EPILOGUE_RESIDUAL)
    assert _lib.lib().tuna_matmul_multi_fused(arr, eps, None, 1, None) == _lib.ERR_INVALID_ARG
    eps[0] = 7
    assert _lib.lib().tuna_matmul_multi_fused(arr, eps, None, 1, None) == _lib.ERR_INVALID_ARG
    ops.matmul_multi([(dx, dq, da, dc, out, m, n, k)], epilogues=[_lib.EPILOGUE_RESIDUAL], residuals=[dres])
    torch.cuda.synchronize()
    ref = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=O.D1) + res.astype(np.float64)
    assert rel_err(out.cpu().numpy().astype(np.float64), ref) <= REL_TOL


def _blockwise_table_entries():
    import json
    import os

    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "tuna_amd", "configs", "param_map_blockwise.json")
    with open(path) as f:
        return sorted(json.load(f), key=lambda s: tuple(int(t) for t in s.split("_")))


@pytest.mark.gpu
@pytest.mark.usefixtures("diagnostic_build")
@pytest.mark.parametrize("key", _blockwise_table_entries())
def test_every_blockwise_table_entry_matches_the_oracle(key):
    """Every tuned entry of the blockwise table at its real size, through the plain entry point (no config: the table
    lookup is what is tested), at the lower edge of its token bucket and at a ragged count inside it: the kernel the
    entry names runs, 64 random 8-row blocks match the oracle's float64 sums over the blockwise D1 weights, and one-hot
    activations read the decoded weights of those rows out exactly (random scales per block)."""
    import torch

    from tuna_amd import _lib, make_configs, ops
    from tuna_amd.quantize import nf4_codebook
    from tuna_amd.synth import make_weights_torch, make_x_torch

    m, n_key, k, bs = (int(t) for t in key.split("_"))
    L = _lib.lib()
    dev = torch.device("cuda")
    q, _ = make_weights_torch(m, k, seed=m + k + bs, device=dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(bs + n_key)
    absmax = (torch.rand((m, k // bs), dtype=torch.float32, device=dev, generator=gen) * 0.015 + 0.005).to(torch.float16).float()
    code = nf4_codebook(dev)
    rng = np.random.default_rng(m + n_key)
    mbs = np.sort(rng.choice(m // 8, size=min(64, m // 8), replace=False))
    rows = (mbs[:, None] * 8 + np.arange(8)[None, :]).ravel()
    q_sub = q[torch.from_numpy(mbs).to(dev)].cpu().numpy()
    a_sub = absmax.cpu().numpy()[rows]
    code_np = code.cpu().numpy()
    lo, hi = make_configs.N_BUCKETS[n_key]
    for n in sorted({lo, min(hi, lo + max(1, lo // 2) + 1)}):
        c, hit = ops.select_config_blockwise(m, n, k, bs)
        fam = ops.blockwise_family(c)
        print(f"blockwise table entry {key} at n={n}: {fam} {c.to_dict()} from_table={hit}", flush=True)
        assert hit or n != lo          # (inside the bucket an entry that cannot make its one pass gives way to a derived config)
        before = L.tuna_blockwise_launches(ops.BLOCKWISE_FAMILIES.index(fam))
        x = make_x_torch(n, k, seed=n, device=dev)
        out = torch.full((n, m), float("nan"), dtype=torch.float16, device=dev)
        ops.matmul_blockwise(x, q, absmax, code, out, m, n, k, bs)
        torch.cuda.synchronize()
        assert L.tuna_blockwise_launches(ops.BLOCKWISE_FAMILIES.index(fam)) > before
        assert not torch.isnan(out).any()
        ref = O.gemm_f64(q_sub, x.cpu().numpy().view(np.uint16), code_np, a_sub, len(rows), n, k, mode=O.D1, block_size=bs)
        e = rel_err(f16_bits_to_f64(out.cpu().numpy().view(np.uint16)[:, rows]), ref)
        assert e <= REL_TOL, e
        nh = min(n, k)
        cols = rng.choice(k, size=nh, replace=False)
        xh = torch.zeros((n, k), dtype=torch.float16, device=dev)
        xh[torch.arange(nh, device=dev), torch.from_numpy(cols).to(dev)] = 1.0
        ops.matmul_blockwise(xh, q, absmax, code, out, m, n, k, bs)
        torch.cuda.synchronize()
        img_sub = O.dequant(q_sub, a_sub, code_np, len(rows), k, mode=O.D1, block_size=bs)
        assert np.array_equal(out.cpu().numpy().view(np.uint16)[:nh][:, rows], img_sub[:, cols].T)
