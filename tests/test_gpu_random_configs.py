"""Seeded random launch configurations of the streaming kernel families against the oracle.

Every case draws a shape, a token count and a config from the same spaces the tuner searches
(narrow-row variants, lean-kernel layouts, the general kernel's seed pool, the 17..128-token streaming kernel), keeps it only if the Python
validator accepts it, and runs it through the C-ABI. A config the Python validator accepts but the library
cannot launch, or a launch that differs from the oracle beyond the GEMM tolerance, fails the test.
Output layout and rounding follow kernel.cu:2649-2754 (fp32 accumulate, one fp16 rounding).
"""
import random

import numpy as np
import pytest
import torch

from helpers import O, REL_TOL, make_inputs_np, rel_err, to_dev
from tuna_amd import make_configs as mc
from tuna_amd import ops, tuner

pytestmark = pytest.mark.gpu

TOKENS = [1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 100]


def draw(rng):
    kind = rng.choice(["narrow", "lean", "general", "mid"])
    n = rng.choice(TOKENS)
    bucket = mc.bucket_of(n)
    if kind == "mid":
        wm, wk = rng.randint(1, 8), rng.choice([1, 2, 4])
        xc = rng.choice([128, 256, 512])
        c = dict(rows_per_wave=64, waves_m=wm, waves_k=wk, split_k=1, prefetch=rng.choice([2, 4, 8]), x_chunk=xc,
                 token_tiles=rng.choice([2, 4, 8]), xcd_swizzle=rng.choice([0, 1]), k_stagger=0, lds_tile_rows=0)
        m, k = 64 * wm * rng.randint(1, 6), xc * rng.randint(1, 4)
        n = rng.choice([17, 20, 32, 33, 50, 64, 65, 100, 128, 130, 200])
        try:
            mc.validate(m, mc.bucket_of(n), k, c)
        except ValueError:
            return None
        return (kind, m, n, k, c) if mc.mid_applies(m, k, c) else None
    if kind == "narrow":
        rows, wk, pf, tt = rng.choice(sorted(mc.NARROW_VARIANTS))
        m = rows * rng.randint(1, 12)
        k = 32 * wk * pf * rng.randint(1, 6)
        c = dict(rows_per_wave=rows, waves_m=0 if rows == 64 else 1, waves_k=wk, split_k=1, prefetch=pf,
                 x_chunk=32 * wk * pf, token_tiles=tt, xcd_swizzle=0, k_stagger=0, lds_tile_rows=0)
    elif kind == "lean":
        wm, wk = rng.randint(1, 8), rng.choice([1, 2, 4, 8, 16])
        if wm * wk > 16:
            return None
        pf, sp = rng.choice([2, 4, 8]), rng.choice([1, 2, 4, 8])
        k = 32 * wk * pf * rng.randint(1, 4) * sp
        m = 64 * wm * rng.randint(1, 6)
        c = dict(rows_per_wave=64, waves_m=wm, waves_k=wk, split_k=sp, prefetch=pf, x_chunk=32 * wk * pf,
                 token_tiles=1, xcd_swizzle=rng.choice([0, 1]), k_stagger=0, lds_tile_rows=0)
        c = tuner.repair(c, m, bucket, k)
        if c is None or c["token_tiles"] != 1 or c["split_k"] != sp:
            return None
    else:
        m, k = 8 * rng.randint(1, 120), 8 * rng.randint(1, 400)
        pool = tuner.seeds(m, bucket, k)
        if not pool:
            return None
        c = rng.choice(pool)
    try:
        mc.validate(m, bucket, k, c)
    except ValueError:
        return None
    return kind, m, n, k, c


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_configs_match_oracle(seed):
    rng = random.Random(seed)
    ran = {"narrow": 0, "lean": 0, "general": 0, "mid": 0}
    for case in range(60):
        drawn = draw(rng)
        if drawn is None:
            continue
        kind, m, n, k, c = drawn
        q, x, code, absmax = make_inputs_np(m, n, k, seed=seed * 1000 + case)
        want = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
        dq, dx, dc, da = to_dev(q, x, code, absmax)
        out = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
        print(f"seed {seed} case {case} {kind} m={m} n={n} k={k} {c}", flush=True)
        ops.matmul(dx, dq, da, dc, out, m, n, k, config=ops.GemmConfig.from_dict(c))
        torch.cuda.synchronize()
        err = rel_err(out.cpu().numpy().astype(np.float64), want)
        assert err <= REL_TOL, (kind, m, n, k, c, err)     # max relative error 1e-2
        ran[kind] += 1
    assert all(v >= 3 for v in ran.values()), ran


@pytest.mark.parametrize("seed", [21, 22])
def test_random_shapes_through_the_dispatcher_match_oracle(seed):
    """No config: the library picks one for every shape and token count, tuned or not (m and k any
    multiples of 8, 1..2500 tokens - every bucket of the dispatcher, kernel.cu:3022-3155)."""
    from helpers import f16_bits_to_f64, run_gemm
    rng = random.Random(seed)
    for case in range(28):
        n = rng.choice([1, 2, 9, 16, 17, 40, 64, 100, 128, 200, 256, 300, 512, 600, 769, 1025, 2500])
        budget = 3e8 // n                                   # keeps the oracle's float64 GEMM in seconds
        k = 8 * rng.randint(1, 600)
        m = 8 * rng.randint(1, max(1, min(400, int(budget // k) // 8)))
        q, x, code, absmax = make_inputs_np(m, n, k, seed=seed * 1000 + case)
        print(f"seed {seed} case {case} dispatcher m={m} n={n} k={k}", flush=True)
        got = run_gemm(q, x, code, absmax, m, n, k, prefill=float("nan"))
        want = O.gemm_f64(q, x, code, absmax, m, n, k, mode=O.D1)
        err = rel_err(f16_bits_to_f64(got), want)
        assert err <= REL_TOL, (m, n, k, err)              # max relative error 1e-2


def test_random_grouped_launches_match_per_group_oracle():
    """Random group counts, sizes and token lists (empty groups included), no config."""
    from helpers import f16_bits_to_f64
    rng = random.Random(31)
    for case in range(12):
        n_groups = rng.choice([1, 2, 3, 8, 16])
        m_group = 64 * rng.randint(1, 8)                 # groups are whole 64-row tiles
        k = 8 * rng.randint(1, 300)
        counts = [rng.choice([0, 0, 1, 3, 16, 17, 40]) for _ in range(n_groups)]
        if sum(counts) == 0:
            counts[rng.randrange(n_groups)] = 5
        offsets = [0]
        for c in counts:
            offsets.append(offsets[-1] + c)
        n_total, m = offsets[-1], m_group * n_groups
        q, x, code, absmax = make_inputs_np(m, n_total, k, seed=3100 + case)
        dq, dx, dc, da = to_dev(q, x, code, absmax)
        out = torch.full((n_total, m_group), float("nan"), dtype=torch.float16, device="cuda")
        print(f"grouped case {case} m_group={m_group} n_groups={n_groups} k={k} counts={counts}", flush=True)
        ops.matmul_grouped(dx, dq, da, dc, out, m_group, n_groups, k, offsets)
        torch.cuda.synchronize()
        got = out.cpu().numpy().astype(np.float64)
        qb = q.reshape(n_groups, m_group // 8, k // 8, 32)
        for e in range(n_groups):
            lo, hi = offsets[e], offsets[e + 1]
            if hi == lo:
                continue
            want = O.gemm_f64(np.ascontiguousarray(qb[e]), np.ascontiguousarray(x[lo:hi]), code,
                              np.ascontiguousarray(absmax[e * m_group:(e + 1) * m_group]), m_group, hi - lo, k, mode=O.D1)
            err = rel_err(got[lo:hi], want)
            assert err <= REL_TOL, (case, e, err)
