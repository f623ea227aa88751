"""Evolutionary tuner of the GEMM tile configs for MI355X (gfx950).

The reference's README names an evolutionary tuner (README.md:32) whose output is
param_map.json (consumed by make_configs.py:85-132), but the tuner itself is not in the
repository.  This one searches the CDNA4 config space of `tuna_gemm_config`
(wave64 workgroups of waves_m x waves_k waves, 64/128/256 rows per wave, the depth of the
per-wave global->register prefetch ring, the LDS staging chunk of x, in-workgroup and
cross-workgroup split-K sized for 256 CUs / 8 XCDs / 160 KB of LDS) and writes entries keyed
"<m>_<n>_<k>" like the reference's.

Search: a seeded population of hand-derived configs, then generations of
(tournament selection -> crossover -> mutation -> validity repair), every candidate timed on
the GPU with HIP events over rotating, cache-defeating weight sets (tuna_time_matmul).

    python -m tuna_amd.tuner --tokens 16 --shapes all --generations 6 --out tuned/param_map.json

Two more passes measure how the lookup treats token counts between the tuned ones: --next-from (from which count
of a bucket the next bucket's entry is faster) and, with the table rebuilt into the library, --derived-range (the
stretch of a bucket where the library's derived config is faster than the table's).
"""
import argparse
import json
import os
import random
import sys
import time

from . import make_configs
from .synth import SHAPES

HERE = os.path.dirname(os.path.abspath(__file__))

GENES = {
    "rows_per_wave": (64, 128, 256),
    "waves_m": (1, 2, 3, 4, 5, 6, 7, 8),
    "waves_k": (1, 2, 4, 8, 16),
    "prefetch": (2, 4, 8),
    "token_tiles": (1, 2, 4),
    "xcd_swizzle": (0, 1),
    "k_stagger": (0, 1, 1, 2, 3, 5, 8, 16),
}
N_CU = 256


def _pow2_floor(v: int) -> int:
    p = 1
    while p * 2 <= v:
        p *= 2
    return p


def repair(c: dict, m: int, n_key: int, k: int):
    """Make a raw gene vector a valid config for the shape, or return None."""
    c = dict(c)
    c.setdefault("k_stagger", 0)
    c.setdefault("lds_tile_rows", 0)
    if c["lds_tile_rows"] > 0 or make_configs.is_narrow(c):
        try:
            make_configs.validate(m, n_key, k, c)
            return c
        except ValueError:
            return None
    steps = -(-k // 32)
    if c["waves_m"] * c["waves_k"] > 16:
        return None
    lo, hi = make_configs.N_BUCKETS[n_key]
    # token tiles: never more tiles than the bucket's largest token count needs
    need = 1 if hi <= 16 or lo < 16 else (2 if lo < 32 else 4)
    c["token_tiles"] = min(c["token_tiles"], need)
    threads = 64 * c["waves_m"] * c["waves_k"]
    unit = 32 * c["waves_k"] * c["prefetch"]      # smallest x chunk: one ring turn of the workgroup
    c["split_k"] = max(0, min(int(c["split_k"]), steps))    # 0 = balanced split
    sps = -(-steps // max(1, c["split_k"]))
    # x chunk: a power of two in [unit, 2*threads/token_tiles], no larger than the split needs
    hi_chunk = _pow2_floor(max(unit, (4 if c["prefetch"] == 8 else 2) * threads // c["token_tiles"]))
    want = max(unit, min(_pow2_floor(max(int(c.get("x_chunk", 1024)), 1)), hi_chunk))
    while want // 2 >= unit and want // 2 >= sps * 32:
        want //= 2
    c["x_chunk"] = want
    while True:
        try:
            make_configs.validate(m, n_key, k, c)
            return c
        except ValueError as e:
            if "LDS" in str(e) and c["x_chunk"] // 2 >= unit:
                c["x_chunk"] //= 2
                continue
            return None


def seeds(m: int, n_key: int, k: int):
    """Hand-derived starting points: fill the 256 CUs with 1-2 workgroups each."""
    out = []
    for rpw in (64, 128):
        for wm, wk in ((1, 4), (1, 8), (2, 4), (2, 2), (4, 2), (1, 16), (2, 8), (4, 4), (4, 1), (8, 1), (1, 2), (16, 1),
                       (8, 2), (2, 1), (7, 1), (7, 2), (14, 1), (3, 4), (3, 2), (5, 2), (6, 2), (5, 1), (6, 1), (3, 1)):
            row_tiles = -(-m // (rpw * wm))
            for target in (0, N_CU, 2 * N_CU, 4 * N_CU):
                split = max(1, round(target / row_tiles)) if target else 0
                for pf in (2, 4, 8):
                    for tt in (1, 2, 4):
                        for xc in (256, 512, 1024, 2048):
                            for sw, stg in ((0, 0), (1, 0), (1, 1), (0, 1)):
                                c = repair(dict(rows_per_wave=rpw, waves_m=wm, waves_k=wk, split_k=split, prefetch=pf,
                                                x_chunk=xc, token_tiles=tt, xcd_swizzle=sw, k_stagger=stg), m, n_key, k)
                                if c is not None:
                                    out.append(c)
    uniq = {json.dumps(c, sort_keys=True): c for c in out}
    return list(uniq.values())


def tiled_space(m: int, n_key: int, k: int):
    """Every config of the many-token kernel (weights decoded once into LDS) worth timing for
    the shape: tile shapes x k splits.  Small enough to time exhaustively."""
    lo, _ = make_configs.N_BUCKETS[n_key]
    if lo < 64:
        return []
    out = []
    steps = -(-k // 64)
    for rows, tokens in sorted(make_configs.TILED_VARIANTS):
        if tokens > max(64, 2 * lo):
            continue
        tiles = -(-m // rows) * -(-lo // tokens)
        for split in (1, 2, 3, 4, 6, 8, 12, 16, 24, 32):
            if split > 1 and (steps // split < 4 or tiles * split > 4 * N_CU):
                continue
            for mfma_rows in (64, 32):   # 16 x 16 x 32 MFMA tiles (any value but 32) / 32 x 32 x 16
                c = dict(rows_per_wave=mfma_rows, waves_m=1, waves_k=1, split_k=split, prefetch=2, x_chunk=64,
                         token_tiles=tokens // 16, xcd_swizzle=0, k_stagger=0, lds_tile_rows=rows)
                try:
                    make_configs.validate(m, n_key, k, c)
                except ValueError:
                    continue
                out.append(c)
    return out


def lean_space(m: int, n_key: int, k: int):
    """Every config whose launch takes the stripped-down kernel for small aligned launches
    (gemm_lean.hpp; the conditions of lean_applies in gemm_launch.hip): 64 rows per wave, one
    token tile, no stagger, a power-of-two split, whole ring turns, all tiles resident at once.
    Small enough to time exhaustively."""
    lo, _ = make_configs.N_BUCKETS[n_key]
    if lo > 64 or k % 32:
        return []
    steps = k // 32
    out = []
    for wm in range(1, 17):
        for wk in (1, 2, 4, 8, 16):
            waves = wm * wk
            if waves > 16 or m % (64 * wm):
                continue
            split = 1
            while split <= steps:
                sps = steps // split
                if steps % split == 0 and sps * 64 <= 8 * 64 * waves:
                    lds = 65536 + max(sps * 1024, waves * 4096) + 16
                    wgs = min(make_configs.LDS_LIMIT // lds, max(1, 20 // waves)) if lds <= make_configs.LDS_LIMIT else 0
                    if (m // (64 * wm)) * split <= N_CU * wgs:
                        for pf in (2, 4, 8):
                            if sps % (wk * pf):
                                continue
                            for sw in (0, 1):
                                c = repair(dict(rows_per_wave=64, waves_m=wm, waves_k=wk, split_k=split, prefetch=pf,
                                                x_chunk=32 * wk * pf, token_tiles=1, xcd_swizzle=sw, k_stagger=0), m, n_key, k)
                                if c is not None and c["split_k"] == split and c["token_tiles"] == 1:
                                    out.append(c)
                split *= 2
    uniq = {json.dumps(c, sort_keys=True): c for c in out}
    return list(uniq.values())


def mid_space(m: int, n_key: int, k: int):
    """Every config whose launch takes the 17..128-token streaming kernel (gemm_mid.hpp; the
    conditions of mid_variant in gemm_mid.hip): 64 rows per wave, k unsplit or split into a power of two
    of parts.  Small enough to time exhaustively."""
    lo, hi = make_configs.N_BUCKETS[n_key]
    out = []
    # tuned at the bucket's lower edge; from 128 tokens on, passes of eight token tiles (on the
    # largest shapes they beat the many-token kernel at every token count)
    # (from 32 tokens on also chunks of fewer token tiles than the count needs: they run side by side and share
    # the weights when they all fit the device, which fills it without a split of k and its hand-over - the
    # mid-size shapes prefer them: 10240 x 8192 at 384 tokens 112 -> 82 us with six chunks of four token tiles)
    for tt in ((1,) if lo <= 16 else (2, 1) if lo <= 32 else (4, 2, 1) if lo <= 64 else (8, 4, 2) if lo <= 256 else (8, 4)):
        for wm in range(1, 17):
            for wk in (1, 2, 4, 8):
                if m % (64 * wm) or wm * wk > 16 or wm * wk < 4:
                    continue
                if tt == 1 and ((m // (64 * wm)) * -(-lo // 16) < 100 or wm * wk < 8):
                    continue        # one token tile: only launches that fill the device unsplit (others: lean, narrow-row)
                for pf in (2, 4, 8):
                    for xc in (128, 256, 512, 1024, 2048):
                        for sw, stg in ((0, 0), (1, 0), (0, 2), (0, 5)):
                            # k split across workgroups (two or more token tiles, no stagger): where the row tiles
                            # alone leave compute units idle, up to about two rounds of workgroups
                            for split in (1, 2, 4, 8, 16):
                                if split > 1 and (tt < 2 or stg or (m // (64 * wm)) * (split // 2) >= 2 * N_CU):
                                    continue
                                c = dict(rows_per_wave=64, waves_m=wm, waves_k=wk, split_k=split, prefetch=pf, x_chunk=xc,
                                         token_tiles=tt, xcd_swizzle=sw, k_stagger=stg, lds_tile_rows=0)
                                try:
                                    make_configs.validate(m, n_key, k, c)
                                except ValueError:
                                    continue
                                if make_configs.mid_applies(m, k, c):
                                    out.append(c)
                                    # the same launch with the packed weights staged through LDS, where that twin exists
                                    cl = dict(c, lds_tile_rows=-1)
                                    try:
                                        make_configs.validate(m, n_key, k, cl)
                                        out.append(cl)
                                    except ValueError:
                                        pass
    return out


def narrow_space(m: int, n_key: int, k: int):
    """Every config of the narrow-row kernel (gemm_narrow.hpp: 16 or 32 rows per workgroup, all
    waves along k, no split) the shape admits.  Small enough to time exhaustively."""
    lo, hi = make_configs.N_BUCKETS[n_key]
    if lo > 512:     # (up to 512 tokens: small shapes run one round of workgroups x token passes side by side)
        return []
    out = []
    for rows, wk, pf, tt in sorted(make_configs.NARROW_VARIANTS):
        if 16 * tt > max(16, hi) or (tt > 1 and 16 * (tt // 2) >= hi):   # no more token tiles than the bucket can fill
            continue
        c = dict(rows_per_wave=rows, waves_m=0 if rows == 64 else 1, waves_k=wk, split_k=1, prefetch=pf, x_chunk=32 * wk * pf,
                 token_tiles=tt, xcd_swizzle=0, k_stagger=0, lds_tile_rows=0)
        try:
            make_configs.validate(m, n_key, k, c)
        except ValueError:
            continue
        if m // rows <= 8 * N_CU:
            out.append(c)
    return out


def mutate(c: dict, rng: random.Random, m, n_key, k):
    c = dict(c)
    for _ in range(rng.choice((1, 1, 2))):
        gene = rng.choice(list(GENES) + ["split_k", "split_k", "x_chunk"])
        if gene == "split_k":
            if rng.random() < 0.2:
                c["split_k"] = 0                                   # balanced split
            elif c["split_k"] == 0:
                c["split_k"] = rng.choice((1, 2, 4, 8))
            else:
                c["split_k"] = max(1, int(round(c["split_k"] * rng.choice((0.5, 0.75, 1.25, 1.5, 2.0)) + rng.choice((-1, 0, 1)))))
        elif gene == "x_chunk":
            c["x_chunk"] = max(64, int(c["x_chunk"] * rng.choice((0.5, 2.0))))
        else:
            c[gene] = rng.choice(GENES[gene])
    return repair(c, m, n_key, k)


def crossover(a: dict, b: dict, rng: random.Random, m, n_key, k):
    c = {g: (a if rng.random() < 0.5 else b)[g] for g in a}
    return repair(c, m, n_key, k)


class Evaluator:
    """Times configs for one shape on the GPU over rotating weight sets."""

    def __init__(self, m, n, k, iters=60, warmup=10):
        import torch

        from . import ops, synth
        from .quantize import nf4_codebook

        self.ops, self.torch = ops, torch
        self.m, self.n, self.k = m, n, k
        self.iters, self.warmup = iters, warmup
        dev = torch.device("cuda")
        bytes_w = m * k // 2
        n_sets = max(2, min(-(-(512 << 20) // bytes_w), 64))
        self.sets = [synth.make_weights_torch(m, k, 777 + i, dev) for i in range(n_sets)]
        self.x = synth.make_x_torch(n, k, 1, dev)
        self.code = nf4_codebook(dev)
        self.out = torch.empty((n, m), dtype=torch.float16, device=dev)
        self.cache = {}

    def __call__(self, c: dict) -> float:
        key = json.dumps(c, sort_keys=True)
        if key not in self.cache:
            cfg = self.ops.GemmConfig.from_dict(c)
            try:
                best = float("inf")
                for _ in range(2):
                    ms = self.ops.time_matmul([s[0] for s in self.sets], [s[1] for s in self.sets], self.x, self.code,
                                              self.out, self.m, self.n, self.k, config=cfg, warmup=self.warmup,
                                              iters=self.iters)
                    best = min(best, ms * 1000.0 / self.iters)
                self.cache[key] = best
            except self.ops.TunaError:
                self.cache[key] = float("inf")
        return self.cache[key]


def tune_shape(m, n, k, generations=6, population=24, seed=0, log=print, max_seed_evals=120, iters=60, extra=()):
    rng = random.Random(seed * 7919 + m * 31 + k)
    n_key = make_configs.bucket_of(n)
    ev = Evaluator(m, n, k, iters=iters, warmup=max(2, iters // 6))
    # what the library would run without a table entry: a tuned entry is never worse than that
    derived = [ev.ops.derive_config(m, n, k).to_dict()]
    if n_key >= 512:
        # far beyond the general kernel's range: the many-token kernel and the streaming kernel
        # with eight token tiles per pass are timed exhaustively, nothing is bred
        scored = sorted((ev(c), json.dumps(c, sort_keys=True)) for c in tiled_space(m, n_key, k) + mid_space(m, n_key, k) + derived)
        log(f"  many-token + streaming kernel: {len(scored)} configs, best {scored[0][0]:.2f} us {scored[0][1]}")
        return json.loads(scored[0][1]), scored[0][0]
    pool = seeds(m, n_key, k)
    rng.shuffle(pool)
    pool = pool[:max_seed_evals] + lean_space(m, n_key, k) + mid_space(m, n_key, k) + tiled_space(m, n_key, k) + derived
    # the winners of the other token buckets of this (m, k), where they are valid here: a config tuned
    # for 16 tokens also runs one token, and is sometimes what the bucket should have
    pool += [c for c in (repair(dict(e), m, n_key, k) for e in extra) if c is not None]
    for c in narrow_space(m, n_key, k):     # a kernel family of its own: timed, not bred
        ev(c)
    scored = sorted(((ev(c), json.dumps(c, sort_keys=True)) for c in pool))
    pop = [json.loads(s) for _, s in scored[:population]]
    log(f"  seeds: {len(pool)} evaluated, best {scored[0][0]:.2f} us {scored[0][1]}")
    for gen in range(generations):
        children = []
        tries = 0
        while len(children) < population and tries < population * 20:
            tries += 1
            a = min(rng.sample(pop, min(3, len(pop))), key=ev)
            if rng.random() < 0.4 and len(pop) > 1:
                b = min(rng.sample(pop, min(3, len(pop))), key=ev)
                child = crossover(a, b, rng, m, n_key, k)
                if child is not None and rng.random() < 0.5:
                    child = mutate(child, rng, m, n_key, k)
            else:
                child = mutate(a, rng, m, n_key, k)
            if child is not None and json.dumps(child, sort_keys=True) not in ev.cache:
                children.append(child)
        for c in children:
            ev(c)
        allc = sorted(((t, s) for s, t in ev.cache.items()))
        pop = [json.loads(s) for _, s in allc[:population]]
        log(f"  gen {gen}: {len(children)} new, best {allc[0][0]:.2f} us {allc[0][1]}")
    for c in tiled_space(m, n_key, k):      # the other kernel family: timed exhaustively
        ev(c)
    best_t, best_s = min(((t, s) for s, t in ev.cache.items()))
    # re-time the top few with more iterations to pick a stable winner
    top = sorted(((t, s) for s, t in ev.cache.items()))[:5]
    ev2 = Evaluator.__new__(Evaluator)
    ev2.__dict__.update(ev.__dict__)
    ev2.cache, ev2.iters, ev2.warmup = {}, 5 * iters, max(2, iters // 2)
    final = sorted((ev2(json.loads(s)), s) for _, s in top)
    log(f"  final: {final[0][0]:.2f} us {final[0][1]}  ({len(ev.cache)} configs tried)")
    return json.loads(final[0][1]), final[0][0]


def blockwise_space(m: int, n_key: int, k: int, bs: int, row_entries=()):
    """Every config of the GEMM with a scale per `bs` weights worth timing for the shape and token bucket: the
    narrow-row variants, the batched kernel's workgroup shapes, the streaming kernel's scale-block twin (workgroup
    shapes of the per-row table's entries for the shape, `row_entries`, and the plain 4 x 4 / 2 x 8 / 8 x 2 ones) and,
    from 32 tokens, the many-token tiles with their k splits.  Small enough to time exhaustively."""
    lo, _ = make_configs.N_BUCKETS[n_key]
    out = []

    def add(c):
        c = dict(c)
        c.setdefault("k_stagger", 0)
        c.setdefault("lds_tile_rows", 0)
        try:
            make_configs.validate_blockwise(m, n_key, k, bs, c)
        except ValueError:
            return
        out.append(c)

    for rows, wk, u, tt in sorted(make_configs.BLOCKWISE_NARROW):
        if tt == 2 and lo <= 16:
            continue
        add(dict(rows_per_wave=rows, waves_m=0 if rows == 64 else 1, waves_k=wk, split_k=1, prefetch=u, x_chunk=512, token_tiles=tt,
                 xcd_swizzle=0))
    for wm in (4, 2, 1):
        for u in (2, 4):
            add(dict(rows_per_wave=64, waves_m=wm, waves_k=16 // wm, split_k=0, prefetch=u, x_chunk=512, token_tiles=1, xcd_swizzle=0))
    if lo <= 64:
        tiles = 4 if lo > 32 else 2 if lo > 16 else 1
        shapes = {(4, 4), (2, 8), (8, 2), (4, 2), (2, 4), (8, 1), (16, 1)}
        shapes |= {(e["waves_m"], e["waves_k"]) for e in row_entries if e.get("rows_per_wave") == 64 and e.get("waves_m", 0) >= 1}
        for wm, wk in sorted(shapes):
            if wm * wk not in (8, 16) or (tiles == 4 and wm * wk != 8):
                continue
            for u in (2, 4):
                for xc in (256, 512, 1024):
                    for stg in (0, 1, 3):
                        add(dict(rows_per_wave=64, waves_m=wm, waves_k=wk, split_k=1, prefetch=u, x_chunk=xc, token_tiles=tiles,
                                 xcd_swizzle=1, k_stagger=stg))
    if lo >= 32:
        steps = -(-k // 64)
        for rows, tokens in sorted(make_configs.BLOCKWISE_TILED):
            if tokens > max(64, 2 * lo):
                continue
            tiles_n = -(-m // rows) * -(-lo // tokens)
            for split in (1, 2, 3, 4, 6, 8, 12, 16):
                if split > 1 and (steps // split < 4 or tiles_n * split > 4 * N_CU):
                    continue
                add(dict(rows_per_wave=64, waves_m=1, waves_k=1, split_k=split, prefetch=2, x_chunk=64, token_tiles=tokens // 16,
                         xcd_swizzle=0, lds_tile_rows=rows))
    uniq = {json.dumps(c, sort_keys=True): c for c in out}
    return list(uniq.values())


class BlockwiseEvaluator:
    """Times blockwise configs for one shape on the GPU over rotating weight sets (tuna_time_matmul_blockwise)."""

    def __init__(self, m, n, k, bs, iters=60, warmup=10):
        import torch

        from . import ops, synth
        from .quantize import nf4_codebook

        self.ops = ops
        self.m, self.n, self.k, self.bs = m, n, k, bs
        self.iters, self.warmup = iters, warmup
        dev = torch.device("cuda")
        n_sets = max(2, min(-(-(512 << 20) // (m * k // 2)), 32))
        self.qs = [synth.make_weights_torch(m, k, 777 + i, dev)[0] for i in range(n_sets)]
        self.scales = [torch.rand((m, k // bs), dtype=torch.float32, device=dev) * 0.015 + 0.005 for _ in range(n_sets)]
        self.x = synth.make_x_torch(n, k, 1, dev)
        self.code = nf4_codebook(dev)
        self.out = torch.empty((n, m), dtype=torch.float16, device=dev)
        self.cache = {}

    def __call__(self, c) -> float:
        key = "derived" if c is None else json.dumps(c, sort_keys=True)
        if key not in self.cache:
            cfg = None if c is None else self.ops.GemmConfig.from_dict(c)
            try:
                best = float("inf")
                for _ in range(2):
                    ms = self.ops.time_matmul_blockwise(self.qs, self.scales, self.x, self.code, self.out, self.m, self.n, self.k,
                                                        self.bs, config=cfg, warmup=self.warmup, iters=self.iters, use_graph=True)
                    best = min(best, ms * 1000.0 / self.iters)
                self.cache[key] = best
            except self.ops.TunaError:
                self.cache[key] = float("inf")
        return self.cache[key]


def tune_blockwise(m, n, k, bs, row_entries=(), iters=60, log=print):
    """Best blockwise config for the shape, its time, and the time of the config the library derives without a table
    entry: the whole space is timed, the top five again with more launches."""
    n_key = make_configs.bucket_of(n)
    ev = BlockwiseEvaluator(m, n, k, bs, iters=iters, warmup=max(2, iters // 6))
    t_derived = ev(None)
    space = blockwise_space(m, n_key, k, bs, row_entries)
    for c in space:
        ev(c)
    top = sorted((t, s) for s, t in ev.cache.items() if s != "derived")[:5]
    ev2 = BlockwiseEvaluator.__new__(BlockwiseEvaluator)
    ev2.__dict__.update(ev.__dict__)
    ev2.cache, ev2.iters, ev2.warmup = {}, 4 * iters, max(2, iters // 2)
    final = sorted((ev2(json.loads(s)), s) for _, s in top)
    t_derived = min(t_derived, ev2(None))
    log(f"  {len(space)} configs; best {final[0][0]:.2f} us ({make_configs.blockwise_family(json.loads(final[0][1]))}) {final[0][1]}; "
        f"derived {t_derived:.2f} us")
    return json.loads(final[0][1]), final[0][0], t_derived


def main_blockwise(args, shapes, tokens):
    """--block-size: tunes tuna_amd/configs/param_map_blockwise.json, keys "<m>_<n>_<k>_<block_size>".  An entry is
    written only where the tuned config beats the derived one by the replace margin (the derived config needs no
    table entry)."""
    base = args.base if args.base.endswith("_blockwise.json") else os.path.splitext(args.base)[0] + "_blockwise.json"
    param_map, row_map = {}, {}
    if os.path.exists(base):
        with open(base) as f:
            param_map = json.load(f)
    row_base = base.replace("_blockwise.json", ".json")
    if os.path.exists(row_base):
        with open(row_base) as f:
            row_map = json.load(f)
    out = args.out if args.out.endswith("_blockwise.json") else os.path.splitext(args.out)[0] + "_blockwise.json"
    os.makedirs(os.path.dirname(os.path.abspath(out)), exist_ok=True)
    for name, m, k in shapes:
        for n in tokens:
            for bs in args.block_size:
                if k % bs or bs >= k:
                    continue
                t0 = time.time()
                print(f"tuning blockwise {name} m={m} n={n} k={k} block={bs}", flush=True)
                rows = [e for key_, e in row_map.items() if key_.split("_")[0] == str(m) and key_.split("_")[2] == str(k)]
                best, us, t_derived = tune_blockwise(m, n, k, bs, rows, iters=args.iters, log=lambda s_: print(s_, flush=True))
                key = f"{m}_{make_configs.bucket_of(n)}_{k}_{bs}"
                margin = args.replace_margin if args.replace_margin > 0 else 1.0
                if us < margin * t_derived:
                    best = dict(best)
                    best["us"] = round(us, 3)
                    best["us_derived"] = round(t_derived, 3)
                    param_map[key] = best
                    print(f"  -> {key}: {us:.2f} us against {t_derived:.2f} derived ({time.time() - t0:.0f} s)", flush=True)
                else:
                    param_map.pop(key, None)
                    print(f"  -> {key}: the derived config stays ({t_derived:.2f} us; best timed {us:.2f})", flush=True)
                with open(out, "w") as f:
                    json.dump(param_map, f, indent=1, sort_keys=True)


def next_from_samples(n_key: int, keys_present=()):
    """Token counts inside an entry's range at which the entry is timed against the next one of its shape."""
    lo, hi = make_configs.key_range(n_key, keys_present)
    if lo == 1:
        return [2, 4, 6, 8, 10, 12, 15]
    span = hi - lo
    # the quarter points, and the first count past every multiple of 16 (32 in the wide ranges) tokens: a launch in
    # chunks of token tiles gains a chunk there, which is where one entry overtakes the other
    step = 16 if span <= 128 else 32
    while span // step > 8:
        step *= 2
    edges = {v + 1 for v in range((lo // step + 1) * step, hi, step)}
    return sorted({lo + 1, lo + span // 4, lo + span // 2, lo + 3 * span // 4, hi} | edges)


def tune_next_from(param_map, keys, iters=40, margin=0.98, log=print):
    """Writes "next_from" into the entries `keys` of param_map: the smallest sampled token count from which the next
    entry of the shape is faster than the entry itself (by the margin) at that count and at every larger sample of
    the entry's range; n_hi + 1 where it never is.  The last entry of a shape, and an entry whose range is not
    followed directly by another entry's, are left alone."""
    for key in keys:
        m, nk, k = (int(t) for t in key.split("_"))
        present = make_configs.keys_of_shape(param_map, m, k)
        lo, hi = make_configs.key_range(nk, present)
        later = [p for p in present if p > nk]
        if not later or make_configs.key_range(min(later), present)[0] != hi + 1:
            continue
        nxt_key = f"{m}_{min(later)}_{k}"
        own = {f: param_map[key].get(f, 0) for f in make_configs.FIELDS}
        nxt = {f: param_map[nxt_key].get(f, 0) for f in make_configs.FIELDS}
        if own == nxt:
            param_map[key].pop("next_from", None)
            continue
        rows = []
        for n in next_from_samples(nk, present):
            ev = Evaluator(m, n, k, iters=max(10, iters // 4) if n >= 256 else iters, warmup=5)
            t_own, t_nxt = ev(own), ev(nxt)
            ev.cache.clear()
            t_own, t_nxt = min(t_own, ev(own)), min(t_nxt, ev(nxt))
            rows.append((n, t_own, t_nxt))
            del ev
        nf = hi + 1
        for n, t_own, t_nxt in reversed(rows):
            if t_nxt < margin * t_own:
                nf = n
            else:
                break
        if rows and nf == rows[0][0]:
            nf = lo + 1
        param_map[key]["next_from"] = int(nf)
        log(f"{key}: next_from {nf}  " + "  ".join(f"n={n}: {a:.2f}/{b:.2f}" for n, a, b in rows))


def derived_stretch(rows, hi, margin):
    """rows: (token count, us with the table's config, us with the derived one) in ascending counts.  The longest run
    of consecutive rows whose derived time is below margin x the table's, as (first count of the run, first count
    after it - hi + 1 when the run reaches the last row); None without such a row."""
    best, i = None, 0
    while i < len(rows):
        j = i
        while j < len(rows) and rows[j][2] < margin * rows[j][1]:
            j += 1
        if j > i and (best is None or j - i > best[1] - best[0]):
            best = (i, j)
        i = max(j, i + 1)
    if best is None:
        return None
    return int(rows[best[0]][0]), int(rows[best[1]][0]) if best[1] < len(rows) else hi + 1


def tune_derived_range(param_map, keys, iters=40, margin=0.95, log=print):
    """Writes "derived_from" / "derived_to" into the entries `keys` of param_map: the longest stretch of sampled token
    counts of the entry's range (above 64 tokens) at which the library's derived config takes less than `margin` of
    the time of what the table hands out there (the entry, or from its next_from on the next one) - from the first
    such sample to the first sample after the stretch that does not.  Entries without such a stretch lose the
    fields.  Shapes of fewer than 24576 rows are skipped above 512 tokens, where the lookup derives already, and every
    shape's open-ended last bucket.  The
    derived configs are the loaded library's: run this again after a change to its derivation rules."""
    from . import ops
    F = make_configs.FIELDS
    for key in keys:
        m, nk, k = (int(t) for t in key.split("_"))
        present = make_configs.keys_of_shape(param_map, m, k)
        lo, hi = make_configs.key_range(nk, present)
        param_map[key].pop("derived_from", None)
        param_map[key].pop("derived_to", None)
        if hi <= 64 or hi >= 128000 or (lo >= 512 and m < 24576):
            continue
        own = {f: param_map[key].get(f, 0) for f in F}
        nf = make_configs.next_from_of(nk, param_map[key], present)
        later = [p for p in present if p > nk]
        nxt = None
        if later and make_configs.key_range(min(later), present)[0] == hi + 1:
            nxt = {f: param_map[f"{m}_{min(later)}_{k}"].get(f, 0) for f in F}
        samples = [n for n in next_from_samples(nk, present) if n > 64 and not (n > 512 and m < 24576)]
        rows = []
        for n in samples:
            table = own
            if nxt is not None and n >= nf:
                try:
                    ops.validate_config(m, n, k, ops.GemmConfig.from_dict(nxt))
                    table = nxt
                except ops.TunaError:
                    pass
            derived = ops.derive_config(m, n, k).to_dict()
            if derived == table:
                rows.append((n, 0.0, 0.0))
                continue
            ev = Evaluator(m, n, k, iters=max(10, iters // 4) if n >= 256 else iters, warmup=5)
            t_tab, t_der = ev(table), ev(derived)
            ev.cache.clear()
            t_tab, t_der = min(t_tab, ev(table)), min(t_der, ev(derived))
            rows.append((n, t_tab, t_der))
            del ev
        best = derived_stretch(rows, hi, margin)
        if best is not None:
            param_map[key]["derived_from"], param_map[key]["derived_to"] = best
        log(f"{key}: derived " + (f"{best[0]}..{best[1] - 1}" if best else "nowhere")
            + "  " + "  ".join(f"n={n}: {a:.2f}/{b:.2f}" for n, a, b in rows))


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--shapes", default="all", help="comma list of shape names or 'all' or 'MxK,...'")
    ap.add_argument("--tokens", default="16", help="comma list of token counts (one per bucket to tune)")
    ap.add_argument("--generations", type=int, default=6)
    ap.add_argument("--population", type=int, default=24)
    ap.add_argument("--max-seed-evals", type=int, default=120)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--iters", type=int, default=60, help="timed launches per candidate (fewer for large token counts)")
    ap.add_argument("--base", default=os.path.join(HERE, "configs", "param_map.json"),
                    help="existing param_map.json to update")
    ap.add_argument("--out", default="tuned/param_map.json")
    ap.add_argument("--replace-margin", type=float, default=0.98,
                    help="an entry of --base is replaced only if the new config takes less than this fraction of its "
                         "time, both timed on this box (0: always replace)")
    ap.add_argument("--eval", default=None, help="JSON config: just time it on the given shapes and exit")
    ap.add_argument("--sub-keys", action="store_true",
                    help="token counts that are keys inside a bucket (24, 48, 96, 192, 384) get an entry of their own "
                         "for the upper part of the bucket, where it beats the lookup without it by --sub-key-margin")
    ap.add_argument("--sub-key-margin", type=float, default=0.95)
    ap.add_argument("--next-from", action="store_true",
                    help="instead of tuning configs: time every entry of --base for the given shapes (all token buckets) "
                         "against the next bucket's entry at several counts inside its bucket and write the hand-over "
                         "count (\"next_from\") into --out")
    ap.add_argument("--derived-range", action="store_true",
                    help="instead of tuning configs: time what the table of --base hands out for the given shapes (all "
                         "token buckets above 64 tokens) against the library's derived config at several counts inside "
                         "each bucket and write the stretch where the derived one wins (\"derived_from\", "
                         "\"derived_to\") into --out; run after --next-from")
    ap.add_argument("--block-size", default=None,
                    help="comma list of scale-block sizes (64, 128, ...): tune the blockwise GEMM's table "
                         "(param_map_blockwise.json beside --base / --out) instead of the per-row one")
    args = ap.parse_args(argv)

    shapes = []
    for tok in (SHAPES if args.shapes == "all" else args.shapes.split(",")):
        if tok in SHAPES:
            shapes.append((tok,) + SHAPES[tok])
        else:
            mm, kk = tok.lower().split("x")
            shapes.append((tok, int(mm), int(kk)))
    tokens = [int(t) for t in args.tokens.split(",")]

    if args.block_size:
        args.block_size = [int(t) for t in args.block_size.split(",")]
        return main_blockwise(args, shapes, tokens)

    if args.next_from or args.derived_range:
        with open(args.base) as f:
            param_map = json.load(f)
        os.makedirs(os.path.dirname(os.path.abspath(args.out)), exist_ok=True)
        for name, m, k in shapes:
            keys = sorted((key for key in param_map if key.split("_")[0] == str(m) and key.split("_")[2] == str(k)),
                          key=lambda s_: int(s_.split("_")[1]))
            if args.next_from:
                tune_next_from(param_map, keys, iters=args.iters, log=lambda s_: print(s_, flush=True))
            if args.derived_range:
                tune_derived_range(param_map, keys, iters=args.iters, log=lambda s_: print(s_, flush=True))
            with open(args.out, "w") as f:
                json.dump(param_map, f, indent=1, sort_keys=True)
        return

    if args.eval:
        c0 = json.loads(args.eval)
        for name, m, k in shapes:
            for n in tokens:
                c = repair(c0, m, make_configs.bucket_of(n), k)
                if c is None:
                    print(f"{name} n={n}: invalid")
                    continue
                t = Evaluator(m, n, k, iters=200, warmup=20)(c)
                print(f"{name} n={n}: {t:.2f} us  {m * k / 2 / t / 1e3:.0f} GB/s  {json.dumps(c)}", flush=True)
        return

    param_map = {}
    if args.base and os.path.exists(args.base):
        with open(args.base) as f:
            param_map = json.load(f)
    os.makedirs(os.path.dirname(os.path.abspath(args.out)), exist_ok=True)
    for name, m, k in shapes:
        for n in tokens:
            t0 = time.time()
            print(f"tuning {name} m={m} n={n} k={k}", flush=True)
            others = [{f: e.get(f, 0) for f in make_configs.FIELDS} for key_, e in param_map.items()
                      if key_.split("_")[0] == str(m) and key_.split("_")[2] == str(k)]
            best, us = tune_shape(m, n, k, args.generations, args.population, args.seed,
                                  log=lambda s: print(s, flush=True), max_seed_evals=args.max_seed_evals,
                                  iters=args.iters, extra=others)
            key = f"{m}_{make_configs.bucket_of(n)}_{k}"
            if args.sub_keys and n in make_configs.SUB_KEYS:
                # an entry of its own for the upper part of the bucket: only where it beats what the lookup hands
                # out at this count without it (the bucket's entry, or the next bucket's) by the margin
                key = f"{m}_{n}_{k}"
                if key not in param_map:
                    from . import ops
                    ev = Evaluator(m, n, k, iters=max(100, 2 * args.iters), warmup=15)
                    c_sel = ops.select_config(m, n, k)[0].to_dict()
                    t_old, t_new = ev(c_sel), ev(dict(best))
                    ev.cache.clear()
                    t_old, t_new = min(t_old, ev(c_sel)), min(t_new, ev(dict(best)))
                    print(f"  lookup without the entry {t_old:.2f} us, new config {t_new:.2f} us on this box", flush=True)
                    if not t_new < args.sub_key_margin * t_old:
                        print(f"  -> {key}: no entry", flush=True)
                        continue
                    us = t_new
            old = param_map.get(key)
            if old is not None and args.replace_margin > 0:
                # Boxes differ by several per cent, so a time recorded with the existing entry says
                # little: the entry is re-timed here, on this box, and kept unless the new config
                # beats it by the margin.
                c_old = {f: old.get(f, 0) for f in make_configs.FIELDS}
                if c_old != {f: best.get(f, 0) for f in make_configs.FIELDS}:
                    ev = Evaluator(m, n, k, iters=max(100, 2 * args.iters), warmup=15)
                    t_old, t_new = ev(c_old), ev(dict(best))
                    ev.cache.clear()
                    t_old, t_new = min(t_old, ev(c_old)), min(t_new, ev(dict(best)))
                    print(f"  existing entry {t_old:.2f} us, new config {t_new:.2f} us on this box", flush=True)
                    if not t_new < args.replace_margin * t_old:
                        print(f"  -> {key}: existing entry kept", flush=True)
                        continue
                    us = t_new
            best = dict(best)
            best["us"] = round(us, 3)
            best["gbs"] = round(m * k / 2 / us / 1e3, 1)
            param_map[key] = best
            with open(args.out, "w") as f:
                json.dump(param_map, f, indent=1, sort_keys=True)
            print(f"  -> {key}: {us:.2f} us, {best['gbs']} GB/s ({time.time() - t0:.0f} s)", flush=True)


if __name__ == "__main__":
    sys.exit(main())
