"""CPU tests of the host side: C ABI surface, config table / generator / validation, tuner's
search-space helpers, quantizer + packer, error behaviour without a GPU."""
import ctypes
import json
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header_name):
    return set(re.findall(r"\b(tuna_[a-z0-9_]+)\s*\(", open(os.path.join(ROOT, "include", header_name)).read()))


def _exported(path):
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", path], check=True, capture_output=True, text=True).stdout
    return {line.split()[-1] for line in out.splitlines() if line.strip()}


def test_product_library_exports_exactly_what_its_header_declares():
    """libtuna_amd.so: every symbol include/tuna_amd.h declares and not one dynamic symbol more - no timing loops,
    no yardstick kernels, no process-wide switches, no kernel launch stubs."""
    from tuna_amd import _lib

    L = _lib._load("product")
    declared = _declared("tuna_amd.h")
    assert declared, "no declarations parsed"
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    for name in declared:
        assert hasattr(L, name), name
    assert _exported(_lib.LIB_PATH) == declared, _exported(_lib.LIB_PATH) ^ declared
    assert L.tuna_version() == 100
    assert L.tuna_status_string(0) == b"ok"
    assert L.tuna_status_string(2) == b"unsupported shape or config"


def test_diagnostic_build_exports_the_product_abi_plus_its_own_header():
    from tuna_amd import _lib

    L = _lib.bench_lib()
    bench_only = _declared("tuna_amd_bench.h")
    assert bench_only == set(_lib.BENCH_SIGNATURES), bench_only ^ set(_lib.BENCH_SIGNATURES)
    assert not bench_only & _declared("tuna_amd.h")
    for name in bench_only | set(_lib.SIGNATURES):
        assert hasattr(L, name), name
    assert _exported(_lib.BENCH_LIB_PATH) == bench_only | _declared("tuna_amd.h")
    # the switches apply to ops while the diagnostic build is the active library, and only then
    assert _lib.lib() is _lib._load("product")
    with _lib.diagnostic_build() as D:
        assert _lib.lib() is D is L
        prev = D.tuna_set_lean_kernels(0)
        assert D.tuna_set_lean_kernels(prev) == 0
    assert _lib.lib() is _lib._load("product")


def test_config_struct_matches_header():
    from tuna_amd._lib import GemmConfig

    header = open(os.path.join(ROOT, "include", "tuna_amd.h")).read()
    body = header[header.index("typedef struct tuna_gemm_config"):header.index("} tuna_gemm_config;")]
    fields = re.findall(r"int32_t\s+([a-z_]+);", body)
    assert tuple(fields) == GemmConfig.FIELDS
    assert ctypes.sizeof(GemmConfig) == 4 * len(fields)


def test_select_config_is_host_only_and_every_table_entry_validates():
    from tuna_amd import make_configs, ops

    table = ops.config_table()
    next_from = ops.config_table_next_from()
    with open(os.path.join(ROOT, "tuna_amd", "configs", "param_map.json")) as f:
        pm = json.load(f)
    derived_ranges = ops.config_table_derived_ranges()
    assert len(table) == len(pm) == len(next_from) == len(derived_ranges)
    assert sum(r != (0, 0) for r in derived_ranges) >= 1
    for (m, lo, hi, k, cfg), nf, (d_from, d_to) in zip(table, next_from, derived_ranges):
        # an entry's key is the lower edge of its range: a bucket key, or a key inside a bucket (which ends the
        # range of the bucket's own entry one token earlier)
        present = make_configs.keys_of_shape(pm, m, k)
        n_key = make_configs.key_of(lo, present)
        key = f"{m}_{n_key}_{k}"
        assert key in pm and (lo, hi) == make_configs.key_range(n_key, present)
        assert n_key == (lo if lo in make_configs.SUB_KEYS else make_configs.bucket_of(lo))
        assert cfg.to_dict() == {f: pm[key][f] for f in cfg.FIELDS}
        assert nf == make_configs.next_from_of(n_key, pm[key], present) and lo < nf <= hi + 1
        # the stretch of the range, if any, where the tuner timed the derived config ahead of the table's
        assert (d_from, d_to) == make_configs.derived_range_of(n_key, pm[key], present)
        assert (d_from, d_to) == (0, 0) or max(lo, 65) <= d_from < d_to <= hi + 1
        inside = {d_from, d_to - 1, max(d_from - 1, lo), min(d_to, hi)} if d_to else set()
        for n in sorted({lo, hi, min(nf, hi), max(nf - 1, lo)} | inside):
            ops.validate_config(m, n, k, cfg)                      # the C side accepts it
            got, hit = ops.select_config(m, n, k)
            assert hit
            # entries are tuned at their bucket's lower edge: counts from the entry's next_from on take the next
            # bucket's entry (fewer passes over the weights) where that one can run n tokens
            eff, eff_lo = cfg.to_dict(), lo
            nxt = pm.get(f"{m}_{make_configs.key_of(hi + 1, present)}_{k}") if n >= nf and hi < 128000 else None
            if nxt is not None:
                nxt_cfg = {f: nxt[f] for f in cfg.FIELDS}
                try:
                    ops.validate_config(m, n, k, ops.GemmConfig.from_dict(nxt_cfg))
                    eff, eff_lo = nxt_cfg, hi + 1
                except ops.TunaError:
                    pass      # (passed over only because it cannot run n tokens)
            # above 512 tokens the entries are tuned at 512, 1024 and 2048 tokens: away from those counts (another
            # number of 128-token tiles) a shape of fewer than 24576 rows takes the pick of the derivation's cost
            # model - far into the open-ended last bucket the 256 x 256 tile
            tuned_at = 512 if eff_lo <= 512 else 1024 if eff_lo <= 769 else 2048
            if (n > 512 and m < 24576 and -(-n // 128) != -(-tuned_at // 128)) or d_from <= n < d_to:
                assert got.to_dict() == ops.derive_config(m, n, k).to_dict()
                if n >= 3000:
                    assert (got.lds_tile_rows, got.token_tiles, got.split_k, got.rows_per_wave) == (256, 16, 1, 64)
                ops.validate_config(m, n, k, got)
            else:
                assert got.to_dict() == eff
        make_configs.validate(m, n_key, k, cfg.to_dict())  # and the generator's twin
        lds, ws = ops.config_footprint(m, lo, k, cfg)
        assert lds == make_configs.lds_bytes(cfg.to_dict()) and lds <= 160 * 1024


@pytest.mark.parametrize("shape", [(8, 1, 8), (64, 16, 64), (4096, 16, 4104), (1000 * 8, 3, 40), (12288, 100, 4096),
                                   (8192, 256, 8192), (8192, 4096, 1024), (229376, 128, 4096), (65536, 300, 4096), (24576, 256, 1024), (24576, 2000, 1024), (32768, 50, 2048), (16384, 100, 8192), (12288, 128, 4096)])
def test_derived_config_is_valid_for_any_shape(shape):
    from tuna_amd import ops

    cfg, _ = ops.select_config(*shape)
    ops.validate_config(*shape, cfg)
    lds, ws = ops.config_footprint(*shape, cfg)
    assert 0 < lds <= 160 * 1024


def test_derived_and_looked_up_configs_are_valid_on_a_sweep_of_shapes_and_token_counts():
    """The rules and the grid cost model behind tuna_select_config, on 4000 seeded shapes (every kind of m and k the
    kernels treat differently: multiples of 8, 64, 256, 512) x token counts from 1 to 5000, and on every table shape x
    150 token counts: each pick passes the library's own validator, fits the LDS, and is what a second call returns;
    the blockwise derivation likewise where the shape admits scale blocks."""
    import json

    import numpy as np

    from tuna_amd import ops

    rng = np.random.default_rng(20241125)
    cases = []
    for _ in range(4000):
        step = int(rng.choice([8, 64, 256, 512]))
        m = int(rng.integers(1, 131072 // step)) * step if rng.random() < 0.3 else int(rng.integers(1, 24576 // step)) * step
        ks = int(rng.choice([8, 64, 256, 512]))
        k = int(rng.integers(1, 16384 // ks)) * ks
        n = int(rng.choice([rng.integers(1, 17), rng.integers(17, 65), rng.integers(65, 256), rng.integers(256, 1025), rng.integers(1025, 5000)]))
        if m * k // 2 < (1 << 32):
            cases.append((m, n, k))
    with open(os.path.join(ROOT, "tuna_amd", "configs", "param_map.json")) as f:
        pairs = sorted({(int(key.split("_")[0]), int(key.split("_")[2])) for key in json.load(f)})
    for (m, k) in pairs:
        cases += [(m, int(n), k) for n in rng.integers(1, 4200, size=150)]
    for (m, n, k) in cases:
        cfg, hit = ops.select_config(m, n, k)
        ops.validate_config(m, n, k, cfg)
        lds, ws = ops.config_footprint(m, n, k, cfg)
        assert 0 < lds <= 160 * 1024, (m, n, k, cfg.to_dict())
        again, hit2 = ops.select_config(m, n, k)
        assert again.to_dict() == cfg.to_dict() and hit2 == hit
        if m % 16 == 0 and k % 256 == 0 and k > 64 and n % 7 == 0:
            bcfg, _ = ops.select_config_blockwise(m, n, k, 64)
            ops.validate_config_blockwise(m, n, k, 64, bcfg)


def test_token_buckets_follow_the_reference_dispatcher():
    from tuna_amd import make_configs as mc

    edges = {1: (1, 15), 16: (16, 31), 32: (32, 63), 64: (64, 127), 128: (128, 255), 256: (256, 511),
             512: (512, 768), 1024: (769, 1024), 2048: (1025, 128000)}
    assert mc.N_BUCKETS == edges
    for n, want in [(1, 1), (15, 1), (16, 16), (31, 16), (32, 32), (768, 512), (769, 1024), (1025, 2048),
                    (128000, 2048)]:
        assert mc.bucket_of(n) == want
    with pytest.raises(ValueError):
        mc.bucket_of(128001)
    # keys inside a bucket (this table's own): m_<sub>_k covers sub .. the bucket's upper edge, and the bucket's entry
    # then ends at sub - 1; shapes without such an entry keep the reference's ranges
    assert mc.SUB_KEYS == {24: 16, 48: 32, 96: 64, 192: 128, 384: 256}
    assert mc.key_range(256, [1, 16, 256, 512]) == (256, 511) and mc.key_range(256, [256, 384, 512]) == (256, 383)
    assert mc.key_range(384, [256, 384, 512]) == (384, 511)
    assert mc.key_of(383, [256, 384]) == 256 and mc.key_of(384, [256, 384]) == 384 and mc.key_of(400, [256]) == 256
    assert mc.default_next_from(256, [256, 384]) == 384 and mc.default_next_from(384, [256, 384]) == 512
    assert mc.default_next_from(64, [64]) == 65 and mc.default_next_from(64, [64, 96]) == 96


def test_invalid_configs_are_rejected_by_both_validators():
    from tuna_amd import make_configs as mc
    from tuna_amd import ops

    good = dict(rows_per_wave=64, waves_m=2, waves_k=4, split_k=2, prefetch=4, x_chunk=512, token_tiles=1,
                xcd_swizzle=0)
    ops.validate_config(4096, 16, 4096, ops.GemmConfig.from_dict(good))
    mc.validate(4096, 16, 4096, good)
    bad = [dict(rows_per_wave=96), dict(prefetch=3), dict(token_tiles=3), dict(waves_m=0), dict(waves_k=3), dict(waves_k=32),
           dict(waves_m=8, waves_k=4), dict(split_k=-1), dict(split_k=129), dict(x_chunk=500), dict(x_chunk=256),
           dict(x_chunk=1 << 16), dict(rows_per_wave=256, prefetch=8)]
    for delta in bad:
        c = dict(good, **delta)
        with pytest.raises(ops.TunaError):
            ops.validate_config(4096, 16, 4096, ops.GemmConfig.from_dict(c))
        with pytest.raises(ValueError):
            mc.validate(4096, 16, 4096, c)
    for m, n, k in [(4100, 16, 4096), (4096, 16, 4100), (0, 16, 8), (8, 0, 8)]:
        with pytest.raises(ops.TunaError):
            ops.validate_config(m, n, k, ops.GemmConfig.from_dict(good))


def test_generator_output_and_its_refusal_of_inconsistent_entries(tmp_path):
    from tuna_amd import make_configs as mc

    pm = {"4096_16_4096": dict(rows_per_wave=64, waves_m=1, waves_k=8, split_k=4, prefetch=2, x_chunk=1024,
                               token_tiles=1, xcd_swizzle=1, us=9.9),
          "4096_1_4096": dict(rows_per_wave=64, waves_m=1, waves_k=8, split_k=4, prefetch=2, x_chunk=1024,
                              token_tiles=1, xcd_swizzle=0, k_stagger=3)}
    text = mc.generate(pm)
    # (k_stagger, lds_tile_rows default to 0; next_from, the fifth value, to 17 in the bucket 16..31 and 10 in 1..15)
    assert "{4096, 16, 31, 4096, 17, {64, 1, 8, 4, 2, 1024, 1, 1, 0, 0}}" in text
    assert "{4096, 1, 15, 4096, 10, {64, 1, 8, 4, 2, 1024, 1, 0, 3, 0}}" in text
    assert "kConfigTableSize = 2" in text
    # a tuned hand-over count is emitted as it is, one outside the bucket refused
    assert "{4096, 16, 31, 4096, 25, {" in mc.generate({"4096_16_4096": dict(pm["4096_16_4096"], next_from=25)})
    assert "{4096, 16, 31, 4096, 32, {" in mc.generate({"4096_16_4096": dict(pm["4096_16_4096"], next_from=32)})  # never
    for bad in (16, 33, 0):
        with pytest.raises(ValueError, match="next_from"):
            mc.generate({"4096_16_4096": dict(pm["4096_16_4096"], next_from=bad)})
    # a key inside a bucket: its entry takes the upper part of the bucket, the bucket's own entry the lower part; it
    # needs the bucket's entry, and no other key is accepted
    e16 = pm["4096_16_4096"]
    text = mc.generate({"4096_16_4096": e16, "4096_24_4096": dict(e16, xcd_swizzle=0)})
    assert "{4096, 16, 23, 4096, 24, {64, 1, 8, 4, 2, 1024, 1, 1," in text and "{4096, 24, 31, 4096, 32, {64, 1, 8, 4, 2, 1024, 1, 0," in text
    assert "{4096, 16, 23, 4096, 20, {" in mc.generate({"4096_16_4096": dict(e16, next_from=20), "4096_24_4096": e16})
    with pytest.raises(ValueError, match="next_from"):
        mc.generate({"4096_16_4096": dict(e16, next_from=25), "4096_24_4096": e16})
    with pytest.raises(ValueError, match="needs the bucket's own entry"):
        mc.generate({"4096_24_4096": e16})
    # the stretch of token counts that takes the derived config follows the config in the row; it lies inside the
    # entry's range, above 64 tokens, and its two fields come together
    e64 = dict(e16, token_tiles=1)
    assert "{4096, 64, 127, 4096, 65, {64, 1, 8, 4, 2, 1024, 1, 1, 0, 0}, 65, 81}," in mc.generate({"4096_64_4096": dict(e64, derived_from=65, derived_to=81)})
    assert "0, 0}, 97, 128}," in mc.generate({"4096_64_4096": dict(e64, derived_from=97, derived_to=128)})
    for bad in (dict(derived_from=64, derived_to=80), dict(derived_from=100, derived_to=129), dict(derived_from=90, derived_to=90), dict(derived_from=70)):
        with pytest.raises(ValueError, match="derived"):
            mc.generate({"4096_64_4096": dict(e64, **bad)})
    with pytest.raises(ValueError, match="derived"):
        mc.generate({"4096_16_4096": dict(e16, derived_from=20, derived_to=24)})
    with pytest.raises(ValueError, match="not a bucket key"):
        mc.generate({"4096_20_4096": e16})
    # the checked-in table is what the generator produces from the checked-in json
    with open(os.path.join(ROOT, "tuna_amd", "configs", "param_map.json")) as f:
        real = json.load(f)
    with open(os.path.join(ROOT, "tuna_amd", "configs", "param_map_blockwise.json")) as f:
        real_blk = json.load(f)
    with open(os.path.join(ROOT, "tuna_amd", "csrc", "config_table.cpp")) as f:
        assert f.read() == mc.generate(real) + mc.generate_blockwise(real_blk)
    # blockwise entries: the config names the kernel family; inconsistent ones are refused with their key
    blk = {"8192_16_8192_64": dict(rows_per_wave=64, waves_m=0, waves_k=8, split_k=1, prefetch=4, x_chunk=512, token_tiles=1, xcd_swizzle=0),
           "57344_16_8192_64": dict(rows_per_wave=64, waves_m=4, waves_k=4, split_k=1, prefetch=4, x_chunk=512, token_tiles=1, xcd_swizzle=1,
                                    k_stagger=5),
           "8192_16_28672_128": dict(rows_per_wave=64, waves_m=4, waves_k=4, split_k=0, prefetch=2, x_chunk=512, token_tiles=1, xcd_swizzle=0),
           "4096_64_4096_64": dict(rows_per_wave=64, waves_m=1, waves_k=1, split_k=2, prefetch=2, x_chunk=64, token_tiles=4, xcd_swizzle=0,
                                   lds_tile_rows=256)}
    text = mc.generate_blockwise(blk)
    assert "{8192, 16, 31, 8192, 64, {64, 0, 8, 1, 4, 512, 1, 0, 0, 0}},  // 8192_16_8192_64: narrow" in text
    assert "// 57344_16_8192_64: streaming" in text and "// 8192_16_28672_128: batched" in text and "// 4096_64_4096_64: many-token" in text
    assert "kBlockwiseTableSize = 4" in text
    for bad_key, bad in (("8192_16_8192_96", blk["8192_16_8192_64"]),                                   # not a power of two
                         ("8192_16_8192_64", dict(blk["8192_16_8192_64"], waves_k=2)),                   # no such narrow variant
                         ("4096_64_4096_64", dict(blk["4096_64_4096_64"], token_tiles=16)),              # the 256 x 256 tile has no scale blocks
                         ("8192_128_8192_64", blk["57344_16_8192_64"])):                                # streaming twin: up to 64 tokens
        with pytest.raises(ValueError, match=bad_key):
            mc.generate_blockwise({bad_key: bad})
    # an entry like the reference's gemm_229376_4096_16 (thread count inconsistent with its warp grid) is refused
    pm["229376_16_4096"] = dict(pm["4096_16_4096"], waves_m=8, waves_k=8)
    with pytest.raises(ValueError, match="229376_16_4096"):
        mc.generate(pm)
    pm.pop("229376_16_4096")
    pm["4096_17_4096"] = pm["4096_16_4096"]  # not a bucket key
    with pytest.raises(ValueError):
        mc.generate(pm)


def test_tuner_repair_seeds_and_mutation_stay_valid():
    import random

    from tuna_amd import make_configs as mc
    from tuna_amd import tuner

    rng = random.Random(0)
    for (m, n, k) in [(4096, 16, 4096), (229376, 16, 4096), (8192, 64, 28672), (8192, 1, 8192)]:
        nk = mc.bucket_of(n)
        pool = tuner.seeds(m, nk, k)
        assert len(pool) > 20
        for c in pool:
            mc.validate(m, nk, k, c)
        c = pool[0]
        for _ in range(200):
            d = tuner.mutate(c, rng, m, nk, k)
            if d is not None:
                mc.validate(m, nk, k, d)
                c = d
            e = tuner.crossover(c, rng.choice(pool), rng, m, nk, k)
            if e is not None:
                mc.validate(m, nk, k, e)
    assert tuner.repair(dict(rows_per_wave=64, waves_m=8, waves_k=8, split_k=1, prefetch=2, x_chunk=512,
                             token_tiles=1, xcd_swizzle=0), 4096, 16, 4096) is None


def test_tuner_hand_over_count_from_timings(monkeypatch):
    """tune_next_from with a stub in place of the GPU evaluator: the hand-over is the smallest sampled count from
    which the next bucket's entry wins at every larger sample, the first count inside the bucket if it wins at all
    of them, none (n_hi + 1) if it loses at the top; identical entries and last-bucket entries are left alone."""
    from tuna_amd import make_configs as mc, tuner

    own = dict(rows_per_wave=64, waves_m=1, waves_k=8, split_k=4, prefetch=2, x_chunk=1024, token_tiles=1, xcd_swizzle=1)
    nxt = dict(own, token_tiles=2, x_chunk=512)
    assert tuner.next_from_samples(64) == [65, 79, 81, 95, 97, 111, 113, 127] and tuner.next_from_samples(1)[0] == 2
    assert all(mc.N_BUCKETS[nk][0] < n <= mc.N_BUCKETS[nk][1] for nk in mc.N_BUCKETS if nk != 2048 for n in tuner.next_from_samples(nk))

    def run(win_from):
        class Stub:
            def __init__(self, m, n, k, iters=0, warmup=0):
                self.n, self.cache = n, {}

            def __call__(self, c):
                is_next = c["token_tiles"] == 2
                return (9.0 if self.n >= win_from else 11.0) if is_next else 10.0

        monkeypatch.setattr(tuner, "Evaluator", Stub)
        pm = {"4096_64_4096": dict(own, us=1.0), "4096_128_4096": dict(nxt), "4096_2048_4096": dict(own)}
        tuner.tune_next_from(pm, list(pm), log=lambda s_: None)
        assert "next_from" not in pm["4096_2048_4096"] and "next_from" not in pm["4096_128_4096"]  # no next entry
        mc.next_from_of(64, pm["4096_64_4096"])  # in range for the generator
        return pm["4096_64_4096"]["next_from"]

    assert run(0) == 65        # the next entry wins everywhere: from the first count inside the bucket
    assert run(95) == 95       # wins from the third sample on
    assert run(127) == 127
    assert run(1000) == 128    # never: n_hi + 1
    pm = {"4096_64_4096": dict(own, next_from=100), "4096_128_4096": dict(own)}
    tuner.tune_next_from(pm, ["4096_64_4096"], log=lambda s_: None)
    assert "next_from" not in pm["4096_64_4096"]  # the same config in both buckets: nothing to hand over
    # with an entry for the upper part of the bucket (key 96): the bucket's entry is sampled in 65..95 and hands over
    # to that entry, which is sampled in 97..127 and hands over to the next bucket's
    assert tuner.next_from_samples(64, [64, 96, 128]) == [65, 71, 79, 81, 87, 95]
    assert tuner.next_from_samples(96, [64, 96, 128]) == [97, 103, 111, 113, 119, 127]
    pm = {"4096_64_4096": dict(own), "4096_96_4096": dict(nxt), "4096_128_4096": dict(own)}
    tuner.tune_next_from(pm, list(pm), log=lambda s_: None)   # (the stub of the last run: two token tiles always lose)
    assert pm["4096_64_4096"]["next_from"] == 96 and pm["4096_96_4096"]["next_from"] == 97
    mc.generate(pm)


def test_tuner_derived_stretch_from_timings(monkeypatch):
    """tune_derived_range with a stub in place of the GPU evaluator: the entry gets the longest run of sampled counts
    at which the derived config is ahead of the table's by the margin, ending at the first sample that is not."""
    from tuna_amd import make_configs as mc, ops, tuner

    rows = [(65, 10, 8), (79, 10, 9.5), (81, 10, 8), (95, 10, 8), (97, 10, 9.2), (111, 10, 11), (127, 10, 9)]
    assert tuner.derived_stretch(rows, 127, 0.93) == (81, 111)
    assert tuner.derived_stretch(rows[:5], 127, 0.93) == (81, 128)        # a run up to the last sample: to the range's end
    assert tuner.derived_stretch(rows, 127, 0.5) is None and tuner.derived_stretch([], 127, 0.93) is None

    own = dict(rows_per_wave=64, waves_m=2, waves_k=8, split_k=1, prefetch=2, x_chunk=512, token_tiles=2, xcd_swizzle=1,
               k_stagger=0, lds_tile_rows=-1)
    wins_below = {"n": 0}

    class Stub:
        def __init__(self, m, n, k, **kw):
            self.n, self.cache = n, {}

        def __call__(self, cfg):   # the table's entries take 10 us; anything else 8 below the set count, 12 from it on
            return 10.0 if cfg == own else (8.0 if self.n < wins_below["n"] else 12.0)

    monkeypatch.setattr(tuner, "Evaluator", Stub)
    pm = {"4096_64_4096": dict(own), "4096_128_4096": dict(own), "4096_32_4096": dict(own, token_tiles=1),
          "4096_2048_4096": dict(own, token_tiles=8, x_chunk=128)}
    wins_below["n"] = 96
    tuner.tune_derived_range(pm, list(pm), log=lambda s_: None)
    derived_differs = ops.derive_config(4096, 80, 4096).to_dict() != own
    assert derived_differs
    assert (pm["4096_64_4096"]["derived_from"], pm["4096_64_4096"]["derived_to"]) == (65, 97)
    assert all("derived_from" not in pm[key_] for key_ in ("4096_128_4096", "4096_32_4096", "4096_2048_4096"))
    assert mc.derived_range_of(64, pm["4096_64_4096"]) == (65, 97)          # in range for the generator
    wins_below["n"] = 0
    tuner.tune_derived_range(pm, list(pm), log=lambda s_: None)
    assert "derived_from" not in pm["4096_64_4096"] and "derived_to" not in pm["4096_64_4096"]   # a stale range goes


def test_tuner_small_launch_config_spaces_are_valid_for_both_validators():
    """The exhaustively timed config spaces of the lean and the narrow-row kernel: every member
    passes the Python validator and the library's, narrow-row members report the footprint the
    twin computes, and the spaces have the members the tuned table relies on."""
    from tuna_amd import make_configs as mc
    from tuna_amd import ops, tuner

    for (m, n, k) in [(4096, 16, 4096), (6144, 1, 4096), (6144, 32, 4096), (8192, 64, 8192), (28672, 16, 4096)]:
        nk = mc.bucket_of(n)
        lean = tuner.lean_space(m, nk, k)
        narrow = tuner.narrow_space(m, nk, k)
        assert narrow and (lean or n >= 64)    # the lean kernel takes 16 tokens per pass: not offered from 64 tokens up
        for c in lean + narrow:
            mc.validate(m, nk, k, c)
            ops.validate_config(m, n, k, ops.GemmConfig.from_dict(c))
        for c in lean:
            assert c["rows_per_wave"] == 64 and c["token_tiles"] == 1 and c["k_stagger"] == 0
            assert c["split_k"] & (c["split_k"] - 1) == 0 and (k // 32) % (c["split_k"] * c["waves_k"] * c["prefetch"]) == 0
        for c in narrow:
            assert mc.is_narrow(c)
            lds, ws = ops.config_footprint(m, n, k, ops.GemmConfig.from_dict(c))
            assert (lds, ws) == (mc.lds_bytes(c), 0)
        tiles = {c["token_tiles"] for c in narrow}
        assert tiles == ({1} if n <= 16 else {1, 2} if n <= 32 else {1, 2, 4})
    # 16 waves x 64 rows x 2 token tiles: 128 KB of reduction planes beside the 64 KB table - refused by both validators
    big = dict(rows_per_wave=64, waves_m=0, waves_k=16, split_k=1, prefetch=2, x_chunk=1024, token_tiles=2, xcd_swizzle=0,
               k_stagger=0, lds_tile_rows=0)
    with pytest.raises(ValueError):
        mc.validate(256, 32, 5120, big)
    with pytest.raises(ops.TunaError):
        ops.validate_config(256, 32, 5120, ops.GemmConfig.from_dict(big))
    # configs only the 17..128-token streaming kernel has (ring 8 with four token tiles, 16 waves with two): valid
    # for both validators while the launch qualifies, refused by both when it does not (too many waves, a split)
    mid = dict(rows_per_wave=64, waves_m=8, waves_k=1, split_k=1, prefetch=8, x_chunk=256, token_tiles=4, xcd_swizzle=0,
               k_stagger=0, lds_tile_rows=0)
    for c, ok in ((mid, True), (dict(mid, waves_m=16, token_tiles=2, prefetch=4), True),
                  (dict(mid, k_stagger=3), True), (dict(mid, waves_m=4, waves_k=4), False), (dict(mid, split_k=2), False)):
        assert mc.mid_applies(229376, 4096, c) == ok
        if ok:
            mc.validate(229376, 64 if c["token_tiles"] == 4 else 32, 4096, c)
            ops.validate_config(229376, 64 if c["token_tiles"] == 4 else 32, 4096, ops.GemmConfig.from_dict(c))
        else:
            with pytest.raises(ValueError):
                mc.validate(229376, 64, 4096, c)
            with pytest.raises(ops.TunaError):
                ops.validate_config(229376, 64, 4096, ops.GemmConfig.from_dict(c))
    space = tuner.mid_space(229376, 64, 4096)
    assert space and all(mc.mid_applies(229376, 4096, c) for c in space)
    # one token tile: offered only where unsplit tiles fill the device (small shapes take the lean or narrow-row kernel)
    assert tuner.mid_space(229376, 16, 4096) and tuner.mid_space(4096, 16, 4096) == []
    # from 128 tokens on: passes of eight token tiles, timed for every larger bucket too
    for n_key in (128, 256, 2048):
        big = tuner.mid_space(57344, n_key, 8192)
        assert big and all(mc.mid_applies(57344, 8192, c) for c in big)
        # 128 and 256 tokens: also passes of 32 and 64 tokens (they share the weights when they all fit the device)
        assert {c["token_tiles"] for c in big} == ({8, 4, 2} if n_key <= 256 else {8, 4})
    # 32 and 64 tokens: also chunks of fewer token tiles than the count needs, side by side
    assert {c["token_tiles"] for c in tuner.mid_space(10240, 32, 8192)} == {2, 1}
    assert {c["token_tiles"] for c in tuner.mid_space(10240, 64, 8192)} == {4, 2, 1}
    # packed weights staged through LDS (lds_tile_rows = -1): offered for 16-wave launches with one token tile, valid
    # for both validators exactly where the twin exists
    sp16 = tuner.mid_space(229376, 16, 4096)
    lds = [c for c in sp16 if c["lds_tile_rows"] == -1]
    assert lds and all(c["waves_m"] * c["waves_k"] == 16 and c["prefetch"] in (2, 4) and c["token_tiles"] == 1 for c in lds)
    for c in lds[:40]:
        mc.validate(229376, 16, 4096, c)
        ops.validate_config(229376, 16, 4096, ops.GemmConfig.from_dict(c))
        assert "weights through LDS" in ops.describe_launch(229376, 16, 4096, ops.GemmConfig.from_dict(c))
    # ... and for the passes of 32 ... 128 tokens (8 or 16 waves, ring 2 or 4; ring 2 with eight token tiles)
    for n_key in (64, 128):
        sp = [c for c in tuner.mid_space(229376, n_key, 4096) if c["lds_tile_rows"] == -1]
        assert sp and all(c["waves_m"] * c["waves_k"] in (8, 16) and c["prefetch"] in (2, 4) for c in sp)
        assert all(c["prefetch"] == 2 for c in sp if c["token_tiles"] == 8)
        for c in sp[:40]:
            mc.validate(229376, n_key, 4096, c)
            ops.validate_config(229376, n_key, 4096, ops.GemmConfig.from_dict(c))
            assert "weights through LDS" in ops.describe_launch(229376, n_key, 4096, ops.GemmConfig.from_dict(c))
    for bad in (dict(lds[0], waves_m=4, waves_k=1), dict(lds[0], prefetch=8, x_chunk=1024), dict(lds[0], token_tiles=8, prefetch=4),
                dict(lds[0], split_k=2), dict(lds[0], lds_tile_rows=-2)):
        with pytest.raises(ValueError):
            mc.validate(229376, 16 if bad["token_tiles"] == 1 else 128, 4096, bad)
        with pytest.raises(ops.TunaError):
            ops.validate_config(229376, 16 if bad["token_tiles"] == 1 else 128, 4096, ops.GemmConfig.from_dict(bad))
    # (narrow-row configs are offered up to the 512-token bucket - token passes side by side - and no further)
    assert tuner.narrow_space(4096, 128, 4096) and tuner.narrow_space(4096, 512, 4096) and tuner.narrow_space(4096, 1024, 4096) == []
    assert tuner.lean_space(4096, 128, 4096) == []
    assert tuner.lean_space(4096, 16, 4104) == []       # k not a multiple of 32: no lean launch


def test_quantizer_matches_nearest_code_and_layout():
    import torch

    from oracle import oracle as O
    from tuna_amd.quantize import quantize_blockwise_dynamic_4bit, unpack_codes

    torch.manual_seed(0)
    m, k = 64, 256
    w = (torch.randn(m, k) * 0.05).half()
    q, (absmax, code) = quantize_blockwise_dynamic_4bit(w, block_size=k, preprocess=True)
    assert q.shape == (m // 8, k // 8, 32) and q.dtype == torch.uint8
    assert absmax.dtype == torch.float32 and absmax.shape == (m,)
    assert torch.equal(absmax, w.abs().amax(dim=1).float())
    codes = unpack_codes(q, m, k).numpy()
    # brute-force nearest entry (lowest index on ties) in float32, like the reference's argmin
    norm = (w / absmax[:, None]).float().numpy()
    cb = O.nf4_codebook()
    want = np.abs(norm[:, :, None] - cb[None, None, :]).argmin(axis=2)
    assert np.array_equal(codes, want)
    # the packed bytes mean the same thing to the oracle
    assert np.array_equal(O.unpack(q.numpy(), m, k), codes)
    # unpacked variant returns flat codes
    flat, _ = quantize_blockwise_dynamic_4bit(w, block_size=k, preprocess=False)
    assert np.array_equal(flat.numpy().reshape(m, k), codes)
    # decoded weights approximate the originals within half the widest code gap times absmax
    img = O.dequant(q.numpy(), absmax.numpy(), cb, m, k, mode=O.D2).view(np.float16).astype(np.float32)
    gap = np.diff(cb).max() / 2
    assert (np.abs(img - w.float().numpy()) <= gap * absmax.numpy()[:, None] + 1e-3).all()


def test_ops_reject_bad_arguments_without_touching_a_gpu():
    import torch

    from tuna_amd import ops

    x = torch.zeros((16, 64), dtype=torch.float16)
    q = torch.zeros((8, 8, 32), dtype=torch.uint8)
    s = torch.ones(64)
    c = torch.zeros(16)
    o = torch.zeros((16, 64), dtype=torch.float16)
    with pytest.raises(ValueError, match="HIP device"):
        ops.matmul(x, q, s, c, o, 64, 16, 64)      # CPU tensors: there is no CPU fallback
    with pytest.raises(ValueError):
        ops.matmul(x, q, s, c, o, 60, 16, 64)
    with pytest.raises(ValueError, match="HIP device"):
        ops.dequant(q, s, c, torch.zeros((64, 64), dtype=torch.float16), 64, 64)


def test_drop_in_module_has_the_reference_signatures():
    import inspect

    import tuna

    assert list(inspect.signature(tuna.matmul).parameters)[:8] == ["x", "q", "s", "c", "o", "m", "n", "k"]
    assert list(inspect.signature(tuna.dequant).parameters)[:6] == ["q", "absmax", "codebook", "o", "m", "k"]


def test_synthetic_inputs_are_deterministic_and_in_range():
    from tuna_amd.synth import SHAPES, make_inputs_np

    a = make_inputs_np(64, 16, 128, seed=3)
    b = make_inputs_np(64, 16, 128, seed=3)
    for u, v in zip(a, b):
        assert np.array_equal(u, v)
    q, x, code, absmax = a
    assert q.dtype == np.uint8 and q.shape == (8, 16, 32)
    assert x.dtype == np.float16 and absmax.dtype == np.float32 and code.dtype == np.float32
    assert (absmax >= 0.004999).all() and (absmax <= 0.02001).all()
    assert np.array_equal(absmax, absmax.astype(np.float16).astype(np.float32))  # fp16-representable scales
    assert len(SHAPES) == 10 and SHAPES["mistral_qkv"] == (6144, 4096)


# ---------------------------------------------------------------------------------------
# balanced split (split_k = 0): the partition arithmetic the kernel and the host share
# ---------------------------------------------------------------------------------------
def _balanced_cfg(**kw):
    from tuna_amd import ops

    base = dict(rows_per_wave=64, waves_m=1, waves_k=8, split_k=0, prefetch=2, x_chunk=1024, token_tiles=1, xcd_swizzle=1)
    base.update(kw)
    return ops.GemmConfig.from_dict(base)


@pytest.mark.parametrize("m,k,cfgkw,nwgs", [
    (6144, 4096, {}, (256, 512, 96, 7, 1)),
    (4096, 4096, dict(waves_k=4, prefetch=4, x_chunk=512), (512, 100)),
    (57344, 8192, dict(waves_m=4, waves_k=4, x_chunk=1024), (256, 255, 33)),
    (229376, 4096, dict(waves_m=8, waves_k=1, x_chunk=512), (512, 256)),
    (4096, 14336, dict(waves_k=8, prefetch=4), (256, 300)),
    (72, 200, dict(waves_k=2, x_chunk=128), (256, 3, 1)),     # ragged rows and k
    (8192, 28672, dict(waves_m=2, waves_k=8, x_chunk=1024), (256, 511)),
])
def test_balanced_split_partitions_every_k_step_once(m, k, cfgkw, nwgs):
    """Every (row tile, k-step) is covered by exactly one segment; a row tile's partial
    segments are consecutive workgroups in k order with the slots the finishing workgroup
    assumes; whole row tiles have a single owner.  Checked through the C ABI, whose
    arithmetic is the inline code the kernel compiles too."""
    from tuna_amd import ops

    cfg = _balanced_cfg(**cfgkw)
    steps = -(-k // 32)
    rows_wg = cfg.rows_per_wave * cfg.waves_m
    row_tiles = -(-m // rows_wg)
    for nw in nwgs:
        segs = {}
        n_launch = None
        # the library clamps the workgroup count to what the launch would start
        w = 0
        while True:
            try:
                sg = ops.config_segments(m, 16, k, cfg, nw, w)
            except ops.TunaError:
                break
            segs[w] = sg
            w += 1
        n_launch = w
        assert 1 <= n_launch <= nw
        cover = np.zeros((row_tiles, steps), dtype=np.int32)
        per_tile = {}
        for w, sg in segs.items():
            partial_slots = []
            for (rt, sb, ns, part) in sg:
                assert 0 <= rt < row_tiles and ns > 0 and sb >= 0 and sb + ns <= steps
                cover[rt, sb:sb + ns] += 1
                per_tile.setdefault(rt, []).append((sb, w, part, ns))
                if part >= 0:
                    partial_slots.append(part)
                else:
                    assert sb == 0 and ns == steps
            assert len(partial_slots) == len(set(partial_slots)) <= 2     # a workgroup owns two slots
        assert (cover == 1).all()
        # balance: workgroups differ by at most one unit (+ a ragged last unit)
        unit = cfg.waves_k * cfg.prefetch
        loads = [sum(s[2] for s in sg) for sg in segs.values()]
        assert max(loads) - min(loads) <= 2 * unit
        for rt, lst in per_tile.items():
            lst.sort()
            first_wg, count, first_slot = ops.config_contributors(m, 16, k, cfg, nw, rt)
            if len(lst) == 1:
                assert lst[0][2] == -1
                continue
            assert count == len(lst)
            assert [w for _, w, _, _ in lst] == list(range(first_wg, first_wg + count))
            assert lst[0][2] == first_slot
            assert all(part == 0 for _, _, part, _ in lst[1:])


def test_fixed_split_segments_match_the_grid():
    from tuna_amd import ops

    cfg = _balanced_cfg(split_k=4)
    segs = [ops.config_segments(6144, 16, 4096, cfg, 0, w) for w in range(8)]
    assert segs[0][0] == (0, 0, 32, 0) and segs[5][0] == (1, 32, 32, 1)
    assert ops.config_contributors(6144, 16, 4096, cfg, 0, 3) == (-1, 4, 0)


def test_gpu_parity_config_families_are_valid_configs():
    """The config families the GPU parity tests launch are accepted by the host validator for
    both of their shapes (a rejected config would fail the GPU test for the wrong reason)."""
    import importlib.util

    from tuna_amd import make_configs, ops

    spec = importlib.util.spec_from_file_location("gpu_parity_cases", os.path.join(ROOT, "tests", "test_gpu_parity.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    for kw in mod.CONFIGS:
        for shape in ((1024, 16, 2048), (520, 37, 1096)):
            ops.validate_config(*shape, mod.cfg(**kw))
    for rows, tt in mod.TILED:
        for (m, n, k, split) in ((512, 256, 512, 1), (520, 300, 1096, 1), (256, 70, 2048, 4), (1024, 129, 200, 3)):
            ops.validate_config(m, n, k, mod.cfg(lds_tile_rows=rows, token_tiles=tt, split_k=split))
    for case in mod.NARROW_CASES:
        m, n, k, rows, wk, pf = case[:6]
        c = mod.narrow_cfg(rows, wk, pf, *case[6:])
        ops.validate_config(m, n, k, c)
        lds, ws = ops.config_footprint(m, n, k, c)
        assert (lds, ws) == (make_configs.lds_bytes(c.to_dict()), 0)
        make_configs.validate(m, make_configs.bucket_of(n), k, c.to_dict())
        assert ops.config_segments(m, n, k, c, 0, m // rows - 1) == [(m // rows - 1, 0, k // 32, -1)]
        assert ops.config_contributors(m, n, k, c, 0, 0) == (-1, 1, 0)
    # the 256 x 256 tile (a kernel of its own): both MFMA shapes, split-K, k in multiples of 64 only; 160 KB of LDS
    # (32 KB table + two buffers of 512 rows) in the C planner and in the generator's twin
    for mfma_rows in (64, 32):
        for (m, n, k, split) in ((512, 256, 512, 1), (520, 300, 1088, 1), (256, 70, 2048, 4), (1024, 129, 192, 3)):
            c = mod.cfg(lds_tile_rows=256, token_tiles=16, split_k=split, rows_per_wave=mfma_rows)
            ops.validate_config(m, n, k, c)
            lds, _ = ops.config_footprint(m, n, k, c)
            assert lds == make_configs.lds_bytes(c.to_dict()) == 160 * 1024
            make_configs.validate(m, make_configs.bucket_of(n), k, c.to_dict())
    ops.validate_config(512, 256, 520, mod.cfg(lds_tile_rows=256, token_tiles=16))          # k not a multiple of 64: the
    make_configs.validate(512, 256, 520, mod.cfg(lds_tile_rows=256, token_tiles=16).to_dict())  # kernel's k-tail variant
    with pytest.raises(ops.TunaError):
        ops.validate_config(512, 256, 512, mod.cfg(lds_tile_rows=96, token_tiles=16))       # no such tile
    with pytest.raises(ops.TunaError):
        ops.validate_config(512, 256, 512, mod.cfg(lds_tile_rows=64, token_tiles=4))        # no 64 x 64 tile


def test_grouped_gemm_argument_checks_need_no_device():
    """tuna_matmul_grouped validates the group description on the host before any HIP call."""
    from tuna_amd import _lib

    L = _lib.lib()

    def call(m_group, n_groups, k, offsets):
        arr = (ctypes.c_int * len(offsets))(*offsets)
        return L.tuna_matmul_grouped(None, None, None, None, None, m_group, n_groups, k, arr, None, 1, None)

    assert call(256, 0, 256, [0]) == 1                    # no groups
    assert call(256, 65, 256, list(range(66))) == 1       # more than 64 groups
    assert call(256, 2, 256, [0, 9, 8]) == 1              # decreasing offsets
    assert call(256, 2, 256, [-1, 3, 8]) == 1             # negative start
    assert call(100, 2, 256, [0, 4, 8]) in (1, 2)         # rows per group not a multiple of 64
    assert b"" != L.tuna_last_error()
    assert call(256, 2, 256, [0, 0, 0]) == 0              # no tokens anywhere: nothing to do, no pointer is touched
    assert call(256, 2, 256, [0, 4, 8]) == 1              # tokens, but null pointers


def test_dequant_rounding_mode_gets_a_runnable_config_for_every_table_shape():
    """tuna_matmul_ex(cfg=NULL, TUNA_DECODE_DEQUANT) must run every tuned shape: the table's entries
    are for the GEMM's own decode (narrow-row, many-token and deep-ring entries have no variant
    with the dequant rounding), so that mode takes a derived streaming config."""
    from tuna_amd import _lib, ops

    for m, lo, hi, k, _cfg in ops.config_table():
        for n in sorted({lo, min(hi, lo + 7), min(hi, 4096)}):
            c, hit = ops.select_config(m, n, k, _lib.DECODE_DEQUANT)
            assert not hit
            assert c.lds_tile_rows == 0 and c.rows_per_wave == 64 and c.prefetch == 2 and c.waves_m >= 1
            assert c.waves_m * c.waves_k <= 8 and c.token_tiles in (1, 2, 4)
            ops.validate_config(m, n, k, c, _lib.DECODE_DEQUANT)
    # the GEMM's own decode still takes the table
    c, hit = ops.select_config(6144, 16, 4096, _lib.DECODE_GEMM)
    assert hit and c.rows_per_wave == 32
    with pytest.raises(ops.TunaError):
        ops.validate_config(6144, 16, 4096, c, _lib.DECODE_DEQUANT)   # narrow-row: GEMM decode only


def test_grouped_launch_gets_a_runnable_config_for_every_table_shape():
    """tuna_matmul_grouped(cfg=NULL) for every tuned shape split into 1, 2 or 8 groups, with all or
    only some groups active: a config is found (no division by a zero waves_m of a narrow-row
    entry, no TUNA_ERR_UNSUPPORTED), its row tile divides the group and it is a streaming config."""
    from tuna_amd import _lib, ops

    seen = 0
    for m, lo, hi, k, _cfg in ops.config_table():
        for groups in (1, 2, 8):
            if m % (64 * groups):
                continue
            m_group = m // groups
            for active in sorted({1, groups}):
                for decode in (_lib.DECODE_GEMM, _lib.DECODE_DEQUANT):
                    c = ops.select_config_grouped(m_group, active, lo, k, decode)
                    assert c.lds_tile_rows == 0 and c.rows_per_wave == 64 and c.waves_m >= 1
                    assert m_group % (64 * c.waves_m) == 0
                    seen += 1
    assert seen > 300
    # the case that used to divide by zero: Mixtral down, all 8 experts active, 4 tokens each
    c = ops.select_config_grouped(4096, 8, 4, 14336)
    assert c.waves_m >= 1 and 4096 % (64 * c.waves_m) == 0
    with pytest.raises(ops.TunaError):
        ops.select_config_grouped(4000, 8, 4, 14336)                   # not a multiple of 64 rows


def test_bench_last_line_stays_compact_whatever_the_detail_holds():
    """The harness that runs bench.py keeps the end of stdout and parses its last line: that line is the
    headline only and stays far below 4 KB even when the detail object is hundreds of kilobytes."""
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench

    shape_row = {"m": 6144, "n": 16, "k": 4096, "us_per_gemm": 7.0, "gbs": 1797.5, "frac_hbm": 0.2247,
                 "kernel": "gemm_narrow_kernel<LW=2,WK=8,U=4,PERM=1,TT=1>", "config": {"rows_per_wave": 32} , "pad": "x" * 4000}
    detail = {
        "metric": bench.METRIC, "value": 1797.5, "unit": "GB/s", "n_gpus": 1, "steps": 20, "warmup": 5,
        "ms_per_step": 0.007, "us_per_gemm": 7.0, "tflops": 115.0, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "benchmark config 1: Mistral-7B QKV projection, M=16 tokens, K=4096, N=6144; " + "y" * 5000,
                   "tile_config": {"rows_per_wave": 32, "waves_m": 1, "waves_k": 8, "split_k": 1, "prefetch": 4, "x_chunk": 512,
                                   "token_tiles": 1, "xcd_swizzle": 0, "k_stagger": 0, "lds_tile_rows": 0},
                   "launch": "stream"},
        "roofline": {"bound": "hbm", "achieved": 1797.5, "peak": 8000.0, "unit": "GB/s", "frac": 0.2247, "traffic": 13919232,
                     "kernel": "tuna::gemm_narrow_kernel<LW=2,WK=8,U=4,PERM=1,TT=1>", "algorithmic_bytes_per_launch": 12582912,
                     "avg_launch_us": 7.0, "extra": "z" * 3000},
        "cpu_baseline": {"value": 3.3, "unit": "GB/s", "cores": 16, "kind": "port", "sample": "s" * 2000, "us_per_gemm": 2507.2,
                         "us_decode": 1.0, "us_matmul": 2.0, "single_thread_us_per_gemm": 36553.9},
        "shapes": {f"shape_{i}": dict(shape_row) for i in range(40)},
        "sweeps": {"token_sweep": {str(t): {f"shape_{i}": dict(shape_row) for i in range(4)} for t in (1, 16, 64, 256, 1024, 4096)}},
        "unit_rates": {f"unit_{i}": 1.0 for i in range(40)},
    }
    assert len(json.dumps(detail)) > 200_000
    text = bench.headline_line(detail, "gpurun_out/bench_detail.json")
    assert "\n" not in text and len(text) < 2048, len(text)
    line = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "dtype", "data"):
        assert line[key] == detail[key], key
    assert line["config"]["workload"].startswith("benchmark config 1") and "model" not in line["config"]
    assert set(line["roofline"]) == set(bench.ROOFLINE_KEYS) and line["roofline"]["frac"] == 0.2247
    assert line["cpu_baseline"]["cores"] == 16 and line["cpu_baseline"]["kind"] == "port"
    assert len(line["frac_hbm_by_shape"]) <= 12
    # no CPU leg and no shape table (profiling runs): still one parseable line
    bare = dict(detail, cpu_baseline=None)
    del bare["shapes"]
    assert json.loads(bench.headline_line(bare))["cpu_baseline"] is None


def test_library_chosen_configs_accept_scales_that_are_only_float_aligned():
    """tuna_matmul(cfg = NULL) with an absmax pointer of the form 4 mod 16 on every shape of the table, at the token
    counts its entries start at: never an argument error (the dispatcher moves off kernels that read the scales
    two or four at a time).  Host only: fake pointers, so this runs where no device can take the launch."""
    import torch

    if torch.cuda.is_available():
        pytest.skip("fake pointers: only where nothing can be launched")
    from tuna_amd import _lib

    L = _lib.lib()
    m_, lo_, hi_, k_ = (ctypes.c_int() for _ in range(4))
    cfg = _lib.GemmConfig()
    seen = set()
    for i in range(L.tuna_config_table_size()):
        assert L.tuna_config_table_entry(i, ctypes.byref(m_), ctypes.byref(lo_), ctypes.byref(hi_), ctypes.byref(k_), ctypes.byref(cfg)) == 0
        for n in {lo_.value, min(hi_.value, lo_.value + 3)}:
            if n > 64 or (m_.value, n, k_.value) in seen:
                continue
            seen.add((m_.value, n, k_.value))
            rc = L.tuna_matmul(0x10000, 0x20000, 0x30000, 0x40004, 0x50000, m_.value, n, k_.value, None)
            assert rc != _lib.ERR_INVALID_ARG, (m_.value, n, k_.value, L.tuna_last_error())
            assert rc in (_lib.ERR_HIP, _lib.ERR_NO_DEVICE, _lib.ERR_WORKSPACE), rc
    assert len(seen) > 40


def test_every_blockwise_table_entry_validates_and_derived_configs_are_runnable():
    """The blockwise table: every entry of param_map_blockwise.json is in the library's table, passes the generator's
    structural check and the library's own validator at the token count it was tuned at, and is what
    tuna_select_config_blockwise returns there; shapes without an entry get a derived config that validates too."""
    from tuna_amd import _lib, make_configs as mc, ops

    with open(os.path.join(ROOT, "tuna_amd", "configs", "param_map_blockwise.json")) as f:
        pm = json.load(f)
    L = _lib.lib()
    assert L.tuna_blockwise_table_size() == len(pm) > 0
    seen = set()
    m_, lo_, hi_, k_, bs_ = (ctypes.c_int() for _ in range(5))
    cfg = _lib.GemmConfig()
    for i in range(len(pm)):
        assert L.tuna_blockwise_table_entry(i, ctypes.byref(m_), ctypes.byref(lo_), ctypes.byref(hi_), ctypes.byref(k_), ctypes.byref(bs_),
                                            ctypes.byref(cfg)) == 0
        n_key = [key for key, (lo, hi) in mc.N_BUCKETS.items() if lo == lo_.value][0]
        key = f"{m_.value}_{n_key}_{k_.value}_{bs_.value}"
        seen.add(key)
        want = {f: int(pm[key].get(f, 0)) for f in mc.FIELDS}
        assert cfg.to_dict() == want, key
        mc.validate_blockwise(m_.value, n_key, k_.value, bs_.value, want)
        ops.validate_config_blockwise(m_.value, lo_.value, k_.value, bs_.value, cfg)
        for n in (lo_.value, hi_.value):
            # (an entry that makes one pass over the weights with the token tiles of the bucket's lower edge cannot
            # take the bucket's upper edge: the lookup then hands out a derived config, which must run as well)
            got, hit = ops.select_config_blockwise(m_.value, n, k_.value, bs_.value)
            ops.validate_config_blockwise(m_.value, n, k_.value, bs_.value, got)
            assert (hit and got.to_dict() == want) or (not hit and n != lo_.value), (key, n)
    assert seen == set(pm)
    for (m, n, k, bs) in [(4096, 16, 4096, 64), (5120, 1, 5120, 128), (3072, 40, 9216, 64), (65536, 16, 4096, 256), (1024, 300, 2048, 64),
                          (16, 1, 256, 64), (49152, 24, 6144, 64), (12288, 100, 4096, 128), (2048, 2000, 1024, 512)]:
        got, hit = ops.select_config_blockwise(m, n, k, bs)
        assert not hit and ops.blockwise_family(got) in ops.BLOCKWISE_FAMILIES
        ops.validate_config_blockwise(m, n, k, bs, got)
    # what cannot run is refused with a reason, not launched
    bad = ops.GemmConfig.from_dict(dict(rows_per_wave=64, waves_m=4, waves_k=4, split_k=1, prefetch=2, x_chunk=512, token_tiles=1, xcd_swizzle=0))
    with pytest.raises(ops.TunaError):
        ops.validate_config_blockwise(4096, 100, 4096, 64, bad)          # the streaming twin: up to 64 tokens
    with pytest.raises(ops.TunaError):
        ops.validate_config_blockwise(4096, 16, 4096, 96, bad)           # not a power of two
