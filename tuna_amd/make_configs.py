"""param_map.json -> csrc/config_table.cpp: the shape -> tile-config table of the GEMM.

Counterpart of the reference's make_configs.py (make_configs.py:1-132), which pastes
param_map.json values into a C++ template to produce configs.cu.  Differences:

* the output is a run-time data table (`kConfigTable`, searched by
  tuna_select_config) instead of 126 compile-time constants feeding template
  instantiations (configs.cu:56-3331, kernel.cu:3018-3156);
* every entry is validated against the kernel's constraints before it is emitted (the
  reference emits inconsistent entries such as gemm_229376_4096_16, whose
  warp_count_m * warp_count_n * 32 != tpb, param_map.json:4034-4069);
* keys are "<m>_<n>_<k>" like the reference's (make_configs.py:111-115), n being the
  lower edge of a token bucket; bucket edges follow kernel.cu:3022-3155.  In addition an entry may sit
  under one of the keys of SUB_KEYS (1.5 times a bucket's lower edge): it covers the bucket from that token
  count up, and the bucket's own entry the counts below.

Usage:  python -m tuna_amd.make_configs [param_map.json] [config_table.cpp]
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
DEFAULT_JSON = os.path.join(HERE, "configs", "param_map.json")
DEFAULT_OUT = os.path.join(HERE, "csrc", "config_table.cpp")

# token buckets of the reference's dispatcher (kernel.cu:3022-3155): key n -> [lo, hi]
N_BUCKETS = {
    1: (1, 15),
    16: (16, 31),
    32: (32, 63),
    64: (64, 127),
    128: (128, 255),
    256: (256, 511),
    512: (512, 768),
    1024: (769, 1024),
    2048: (1025, 128000),
}

# Optional keys inside a bucket (no counterpart in the reference's table): an entry m_<sub>_k covers the token
# counts from <sub> to the upper edge of the bucket it sits in, and that bucket's own entry then ends at <sub> - 1.
# An entry is tuned at the lower edge of its range, and the best launch at 1.5 times that count is often another
# one (another number of token chunks side by side, another tile of the many-token kernel).
SUB_KEYS = {24: 16, 48: 32, 96: 64, 192: 128, 384: 256}

FIELDS = ("rows_per_wave", "waves_m", "waves_k", "split_k", "prefetch", "x_chunk",
          "token_tiles", "xcd_swizzle", "k_stagger", "lds_tile_rows")

LUT_BYTES = 256 * 64 * 4
LDS_LIMIT = 160 * 1024
STEP_K = 32

# (rows_per_wave / 64, prefetch, token_tiles) variants compiled for <= 8 waves (<= 256 VGPRs),
# for <= 8 waves with <= 128 VGPRs (two workgroups per CU) and for 16-wave workgroups;
# must match kVariants in csrc/gemm_launch.hip
VARIANTS_512 = {(1, 2, 1), (1, 2, 2), (1, 2, 4), (1, 4, 1), (1, 4, 2), (1, 8, 1), (1, 8, 2), (2, 2, 1), (2, 4, 1)}
VARIANTS_512_2WG = {(1, 2, 1), (1, 4, 1)}
VARIANTS_1024 = {(1, 2, 1), (1, 4, 1)}


# (prefetch, token_tiles, x pieces per thread, max threads) of the 17..128-token streaming kernel; must match
# kMid in csrc/gemm_mid.hip
MID_VARIANTS = ({(u, tt, xb, 512) for u in (2, 4, 8) for tt in (2, 4) for xb in (4, 8)}
                | {(2, 8, 4, 512), (2, 8, 8, 512), (2, 2, 4, 1024), (4, 2, 4, 1024)}
                | {(u, 1, xb, 512) for u in (2, 4, 8) for xb in (4, 8)} | {(u, 1, 4, 1024) for u in (2, 4, 8)})

# ... of those, the ones with a twin for k split across workgroups (fn_split of kMid)
MID_SPLIT_VARIANTS = ({(u, tt, xb, 512) for u in (2, 4) for (tt, xb) in ((2, 4), (4, 4), (4, 8))}
                      | {(2, 2, 4, 1024), (4, 2, 4, 1024)})

# (rows, waves_k, prefetch, token_tiles) of the narrow-row kernel; must match kNarrow in csrc/gemm_launch.hip
NARROW_VARIANTS = (
    {(r, wk, pf, 1) for r in (16, 32, 64) for wk in (4, 8, 16) for pf in (2, 4, 8)}
    | {(16, 1, 2, 1), (16, 2, 2, 1), (32, 1, 2, 1), (32, 2, 2, 1)}
    | {(r, wk, pf, 2) for r in (16, 32, 64) for wk in (4, 8, 16) for pf in (2, 4)}
    | {(r, wk, pf, 4) for r in (16, 32) for wk in (4, 8) for pf in (2, 4)} | {(64, 4, 2, 4), (64, 8, 2, 4)}
    | {(24, 8, 2, 1), (24, 8, 4, 1), (24, 8, 8, 1), (24, 16, 2, 1), (24, 16, 4, 1)})

# (rows, tokens) tiles of the many-token kernels; must match kTiled in csrc/gemm_tiled.hip, plus the 256 x 256 tile
# of csrc/gemm_wide.hip (one wave per SIMD)
TILED_VARIANTS = {(256, 256), (256, 128), (256, 64), (128, 256), (128, 128), (64, 256), (64, 128)}
WIDE_LUT_BYTES = 256 * 32 * 4


def _pow2(v: int) -> bool:
    return v > 0 and (v & (v - 1)) == 0


def bucket_of(n: int):
    """Token count -> bucket key."""
    for key, (lo, hi) in N_BUCKETS.items():
        if lo <= n <= hi:
            return key
    raise ValueError(f"n={n} outside every token bucket")


def key_range(n_key: int, keys_present=()) -> tuple:
    """The token counts [lo, hi] that the entry under key `n_key` covers when the entries of its (m, k) have the keys
    `keys_present`: a bucket's range, cut short by a sub key inside it where there is one."""
    if n_key in SUB_KEYS:
        return n_key, N_BUCKETS[SUB_KEYS[n_key]][1]
    lo, hi = N_BUCKETS[n_key]
    subs = [s for s, parent in SUB_KEYS.items() if parent == n_key and s in keys_present]
    return lo, (min(subs) - 1 if subs else hi)


def key_of(n: int, keys_present=()) -> int:
    """Token count -> the key of the entry that covers it, among the keys `keys_present` of one (m, k)."""
    nk = bucket_of(n)
    subs = [s for s, parent in SUB_KEYS.items() if parent == nk and s in keys_present and n >= s]
    return max(subs) if subs else nk


def keys_of_shape(param_map: dict, m: int, k: int) -> list:
    """The token keys of the entries that `param_map` holds for (m, k), ascending."""
    return sorted(int(key.split("_")[1]) for key in param_map if key.split("_")[0] == str(m) and key.split("_")[2] == str(k))


def is_narrow(c: dict) -> bool:
    """The config selects the narrow-row kernel: rows_per_wave 16, 24 or 32, or 64 with waves_m 0."""
    return c.get("lds_tile_rows", 0) == 0 and (c["rows_per_wave"] in (16, 24, 32) or (c["rows_per_wave"] == 64 and c["waves_m"] == 0))


def validate(m: int, n_key: int, k: int, c: dict) -> None:
    """Raise ValueError unless config `c` can run shape (m, n in bucket n_key, k)."""
    c = {"k_stagger": 0, "lds_tile_rows": 0, **c}  # entries written before the fields existed
    missing = [f for f in FIELDS if f not in c]
    if missing:
        raise ValueError(f"missing fields {missing}")
    if m <= 0 or k <= 0 or m % 8 or k % 8:
        raise ValueError("m and k must be positive multiples of 8")
    if n_key not in N_BUCKETS and n_key not in SUB_KEYS:
        raise ValueError(f"n={n_key} is not a bucket key {sorted(N_BUCKETS)} nor a key inside a bucket {sorted(SUB_KEYS)}")
    if c["lds_tile_rows"] not in (0, -1, 64, 128, 256):
        raise ValueError("lds_tile_rows must be 0, -1 (packed weights through LDS), 64, 128 or 256")
    if c["lds_tile_rows"] > 0:
        # many-token kernel: only the tile shape and the split matter
        if (c["lds_tile_rows"], 16 * c["token_tiles"]) not in TILED_VARIANTS:
            raise ValueError(f"no many-token kernel for a {c['lds_tile_rows']} x {16 * c['token_tiles']} tile")
        if c["rows_per_wave"] == 32 and (c["lds_tile_rows"], 16 * c["token_tiles"]) == (64, 128):
            raise ValueError("the 64 x 128 tile has no 32 x 32 MFMA variant (one 16-token tile per wave)")
        if not 1 <= c["split_k"] <= -(-k // 64):
            raise ValueError("split_k of the many-token kernel must be in 1..ceil(k/64)")
        return
    if is_narrow(c):
        # narrow-row kernel: one workgroup per 16, 32 or 64 rows, all waves along k, no split
        if (c["waves_m"], c["split_k"], c["k_stagger"]) != (0 if c["rows_per_wave"] == 64 else 1, 1, 0):
            raise ValueError("the narrow-row kernel needs waves_m=1 (0 with rows_per_wave 64), split_k=1, k_stagger=0")
        if (c["rows_per_wave"], c["waves_k"], c["prefetch"], c["token_tiles"]) not in NARROW_VARIANTS:
            raise ValueError("no narrow-row kernel for this rows_per_wave / waves_k / prefetch / token_tiles")
        if c["x_chunk"] != STEP_K * c["waves_k"] * c["prefetch"]:
            raise ValueError("the narrow-row kernel stages no x: x_chunk must be 32*waves_k*prefetch, the k of one ring turn")
        if m % c["rows_per_wave"] or k % (STEP_K * c["waves_k"] * c["prefetch"]):
            raise ValueError("rows_per_wave 16, 24 or 32 needs m a multiple of it and k a multiple of 32*waves_k*prefetch")
        if m * k // 2 >= 1 << 32 or k * 32 >= 1 << 32:
            raise ValueError("operands exceed the kernel's 32-bit offsets")
        if lds_bytes(c) > LDS_LIMIT:
            raise ValueError(f"needs {lds_bytes(c)} bytes of LDS (limit {LDS_LIMIT})")
        return
    if c["rows_per_wave"] not in (64, 128, 256):
        raise ValueError("rows_per_wave must be 16, 24, 32 (narrow-row kernel), 64, 128 or 256")
    if c["prefetch"] not in (2, 4, 8):
        raise ValueError("prefetch must be 2, 4 or 8")
    if c["token_tiles"] not in (1, 2, 4, 8):
        raise ValueError("token_tiles must be 1, 2, 4 or 8")
    wm, wk = c["waves_m"], c["waves_k"]
    if wm < 1 or not _pow2(wk) or wm * wk > 16:
        raise ValueError("waves_m must be >= 1 and waves_k a power of two, with waves_m * waves_k <= 16")
    if m * k // 2 >= 1 << 32:
        raise ValueError("packed weights exceed the kernel's 32-bit offsets")
    steps = -(-k // STEP_K)
    if not 0 <= c["split_k"] <= steps:
        raise ValueError(f"split_k must be in 0..{steps} (0 = balanced split)")
    unit = STEP_K * wk * c["prefetch"]
    if not _pow2(c["x_chunk"]) or c["x_chunk"] < unit:
        raise ValueError(f"x_chunk must be a power of two >= {unit}")
    rw = c["rows_per_wave"] // 64
    key = (rw, c["prefetch"], c["token_tiles"])
    threads = 64 * wm * wk
    if key not in (VARIANTS_512 if threads <= 512 else VARIANTS_1024) and not mid_applies(m, k, c):
        raise ValueError(f"no kernel variant {key} for {threads} threads")
    if c["x_chunk"] * c["token_tiles"] > (4 if c["prefetch"] == 8 else 2) * threads:
        raise ValueError("x_chunk * token_tiles too large for the x staging (4 pieces per thread, 8 with prefetch 8)")
    if not 0 <= c["k_stagger"] <= 4096:
        raise ValueError("k_stagger must be in 0..4096")
    if lds_bytes(c) > LDS_LIMIT:
        raise ValueError(f"needs {lds_bytes(c)} bytes of LDS (limit {LDS_LIMIT})")
    if c["lds_tile_rows"] == -1 and not mid_lds_applies(m, k, c):
        raise ValueError("lds_tile_rows -1 needs a launch of 8 or 16 waves the streaming kernel takes, prefetch 2 or 4 "
                         "(2 with eight token tiles) and x chunks that leave room for the weight rings")


# (prefetch, token_tiles, x pieces per thread, max threads) of the streaming kernel's twins that stage the packed
# weights through LDS; must match the fn_lds entries of kMid in csrc/gemm_mid.hip
MID_LDS_VARIANTS = ({(u, 2, 4, 512) for u in (2, 4)} | {(u, 4, xb, 512) for u in (2, 4) for xb in (4, 8)}
                    | {(2, 8, 4, 512), (2, 8, 8, 512), (2, 2, 4, 1024), (4, 2, 4, 1024), (2, 1, 4, 1024), (4, 1, 4, 1024)})


def _mid_variant(m: int, k: int, c: dict, lds_path: bool):
    """(variant key, x chunk) of the streaming kernel for a dense launch of this config, or None
    (mirrors mid_variant and mid_x_chunk in csrc/gemm_mid.hip)."""
    tt, wm, wk = c["token_tiles"], c["waves_m"], c["waves_k"]
    if c["rows_per_wave"] != 64 or tt not in (1, 2, 4, 8) or not 0 <= c["k_stagger"] <= 4096:
        return None
    split = c["split_k"]
    # k split across workgroups: 2..256 equal parts, a power of two, two or more token tiles, no stagger
    if split != 1 and (not _pow2(split) or split > 256 or tt < 2 or c["k_stagger"] != 0):
        return None
    if k % STEP_K or k >= 1 << 23 or not _pow2(wk) or wm < 1 or wm * wk > 16 or m % (64 * wm):
        return None
    threads = 64 * wm * wk
    ring = (threads // 64) * c["prefetch"] * 1024 if lds_path and threads in (512, 1024) and c["prefetch"] in (2, 4) else 0
    xc = c["x_chunk"]
    cap = (LDS_LIMIT - LUT_BYTES - ring) // (2 * tt * 32)
    while xc > cap:
        xc //= 2
    if xc < wk * c["prefetch"] * STEP_K or k % (xc * split):
        return None
    per_thread = -(-(tt * 2 * xc) // threads)
    if per_thread > 8:
        return None
    key = (c["prefetch"], tt, 4 if per_thread <= 4 else 8, 512 if threads <= 512 else 1024)
    if split != 1 and key not in MID_SPLIT_VARIANTS:
        return None
    return (key, xc) if key in MID_VARIANTS else None


def mid_lds_applies(m: int, k: int, c: dict) -> bool:
    """True if the streaming kernel's twin with the packed weights staged through LDS takes a dense
    launch of this config (mirrors mid_lds_applies in csrc/gemm_mid.hip)."""
    v = _mid_variant(m, k, c, True)
    threads = 64 * c["waves_m"] * c["waves_k"]
    if v is None or v[0] not in MID_LDS_VARIANTS or threads not in (512, 1024):
        return False
    xc, tt, waves = v[1], c["token_tiles"], threads // 64
    pieces = (xc // 32) * tt
    if pieces % waves or pieces // waves not in (1, 2, 4):
        return False
    x_lds, red_lds = 2 * tt * 32 * xc, 2 * waves * 1024
    return x_lds >= red_lds and LUT_BYTES + x_lds + waves * c["prefetch"] * 1024 <= LDS_LIMIT


def mid_applies(m: int, k: int, c: dict) -> bool:
    """True if a dense launch of this config is taken by the 17..128-token streaming kernel
    (mirrors mid_variant in csrc/gemm_mid.hip)."""
    return _mid_variant(m, k, c, c.get("lds_tile_rows", 0) == -1) is not None


def lds_bytes(c: dict) -> int:
    """Dynamic LDS of a launch: decode table + max(x chunk, reduction buffers).

    The reduction buffers are 2 x 1 plane (1 KB) per wave, or 2 x 4 planes (1 x 4 for a wave with one
    64-row group and token tile) when that costs no occupancy (mirrors plan_gemm in csrc/api.cpp)."""
    if c.get("lds_tile_rows", 0) > 0:
        # many-token kernel: decode table + two buffers of (weight tile + activation tile), 128 bytes per row
        wide = (c["lds_tile_rows"], 16 * c["token_tiles"]) == (256, 256)
        return (WIDE_LUT_BYTES if wide else LUT_BYTES) + 2 * (c["lds_tile_rows"] + 16 * c["token_tiles"]) * 128
    if is_narrow(c):
        # narrow-row kernel: decode table + one accumulator plane (1 KB) per wave and 16 rows
        return LUT_BYTES + c["waves_k"] * ((c["rows_per_wave"] + 15) // 16) * c["token_tiles"] * 1024
    threads = 64 * c["waves_k"] * c["waves_m"]
    x = c["token_tiles"] * 16 * c["x_chunk"] * 2
    plane = c["waves_k"] * c["waves_m"] * 1024
    small = LUT_BYTES + max(x, 2 * plane)
    one_group = c["rows_per_wave"] == 64 and c["token_tiles"] == 1     # nothing to alternate with: one buffer
    big = LUT_BYTES + max(x, (4 if one_group else 8) * plane)
    two_wgs = threads <= 512 and 2 * small <= LDS_LIMIT
    return big if big <= LDS_LIMIT and (big == small or not two_wgs) else small


# ---- the GEMM with scale blocks finer than a row: entries keyed "<m>_<n>_<k>_<block_size>" -------------------------
# Narrow-row scale-block variants (rows per workgroup, waves along k, ring, token tiles); must match kBlockwise in
# csrc/gemm_launch.hip
BLOCKWISE_NARROW = ({(16, 4, 2, 1), (16, 8, 4, 1), (16, 16, 2, 1), (32, 8, 2, 1), (32, 8, 4, 1), (32, 16, 2, 1), (64, 4, 4, 1),
                     (64, 8, 2, 1), (64, 8, 4, 1), (64, 16, 2, 1)}
                    | {(16, 4, 2, 2), (16, 8, 4, 2), (32, 8, 2, 2), (32, 8, 4, 2), (64, 8, 2, 2), (64, 8, 4, 2)})
# many-token tiles with a scale-block variant (16 x 16 x 32 MFMA; not the 256 x 256 tile)
BLOCKWISE_TILED = {(64, 128), (64, 256), (128, 64), (128, 128), (128, 256), (256, 64), (256, 128)}
BLOCKWISE_FAMILIES = ("narrow", "batched", "many-token", "streaming")


def blockwise_family(c: dict) -> str:
    """Which kernel a blockwise config names (mirrors blockwise_family in csrc/api.cpp)."""
    if c.get("lds_tile_rows", 0) > 0:
        return "many-token"
    if is_narrow(c):
        return "narrow"
    if c["split_k"] == 0:
        return "batched"
    return "streaming"


def validate_blockwise(m: int, n: int, k: int, bs: int, c: dict) -> None:
    """Raise ValueError unless `c` is a runnable blockwise config for (m, n in bucket n, k, block size bs): the
    structural checks of run_blockwise in csrc/api.cpp (the library's own validator, tuna_validate_config_blockwise,
    is the full check and is run over the generated table by the tests)."""
    if n not in N_BUCKETS:
        raise ValueError(f"n={n} is not a token bucket key")
    if bs < 64 or bs & (bs - 1) or k % bs or bs >= k or m % 16 or k % 256:
        raise ValueError(f"block_size={bs}: a power of two >= 64 that divides k={k} (k a multiple of 256, m={m} of 16)")
    fam = blockwise_family(c)
    lo, _ = N_BUCKETS[n]
    if fam == "narrow":
        key = (c["rows_per_wave"], c["waves_k"], c["prefetch"], c["token_tiles"])
        if key not in BLOCKWISE_NARROW:
            raise ValueError(f"no narrow-row scale-block variant {key}")
        if m % c["rows_per_wave"] or k % (STEP_K * c["waves_k"] * c["prefetch"]):
            raise ValueError("narrow-row variant does not divide the shape")
    elif fam == "batched":
        if c["waves_m"] not in (1, 2, 4) or c["waves_m"] * c["waves_k"] != 16 or c["prefetch"] not in (2, 4):
            raise ValueError("batched kernel: 1, 2 or 4 waves along the rows of 16, ring 2 or 4")
        if m % (64 * c["waves_m"]) or k % (STEP_K * c["waves_k"] * c["prefetch"]) or k // bs < 2:
            raise ValueError("batched kernel: row tile or ring turn does not divide the shape")
    elif fam == "many-token":
        if (c["lds_tile_rows"], 16 * c["token_tiles"]) not in BLOCKWISE_TILED or c["split_k"] < 1:
            raise ValueError("no many-token scale-block variant with that tile")
    else:
        tiles = 4 if lo > 32 else 2 if lo > 16 else 1
        if lo > 64 or c["token_tiles"] != tiles or c["split_k"] != 1 or c["rows_per_wave"] != 64 or c["waves_m"] < 1:
            raise ValueError("streaming twin: up to 64 tokens in one pass, unsplit, 64 rows per wave")
        if m % (64 * c["waves_m"]) or c["prefetch"] not in (2, 4) or c["waves_m"] * c["waves_k"] not in (8, 16):
            raise ValueError("streaming twin: 8 or 16 waves, ring 2 or 4, whole row tiles")


def generate_blockwise(param_map: dict) -> str:
    rows = []
    for key in sorted(param_map, key=lambda s: tuple(int(t) for t in s.split("_"))):
        m, n, k, bs = (int(t) for t in key.split("_"))
        c = param_map[key]
        try:
            validate_blockwise(m, n, k, bs, c)
        except ValueError as e:
            raise ValueError(f"blockwise param_map entry {key}: {e}") from None
        lo, hi = N_BUCKETS[n]
        vals = ", ".join(str(int(c.get(f, 0))) for f in FIELDS)
        rows.append(f"    {{{m}, {lo}, {hi}, {k}, {bs}, {{{vals}}}}},  // {key}: {blockwise_family(c)}")
    body = "\n".join(rows)
    return f"""
// Scale blocks finer than a row: (m, token bucket, k, block_size) -> config, searched by tuna_select_config_blockwise.
// Generated from tuna_amd/configs/param_map_blockwise.json.  Entry: m, n_lo, n_hi, k, block_size, {{config}}
namespace tuna {{

const BlockwiseTableEntry kBlockwiseTable[] = {{
{body}
    {{0, 0, 0, 0, 0, {{0, 0, 0, 0, 0, 0, 0, 0, 0, 0}}}},  // sentinel (not counted)
}};
const int kBlockwiseTableSize = {len(rows)};

}}  // namespace tuna
"""


def default_next_from(n_key: int, keys_present=()) -> int:
    """Where an entry without a tuned "next_from" hands over to the next bucket's entry: entries are tuned at the
    lower edge of their bucket, and a count inside one of the buckets 16.., 32.., 64.., 128.. takes two passes over
    the weights with such an entry but one with the next bucket's (from 10 tokens in the first bucket); the other
    buckets keep their entry throughout (n_hi + 1: never)
    (with keys inside buckets: `keys_present`, the keys of the entry's (m, k), gives the range; an entry whose range
    a sub key starts or ends keeps its entry throughout)"""
    lo, hi = key_range(n_key, keys_present)
    if n_key in SUB_KEYS or hi != N_BUCKETS[n_key][1]:
        return hi + 1
    if lo == 1:
        return 10
    return lo + 1 if 16 <= lo <= 128 else hi + 1


def next_from_of(n_key: int, c: dict, keys_present=()) -> int:
    """The entry's "next_from" (the token count from which the lookup hands out the next entry of its (m, k) instead;
    written by the tuner, which times both entries inside the range), checked: n_lo < next_from <= n_hi + 1."""
    lo, hi = key_range(n_key, keys_present)
    nf = int(c.get("next_from", default_next_from(n_key, keys_present)))
    if not lo < nf <= hi + 1:
        raise ValueError(f"next_from={nf} outside {lo + 1}..{hi + 1}")
    return nf


def derived_range_of(n_key: int, c: dict, keys_present=()):
    """The entry's "derived_from" / "derived_to": the lookup hands out the derived config instead of the table's for
    token counts in [derived_from, derived_to) (written by the tuner, which times both at the sampled counts of the
    range; absent: (0, 0), nowhere).  Checked: both or neither, inside the entry's range, and above 64 tokens (below,
    every count of a bucket has the same grid but for one chunk, and the entries are tuned for it)."""
    if "derived_from" not in c and "derived_to" not in c:
        return 0, 0
    lo, hi = key_range(n_key, keys_present)
    try:
        a, b = int(c["derived_from"]), int(c["derived_to"])
    except KeyError:
        raise ValueError("derived_from and derived_to come together") from None
    if not (max(lo, 65) <= a < b <= hi + 1):
        raise ValueError(f"derived range {a}..{b} outside {max(lo, 65)}..{hi + 1}")
    return a, b


def generate(param_map: dict) -> str:
    rows = []
    for key in sorted(param_map, key=lambda s: tuple(int(t) for t in s.split("_"))):
        m, n, k = (int(t) for t in key.split("_"))
        c = param_map[key]
        present = keys_of_shape(param_map, m, k)
        try:
            validate(m, n, k, c)
            if n in SUB_KEYS and SUB_KEYS[n] not in present:
                raise ValueError(f"a key inside a bucket needs the bucket's own entry ({m}_{SUB_KEYS[n]}_{k})")
            nf = next_from_of(n, c, present)
            dr = derived_range_of(n, c, present)
        except ValueError as e:
            raise ValueError(f"param_map entry {key}: {e}") from None
        lo, hi = key_range(n, present)
        vals = ", ".join(str(int(c.get(f, 0))) for f in FIELDS)
        tail = f", {dr[0]}, {dr[1]}" if dr != (0, 0) else ""
        rows.append(f"    {{{m}, {lo}, {hi}, {k}, {nf}, {{{vals}}}{tail}}},  // {key}")
    body = "\n".join(rows)
    return f"""// GENERATED by tuna_amd/make_configs.py from tuna_amd/configs/param_map.json - do not edit.
// Shape -> tile-config table, searched linearly by tuna_select_config.
// Entry: m, n_lo, n_hi, k, next_from, {{{", ".join(FIELDS)}}}[, derived_from, derived_to]
#include "tuna_internal.h"

namespace tuna {{

const TableEntry kConfigTable[] = {{
{body}
    {{0, 0, 0, 0, 0, {{0, 0, 0, 0, 0, 0, 0, 0, 0, 0}}}},  // sentinel (not counted)
}};
const int kConfigTableSize = {len(rows)};

}}  // namespace tuna
"""


def main(argv):
    src = argv[1] if len(argv) > 1 else DEFAULT_JSON
    dst = argv[2] if len(argv) > 2 else DEFAULT_OUT
    with open(src) as f:
        param_map = json.load(f)
    text = generate(param_map)
    # the blockwise table sits beside the per-row one: <stem>_blockwise.json (absent: an empty table)
    src_blk = os.path.splitext(src)[0] + "_blockwise.json"
    blockwise = {}
    if os.path.exists(src_blk):
        with open(src_blk) as f:
            blockwise = json.load(f)
    text += generate_blockwise(blockwise)
    with open(dst, "w") as f:
        f.write(text)
    print(f"{dst}: {len(param_map)} entries, {len(blockwise)} blockwise entries")


if __name__ == "__main__":
    main(sys.argv)
