#!/usr/bin/env python3
"""Benchmark of the FP16 x 4-bit GEMM on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one GEMM of the headline workload (Mistral-7B QKV projection at 16 tokens:
out[16, 6144] = x[16, 4096] . W[6144, 4096]^T, benchmark configuration 1) on one of a rotating set
of distinct, HBM-resident weight matrices, so that neither L2 nor the 256 MB Infinity Cache
can serve re-reads.  W warm-up steps, then exactly K timed steps bracketed by HIP events on
the launch stream (tuna_time_matmul, inside the C library, so that no Python overhead sits
between launches).  The LAST line printed is one compact JSON object (under 2 KB, headline_line()):

  value        packed-weight bytes (m*k/2) per second, GB/s  - the roofline quantity
  ms_per_step  milliseconds per GEMM (x1000 = the metric's "us/GEMM")
  roofline     achieved / peak HBM bandwidth for the GEMM kernel (algorithmic bytes = m*k/2)
  cpu_baseline the CPU oracle's dequantize-then-matmul on benchmark configuration 0, host cores
  frac_hbm_by_shape   fraction of 8 TB/s for every 16-token layer shape of the benchmark configurations

Everything else - the per-shape table with configs and kernels, the same shapes eight to a launch, the
Llama-70B 80-layer sweep, the token sweep, the dequant / quantizer / blockwise timings and the yardsticks -
goes into one "detail" JSON object that is printed on an earlier line and written to the file DETAIL_FILE names.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Kernel arguments placed in device memory by the HIP runtime instead of host memory: the
# command processor then reads them locally, which takes about 1 us off every launch of a
# 10 us kernel.  A runtime setting of the process (read when HIP initialises), recommended
# for serving processes; the caller's own value wins.
os.environ.setdefault("HIP_FORCE_DEV_KERNARG", "1")

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = 2500.0  # dense fp16 matrix peak of the MI355X, published
METRIC = "us/GEMM + HBM GB/s (frac of ~8 TB/s) at M=16, Mistral/Llama-70B shapes"
HEADLINE = "mistral_qkv"
TOKENS = 16
CACHE_BYTES = 256 << 20  # Infinity Cache; the rotation streams at least twice this between re-uses

# HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE in KiB per dispatch, each
# scaled by the same counter's reading for the copy kernel of known size: factors 2.000 and 1.000), from the
# summaries under profiles/.  Keyed by shape AND by the kernel the profile was taken of: when the table or
# the dispatcher picks another kernel for the shape, the entry no longer applies and `traffic` is null.
MEASURED_TRAFFIC = {
    # profiles/gemm_kernels_hbm_traffic_all_16_token_shapes.md
    ("mistral_attn_out", "gemm_narrow_kernel<LW=1,WK=8,U=8,PERM=1,TT=1>"): (4666.0, 128.0),
    ("mistral_qkv", "gemm_narrow_kernel<LW=2,WK=8,U=4,PERM=1,TT=1>"): (6707.1, 192.0),
    ("mistral_gate_up", "gemm_mid_kernel<U=2,TT=1,XB=4,1024 threads,weights through LDS> x_chunk=512"): (29325.8, 896.0),
    ("mistral_down", "gemm_lean_kernel<WK=4,U=2,512 threads> split_k=8"): (17215.1, 2185.0),
    ("llama70b_qkv", "gemm_lean_kernel<WK=4,U=2,1024 threads> split_k=4"): (22859.5, 2886.2),
    ("llama70b_attn_out", "gemm_lean_kernel<WK=4,U=8,512 threads> split_k=4"): (18547.0, 2314.0),
    ("llama70b_gate_up", "gemm_mid_kernel<U=4,TT=1,XB=4,1024 threads,weights through LDS> x_chunk=512"): (116004.4, 1792.0),
    ("llama70b_down", "gemm_multi_kernel<U=2> waves_m=4 waves_k=4"): (65442.8, 4361.0),
    ("mixtral_gate_up_8e", "gemm_mid_kernel<U=4,TT=1,XB=4,1024 threads> x_chunk=1024"): (231760.9, 8960.0),
    ("mixtral_down_8e", "gemm_mid_kernel<U=2,TT=1,XB=4,1024 threads,weights through LDS> x_chunk=512"): (116656.2, 1024.0),
}


def traffic_bytes(shape_name, kernel):
    kib = MEASURED_TRAFFIC.get((shape_name, kernel))
    return int((kib[0] * 2.000 + kib[1] * 1.000) * 1024) if kib else None


def roofline_block(shape_name, r):
    """The `roofline` object of one timed shape `r` (a time_shape result): packed-weight bytes against HBM up
    to 64 tokens, flops against the dense fp16 matrix peak from 128 tokens (the ridge of the op is about 64)."""
    if r["n"] >= 128:
        return {
            "bound": "mfma", "achieved": r["tflops"], "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(r["tflops"] / MFMA_PEAK_TFLOPS, 4), "traffic": None, "kernel": "tuna::" + r["kernel"],
            "algorithmic_flops_per_launch": 2 * r["m"] * r["n"] * r["k"], "avg_launch_us": r["us_per_gemm"],
        }
    return {
        "bound": "hbm", "achieved": r["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(r["gbs"] / HBM_PEAK_GBS, 4),
        "traffic": traffic_bytes(shape_name, r["kernel"]) if r["n"] == TOKENS else None,
        "kernel": "tuna::" + r["kernel"],
        "algorithmic_bytes_per_launch": r["packed_bytes"],
        "avg_launch_us": r["us_per_gemm"],
    }


def n_sets_for(bytes_per_set: int, cap_bytes: int) -> int:
    n = max(2, -(-2 * CACHE_BYTES // bytes_per_set))
    return max(2, min(n, max(2, cap_bytes // bytes_per_set)))


def time_shape(ops, synth, torch, dev, m, n, k, steps, warmup, seed0=0, use_graph=False, cfg=None, sets=None, settle=0,
               settle_ms=0.0):
    """-> dict with us_per_gemm, GB/s, TFLOP/s, roofline fraction for one shape.  `settle` untimed
    launches run before the warm-up (clocks and caches of a box that has just been idle); `settle_ms`
    asks for that many milliseconds of them instead (the count comes from a five-launch estimate)."""
    bytes_w = m * k // 2
    if sets is None:
        ns = n_sets_for(bytes_w, 24 << 30)
        sets = [synth.make_weights_torch(m, k, seed0 + i, dev) for i in range(ns)]
    qs = [s[0] for s in sets]
    ams = [s[1] for s in sets]
    x = synth.make_x_torch(n, k, seed0, dev)
    from tuna_amd.quantize import nf4_codebook

    code = nf4_codebook(dev)
    out = torch.empty((n, m), dtype=torch.float16, device=dev)
    torch.cuda.synchronize()
    if settle_ms > 0:
        est = ops.time_matmul(qs, ams, x, code, out, m, n, k, config=cfg, warmup=1, iters=5, use_graph=False) / 5.0
        settle = max(settle, min(20000, int(settle_ms / max(est, 1e-4)) + 1))
    if settle > 0:
        ops.time_matmul(qs, ams, x, code, out, m, n, k, config=cfg, warmup=0, iters=settle, use_graph=False)
    ms = ops.time_matmul(qs, ams, x, code, out, m, n, k, config=cfg, warmup=warmup, iters=steps, use_graph=use_graph)
    us = ms * 1000.0 / steps
    gbs = bytes_w / (us * 1e-6) / 1e9
    used, hit = ops.select_config(m, n, k)
    return {
        "m": m, "n": n, "k": k, "packed_bytes": bytes_w, "weight_sets": len(qs),
        "us_per_gemm": round(us, 3), "gbs": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4),
        "tflops": round(2.0 * m * n * k / (us * 1e-6) / 1e12, 2),
        "config": (cfg or used).to_dict(), "config_from_table": bool(hit) if cfg is None else None,
        "launch": "graph" if use_graph else "stream",
        "kernel": ops.describe_launch(m, n, k, cfg),
    }


def mfma_shapes(ops, synth, torch, dev, tokens):
    """The many-token kernel's 256 x 128 tile with v_mfma_f32_16x16x32_f16 and with v_mfma_f32_32x32x16_f16
    (rows_per_wave 64 / 32 in the config), same inputs, alternating, on two Llama-70B shapes."""
    out = {}
    for name in ("llama70b_gate_up", "llama70b_qkv"):
        m, k = synth.SHAPES[name]
        sets = [synth.make_weights_torch(m, k, 40 + i, dev) for i in range(3)]
        row = {}
        for rep in range(2):
            for label, rpw in (("mfma_16x16x32", 64), ("mfma_32x32x16", 32)):
                c = ops.GemmConfig(rows_per_wave=rpw, waves_m=1, waves_k=1, split_k=1, prefetch=2, x_chunk=64, token_tiles=8,
                                   xcd_swizzle=0, k_stagger=0, lds_tile_rows=256)
                r = time_shape(ops, synth, torch, dev, m, tokens, k, 20, 5, cfg=c, sets=sets)
                if label not in row or r["us_per_gemm"] < row[label]["us"]:
                    row[label] = {"us": r["us_per_gemm"], "tflops": r["tflops"], "kernel": r["kernel"]}
        out[name] = {"tokens": tokens, **row}
        del sets
        torch.cuda.empty_cache()
    return out


def cpu_baseline(m, n, k, budget_s=12.0):
    """The oracle's dequantize (D2) + fp32 matmul on the host cores (checker code timed as a
    reported baseline only)."""
    import numpy as np

    from oracle import oracle as O
    from tuna_amd.synth import make_inputs_np

    q, x, code, absmax = make_inputs_np(m, n, k, seed=0)
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count() or 1
    cores = max(1, min(cores, O.max_threads() if O.max_threads() > 0 else cores))
    xb = x.view(np.uint16)
    # single-thread figure (one pass) and the all-cores figure (median over the budget)
    _, td1, tm1, _ = O.cpu_baseline(q, xb, code, absmax, m, n, k, threads=1)
    times, dec, mat = [], [], []
    O.cpu_baseline(q, xb, code, absmax, m, n, k, threads=cores)  # warm-up
    t_end = time.perf_counter() + budget_s
    while time.perf_counter() < t_end or len(times) < 3:
        _, td, tm, _ = O.cpu_baseline(q, xb, code, absmax, m, n, k, threads=cores)
        times.append(td + tm)
        dec.append(td)
        mat.append(tm)
        if len(times) >= 200:
            break
    med = float(np.median(times))
    bytes_w = m * k // 2
    return {
        "value": round(bytes_w / med / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
        "sample": f"benchmark config 0, seed 0: {len(times)} full GEMMs m={m} n={n} k={k} (decode to fp16, then "
                  f"fp32-accumulate matmul), median of total; oracle/tuna_oracle.c with OpenMP",
        "us_per_gemm": round(med * 1e6, 1), "us_decode": round(float(np.median(dec)) * 1e6, 1),
        "us_matmul": round(float(np.median(mat)) * 1e6, 1),
        "single_thread_us_per_gemm": round((td1 + tm1) * 1e6, 1),
    }


READ_VARIANTS = {0: "nontemporal x8", 1: "plain x8", 2: "nontemporal x16", 3: "plain x16", 4: "nontemporal x4", 5: "plain x4"}


def read_sweep(ops, torch, dev, nbytes=2 << 30, iters=5):
    """Rate of the read-only kernel over `nbytes` for every (workgroups, variant): {label: GB/s}."""
    big = torch.full((nbytes,), 3, dtype=torch.uint8, device=dev)
    out = {}
    for variant, vname in READ_VARIANTS.items():
        for blocks in (256, 512, 1024, 2048, 4096, 8192):
            ms = ops.time_read(big, blocks=blocks, variant=variant, warmup=2, iters=iters) / iters
            out[f"{vname}, {blocks} workgroups"] = round(nbytes / (ms * 1e-3) / 1e9, 1)
    del big
    torch.cuda.empty_cache()
    return out


def copy_yardstick(ops, torch, dev, mib):
    """The plain copy kernel over `mib` mebibytes: the known-traffic launch the HBM counters are scaled by."""
    nb = mib << 20
    src = torch.full((nb,), 7, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    ms = ops.time_copy(src, dst, warmup=2, iters=10)
    return {"bytes_read": nb, "bytes_written": nb, "us": round(ms * 100.0, 2),
            "gbs_read_plus_write": round(2 * nb / (ms * 1e-4) / 1e9, 1)}


def multi_stream(ops, synth, torch, dev, names=("mistral_attn_out", "mistral_qkv"), tokens=TOKENS, iters=1024):
    """Independent GEMMs (rotating weights, one output buffer per stream) dealt round-robin to 1, 2 and 4 streams of
    the default priority, and the empty kernel the same way: us per GEMM over all streams.  Beside the single-stream
    headline, never instead of it: a decoder layer's GEMMs depend on each other and run on one stream."""
    from tuna_amd.quantize import nf4_codebook

    code = nf4_codebook(dev)
    out = {"empty_kernel_us": {f"{ns}_{mode}": round(ops.time_empty_launches(dev, n_streams=ns, use_graph=mode == "graph", iters=2048) * 1000.0 / 2048, 3)
                               for ns in (1, 2, 4) for mode in ("stream", "graph")}}
    for nm in names:
        m, k = synth.SHAPES[nm]
        ns_sets = n_sets_for(m * k // 2, 2 << 30)
        sets = [synth.make_weights_torch(m, k, 6000 + i, dev) for i in range(ns_sets)]
        x = synth.make_x_torch(tokens, k, 5, dev)
        row = {}
        for ns in (1, 2, 4):
            outs = [torch.empty((tokens, m), dtype=torch.float16, device=dev) for _ in range(ns)]
            for mode in ("stream", "graph"):
                args = ([s_[0] for s_ in sets], [s_[1] for s_ in sets], x, code, outs, m, tokens, k)
                ops.time_matmul_streams(*args, warmup=50, iters=256, use_graph=mode == "graph")
                ms = ops.time_matmul_streams(*args, warmup=50, iters=iters, use_graph=mode == "graph")
                us = ms * 1000.0 / iters
                row[f"{ns}_{mode}"] = {"us_per_gemm": round(us, 3), "frac_hbm": round(m * k / 2 / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}
        out[nm] = row
        del sets
        torch.cuda.empty_cache()
    return out


def handover_yardstick(ops, dev):
    """One producer -> consumer step of a split-K hand-over between two workgroups, on one XCD and across XCDs, with the
    kernels' device-coherent accesses (sc1 stores and loads) and with accesses that stay in the XCD's L2: nanoseconds
    on an otherwise idle device, and whether the consumer read what the producer wrote."""
    out = {}
    for place, same in (("same_xcd", True), ("neighbouring_xcds", False)):
        for label, st, ld, reuse in (("sc1_store_sc1_load", 1, 1, 1), ("plain_store_sc1_load", 0, 1, 1),
                                     ("plain_store_plain_load", 0, 0, 1), ("plain_store_plain_load_fresh_lines", 0, 0, 0)):
            out[f"{place}:{label}"] = ops.measure_handover(dev, same, st, ld, reuse)
    return out


def launch_floor(ops, torch, dev, headline_bytes):
    # a kernel that does nothing, 192 workgroups of 512 threads: replayed from a HIP graph (what the device needs
    # per launch) and enqueued launch by launch (where the host's enqueue time can be the longer of the two)
    us_empty = ops.time_empty_launches(dev, use_graph=True, iters=2000) * 1000.0 / 2000
    us_empty_stream = ops.time_empty_launches(dev, use_graph=False, iters=2000) * 1000.0 / 2000
    sweep = read_sweep(ops, torch, dev)
    best = max(sweep, key=sweep.get)
    rate = sweep[best]
    return {
        "empty_launch_us": round(us_empty, 3),
        "empty_launch_enqueued_one_by_one_us": round(us_empty_stream, 3),
        "read_kernel_gbs": rate,
        "read_kernel_best": best,
        "read_kernel_frac_of_peak": round(rate / HBM_PEAK_GBS, 4),
        "read_kernel_sweep_gbs": sweep,
        "headline_bytes_at_read_rate_us": round(headline_bytes / rate / 1e3, 3),
        "floor_us": round(us_empty + headline_bytes / rate / 1e3, 3),
    }


def unit_rates(ops, dev):
    """Yardsticks of the many-token kernels: what the matrix cores and the LDS of this box deliver to the MFMA
    shapes and LDS access patterns those kernels use (best of three timings each)."""
    names = ["mfma_16x16x32_f16_one_wave_per_simd_tflops", "mfma_16x16x32_f16_two_waves_per_simd_tflops",
             "mfma_32x32x16_f16_one_wave_per_simd_tflops", "lds_fragment_reads_b128_bytes_per_clk_per_cu",
             "lds_table_reads_b32_bytes_per_clk_per_cu", "lds_tile_writes_b128_bytes_per_clk_per_cu",
             "lds_tile_writes_b64_bytes_per_clk_per_cu", "lds_linear_writes_b128_bytes_per_clk_per_cu",
             "lds_table_reads_b32_copy_per_32_lanes_bytes_per_clk_per_cu", "lds_table_reads_b32_copy_per_16_lanes_bytes_per_clk_per_cu",
             "mfma_32x32x16_f16_random_operands_one_wave_per_simd_tflops", "mfma_16x16x32_f16_random_operands_two_waves_per_simd_tflops",
             "mfma_16x16x32_f16_random_operands_one_wave_per_simd_tflops", "mfma_32x32x16_f16_random_operands_two_waves_per_simd_tflops",
             "lds_table_reads_b32_16_waves_bytes_per_clk_per_cu", "lds_fragment_reads_b128_16_waves_bytes_per_clk_per_cu",
             "lds_tile_writes_b128_16_waves_bytes_per_clk_per_cu",
             "mixed_64_token_k_step_mfma_only_us", "mixed_64_token_k_step_lds_reads_only_us",
             "mixed_64_token_k_step_both_in_every_wave_us", "mixed_64_token_k_step_four_mfma_waves_four_lds_waves_us",
             "mixed_64_token_k_step_reads_between_the_mfmas_us"]
    out = {}
    for unit, nm in enumerate(names):
        best = 0.0
        for _ in range(3):
            ms, work = ops.time_unit_rate(unit, dev, warmup=1, iters=4)
            best = max(best, work * 4 / (ms * 1e-3))
        if nm.startswith("mixed"):
            out[nm] = round(work / best * 1e6, 1)  # microseconds per launch (1024 k-steps per wave, 8 waves per CU)
        else:
            out[nm] = round(best / 1e12, 1) if nm.startswith("mfma") else round(best / 256 / 2.4e9, 1)
    out["note"] = ("LDS rates per compute unit at the 2.4 GHz peak clock, 256 compute units, from 8 waves per compute unit unless the name "
                   "says 16 (reads are latency-bound at 8); the random-operand MFMA rates (operands "
                   "of pseudo-random fp16 values instead of one pair of small regular numbers) are what the matrix cores sustain "
                   "on real data: the practical ceiling of the many-token kernels")
    return out


def time_dequant_shapes(ops, synth, torch, dev, names=("mistral_attn_out", "mistral_gate_up", "llama70b_down")):
    from tuna_amd.quantize import nf4_codebook

    deq = {}
    for nm in names:
        dm, dk = synth.SHAPES[nm]
        sets = [synth.make_weights_torch(dm, dk, 50 + i, dev) for i in range(max(2, min(8, (1 << 30) // (dm * dk // 2))))]
        img = torch.empty((dm, dk), dtype=torch.float16, device=dev)
        ms = ops.time_dequant([s[0] for s in sets], [s[1] for s in sets], nf4_codebook(dev), img, dm, dk, 10, 100)
        us = ms * 10.0
        gbs = 2.5 * dm * dk / (us * 1e-6) / 1e9
        deq[nm] = {"m": dm, "k": dk, "us": round(us, 2), "gbs_in_plus_out": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4),
                   "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "kernel": "tuna::dequant_kernel",
                                "algorithmic_bytes_per_launch": int(2.5 * dm * dk), "avg_launch_us": round(us, 2)}}
        del sets, img
        torch.cuda.empty_cache()
    return deq


def time_quantize(ops, synth, torch, dev):
    """Device quantizer + packer (fp16 weights in, packed codes and scales out) on 4096 x 4096, per-row and
    per-64 scales: back-to-back launches through the C ABI on preallocated buffers, HIP events around them."""
    import ctypes

    from tuna_amd import _lib
    from tuna_amd.quantize import nf4_codebook

    qm, qk = synth.SHAPES["mistral_attn_out"]
    L = _lib.lib()
    code = nf4_codebook(dev)
    ws = [(torch.randn((qm, qk), device=dev) * 0.02).to(torch.float16) for _ in range(16)]   # 16 x 33.5 MB: beyond the caches
    q = torch.empty((qm // 8, qk // 8, 32), dtype=torch.uint8, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    res = {}
    for label, bs in (("per_row", qk), ("per_64", 64)):
        absmax = torch.empty((qm * (qk // bs),), dtype=torch.float32, device=dev)
        def launch(i):
            _lib.check(L.tuna_quantize_blockwise(ws[i % len(ws)].data_ptr(), code.data_ptr(), q.data_ptr(), absmax.data_ptr(), qm, qk,
                                                 bs, stream))
        for i in range(5):
            launch(i)
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        iters = 100
        ev0.record()
        for i in range(iters):
            launch(i)
        ev1.record()
        torch.cuda.synchronize()
        us = ev0.elapsed_time(ev1) * 1000.0 / iters
        nbytes = 2.5 * qm * qk + 4 * qm * (qk // bs)    # fp16 in, half a byte per weight and the scales out
        gbs = nbytes / (us * 1e-6) / 1e9
        res[label] = {"m": qm, "k": qk, "block_size": bs, "us": round(us, 2), "gbs_fp16_in": round(2.0 * qm * qk / (us * 1e-6) / 1e9, 1),
                      "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                   "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "kernel": "tuna::quantize_kernel",
                                   "algorithmic_bytes_per_launch": int(nbytes), "avg_launch_us": round(us, 2)}}
    return res


def time_blockwise(ops, synth, torch, dev, names=("mistral_qkv", "mistral_gate_up", "llama70b_qkv", "llama70b_gate_up", "llama70b_down"),
                   block_size=64, tokens=16):
    """tuna_matmul_blockwise (one fp32 scale per `block_size` weights of a row, the layout of block-quantized NF4
    checkpoints) on some of the 16-token shapes: calls through the C ABI over rotating weights, recorded once into a
    HIP graph and replayed (a call from Python costs about 10 us, more than the smaller launches take), HIP events
    around the replays on torch's stream.  Algorithmic bytes: packed weights + scales."""
    from tuna_amd import _lib
    from tuna_amd.quantize import nf4_codebook

    L = _lib.lib()
    code = nf4_codebook(dev)
    out = {}
    for nm in names:
        m, k = synth.SHAPES[nm]
        nsets = max(2, min(24, int(600e6 // (m * k // 2))))
        sets = [synth.make_weights_torch(m, k, 70 + i, dev) for i in range(nsets)]
        scales = [torch.rand((m, k // block_size), dtype=torch.float32, device=dev) * 0.015 + 0.005 for _ in range(nsets)]
        x = synth.make_x_torch(tokens, k, 3, dev)
        o = torch.empty((tokens, m), dtype=torch.float16, device=dev)
        before = [L.tuna_blockwise_launches(i) for i in range(4)]
        calls = 4 * nsets
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            for i in range(nsets):  # (the library's workspace exists before the capture starts)
                ops.matmul_blockwise(x, sets[i][0], scales[i], code, o, m, tokens, k, block_size)
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for i in range(calls):
                    ops.matmul_blockwise(x, sets[i % nsets][0], scales[i % nsets], code, o, m, tokens, k, block_size)
        torch.cuda.synchronize()
        took = [L.tuna_blockwise_launches(i) - before[i] for i in range(4)]
        kernel = ("tuna::gemm_narrow_kernel", "tuna::gemm_multi_kernel", "tuna::gemm_tiled_kernel", "tuna::gemm_mid_kernel")[took.index(max(took))]
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        replays = max(3, 300 // calls)
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for _ in range(replays):
            graph.replay()
        ev1.record()
        torch.cuda.synchronize()
        us = ev0.elapsed_time(ev1) * 1000.0 / (replays * calls)
        del graph
        nbytes = m * k // 2 + 4 * m * (k // block_size)
        gbs = nbytes / (us * 1e-6) / 1e9
        out[nm] = {"m": m, "k": k, "block_size": block_size, "us": round(us, 2),
                   "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                                "kernel": kernel + " (scale blocks)",
                                "algorithmic_bytes_per_launch": nbytes, "avg_launch_us": round(us, 2)}}
        del sets, scales
        torch.cuda.empty_cache()
    return out


def multi_layer_sweep(ops, synth, torch, dev, names, n, layers, iters=None, seed0=10_000):
    """`layers` calls of tuna_matmul_multi, each with the GEMMs `names` of one layer (distinct seeded weights per
    layer), back to back: us per call, packed-weight GB/s.  The independent-problems reading of a layer: what
    a benchmark sweep or a batch of unrelated projections can use; a real decoder layer's GEMMs feed one another."""
    from tuna_amd.quantize import nf4_codebook

    code = nf4_codebook(dev)
    batches, total_bytes = [], 0
    xs = {nm: synth.make_x_torch(n, synth.SHAPES[nm][1], seed0, dev) for nm in names}
    outs = [torch.empty((n, synth.SHAPES[nm][0]), dtype=torch.float16, device=dev) for nm in names]  # one per problem of a launch
    for layer in range(layers):
        b = []
        for j, nm in enumerate(names):
            m, k = synth.SHAPES[nm]
            q, a = synth.make_weights_torch(m, k, seed0 + layer * len(names) + j, dev)
            b.append((xs[nm], q, a, code, outs[j], m, n, k))
        batches.append(b)
    total_bytes = sum(synth.SHAPES[nm][0] * synth.SHAPES[nm][1] // 2 for nm in names)
    iters = iters or 2 * layers
    best = None
    for use_graph in (False, True):
        ms = ops.time_matmul_multi(batches, warmup=layers, iters=iters, use_graph=use_graph)
        us = ms * 1000.0 / iters
        if best is None or us < best[0]:
            best = (us, "graph" if use_graph else "stream")
    us = best[0]
    del batches
    torch.cuda.empty_cache()
    return {
        "launch": "multi", "gemms_per_launch": len(names), "us_per_launch": round(us, 2),
        "us_per_gemm_mean": round(us / len(names), 3), "ms_all": round(us * layers / 1000, 3),
        "packed_bytes_per_launch": total_bytes, "gbs": round(total_bytes / (us * 1e-6) / 1e9, 1),
        "frac_hbm": round(total_bytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4), "enqueue": best[1],
        "kernel": "tuna::gemm_multi_kernel",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--no-shapes", action="store_true", help="skip the per-shape table")
    ap.add_argument("--no-sweeps", action="store_true", help="skip the 80-layer and token sweeps")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--only-headline", action="store_true", help="headline workload only (profiling runs)")
    ap.add_argument("--workload", default=HEADLINE, help="shape name, or <rows>x<k>, timed as the headline (profiling runs)")
    ap.add_argument("--tokens", type=int, default=TOKENS, help="token count of the headline workload")
    ap.add_argument("--launch", choices=("both", "stream", "graph"), default="both")
    ap.add_argument("--settle", type=int, default=300,
                    help="untimed launches before the warm-up of the headline (a box that was idle ramps its clocks)")
    ap.add_argument("--only", choices=("read", "dequant", "quantize", "multi", "mfma", "rates", "blockwise", "streams", "handover"), default=None,
                    help="profiling runs: launch only the read-kernel sweep / the dequant kernel / the quantizer / "
                         "the Llama-70B layer set through tuna_matmul_multi (16 layers) / the many-token kernel with "
                         "16x16x32 and with 32x32x16 MFMA tiles (Llama-70B gate+up and QKV, --tokens, default 1024) / the "
                         "matrix-core and LDS yardstick kernels / the blockwise GEMM (a scale per 64 weights) / the two "
                         "smallest shapes dealt to 1, 2 and 4 streams")
    ap.add_argument("--weight-path", choices=("table", "registers", "lds"), default="table",
                    help="headline workload: the table's config as it is, or with the packed weights forced through "
                         "registers / staged through LDS (lds_tile_rows 0 / -1; A/B runs of the two weight paths)")
    ap.add_argument("--copy-yardstick", type=int, default=0, metavar="MIB",
                    help="also launch the plain copy kernel over MIB mebibytes (counter runs: the known-traffic "
                         "launch the HBM counters of the GEMM kernel are scaled by)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)
    if args.only_headline:
        args.no_shapes = args.no_sweeps = args.no_cpu = True

    import torch

    from tuna_amd import _lib, ops, synth

    # The timing loops (HIP events around back-to-back launches, no Python in between) and the yardstick kernels
    # live in the diagnostic build, libtuna_amd_bench.so: the product library's own object files plus those tools.
    # Every GEMM this program times is launched through that library's tuna_matmul_ex / tuna_matmul_multi.
    _lib.use_diagnostic_build()

    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.only:
        if args.only == "read":
            res = {"read_kernel_sweep_gbs": read_sweep(ops, torch, dev)}
        elif args.only == "dequant":
            res = {"dequant": time_dequant_shapes(ops, synth, torch, dev)}
        elif args.only == "quantize":
            res = {"quantize": time_quantize(ops, synth, torch, dev)}
        elif args.only == "rates":
            res = {"unit_rates": unit_rates(ops, dev)}
        elif args.only == "handover":
            res = {"handover_yardstick": handover_yardstick(ops, dev)}
        elif args.only == "streams":
            res = {"headline_multi_stream": multi_stream(ops, synth, torch, dev, iters=256)}
        elif args.only == "blockwise":
            res = {"blockwise_gemm_block_64": time_blockwise(ops, synth, torch, dev)}
        elif args.only == "mfma":
            res = {"many_token_kernel_mfma_shapes": mfma_shapes(ops, synth, torch, dev, 1024 if args.tokens == TOKENS else args.tokens)}
        else:
            names = ["llama70b_qkv", "llama70b_attn_out", "llama70b_gate_up", "llama70b_down"]
            res = {"llama70b_layers_multi": multi_layer_sweep(ops, synth, torch, dev, names, args.tokens, layers=16)}
        if args.copy_yardstick > 0:
            res["copy_yardstick"] = copy_yardstick(ops, torch, dev, args.copy_yardstick)
        print(json.dumps(res))
        return

    if args.workload in synth.SHAPES:
        m, k = synth.SHAPES[args.workload]
    else:                                   # (profiling runs of a shape outside the benchmark set: "<rows>x<k>")
        m, k = (int(t) for t in args.workload.lower().split("x"))
    n = args.tokens
    head_cfg = None
    if args.weight_path != "table":
        head_cfg, _ = ops.select_config(m, n, k)
        head_cfg.lds_tile_rows = -1 if args.weight_path == "lds" else 0
        ops.validate_config(m, n, k, head_cfg)   # raises where the shape's config has no such twin
    res_stream = res_graph = None
    if args.launch in ("both", "stream"):
        res_stream = time_shape(ops, synth, torch, dev, m, n, k, args.steps, args.warmup, use_graph=False, cfg=head_cfg,
                                settle=args.settle)
    if args.launch in ("both", "graph"):
        res_graph = time_shape(ops, synth, torch, dev, m, n, k, args.steps, args.warmup, use_graph=True, cfg=head_cfg,
                               settle=args.settle)
    cands = [r for r in (res_stream, res_graph) if r is not None]
    head = min(cands, key=lambda r: r["us_per_gemm"])
    line = {
        "metric": METRIC,
        "value": head["gbs"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(head["us_per_gemm"] / 1000.0, 6),
        "us_per_gemm": head["us_per_gemm"],
        "tflops": head["tflops"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": f"{'benchmark config 1: Mistral-7B QKV projection' if args.workload == HEADLINE else args.workload}, "
                        f"M={n} tokens, K={k}, N={m}; "
                        f"uniform 4-bit codes, fp16 scales U(0.005,0.02), x ~ N(0,1)*0.1; "
                        f"{head['weight_sets']} distinct weight matrices rotated",
            "tile_config": head["config"],
            "launch": head["launch"],
        },
        "roofline": roofline_block(args.workload, head),
        "headline_stream_launch": res_stream,
        "headline_graph_launch": res_graph,
    }

    # Yardsticks for the fixed cost of a launch, measured in the same run: back-to-back launches of a
    # read kernel over 4 KB (nothing to stream: the time per launch is what any kernel pays on this box)
    # and the best rate a read-only kernel reaches over 2 GB (sweep over workgroup counts, loads in flight
    # and nontemporal / plain loads).  A launch that streams the headline's packed bytes at that rate
    # cannot take less than their sum.
    if not args.only_headline:
        line["launch_floor"] = launch_floor(ops, torch, dev, head["packed_bytes"])
        line["unit_rates"] = unit_rates(ops, dev)
        line["headline_multi_stream"] = multi_stream(ops, synth, torch, dev)
        line["handover_yardstick"] = handover_yardstick(ops, dev)

    if args.copy_yardstick > 0:
        line["copy_yardstick"] = copy_yardstick(ops, torch, dev, args.copy_yardstick)

    if not args.no_shapes:
        shapes = {}
        steps = max(50, min(args.steps, 300))
        for name, (sm, sk) in synth.SHAPES.items():
            r_s = time_shape(ops, synth, torch, dev, sm, n, sk, steps, max(10, args.warmup // 5), seed0=1000, settle_ms=10.0)
            r_g = time_shape(ops, synth, torch, dev, sm, n, sk, steps, max(10, args.warmup // 5), seed0=1000,
                             use_graph=True)
            best = r_g if r_g["us_per_gemm"] < r_s["us_per_gemm"] else r_s
            best["us_stream"] = r_s["us_per_gemm"]
            best["us_graph"] = r_g["us_per_gemm"]
            best["roofline"] = roofline_block(name, best)
            shapes[name] = best
            torch.cuda.empty_cache()
        line["shapes"] = shapes
        line["min_frac_hbm_over_shapes"] = min(v["frac_hbm"] for v in shapes.values())
        # every shape again as batches of 8 independent problems per launch (tuna_matmul_multi, distinct weights):
        # what the per-launch fixed time costs each shape, beside the one-GEMM-per-launch numbers above
        shapes_multi = {}
        for name in synth.SHAPES:
            sets = max(2, min(16, (4 << 30) // (8 * synth.SHAPES[name][0] * synth.SHAPES[name][1] // 2)))
            r = multi_layer_sweep(ops, synth, torch, dev, [name] * 8, n, layers=sets, iters=max(20, 2 * sets), seed0=3000)
            shapes_multi[name] = {"launch": "multi", "gemms_per_launch": 8, "us_per_gemm": r["us_per_gemm_mean"],
                                  "gbs": r["gbs"], "frac_hbm": r["frac_hbm"], "enqueue": r["enqueue"], "kernel": r["kernel"]}
        line["shapes_multi_x8"] = shapes_multi
        line["min_frac_hbm_over_shapes_multi_x8"] = min(v["frac_hbm"] for v in shapes_multi.values())
        line["dequant"] = time_dequant_shapes(ops, synth, torch, dev)
        line["quantize"] = time_quantize(ops, synth, torch, dev)
        line["blockwise_gemm_block_64"] = time_blockwise(ops, synth, torch, dev)

    if not args.no_shapes:
        # Mixtral gate+up with a router: 16 tokens x top-2 = 32 (token, expert) rows spread over the 8
        # experts; each expert multiplies only its own rows (grouped GEMM, one launch).  "dense" is
        # the reference's all-experts-on-all-tokens reading of the same weights.
        from tuna_amd.quantize import nf4_codebook

        gm, gk = 28672, 4096
        sets = [synth.make_weights_torch(8 * gm, gk, 4000 + i, dev) for i in range(3)]
        moe = {}
        for label, counts in (("balanced_4_per_expert", [4] * 8), ("skewed", [9, 0, 6, 1, 0, 11, 5, 0]),
                              ("two_experts", [16, 0, 0, 0, 16, 0, 0, 0]),
                              ("prefill_256_per_expert", [256] * 8), ("prefill_skewed", [700, 3, 0, 90, 1024, 40, 0, 191])):
            offs = [0]
            for cnt in counts:
                offs.append(offs[-1] + cnt)
            xg = synth.make_x_torch(offs[-1], gk, 7, dev)
            og = torch.empty((offs[-1], gm), dtype=torch.float16, device=dev)
            big = max(counts) > 64  # (groups of more than 64 tokens run as dense GEMMs of their own: fewer, longer calls)
            it = 12 if big else 100
            ms = ops.time_matmul_grouped([s_[0] for s_ in sets], [s_[1] for s_ in sets], xg, nf4_codebook(dev), og, gm, 8, gk,
                                         offs, warmup=3 if big else 10, iters=it, use_graph=True)
            us = ms * 1e3 / it
            active = sum(1 for cnt in counts if cnt)
            moe[label] = {"tokens_per_expert": counts, "us": round(us, 2), "active_experts": active,
                          "packed_bytes_read": active * gm * gk // 2,
                          "gbs": round(active * gm * gk / 2 / (us * 1e-6) / 1e9, 1),
                          "tflops": round(2.0 * offs[-1] * gm * gk / (us * 1e-6) / 1e12, 1)}
        del sets
        torch.cuda.empty_cache()
        line["mixtral_gate_up_routed"] = moe

    if not args.no_sweeps:
        sweeps = {}
        # Llama-70B decoder layer x 80 layers, distinct seeded weights per layer (34.2 GB resident)
        names = ["llama70b_qkv", "llama70b_attn_out", "llama70b_gate_up", "llama70b_down"]
        try:
            layer_us = {}
            total_bytes = 0
            for nm in names:
                sm, sk = synth.SHAPES[nm]
                sets = [synth.make_weights_torch(sm, sk, 10_000 + layer, dev) for layer in range(80)]
                r = time_shape(ops, synth, torch, dev, sm, n, sk, 160, 80, sets=sets, use_graph=True)
                layer_us[nm] = r["us_per_gemm"]
                total_bytes += sm * sk // 2
                del sets
                torch.cuda.empty_cache()
            tot = sum(layer_us.values())
            sweeps["llama70b_80_layers"] = {
                "us_per_gemm": layer_us, "us_per_layer": round(tot, 2), "ms_80_layers": round(tot * 80 / 1000, 3),
                "packed_bytes_per_layer": total_bytes, "gbs": round(total_bytes / (tot * 1e-6) / 1e9, 1),
                "frac_hbm": round(total_bytes / (tot * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            }
        except torch.OutOfMemoryError as e:  # pragma: no cover
            sweeps["llama70b_80_layers"] = {"error": str(e)[:200]}
        # the same 80 layers with the four GEMMs of a layer in ONE launch (tuna_matmul_multi): one call per layer
        try:
            sweeps["llama70b_80_layers_multi"] = multi_layer_sweep(ops, synth, torch, dev, names, n, layers=80)
        except torch.OutOfMemoryError as e:  # pragma: no cover
            sweeps["llama70b_80_layers_multi"] = {"error": str(e)[:200]}
        # token sweep on the Llama-70B layer set: the lower edges of the token buckets (where the table's entries are
        # tuned) and counts inside them (24, 100, 384: served by the entry their bucket's next_from points to, or an
        # entry of their own; 1536: between two tuning counts, where shapes of fewer than 24576 rows take the pick
        # of the derivation's cost model)
        tok = {}
        for nt in (1, 16, 24, 64, 100, 256, 384, 1024, 1536, 4096):
            row = {}
            for nm in names:
                sm, sk = synth.SHAPES[nm]
                r = time_shape(ops, synth, torch, dev, sm, nt, sk, 100, 20, seed0=2000, use_graph=True, settle_ms=25.0)
                row[nm] = {"us": r["us_per_gemm"], "gbs": r["gbs"], "tflops": r["tflops"], "kernel": r["kernel"],
                           "roofline": roofline_block(nm, r)}
                torch.cuda.empty_cache()
            tok[str(nt)] = row
        sweeps["token_sweep_llama70b"] = tok
        line["sweeps"] = sweeps

    # The published matrix peak is reached on regular operands only; beside every fraction of it, the fraction of
    # what this box's matrix cores sustained on pseudo-random operands in this run (the faster of the two MFMA
    # shapes, two waves per SIMD).
    sustained = max((v for key, v in line.get("unit_rates", {}).items() if "random_operands" in key), default=None)
    if sustained:
        def annotate(obj):
            if isinstance(obj, dict):
                if obj.get("bound") == "mfma" and "achieved" in obj:
                    obj["sustained_on_random_operands"] = sustained
                    obj["frac_of_sustained"] = round(obj["achieved"] / sustained, 4)
                for v in obj.values():
                    annotate(v)
        annotate(line)

    if not args.no_cpu:
        # benchmark configuration 0: the CPU path on the Mistral attention out-proj shape, 16 tokens, seed 0
        cm, ck = synth.SHAPES["mistral_attn_out"]
        line["cpu_baseline"] = cpu_baseline(cm, TOKENS, ck)
    else:
        line["cpu_baseline"] = None

    detail_path = write_detail(line)
    print(json.dumps({"detail": line}))
    print(headline_line(line, detail_path))


DETAIL_FILE = os.path.join("gpurun_out", "bench_detail.json")
HEADLINE_KEYS = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "us_per_gemm", "tflops",
                 "higher_is_better", "scaling", "vs_baseline", "dtype", "data")
ROOFLINE_KEYS = ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "algorithmic_bytes_per_launch",
                 "avg_launch_us")
CPU_KEYS = ("value", "unit", "cores", "kind", "sample", "us_per_gemm", "single_thread_us_per_gemm")


def write_detail(detail):
    """Writes the full result object beside the repository's other GPU-run outputs; -> the relative path, or None
    where the directory cannot be written."""
    try:
        os.makedirs(os.path.join(ROOT, os.path.dirname(DETAIL_FILE)), exist_ok=True)
        with open(os.path.join(ROOT, DETAIL_FILE), "w") as f:
            json.dump(detail, f, indent=1)
        return DETAIL_FILE
    except OSError:
        return None


def headline_line(detail, detail_path=None):
    """The last line bench.py prints: the headline measurement only, as compact JSON of well under 2 KB whatever the
    detail object holds (the harness that runs the bench keeps the end of stdout and parses its last line)."""
    line = {key: detail.get(key) for key in HEADLINE_KEYS}
    cfg = detail.get("config") or {}
    line["config"] = {"workload": str(cfg.get("workload", ""))[:300], "launch": cfg.get("launch"),
                      "timed_launches": detail.get("steps"), "tile_config": cfg.get("tile_config")}
    roof = detail.get("roofline") or {}
    line["roofline"] = {key: roof.get(key) for key in ROOFLINE_KEYS}
    cpu = detail.get("cpu_baseline")
    line["cpu_baseline"] = None if cpu is None else {key: (str(cpu.get(key))[:200] if key == "sample" else cpu.get(key))
                                                     for key in CPU_KEYS}
    shapes = detail.get("shapes") or {}
    if shapes:
        line["frac_hbm_by_shape"] = {name: r.get("frac_hbm") for name, r in list(shapes.items())[:12]}
    line["detail"] = detail_path
    return json.dumps(line, separators=(",", ":"))


if __name__ == "__main__":
    main()
