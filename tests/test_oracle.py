"""CPU tests of the oracle itself: it is pinned here before any GPU result is compared to it.

Pins used (none of them re-types the oracle's own formula):
  * float conversions  : numpy's IEEE-754 float16 casts, exhaustively / on dense sweeps incl. ties
  * codebook           : fp32 and fp16 bit patterns of the literals in the reference harness
  * packed layout      : closed-form bit positions + brute force + the product's independent packer
  * decode D1 / D2     : numpy float16 / float32 arithmetic over 16 codes x all 65536 scale patterns,
                         and the known-answer rows for scale 0x211f
  * GEMM               : numpy float64 matmul on the decoded image, linearity, one-hot read-out,
                         row permutation
"""
import hashlib
import json
import os

import numpy as np
import pytest

from oracle import oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# fp32 / fp16 bit patterns of the 16 NF4 constants of the reference harness (test.py:19-37)
CODE_F32_BITS = ("bf800000 bf3239b1 bf066b30 beca32a0 be91a24d be3d353f bdba7871 00000000 "
                 "3da2faff 3e24cae3 3e7c04dd 3ead033a 3ee1a4b8 3f1007ab 3f3913b3 3f800000").split()
CODE_F16_BITS = "bc00 b992 b833 b652 b48d b1ea add4 0000 2d18 3126 33e0 3568 370d 3880 39c9 3c00".split()
# decode known answers for the fp16 scale 0x211f (~0.01)
KAT_D1 = "a11f 9f22 9d60 9c0c 99d4 9792 9376 0000 1285 1697 190b 1aec 1c83 1dc3 1f68 211f".split()
KAT_D2 = "a11f 9f21 9d61 9c0b 99d4 9792 9376 0000 1285 1698 190b 1aec 1c84 1dc3 1f68 211f".split()


def test_f16_to_f32_exhaustive():
    h = np.arange(65536, dtype=np.uint16)
    got = O.f16_to_f32(h)
    want = h.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])


def _same_f16(got_bits, want_f16):
    want_bits = want_f16.view(np.uint16)
    nan = np.isnan(want_f16)
    assert np.array_equal(got_bits[~nan], want_bits[~nan])
    assert ((got_bits[nan] & 0x7c00) == 0x7c00).all() and ((got_bits[nan] & 0x3ff) != 0).all()


def test_f32_to_f16_ties_neighbours_and_random():
    # every representable half, the midpoint between neighbours (exact ties) and one float ulp either side
    h = np.arange(0, 0x7c00, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)  # exact in float32
    cases = [mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)), lo.astype(np.float32)]
    v = np.concatenate(cases + [-c for c in cases])
    with np.errstate(over="ignore"):
        _same_f16(O.f32_to_f16(v), v.astype(np.float16))
    rng = np.random.default_rng(0)
    bits = rng.integers(0, 2 ** 32, size=4_000_000, dtype=np.uint64).astype(np.uint32)
    v = bits.view(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        _same_f16(O.f32_to_f16(v), v.astype(np.float16))


def test_f64_to_f16_direct_rounding():
    rng = np.random.default_rng(1)
    v = np.concatenate([rng.standard_normal(500_000) * 10.0 ** rng.integers(-9, 6, 500_000),
                        np.array([0.0, -0.0, 65504.0, 65519.999, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25,
                                  2.0 ** -25 * 1.0000001, 5.96e-8, np.inf, -np.inf])])
    with np.errstate(over="ignore"):
        _same_f16(O.f64_to_f16(v), v.astype(np.float16))
    # a double that rounds differently when it goes through float32 first (double rounding)
    x = 1.0 + 2.0 ** -11 + 2.0 ** -40  # just above a half tie: must round up
    assert O.f64_to_f16(np.array([x]))[0] == np.float16(1.0 + 2.0 ** -10).view(np.uint16)


def test_codebook_bit_patterns():
    cb = O.nf4_codebook()
    assert ["%08x" % b for b in cb.view(np.uint32)] == CODE_F32_BITS
    assert ["%04x" % b for b in O.f32_to_f16(cb)] == CODE_F16_BITS
    from tuna_amd.quantize import NF4_CODE
    assert np.array_equal(np.array(NF4_CODE, np.float32), cb)  # the product carries the same constants


def test_decode_known_answers():
    cb = O.nf4_codebook()
    s = np.full(16, np.array([0x211f], np.uint16).view(np.float16)[0], np.float32)
    assert ["%04x" % b for b in O.decode(cb, s, O.D1)] == KAT_D1
    assert ["%04x" % b for b in O.decode(cb, s, O.D2)] == KAT_D2


def test_decode_exhaustive_against_numpy_arithmetic():
    """16 NF4 codes x every finite fp16 scale pattern, D1 via numpy float16 multiply (one
    rounding of an exact product), D2 via numpy float32 multiply then a float16 cast."""
    cb = O.nf4_codebook()
    h = np.arange(65536, dtype=np.uint16)
    h = h[np.isfinite(h.view(np.float16))]
    scales = h.view(np.float16).astype(np.float32)
    code = np.repeat(cb, scales.size)
    s = np.tile(scales, 16)
    with np.errstate(over="ignore", invalid="ignore"):
        want1 = (code.astype(np.float16) * s.astype(np.float16))  # numpy rounds the fp16 product once
        want2 = (code * s).astype(np.float16)
    d1 = O.decode(code, s, O.D1)
    d2 = O.decode(code, s, O.D2)
    assert np.array_equal(d1, want1.view(np.uint16))
    assert np.array_equal(d2, want2.view(np.uint16))
    # the two decodes are at most one ulp apart, and equal for the codes -1, 0, +1
    key = lambda b: np.where(b & 0x8000, -(b & 0x7fff).astype(np.int32), (b & 0x7fff).astype(np.int32))
    assert np.abs(key(d1) - key(d2)).max() <= 1
    for c in (0, 7, 15):
        sl = slice(c * scales.size, (c + 1) * scales.size)
        assert np.array_equal(d1[sl], d2[sl])
    # in the benchmark's scale range the decodes differ on about a fifth of the (code, scale) pairs
    in_range = (s >= 0.005) & (s <= 0.02)
    frac = float((d1[in_range] != d2[in_range]).mean())
    assert 0.15 < frac < 0.25


def test_decode_with_float32_scales_that_are_not_halves():
    """absmax is float32 in memory: D1 rounds it to fp16 first, D2 does not."""
    rng = np.random.default_rng(3)
    s = rng.uniform(1e-4, 4.0, 200_000).astype(np.float32)
    code = rng.standard_normal(200_000).astype(np.float32)
    want1 = code.astype(np.float16) * s.astype(np.float16)
    want2 = (code * s).astype(np.float16)
    assert np.array_equal(O.decode(code, s, O.D1), want1.view(np.uint16))
    assert np.array_equal(O.decode(code, s, O.D2), want2.view(np.uint16))


def test_pack_closed_form_and_bruteforce():
    for m, k in [(8, 8), (16, 24), (64, 40)]:
        rng = np.random.default_rng(m * k)
        codes = rng.integers(0, 16, size=(m, k), dtype=np.uint8)
        q = O.pack(codes)
        assert q.shape == (m // 8, k // 8, 32)
        # closed form: weight (r, c) is in byte (r%8)*4 + (c%8)//2 of block (r//8, c//8), even column high nibble
        for r in range(m):
            for c in range(k):
                b = q[r // 8, c // 8, (r % 8) * 4 + (c % 8) // 2]
                assert ((b >> 4) if c % 2 == 0 else (b & 15)) == codes[r, c]
        # as little-endian dwords: dword r of a block is one row, column c at bit 8*(c//2) + 4*(1 - c%2)
        d = q.view("<u4")
        for r in range(m):
            for c in range(k):
                w = int(d[r // 8, c // 8, r % 8])
                assert (w >> (8 * ((c % 8) // 2) + 4 * (1 - c % 2))) & 15 == codes[r, c]
        assert np.array_equal(O.unpack(q, m, k), codes)


def test_pack_matches_the_products_independent_packer():
    """The product's packer follows the reshape/permute statement of the reference harness; the
    oracle's follows the byte addressing of the reference kernel.  They must agree."""
    import torch

    from tuna_amd.quantize import pack_codes, pack_codes_np, unpack_codes

    rng = np.random.default_rng(9)
    codes = rng.integers(0, 16, size=(128, 264), dtype=np.uint8)
    q = O.pack(codes)
    assert np.array_equal(pack_codes(torch.from_numpy(codes)).numpy(), q)
    assert np.array_equal(pack_codes_np(codes), q)
    assert np.array_equal(unpack_codes(torch.from_numpy(q), 128, 264).numpy(), codes)
    # uniform random bytes are a valid packed matrix of uniform random codes
    qq = rng.integers(0, 256, size=(4, 5, 32), dtype=np.uint8)
    assert np.array_equal(O.pack(O.unpack(qq, 32, 40)), qq)


def test_dequant_is_unpack_then_decode():
    m, k = 64, 136
    rng = np.random.default_rng(4)
    codes = rng.integers(0, 16, size=(m, k), dtype=np.uint8)
    q = O.pack(codes)
    absmax = rng.uniform(0.005, 0.02, m).astype(np.float16).astype(np.float32)
    cb = O.nf4_codebook()
    for mode, ref in ((O.D1, lambda: cb.astype(np.float16)[codes] * absmax.astype(np.float16)[:, None]),
                      (O.D2, lambda: (cb[codes] * absmax[:, None]).astype(np.float16))):
        got = O.dequant(q, absmax, cb, m, k, mode=mode)
        assert np.array_equal(got, ref().view(np.uint16))


def _inputs(m, n, k, seed):
    from tuna_amd.synth import make_inputs_np
    return make_inputs_np(m, n, k, seed)


def test_gemm_against_numpy_float64():
    m, n, k = 72, 5, 200
    q, x, cb, absmax = _inputs(m, n, k, 2)
    for mode in (O.D1, O.D2):
        w = O.dequant(q, absmax, cb, m, k, mode=mode).view(np.float16).astype(np.float64)
        want = x.astype(np.float64) @ w.T
        got64 = O.gemm_f64(q, x, cb, absmax, m, n, k, mode=mode)
        assert np.allclose(got64, want, rtol=1e-12, atol=1e-15)
        got16 = O.gemm(q, x, cb, absmax, m, n, k, mode=mode, acc64=True)
        assert np.array_equal(got16, want.astype(np.float16).view(np.uint16))
        got32 = O.gemm(q, x, cb, absmax, m, n, k, mode=mode, acc64=False).view(np.float16).astype(np.float64)
        assert np.abs(got32 - want).max() <= 2e-3 * np.abs(want).max()
    rows = np.array([3, 70, 8, 8, 41], np.int32)
    sub = O.gemm(q, x, cb, absmax, m, n, k, mode=O.D1, rows=rows)
    full = O.gemm(q, x, cb, absmax, m, n, k, mode=O.D1)
    assert np.array_equal(sub, full[:, rows])


def test_gemm_invariants():
    m, n, k = 64, 16, 128
    q, x, cb, absmax = _inputs(m, n, k, 5)
    # zero activations
    z = O.gemm(q, np.zeros_like(x), cb, absmax, m, n, k)
    assert not (z & 0x7fff).any()
    # one-hot activations read out decoded columns exactly
    cols = np.arange(n) * 7 % k
    xh = np.zeros((n, k), np.float16)
    xh[np.arange(n), cols] = 1
    img = O.dequant(q, absmax, cb, m, k, mode=O.D1)
    out = O.gemm(q, xh, cb, absmax, m, n, k, mode=O.D1)
    assert np.array_equal(out.view(np.float16).astype(np.float32), img[:, cols].T.view(np.float16).astype(np.float32))
    # linearity in x (float64 sums)
    a = O.gemm_f64(q, x, cb, absmax, m, n, k)
    b = O.gemm_f64(q, (x * np.float16(2)).astype(np.float16), cb, absmax, m, n, k)
    assert np.array_equal(b, 2 * a)
    # permuting 8-row blocks of the weights permutes the outputs
    perm = np.random.default_rng(0).permutation(m // 8)
    rows = (perm[:, None] * 8 + np.arange(8)).ravel()
    c = O.gemm_f64(q[perm], x, cb, absmax[rows], m, n, k)
    assert np.array_equal(c, a[:, rows])


def test_cpu_baseline_matches_gemm_d2():
    m, n, k = 128, 16, 512
    q, x, cb, absmax = _inputs(m, n, k, 7)
    out, td, tm, thr = O.cpu_baseline(q, x, cb, absmax, m, n, k, threads=2)
    ref = O.gemm_f64(q, x, cb, absmax, m, n, k, mode=O.D2)
    got = out.view(np.float16).astype(np.float64)
    assert np.abs(got - ref).max() <= 2e-3 * np.abs(ref).max()
    assert td >= 0 and tm >= 0 and thr == 2


def test_golden_fixtures():
    """Fixtures written by tests/golden/make_golden.py from this oracle (the reference holds no
    vectors of its own): they freeze the oracle's behaviour across rounds."""
    with open(os.path.join(GOLDEN, "golden.json")) as f:
        g = json.load(f)
    cb = O.nf4_codebook()
    # decode tables over the benchmark's scale range: 16 codes x 2049 fp16 scales in [0.005, 0.02]
    lo = int(np.float16(0.005).view(np.uint16))
    h = np.arange(lo, lo + 2049, dtype=np.uint16)
    scales = h.view(np.float16).astype(np.float32)
    for mode, key in ((O.D1, "decode_d1_sha256"), (O.D2, "decode_d2_sha256")):
        tab = O.decode(np.repeat(cb, scales.size), np.tile(scales, 16), mode)
        assert hashlib.sha256(tab.tobytes()).hexdigest() == g[key]
    blk = np.load(os.path.join(GOLDEN, "block_64x128.npz"))
    assert np.array_equal(O.dequant(blk["q"], blk["absmax"], cb, 64, 128, mode=O.D2), blk["image_d2"])
    assert np.array_equal(O.dequant(blk["q"], blk["absmax"], cb, 64, 128, mode=O.D1), blk["image_d1"])
    gm = np.load(os.path.join(GOLDEN, "gemm_256x16x128.npz"))
    out = O.gemm(gm["q"], gm["x"], cb, gm["absmax"], 256, 16, 128, mode=O.D1)
    assert np.array_equal(out, gm["out_d1"])
    out = O.gemm(gm["q"], gm["x"], cb, gm["absmax"], 256, 16, 128, mode=O.D2)
    assert np.array_equal(out, gm["out_d2"])


# ----------------------------------------------------------------------------- quantizer
def _quantize_numpy_model(w, code):
    """Independent model of test.py:7-68 with one block per row: numpy float32 division,
    |difference| in float32, argmin with the first index on ties, then the product's packer."""
    from tuna_amd.quantize import pack_codes_np

    wf = w.astype(np.float32)
    a = np.abs(wf).max(axis=1)
    with np.errstate(divide="ignore", invalid="ignore"):
        nv = (wf / a[:, None]).astype(np.float32)
    d = np.abs((nv[None] - code[:, None, None]).astype(np.float32))
    idx = d.argmin(axis=0).astype(np.uint8)           # all-zero rows: every distance is NaN, argmin gives 0
    return pack_codes_np(idx), a.astype(np.float32)


def _quantizer_inputs(rng, m, k):
    from tuna_amd.quantize import NF4_CODE

    code = np.array(NF4_CODE, np.float32)
    w = (rng.standard_normal((m, k)) * 0.03).astype(np.float16)
    if m >= 8 and k >= 16:
        w[1] = 0                                      # all-zero row
        w[2] = 0
        w[2, 5] = np.float16(-0.25)                   # a single non-zero: the negative extreme
        mids = ((code[:-1] + code[1:]) / 2).astype(np.float32)
        w[3, :15] = (mids * 0.5).astype(np.float16)   # (nearly) halfway between neighbouring codes
        w[3, 15] = np.float16(0.5)
        w[4] = np.float16(6e-8)                       # fp16 subnormals
        w[4, 0] = np.float16(-1.2e-7)
    return w, code


@pytest.mark.parametrize("m,k", [(8, 8), (8, 16), (64, 256), (72, 1096)])
def test_quantizer_oracle_matches_numpy_model(m, k):
    rng = np.random.default_rng(m * 131 + k)
    w, code = _quantizer_inputs(rng, m, k)
    q, absmax = O.quantize(w.view(np.uint16), code, m, k)
    q_ref, a_ref = _quantize_numpy_model(w, code)
    assert np.array_equal(absmax, a_ref)
    assert np.array_equal(q, q_ref)
    # an arbitrary (unsorted) codebook is handled the same way
    code2 = rng.standard_normal(16).astype(np.float32)
    q2, _ = O.quantize(w.view(np.uint16), code2, m, k)
    assert np.array_equal(q2, _quantize_numpy_model(w, code2)[0])


def test_quantizer_oracle_matches_torch_semantics_incl_all_zero_rows():
    """The reference's quantizer is torch code (test.py:41-53): fp16 / fp32 division, |a - b|, and
    torch.argmin, whose result on an all-NaN column (an all-zero row divided by its absmax 0) is
    index 0.  The same torch expressions on the CPU pin the oracle for that input too."""
    import torch

    rng = np.random.default_rng(77)
    m, k = 16, 64
    w, code = _quantizer_inputs(rng, m, k)
    wt = torch.from_numpy(w.copy())
    ct = torch.from_numpy(code.copy())
    absmax = torch.max(wt.abs(), dim=1)[0].float()
    normalized = torch.divide(wt, absmax.unsqueeze(-1)).flatten()
    assert normalized.dtype == torch.float32
    cand = torch.sub(normalized.unsqueeze(0), ct.unsqueeze(-1)).abs()
    idx = torch.argmin(cand, keepdim=True, dim=0).flatten().to(torch.uint8).numpy().reshape(m, k)
    assert (idx[1] == 0).all() and torch.isnan(normalized.reshape(m, k)[1]).all()   # the all-zero row
    from tuna_amd.quantize import pack_codes_np

    q, a = O.quantize(w.view(np.uint16), code, m, k)
    assert np.array_equal(a, absmax.numpy())
    assert np.array_equal(q, pack_codes_np(idx))
    assert (q.reshape(m // 8, k // 8, 8, 4)[0, :, 1] == 0).all()                    # bytes 0x00, not 0x77


def test_quantizer_round_trip_recovers_the_codes():
    """Weights that are exactly code * scale quantize back to the same codes and scale
    (code gaps are far larger than an fp16 rounding), and dequantize to the same weights."""
    from tuna_amd.quantize import NF4_CODE, pack_codes_np

    rng = np.random.default_rng(5)
    m, k = 32, 128
    code = np.array(NF4_CODE, np.float32)
    idx = rng.integers(0, 16, size=(m, k)).astype(np.uint8)
    idx[:, 0] = 15                                    # every row contains the extreme code: absmax = scale
    scale = rng.uniform(0.005, 0.02, size=m).astype(np.float16).astype(np.float32)
    w_bits = O.dequant(pack_codes_np(idx), scale, code, m, k, mode=O.D2)
    q, absmax = O.quantize(w_bits, code, m, k)
    assert np.array_equal(absmax, scale)
    assert np.array_equal(q, pack_codes_np(idx))
    assert np.array_equal(O.dequant(q, absmax, code, m, k, mode=O.D2), w_bits)


# ----------------------------------------------------------------------------- scale blocks finer than a row
@pytest.mark.parametrize("bs", [8, 64, 128, 256])
def test_blockwise_dequant_and_gemm_against_numpy(bs):
    """One scale per block of `bs` weights of a row, absmax [m, k/bs] (the quantizer's layout,
    test.py:15-17): dequant against a numpy gather with the scales expanded per element and the
    elementwise decode (pinned exhaustively above), the GEMM against numpy float64 matmul."""
    rng = np.random.default_rng(bs)
    m, n, k = 64, 5, 512
    idx = rng.integers(0, 16, size=(m, k)).astype(np.uint8)
    q = O.pack(idx)
    code = O.nf4_codebook()
    absmax = rng.uniform(0.004, 0.03, size=(m, k // bs)).astype(np.float32)
    per_elem = np.repeat(absmax, bs, axis=1)                       # [m, k]
    for mode in (O.D1, O.D2):
        want = O.decode(code[idx].ravel(), per_elem.ravel(), mode).reshape(m, k)
        got = O.dequant(q, absmax, code, m, k, mode=mode, block_size=bs)
        assert np.array_equal(got, want)
        x = (rng.standard_normal((n, k)) * 0.1).astype(np.float16)
        ref = x.astype(np.float64) @ want.view(np.float16).astype(np.float64).T
        got64 = O.gemm_f64(q, x.view(np.uint16), code, absmax, m, n, k, mode=mode, block_size=bs)
        assert np.allclose(got64, ref, rtol=1e-12, atol=1e-12)
    # block_size == k is the per-row function
    a_row = rng.uniform(0.004, 0.03, size=m).astype(np.float32)
    assert np.array_equal(O.dequant(q, a_row, code, m, k, block_size=k), O.dequant(q, a_row, code, m, k))


@pytest.mark.parametrize("bs", [8, 64, 128])
def test_blockwise_quantizer_oracle_matches_torch_semantics(bs):
    """The reference's quantizer with block_size < k is torch code (test.py:15-53); the product's
    torch restatement of it (tuna_amd/quantize.py) run on the CPU pins the oracle's blockwise
    quantizer, including a block of zeros (index 0) and near-midpoint inputs."""
    import torch

    from tuna_amd.quantize import quantize_blockwise_dynamic_4bit

    rng = np.random.default_rng(100 + bs)
    m, k = 16, 256
    w, code = _quantizer_inputs(rng, m, k)
    w[5, bs:2 * bs] = 0                                            # one all-zero block inside a non-zero row
    qt, (at, _c) = quantize_blockwise_dynamic_4bit(torch.from_numpy(w.copy()), block_size=bs, preprocess=True)
    q, a = O.quantize(w.view(np.uint16), code, m, k, block_size=bs)
    assert np.array_equal(a.ravel(), at.numpy())
    assert np.array_equal(q, qt.numpy())
    # round trip: dequant of the quantized weights stays within half the widest code gap of the block's scale
    img = O.dequant(q, a, code, m, k, mode=O.D2, block_size=bs).view(np.float16).astype(np.float32)
    gap = np.diff(code).max() / 2
    assert (np.abs(img - w.astype(np.float32)) <= gap * np.repeat(a, bs, axis=1) + 1e-6).all()
