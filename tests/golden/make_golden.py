"""Writes the golden fixtures of tests/golden from the CPU oracle.

The reference holds no golden vectors, known-answer tests or fixtures for this path (its
only check prints two tensors), so these freeze the oracle - which tests/test_oracle.py pins
against numpy arithmetic and the bit patterns of the reference's literals - for later rounds
and for the GPU box.  Run from the repository root:  python tests/golden/make_golden.py
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import oracle as O  # noqa: E402
from tuna_amd.synth import make_inputs_np  # noqa: E402


def main():
    cb = O.nf4_codebook()
    lo = int(np.float16(0.005).view(np.uint16))
    h = np.arange(lo, lo + 2049, dtype=np.uint16)
    scales = h.view(np.float16).astype(np.float32)
    out = {"scale_bits_first": lo, "scale_count": 2049}
    for mode, key in ((O.D1, "decode_d1_sha256"), (O.D2, "decode_d2_sha256")):
        tab = O.decode(np.repeat(cb, scales.size), np.tile(scales, 16), mode)
        out[key] = hashlib.sha256(tab.tobytes()).hexdigest()
    with open(os.path.join(HERE, "golden.json"), "w") as f:
        json.dump(out, f, indent=1)

    q, _, _, absmax = make_inputs_np(64, 1, 128, seed=101)
    np.savez_compressed(os.path.join(HERE, "block_64x128.npz"), q=q, absmax=absmax,
                        image_d1=O.dequant(q, absmax, cb, 64, 128, mode=O.D1),
                        image_d2=O.dequant(q, absmax, cb, 64, 128, mode=O.D2))

    q, x, _, absmax = make_inputs_np(256, 16, 128, seed=202)
    xb = x.view(np.uint16)
    np.savez_compressed(os.path.join(HERE, "gemm_256x16x128.npz"), q=q, x=xb, absmax=absmax,
                        out_d1=O.gemm(q, xb, cb, absmax, 256, 16, 128, mode=O.D1),
                        out_d2=O.gemm(q, xb, cb, absmax, 256, 16, 128, mode=O.D2))
    print("wrote", sorted(os.listdir(HERE)))


if __name__ == "__main__":
    main()
