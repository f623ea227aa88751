"""Deterministic synthetic inputs of the benchmark configurations.

Distributions: 4-bit codes uniform in 0..15, scales ~ U(0.005, 0.02) rounded to fp16 and
stored as float32 (one per weight row), activations ~ N(0, 1) * 0.1 in fp16, codebook =
the NF4 constants.  Uniform codes packed by the layout bijection are uniform bytes, so
the packed tensor is drawn directly.
"""
import numpy as np

from .quantize import NF4_CODE

# (name, m = output features, k) of the 16-token layer shapes, in the order of the benchmark configurations
SHAPES = {
    "mistral_attn_out": (4096, 4096),
    "mistral_qkv": (6144, 4096),
    "mistral_gate_up": (28672, 4096),
    "mistral_down": (4096, 14336),
    "llama70b_qkv": (10240, 8192),
    "llama70b_attn_out": (8192, 8192),
    "llama70b_gate_up": (57344, 8192),
    "llama70b_down": (8192, 28672),
    "mixtral_gate_up_8e": (229376, 4096),
    "mixtral_down_8e": (32768, 14336),
}


def make_inputs_np(m: int, n: int, k: int, seed: int = 0):
    """(q uint8 [m/8,k/8,32], x fp16 [n,k], code fp32 [16], absmax fp32 [m]) as numpy arrays."""
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 256, size=(m // 8, k // 8, 32), dtype=np.uint8)
    absmax = rng.uniform(0.005, 0.02, size=m).astype(np.float16).astype(np.float32)
    x = (rng.standard_normal((n, k)) * 0.1).astype(np.float16)
    code = np.array(NF4_CODE, dtype=np.float32)
    return q, x, code, absmax


def make_weights_torch(m: int, k: int, seed: int, device):
    """(q, absmax) drawn on `device` with a seeded torch generator (large sweeps)."""
    import torch

    g = torch.Generator(device=device)
    g.manual_seed(int(seed))
    q = torch.randint(0, 256, (m // 8, k // 8, 32), dtype=torch.uint8, device=device, generator=g)
    absmax = torch.empty(m, dtype=torch.float32, device=device).uniform_(0.005, 0.02, generator=g)
    absmax = absmax.half().float()
    return q, absmax


def make_x_torch(n: int, k: int, seed: int, device):
    import torch

    g = torch.Generator(device=device)
    g.manual_seed(int(seed) + 7919)
    return (torch.randn(n, k, dtype=torch.float32, device=device, generator=g) * 0.1).half()
