"""Host-side quantizer and packer: the layout contract of the packed weights.

Counterpart of the reference harness's ``quantize_blockwise_dynamic_4bit``
(test.py:7-68): per-row absmax scaling, nearest-codebook-entry quantization with the 16
NF4 constants (test.py:19-37), and the blocked nibble packing (test.py:55-65) that the
kernels read.  Works on CPU or HIP tensors; nothing here is on the GEMM hot path.
"""
import numpy as np
import torch

# The NF4 codebook of the reference harness (test.py:19-37), float32.
NF4_CODE = (
    -1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453,
    -0.28444138169288635, -0.18477343022823334, -0.09105003625154495, 0.0,
    0.07958029955625534, 0.16093020141124725, 0.24611230194568634, 0.33791524171829224,
    0.44070982933044434, 0.5626170039176941, 0.7229568362236023, 1.0,
)


def nf4_codebook(device="cpu") -> torch.Tensor:
    return torch.tensor(NF4_CODE, dtype=torch.float32, device=device)


def pack_codes(codes: torch.Tensor) -> torch.Tensor:
    """uint8 codes [..., m, k] (values 0..15) -> packed uint8 [..., m/8, k/8, 32].

    Byte b of block (mb, kb) holds row mb*8 + b//4, column kb*8 + 2*(b%4) in the high
    nibble and the next column in the low nibble (test.py:58-65; the inverse is what
    kernel.cu:3221-3228 decodes)."""
    *lead, m, k = codes.shape
    if m % 8 or k % 8:
        raise ValueError("m and k must be multiples of 8")
    c = codes.to(torch.uint8).reshape(*lead, m // 8, 8, k // 8, 4, 2)
    nd = len(lead)
    c = c.permute(*range(nd), nd, nd + 2, nd + 1, nd + 3, nd + 4)  # [..., m/8, k/8, 8, 4, 2]
    packed = (c[..., 0] << 4) | (c[..., 1] & 15)
    return packed.reshape(*lead, m // 8, k // 8, 32).contiguous()


def unpack_codes(q: torch.Tensor, m: int, k: int) -> torch.Tensor:
    """Inverse of pack_codes: packed uint8 [..., m/8, k/8, 32] -> codes [..., m, k]."""
    lead = q.shape[:-3]
    nd = len(lead)
    b = q.reshape(*lead, m // 8, k // 8, 8, 4)
    c = torch.stack(((b >> 4) & 15, b & 15), dim=-1)  # [..., m/8, k/8, 8, 4, 2]
    c = c.permute(*range(nd), nd, nd + 2, nd + 1, nd + 3, nd + 4)
    return c.reshape(*lead, m, k).contiguous()


def quantize_blockwise_dynamic_4bit(inp: torch.Tensor, block_size: int = 4096, preprocess: bool = False):
    """Same contract as test.py:7-68: returns (codes or packed bytes, (absmax fp32, code fp32)).

    `block_size` elements share one absmax (the kernels need block_size == k: one scale
    per weight row).  Ties in the nearest-entry search go to the lower index, like the
    argmin of test.py:53."""
    if inp.numel() % 128 or block_size % 4:
        raise ValueError("numel must be a multiple of 128 and block_size of 4")
    code = nf4_codebook(inp.device)
    blocks = inp.reshape(-1, block_size)
    absmax = blocks.abs().amax(dim=1).float()
    normalized = (blocks / absmax.unsqueeze(-1)).flatten()
    idx = torch.empty(normalized.numel(), dtype=torch.uint8, device=inp.device)
    step = 1 << 19
    for lo in range(0, normalized.numel(), step):
        seg = normalized[lo:lo + step]
        idx[lo:lo + step] = (seg.unsqueeze(0) - code.unsqueeze(1)).abs().argmin(dim=0).to(torch.uint8)
    if preprocess:
        m, k = inp.shape[-2:]
        idx = pack_codes(idx.reshape(*inp.shape[:-2], m, k))
    return idx, (absmax, code)


def pack_codes_np(codes: np.ndarray) -> np.ndarray:
    """numpy twin of pack_codes for host-only tooling."""
    m, k = codes.shape
    c = codes.astype(np.uint8).reshape(m // 8, 8, k // 8, 4, 2).transpose(0, 2, 1, 3, 4)
    return ((c[..., 0] << 4) | (c[..., 1] & 15)).reshape(m // 8, k // 8, 32).copy()
