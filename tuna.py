"""Drop-in module named like the reference's extension (setup.py:9-15, extension.cpp:51-55):
``import tuna; tuna.matmul(x, q, a, c, out, M, N, K)`` as called in test.py:85."""
from tuna_amd.ops import dequant, matmul  # noqa: F401
