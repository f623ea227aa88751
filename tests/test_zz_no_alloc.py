"""The allocation-free entry point (tuna_matmul_static) against tuna_matmul_ex, through the C ABI."""
import numpy as np
import pytest

from helpers import make_inputs_np, to_dev

pytestmark = pytest.mark.gpu


def _both(m, n, k, seed, config=None):
    import torch

    from tuna_amd import ops

    q, x, code, absmax = make_inputs_np(m, n, k, seed=seed)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    ref = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    got = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul(dx, dq, da, dc, ref, m, n, k, config=config)
    ops.matmul_static(dx, dq, da, dc, got, m, n, k, config=config)
    torch.cuda.synchronize()
    return got.cpu().numpy().view(np.uint16), ref.cpu().numpy().view(np.uint16)


def test_static_scratch_entry_point_equals_the_allocating_one_on_two_calls_in_a_row():
    """Two split-K launches in a row through tuna_matmul_static, the second with a smaller input:
    both share the device's static array (partial sums of the first call are still in it, the
    counters were returned to zero by the kernel) and both must give the bits of tuna_matmul_ex."""
    from tuna_amd import _lib, ops

    assert _lib.lib().tuna_init() == 0
    cases = [(8192, 16, 8192), (4096, 16, 14336), (1024, 5, 2048)]
    for i, (m, n, k) in enumerate(cases):
        used, _hit = ops.select_config(m, n, k)
        lds, ws = ops.config_footprint(m, n, k, used)
        print(f"static scratch case m={m} n={n} k={k} cfg={used.to_dict()} workspace={ws}", flush=True)
        if i < 2:
            assert 0 < ws <= 16 << 20          # the tuned entries of these shapes split k across workgroups
        got, ref = _both(m, n, k, seed=90 + i)
        assert not np.isnan(got.view(np.float16)).any()
        assert np.array_equal(got, ref)
    # an explicit config: balanced split, then a fixed split of a smaller problem
    from test_gpu_parity import cfg

    got, ref = _both(2048, 40, 4096, 7, cfg(split_k=0, waves_m=1, waves_k=8, prefetch=2, x_chunk=512))
    assert np.array_equal(got, ref)
    got, ref = _both(512, 16, 1024, 8, cfg(split_k=4, x_chunk=256, prefetch=2))
    assert np.array_equal(got, ref)


def test_static_scratch_entry_point_rejects_what_does_not_fit():
    import torch

    from test_gpu_parity import cfg
    from tuna_amd import _lib, ops

    m, n, k = 1024, 16 * 40, 2048
    big = cfg(split_k=0, waves_m=1, waves_k=8, prefetch=2, x_chunk=512)   # 40 chunks x 64 workgroups x 8 KB = 20 MB
    assert ops.config_footprint(m, n, k, big)[1] > 16 << 20
    q, x, code, absmax = make_inputs_np(m, n, k, seed=1)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    out = torch.zeros((n, m), dtype=torch.float16, device="cuda")
    with pytest.raises(ops.TunaError) as ei:
        ops.matmul_static(dx, dq, da, dc, out, m, n, k, config=big)
    assert ei.value.status == _lib.ERR_WORKSPACE
    ops.matmul(dx, dq, da, dc, out, m, n, k, config=big)                  # the allocating entry point takes it
    torch.cuda.synchronize()
