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


def test_static_scratch_entry_point_allocates_no_device_memory_on_a_stream_without_a_workspace():
    """What the entry point exists for: split-K launches through tuna_matmul_static on a stream the library has never
    uses (it owns no workspace there: they are all released first) leave the device's free memory exactly where it was - the allocating entry
    point would have taken 64 MB for that stream - and still give the bits of tuna_matmul_ex.  Runs before any other
    call of this file touches the streams used here."""
    import torch

    from tuna_amd import _lib, ops

    assert _lib.lib().tuna_init() == 0
    m, n, k = 8192, 16, 8192
    used, _hit = ops.select_config(m, n, k)
    assert ops.config_footprint(m, n, k, used)[1] > 0          # the tuned entry splits k across workgroups
    q, x, code, absmax = make_inputs_np(m, n, k, seed=123)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    got = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    ref = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    small = torch.full((5, 1024), float("nan"), dtype=torch.float16, device="cuda")
    q2, x2, code2, absmax2 = make_inputs_np(1024, 5, 2048, seed=124)
    dq2, dx2, dc2, da2 = to_dev(q2, x2, code2, absmax2)
    torch.cuda.synchronize()
    # (torch hands out streams from a pool that earlier tests used too: drop every workspace the library holds)
    assert _lib.lib().tuna_release_workspaces() == 0
    warm, fresh = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(warm):                              # (loads both kernels, finds the array's address)
        ops.matmul_static(dx, dq, da, dc, got, m, n, k)
        ops.matmul_static(dx2, dq2, da2, dc2, small, 1024, 5, 2048)
    with torch.cuda.stream(fresh):                             # (the runtime sets a stream's queue up at its first launch)
        got.fill_(float("nan"))
        small.fill_(float("nan"))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    with torch.cuda.stream(fresh):
        ops.matmul_static(dx, dq, da, dc, got, m, n, k)
        ops.matmul_static(dx2, dq2, da2, dc2, small, 1024, 5, 2048)     # a smaller launch over the first one's partial sums
    fresh.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "tuna_matmul_static allocated device memory"
    with torch.cuda.stream(fresh):
        ops.matmul(dx, dq, da, dc, ref, m, n, k)                   # now the stream gets its workspace
    fresh.synchronize()
    assert torch.cuda.mem_get_info()[0] < free_before
    assert np.array_equal(got.cpu().numpy().view(np.uint16), ref.cpu().numpy().view(np.uint16))
    ref2 = torch.full((5, 1024), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul(dx2, dq2, da2, dc2, ref2, 1024, 5, 2048)
    torch.cuda.synchronize()
    assert np.array_equal(small.cpu().numpy().view(np.uint16), ref2.cpu().numpy().view(np.uint16))


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


def test_static_scratch_entry_point_reduces_a_split_of_the_library_that_would_not_fit():
    """Where the library picks the config itself and its pick splits k of a many-token tile into more partial tiles
    than the static scratch holds, the entry point runs the same tile with the largest split that fits: the bits of
    tuna_matmul_ex with that config."""
    import torch

    from tuna_amd import ops

    m, n, k = 2560, 600, 6912
    pick, hit = ops.select_config(m, n, k)
    assert not hit and pick.lds_tile_rows > 0 and pick.split_k > 2
    assert ops.config_footprint(m, n, k, pick)[1] > 16 << 20          # 60 tiles of 128 x 256 x 4 splits: 30 MB
    fits = ops.GemmConfig.from_dict(pick.to_dict())
    while ops.config_footprint(m, n, k, fits)[1] > 16 << 20:
        fits.split_k -= 1
    assert 1 < fits.split_k < pick.split_k
    q, x, code, absmax = make_inputs_np(m, n, k, seed=5)
    dq, dx, dc, da = to_dev(q, x, code, absmax)
    got = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    ref = torch.full((n, m), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_static(dx, dq, da, dc, got, m, n, k)
    ops.matmul(dx, dq, da, dc, ref, m, n, k, config=fits)
    torch.cuda.synchronize()
    assert not torch.isnan(got).any()
    assert np.array_equal(got.cpu().numpy().view(np.uint16), ref.cpu().numpy().view(np.uint16))
    with pytest.raises(ops.TunaError):                                  # a config the caller names is taken as it is
        ops.matmul_static(dx, dq, da, dc, got, m, n, k, config=pick)


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
