"""egg_newton_schulz_static (Newton-Schulz with the workspace in a static device array: no context, no allocation)
against egg_newton_schulz (the same kernels with a context's buffers) through the C ABI.  Both run the same kernels in
the same order, so the results must be identical bit for bit; the fp64 oracle bounds both.  Two calls in a row share
the static workspace, the second on a smaller matrix, then a larger one again."""
import ctypes as C

import numpy as np
import pytest


@pytest.mark.gpu
def test_static_newton_schulz_matches_the_context_entry_point(pkg, orc, dev):
    import torch
    ctx = pkg.Context(pkg.default_config(use_muon=1, hidden=512, head_dim=64, n_layers=1, seq_len=32, population=8))
    rng = np.random.default_rng(77)
    torch.cuda.synchronize()
    for rows, cols, iters in ((512, 2048, 5), (128, 256, 5), (2048, 512, 4), (64, 96, 5), (512, 512, 5)):
        X = rng.integers(-300, 301, (rows, cols)).astype(np.float32)
        a = torch.from_numpy(X).to(dev)
        b = torch.from_numpy(X).to(dev)
        ctx.newton_schulz(a.data_ptr(), rows, cols, iters)
        ctx.sync()
        pkg.newton_schulz_static(b.data_ptr(), rows, cols, iters, stream=None)
        torch.cuda.synchronize()
        ga, gb = a.cpu().numpy(), b.cpu().numpy()
        assert np.array_equal(ga.view(np.int32), gb.view(np.int32)), (rows, cols, iters)
        ref = X.astype(np.float64)
        orc.lib().orc_newton_schulz_f64(ref.ctypes.data_as(C.c_void_p), rows, cols, iters)
        err = np.linalg.norm(gb - ref) / np.linalg.norm(ref)
        assert err < 1e-5, (rows, cols, err)
        del a, b
    # on a caller's stream as well
    s = torch.cuda.Stream()
    X = rng.integers(-300, 301, (256, 1024)).astype(np.float32)
    a, b = torch.from_numpy(X).to(dev), torch.from_numpy(X).to(dev)
    torch.cuda.synchronize()
    ctx.newton_schulz(a.data_ptr(), 256, 1024, 5)
    ctx.sync()
    pkg.newton_schulz_static(b.data_ptr(), 256, 1024, 5, stream=s.cuda_stream)
    s.synchronize()
    assert torch.equal(a, b)
    del a, b
    ctx.close()


@pytest.mark.gpu
def test_static_newton_schulz_leaves_the_free_device_memory_unchanged(pkg, dev):
    """hipMemGetInfo around a series of calls (every input allocated beforehand, one warm-up call so that the code
    object and its static array are resident): the free byte count must not move, whatever allocator a hipMalloc
    inside the library would have gone through.  A fresh 256 MiB tensor afterwards shows that the counter does see
    device allocations."""
    import torch
    shapes = ((512, 2048, 5), (128, 256, 5), (2048, 512, 4), (64, 96, 5), (512, 512, 5))
    gen = torch.Generator(device="cpu").manual_seed(5)
    xs = [torch.randint(-300, 301, (r, c), generator=gen).float().to(dev) for r, c, _ in shapes]
    s = torch.cuda.Stream()
    pkg.newton_schulz_static(xs[0].data_ptr(), *shapes[0], stream=None)
    torch.cuda.synchronize()
    torch.cuda.empty_cache()          # so that the tensor at the end needs a fresh device allocation
    free_before = torch.cuda.mem_get_info(dev)[0]
    for rep in range(3):
        for x, (r, c, it) in zip(xs, shapes):
            pkg.newton_schulz_static(x.data_ptr(), r, c, it, stream=s.cuda_stream if rep == 1 else None)
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info(dev)[0]
    assert free_after == free_before, (free_before, free_after)
    big = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
    assert torch.cuda.mem_get_info(dev)[0] <= free_before - (128 << 20)      # the driver's figure moves in its own granules
    del big


@pytest.mark.gpu
def test_static_newton_schulz_refuses_what_does_not_fit(pkg, dev):
    import torch
    x = torch.zeros(32 * 32, dtype=torch.float32, device=dev)
    for rows, cols in ((1024, 2048), (2048, 1024), (544, 544), (512, 2080)):
        with pytest.raises(pkg.EggError, match="static workspace"):
            pkg.newton_schulz_static(x.data_ptr(), rows, cols, 5)
    for rows, cols, iters in ((48, 64, 5), (0, 64, 5), (64, 64, -1)):
        with pytest.raises(pkg.EggError, match="multiples of 32"):
            pkg.newton_schulz_static(x.data_ptr(), rows, cols, iters)
    with pytest.raises(pkg.EggError):
        pkg.newton_schulz_static(0, 64, 64, 5)
