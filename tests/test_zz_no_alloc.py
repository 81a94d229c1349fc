"""The entry point that allocates nothing (``p2hip_orbit_mean_static``): called through the C ABI,
its output must equal, bit for bit, what ``p2hip_orbit_mean`` gives with a caller-allocated
workspace — on two calls in a row, the second with a smaller input, so that whatever the first
call left in the library's static array cannot leak into the second."""
import ctypes

import numpy as np
import pytest
import torch

H = 1326
SCRATCH_FLOATS = 4 * 1024 * 1024


def test_static_variant_refuses_what_does_not_fit_without_touching_a_gpu():
    """Argument and size checks come before any HIP call, so they can run anywhere."""
    from poker2_amd import _lib
    lib = _lib.load()
    fake = 4096                                   # non-null, 8-byte aligned, never dereferenced by the checks
    assert lib.p2hip_orbit_mean_static(None, 4, 8, None, 0, None, 2, None) == 1
    assert lib.p2hip_orbit_mean_static(fake, -1, 8, fake, 0, fake, 2, None) == 1
    assert lib.p2hip_orbit_mean_static(fake, 4, 8, fake, 0, fake, 0, None) == 1
    # n = 0 is the set-up call: it resolves the array's address on the current device and launches nothing;
    # without a device it reports the HIP error instead of resolving anything
    rc = lib.p2hip_orbit_mean_static(None, 0, 0, None, 0, None, 1, None)
    assert (rc == 0) == torch.cuda.is_available()
    n, shares = 800, 2                            # 2 * 800 * 2652 = 4 243 200 floats > 4 194 304
    assert shares * n * 2 * H > SCRATCH_FLOATS
    assert lib.p2hip_orbit_mean_static(fake, n, 8, fake, 0, fake, shares, None) == 2  # hipErrorOutOfMemory
    text = open(_lib.os.path.join(_lib.os.path.dirname(_lib.LIB_PATH), "..", "include", "p2hip.h")).read()
    assert f"#define P2HIP_ORBIT_SCRATCH_FLOATS (4 * 1024 * 1024)" in text


@pytest.mark.gpu
def test_static_variant_equals_the_workspace_variant_on_two_calls_in_a_row():
    from poker2_amd import _lib
    lib = _lib.load()
    assert torch.cuda.is_available()
    dev = torch.device("cuda")
    stream = _lib.stream_ptr()
    gen = torch.Generator(device="cpu").manual_seed(17)

    def both(n, k, shares, accumulate):
        hv = torch.randn(n, k, 2, H, generator=gen).to(dev)
        w = torch.rand(k, generator=gen).to(dev)
        base = torch.randn(n, 2, H, generator=gen).to(dev)
        ref, got = base.clone(), base.clone()
        ws = torch.empty(shares, n, 2, H, device=dev)
        torch.cuda.synchronize()
        print(f"orbit_mean n={n} flops={k} shares={shares} accumulate={accumulate}", flush=True)
        _lib.check(lib.p2hip_orbit_mean(hv.data_ptr(), n, k, w.data_ptr(), accumulate, ref.data_ptr(),
                                        ws.data_ptr(), shares, stream), "p2hip_orbit_mean")
        before = torch.cuda.memory_allocated()
        _lib.check(lib.p2hip_orbit_mean_static(hv.data_ptr(), n, k, w.data_ptr(), accumulate, got.data_ptr(),
                                               shares, stream), "p2hip_orbit_mean_static")
        assert torch.cuda.memory_allocated() == before
        torch.cuda.synchronize()
        assert torch.equal(ref, got), f"n={n} k={k} shares={shares}: max diff {(ref - got).abs().max().item():.3e}"
        assert torch.isfinite(got).all()
        return got

    from poker2_amd import chance_node_helper as K
    K.orbit_scratch_init()                                  # the per-device set-up call (n = 0), twice: idempotent
    K.orbit_scratch_init()
    first = both(n=24, k=40, shares=16, accumulate=0)       # 16 * 24 * 2652 floats = 1.0 M of the 4 M array
    second = both(n=5, k=7, shares=3, accumulate=1)         # smaller, other share layout, on top of `out`
    assert first.shape == (24, 2, H) and second.shape == (5, 2, H)
    both(n=3, k=2, shares=2, accumulate=0)                  # shares holding one flop each
    both(n=4, k=9, shares=1, accumulate=0)                  # one share: the array is not used at all
    # the largest request that fits, then one beyond it
    n_max = SCRATCH_FLOATS // (2 * 2 * H)
    both(n=n_max, k=2, shares=2, accumulate=0)
    fake = first.data_ptr()
    assert lib.p2hip_orbit_mean_static(fake, n_max + 1, 2, fake, 0, fake, 2, stream) == 2
    # the Python wrapper's switch reaches the same entry point
    hv = torch.randn(6, 300, 2, H, generator=gen).to(dev)
    w = torch.rand(300, generator=gen).to(dev)
    a = K.orbit_mean(hv, w)
    b = K.orbit_mean(hv, w, out=torch.zeros(6, 2, H, device=dev), static_scratch=True)
    assert torch.equal(a, b)
    with pytest.raises(ValueError):
        K.orbit_mean(hv, w, static_scratch=True)            # no output tensor given
