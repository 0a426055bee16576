"""mynn_attention_noalloc: the attention entry point that allocates nothing (its partial results live in a fixed
device array of the library) against mynn_attention on the same operands, through the C ABI."""
import numpy as np
import pytest

import oracle as orc
from conftest import max_abs_rel

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def g():
    import gpu_util

    return gpu_util


def operands(g, rng, B, Hq, Hkv, D, L, dt):
    q = g.to_dev(orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt), dt)
    k = g.to_dev(orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt), dt)
    v = g.to_dev(orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt), dt)
    return q, k, v


def test_no_alloc_attention_equals_the_allocating_entry_point_twice_in_a_row(g):
    """Two calls in a row, the second on a smaller input that finds the array as the first call left it: both bit for
    bit what mynn_attention returns (same kernels, same key ranges), and within tolerance of the oracle.  The first
    shape takes the streaming kernel with its key ranges merged by a second launch, the second the per-slice kernel;
    both park partial results in the array.  No device memory is allocated between the two measurements."""
    import torch

    dt = orc.F16
    rng = np.random.default_rng(41)
    lib = g.mynn.lib()
    shapes = [(4, 32, 4, 64, 4096, 4001), (1, 32, 4, 64, 1500, 1337)]
    prepared = []
    for B, Hq, Hkv, D, L, active in shapes:
        need = lib.mynn_attention_workspace_bytes(B, 1, L, Hq, Hkv, D, dt, 0)
        assert 0 < need <= 8 << 20, need  # the shape does use scratch memory, and it fits the fixed array
        q, k, v = operands(g, rng, B, Hq, Hkv, D, L, dt)
        want = g.mynn.attention(q, k, v, 0.125, active=active)
        prepared.append((q, k, v, active, want, torch.zeros_like(q)))
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    for q, k, v, active, want, out in prepared:
        g.mynn.attention_noalloc(q, k, v, 0.125, out, active=active)
    torch.cuda.synchronize()
    # neither torch's allocator nor the device's free memory (which a hipMalloc inside the library would lower) moved
    assert torch.cuda.memory_allocated() == before and torch.cuda.mem_get_info()[0] == free_before
    for q, k, v, active, want, out in prepared:
        assert torch.equal(out, want)
        ref = orc.attention(g.to_host(q), g.to_host(k), g.to_host(v), dt, 0.125, False, active)
        assert max_abs_rel(g.f32(g.to_host(out), dt), g.f32(ref, dt)) <= 1e-2
    # and once more in the other order, with the length read on the device
    for q, k, v, active, want, out in reversed(prepared):
        out.zero_()
        d_active = torch.tensor([active], dtype=torch.int32, device="cuda")
        g.mynn.attention_noalloc(q, k, v, 0.125, out, active=k.shape[2], d_active=d_active)
        assert torch.equal(out, g.mynn.attention(q, k, v, 0.125, active=k.shape[2], d_active=d_active))


def test_no_alloc_attention_refuses_what_does_not_fit_the_fixed_array(g):
    """A shape whose partial results need more than the 8 MiB array is refused with a clear error (the operands are
    real and full-sized: a call that got through would simply run)."""
    import torch

    dt = orc.F32
    B, Hq, Hkv, D, L = 16, 64, 8, 128, 4096
    lib = g.mynn.lib()
    assert lib.mynn_attention_workspace_bytes(B, 1, L, Hq, Hkv, D, dt, 0) > 8 << 20
    q = torch.zeros((B, Hq, 1, D), device="cuda")
    k = torch.zeros((B, Hkv, L, D), device="cuda")
    v = torch.zeros((B, Hkv, L, D), device="cuda")
    out = torch.empty_like(q)
    with pytest.raises(g.mynn.MynnError, match="fixed array"):
        g.mynn.attention_noalloc(q, k, v, D ** -0.5, out)
    # a shape that needs no scratch at all is served whatever its size
    g.mynn.attention_noalloc(q[:, :, :, :], k[:, :, :64].contiguous(), v[:, :, :64].contiguous(), D ** -0.5, out)
    torch.cuda.synchronize()
    assert not out.any()
