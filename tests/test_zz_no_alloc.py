"""fastmax_forward_static (the entry point that allocates nothing: its workspace is a static device
array inside the library) against fastmax_forward, through the C ABI: same kernels on the same inputs,
so the results must be the same bits.  Two calls in a row, the second on a smaller problem (the buffer
still holds the first call's contents), then a problem with moment states, then the size limit."""
import ctypes as C
import math

import pytest
import torch

from reproducing_fastmax_results_amd import _capi

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def lib():
    return _capi.get_lib()


def _pair(lib, bh, n, d, dtype, seed, first=False, **kw):
    gen = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(bh, n, d, generator=gen).to(dtype).to(DEV) for _ in range(3))
    o1, g1 = lib.forward(q, k, v, **kw)
    o2 = torch.full_like(o1, float("nan"))
    g2 = torch.full_like(g1, float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info()[0]               # the driver's own count of free device memory
    lib.forward_static(q, k, v, o2, g2, **kw)
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before     # torch's allocator saw nothing
    if not first:
        # nor did the device: a hipMalloc inside the library would lower the driver's free count (the very first
        # call on a device looks the static array's address up, which is allowed to load the code object)
        assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(o1, o2) and torch.equal(g1, g2), f"bh={bh} n={n} d={d} {dtype}"


def test_static_scratch_forward_matches_forward(lib):
    print("case no-alloc forward", flush=True)
    kw = dict(mask=True, inv_tau=1.0 / (8.0 * math.sqrt(64)), p=2)
    _pair(lib, 8, 2048, 64, torch.bfloat16, 1, first=True, **kw)          # first call on this device: looks the buffer up
    _pair(lib, 3, 333, 64, torch.bfloat16, 2, **kw)           # smaller, straight after, on the used buffer
    _pair(lib, 2, 1100, 64, torch.float32, 3, chunk=256, **kw)                 # through moment states
    _pair(lib, 2, 300, 32, torch.bfloat16, 4, mask=False, inv_tau=0.1, p=1)
    _pair(lib, 3, 130, 64, torch.bfloat16, 5, mask=True, inv_tau=0.1, p=1)


def test_static_scratch_limit(lib):
    # a problem whose workspace exceeds the static buffer is refused before anything is launched
    q = torch.zeros(16, 65536, 64, dtype=torch.bfloat16, device=DEV)
    d = lib.make_desc(q, q, q, mask=True, inv_tau=0.1, a0=1.0, a1=1.0, a2=0.5, p=2)
    need, _ = lib.workspace_bytes(d)
    assert need > _capi.STATIC_SCRATCH_BYTES
    o, g = torch.empty_like(q), torch.empty(16, 65536, device=DEV)
    with pytest.raises(_capi.FastmaxError, match="static buffer"):
        lib.forward_static(q, q, q, o, g, mask=True, inv_tau=0.1, p=2)
