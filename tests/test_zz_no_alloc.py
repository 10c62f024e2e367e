"""The routing entry point that allocates nothing (static device scratch) against moe_a2a_route
with a caller-owned workspace: same outputs bit for bit, two calls in a row, the second smaller."""
import pytest
import torch

from kernel_amd import _lib

pytestmark = pytest.mark.gpu

E_CAPACITY = -7


def route_both(lib, dev, T, K, E, W, seed, max_recv=0):
    g = torch.Generator().manual_seed(seed)
    idx = torch.randint(0, E, (T, K), generator=g, dtype=torch.int32).to(dev)
    per_rank = T // W
    rs = torch.tensor([min(r * per_rank, T) for r in range(W)] + [T], dtype=torch.int32, device=dev)
    R = T * K
    rows = E * max_recv if max_recv else R

    def outputs():
        i32 = dict(dtype=torch.int32, device=dev)
        return dict(counts=torch.full((E,), -1, **i32), offsets=torch.full((E + 1,), -1, **i32),
                    soe=torch.full((R,), -1, **i32), sos=torch.full((rows,), -1, **i32),
                    meta=torch.full((rows, 5), -1, **i32), status=torch.zeros(1, **i32))

    st = torch.cuda.current_stream().cuda_stream
    a, b = outputs(), outputs()
    ws = torch.empty(max(lib.moe_a2a_workspace_bytes(T, K, E), 256), dtype=torch.uint8, device=dev)
    rc = lib.moe_a2a_route(idx.data_ptr(), rs.data_ptr(), 0, T, K, E, W, max_recv, a["counts"].data_ptr(),
                           a["offsets"].data_ptr(), a["soe"].data_ptr(), a["sos"].data_ptr(), a["meta"].data_ptr(),
                           a["status"].data_ptr(), ws.data_ptr(), ws.numel(), st)
    assert rc == 0, rc
    free_before = torch.cuda.mem_get_info()[0]
    rc = lib.moe_a2a_route_noalloc(idx.data_ptr(), rs.data_ptr(), 0, T, K, E, W, max_recv, b["counts"].data_ptr(),
                                   b["offsets"].data_ptr(), b["soe"].data_ptr(), b["sos"].data_ptr(),
                                   b["meta"].data_ptr(), b["status"].data_ptr(), st)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before  # nothing was allocated behind the call
    for key in a:
        assert torch.equal(a[key], b[key]), f"{key} differs (T={T}, K={K}, E={E})"
    assert int(a["counts"].sum()) == R and int(a["offsets"][-1]) == R


def test_route_noalloc_equals_route_two_calls_in_a_row(gpu_device):
    lib = _lib.load()
    assert lib.moe_a2a_route_noalloc_max_ints() == 1 << 20
    # both calls need the count matrix (more than 32 768 entries); the second is smaller, so cells of
    # the shared static array that the first call wrote lie beyond what the second one uses
    route_both(lib, gpu_device, T=16384, K=4, E=128, W=8, seed=1)   # 64 tiles x 128 experts
    route_both(lib, gpu_device, T=9000, K=4, E=64, W=8, seed=2)     # 36 tiles x 64 experts
    route_both(lib, gpu_device, T=33000, K=8, E=256, W=8, seed=3)   # 258 tiles: the three-launch form
    route_both(lib, gpu_device, T=5000, K=8, E=32, W=4, seed=4, max_recv=5000)  # padded layout, smaller again
    route_both(lib, gpu_device, T=300, K=8, E=256, W=8, seed=5)     # a small table needs no scratch at all
    route_both(lib, gpu_device, T=16384, K=4, E=128, W=8, seed=1)   # and the first shape once more


def test_route_noalloc_rejects_what_does_not_fit(gpu_device):
    lib = _lib.load()
    A = 0x1000
    # 132 000 x 8 entries = 1032 tiles x 1024 experts > 2^20 cells: refused on the host, nothing launched
    assert lib.moe_a2a_route_noalloc(A, None, 0, 132000, 8, 1024, 8, 0, A, A, A, A, A, None, None) == E_CAPACITY
    assert b"static scratch" in lib.moe_a2a_strerror(E_CAPACITY)
    assert lib.moe_a2a_route_noalloc(A, None, 0, 4, 0, 8, 2, 0, A, A, A, A, A, None, None) == -2  # K = 0
    assert lib.moe_a2a_route_noalloc(A, None, 0, 4, 2, 8, 2, 0, None, A, A, A, A, None, None) == -1
