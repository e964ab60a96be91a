"""The entry point that allocates nothing (``sparse_hip_permute_build_static``) gives, bit
for bit, what ``sparse_hip_permute_build`` gives with a caller workspace -- on two calls in
a row, the second with a smaller input, since every call on a GPU shares one built-in array
that keeps the previous call's contents."""
import pytest
import torch

from sparse_amd import _lib

pytestmark = pytest.mark.gpu


def _outputs(T, K, E, device):
    i32 = dict(device=device, dtype=torch.int32)
    # poisoned so that an entry the kernel leaves unwritten shows up in the comparison
    return [torch.full((T * K,), -7, **i32), torch.full((T * K,), -7, **i32), torch.full((E + 1,), -7, **i32),
            torch.full((E,), -7, **i32), torch.full((1,), -7, **i32)]


def _topi(T, K, E, seed, device):
    g = torch.Generator().manual_seed(seed)
    scores = torch.rand(T, E, generator=g)
    scores[:, : E // 3] += 0.5  # uneven segments, some experts unused at small T
    return torch.topk(scores, K, dim=1).indices.to(torch.int64).contiguous().to(device)


def _both(lib, topi, E, first_call=False):
    T, K = topi.shape
    device = topi.device
    st = torch.cuda.current_stream().cuda_stream
    want = _outputs(T, K, E, device)
    nbytes = lib.sparse_hip_permute_ws_bytes(T, K, E)
    ws = torch.empty((max(1, nbytes // 4),), device=device, dtype=torch.int32)
    _lib.check(lib.sparse_hip_permute_build(topi.data_ptr(), T, K, E, *[t.data_ptr() for t in want], ws.data_ptr(),
                                            st), "sparse_hip_permute_build")
    got = _outputs(T, K, E, device)
    # two views of "allocates nothing": torch's own allocator, and the device's free memory as the
    # runtime reports it (hipMemGetInfo), which a hipMalloc inside the library would lower.  The very first
    # call on a device may resolve the built-in array's address, so the free-memory check starts with the
    # second.
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    _lib.check(lib.sparse_hip_permute_build_static(topi.data_ptr(), T, K, E, *[t.data_ptr() for t in got], st),
               "sparse_hip_permute_build_static")
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    if not first_call:
        assert torch.cuda.mem_get_info()[0] == free_before, "device free memory changed across the call"
    return want, got


@pytest.mark.parametrize("E,K", [(64, 6), (60, 4)])
def test_static_scratch_permute_equals_workspace_permute(device, E, K):
    lib = _lib.load()
    # large, then smaller ones (several blocks each), then one block
    for n, (T, seed) in enumerate(((20000, 1), (4096, 4), (700, 2), (9, 3))):
        topi = _topi(T, K, E, seed, device)
        want, got = _both(lib, topi, E, first_call=(n == 0))
        n_act = int(want[4].item())
        assert int(got[4].item()) == n_act
        for name, w, g in zip(("perm", "inv_perm", "seg_offsets", "active_eids"), want, got):
            if name == "active_eids":
                w, g = w[:n_act], g[:n_act]
            assert torch.equal(w, g), f"{name} differs at T={T}"


def test_static_scratch_permute_rejects_oversize(device):
    lib = _lib.load()
    T = _lib.PERMUTE_STATIC_MAX_TOKENS + 1
    rc = lib.sparse_hip_permute_build_static(1, T, 1, 8, 1, 1, 1, 1, 1, None)
    assert rc == -1
    assert b"exceeds the built-in scratch" in lib.sparse_hip_last_error()
    with pytest.raises(ValueError):
        _lib.check(rc, "sparse_hip_permute_build_static")
