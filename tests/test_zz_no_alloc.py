"""The entry point that allocates nothing (tamd_routing_metadata_static: workspace in a static device array) against
tamd_routing_metadata on the same inputs, through the C ABI: bit-exact tables, two calls in a row with the second
on a smaller input, sizes beyond the fixed capacity rejected."""
import pytest
import torch

from triton_amd import _lib
from triton_amd.tensor_details.ragged_tensor import alloc_tables

pytestmark = pytest.mark.gpu


def _poison_static_workspace(device):
    """Fills the static array with garbage through an ordinary call on other data, so that a following call cannot rely
    on anything in it being zero (or being its own earlier output)."""
    E, k, T = 128, 4, 40000
    junk = torch.randint(0, E, (T, k), dtype=torch.int16, device=device)
    _run(junk, E, k, static=True)


def _run(indx, E, k, static):
    dev = indx.device
    n = indx.numel()
    L = _lib.lib()
    col_sum = torch.full((E, ), -7, dtype=torch.int32, device=dev)
    combined = torch.full((3 * n, ), -7, dtype=torch.int32, device=dev)
    offs, sched, width = alloc_tables(E, n, dev)
    offs.fill_(-7)
    sched.fill_(-7)
    args = [_lib.ptr(indx), int(indx.dtype == torch.int16), n, E, k, _lib.ptr(col_sum), _lib.ptr(combined),
            _lib.ptr(combined[n:]), _lib.ptr(combined[2 * n:]), _lib.ptr(offs), offs.stride(0), _lib.ptr(sched),
            sched.stride(0), width]
    if static:
        rc = L.tamd_routing_metadata_static(*args, _lib.stream_ptr(dev))
    else:
        ws = torch.empty(L.tamd_bitmatrix_metadata_workspace(n, E), dtype=torch.int32, device=dev)
        rc = L.tamd_routing_metadata(*args, _lib.ptr(ws), _lib.stream_ptr(dev))
    assert rc == 0, rc
    torch.cuda.synchronize()
    return col_sum, combined, offs[:, :E + 1].clone(), sched[:, :width].clone()


def test_static_workspace_entry_point_matches_the_allocating_one(device):
    torch.manual_seed(11)
    assert _lib.lib().tamd_routing_metadata_static_init() == 0
    # (rows, experts, k): the first needs the three-launch path with ~1.4 MB of workspace, the second and third the
    # two-launch path, the fourth takes the single-workgroup path (no workspace at all)
    for T, E, k, dt in ((40000, 128, 4, torch.int16), (4096, 128, 4, torch.int16), (1500, 96, 4, torch.int32),
                        (64, 128, 4, torch.int16)):
        indx = torch.stack([torch.randperm(E)[:k] for _ in range(T)]).to(dt)
        indx[T - T // 8:] = -1  # dropped rows at the end
        indx = indx.to(device)
        want = _run(indx, E, k, static=False)
        _poison_static_workspace(device)
        got = _run(indx, E, k, static=True)
        for name, a, b in zip(("col_sum", "index arrays", "offsets", "schedule"), got, want):
            assert torch.equal(a, b), f"{name} differ for T={T}, E={E}"


def test_static_entry_point_allocates_no_device_memory(device):
    """Device memory in use (the driver's count and torch's) is the same before and after calls of the entry point
    once the per-device set-up has run."""
    L = _lib.lib()
    assert L.tamd_routing_metadata_static_init() == 0
    torch.manual_seed(5)
    E, k = 128, 4
    cases = []
    for T in (4096, 40000, 64):
        indx = torch.stack([torch.randperm(E)[:k] for _ in range(T)]).to(torch.int16).to(device)
        n = indx.numel()
        col_sum = torch.empty((E, ), dtype=torch.int32, device=device)
        combined = torch.empty((3 * n, ), dtype=torch.int32, device=device)
        offs, sched, width = alloc_tables(E, n, device)
        cases.append((indx, n, col_sum, combined, offs, sched, width))
    def call(indx, n, col_sum, combined, offs, sched, width):
        return L.tamd_routing_metadata_static(_lib.ptr(indx), 1, n, E, k, _lib.ptr(col_sum), _lib.ptr(combined),
                                              _lib.ptr(combined[n:]), _lib.ptr(combined[2 * n:]), _lib.ptr(offs),
                                              offs.stride(0), _lib.ptr(sched), sched.stride(0), width,
                                              _lib.stream_ptr(device))

    for case in cases:  # every kernel the three paths launch has run once (the runtime loads code objects lazily)
        assert call(*case) == 0
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info(device)
    torch0, reserved0 = torch.cuda.memory_allocated(device), torch.cuda.memory_reserved(device)
    for case in cases:
        rc = call(*case)
        assert rc == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info(device)
    assert torch.cuda.memory_allocated(device) == torch0 and torch.cuda.memory_reserved(device) == reserved0
    assert free1 == free0, f"device memory in use changed by {free0 - free1} bytes"


def test_static_workspace_capacity_is_enforced(device):
    L = _lib.lib()
    cap = L.tamd_routing_metadata_static_max_workspace()
    assert cap == 1 << 20
    n, E = 1 << 22, 1024  # needs n / 64 * E ints: far beyond the capacity
    assert L.tamd_bitmatrix_metadata_workspace(n, E) > cap
    dummy = torch.zeros(8, dtype=torch.int32, device=device)
    rc = L.tamd_routing_metadata_static(_lib.ptr(dummy), 0, n, E, 4, _lib.ptr(dummy), _lib.ptr(dummy), _lib.ptr(dummy),
                                        _lib.ptr(dummy), _lib.ptr(dummy), E + 1, _lib.ptr(dummy), 1 << 30, 0,
                                        _lib.stream_ptr(device))
    assert rc == _lib.E_TOO_LARGE
    with pytest.raises(ValueError, match="capacity"):
        _lib.check(rc, "routing (static workspace)")
