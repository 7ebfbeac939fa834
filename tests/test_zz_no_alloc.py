"""mts_moe_route_static (the entry point that allocates nothing) against mts_moe_route.

The chunk counters of the static variant live in an array inside the library's device image; the
call itself must leave the allocator alone and must give the same integers as the workspace variant,
also when a smaller problem follows a larger one in the same array.
"""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _route(lib, idx, E, static, block_m=64):
    from minitrain_amd import _lib

    T, K = idx.shape
    TK = T * K
    dev = idx.device
    i32 = dict(dtype=torch.int32, device=dev)
    max_tiles = min(TK, -(-TK // block_m) + E - 1)
    outs = dict(
        counts=torch.full((E,), -7, **i32), expert_start=torch.full((E + 1,), -7, **i32),
        s_scatter=torch.full((TK,), -7, **i32), s_reverse=torch.full((TK,), -7, **i32),
        x_gather=torch.full((TK,), -7, **i32), tile_row_start=torch.full((max_tiles,), -7, **i32),
        tile_expert=torch.full((max_tiles,), -7, **i32), tile_count=torch.full((1,), -7, **i32),
    )
    stream = _lib.stream_of(idx)
    ptrs = [outs[k].data_ptr() for k in ("counts", "expert_start", "s_scatter", "s_reverse", "x_gather",
                                         "tile_row_start", "tile_expert", "tile_count")]
    if static:
        # two views of "allocates nothing": torch's caching allocator saw no request, and the device's own count
        # of free bytes (which a raw hipMalloc / hipFree inside the library would move) is where it was
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
        free_before = torch.cuda.mem_get_info(dev)[0]
        rc = lib.mts_moe_route_static(idx.data_ptr(), T, K, E, block_m, *ptrs, stream)
        free_during = torch.cuda.mem_get_info(dev)[0]
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before
        assert free_during == free_before == torch.cuda.mem_get_info(dev)[0]
    else:
        ws_bytes = lib.mts_moe_route_workspace_bytes(T, K, E)
        ws = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=dev)
        rc = lib.mts_moe_route(idx.data_ptr(), T, K, E, block_m, *ptrs, ws.data_ptr(), ws_bytes, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    n = int(outs["tile_count"].item())
    outs["tile_row_start"], outs["tile_expert"] = outs["tile_row_start"][:n], outs["tile_expert"][:n]
    return outs


def _indices(seed, T, K, E, dropped=False):
    g = torch.Generator().manual_seed(seed)
    idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).int()
    if dropped:
        idx[torch.rand(T, K, generator=g) < 0.2] = -1
    return idx.cuda()


def test_static_route_equals_workspace_route_on_consecutive_calls():
    from minitrain_amd import _lib

    lib = _lib.load()
    # a larger problem first, then smaller ones in the same array (which still holds the larger one's counters)
    cases = [(1, 24576, 2, 8, False), (2, 3000, 3, 64, True), (3, 1, 1, 4, False), (4, 700, 8, 1024, False)]
    # the first static call on a device looks the array's address up (and may load the code object): made here,
    # before any call whose free-memory reading is compared
    _route(lib, _indices(0, 64, 2, 8), 8, static=False)
    warm = _indices(0, 64, 2, 8)
    ptr_args = [torch.empty(64 * 2 + 16, dtype=torch.int32, device="cuda") for _ in range(8)]
    assert lib.mts_moe_route_static(warm.data_ptr(), 64, 2, 8, 64, *[t.data_ptr() for t in ptr_args], _lib.stream_of(warm)) == 0
    torch.cuda.synchronize()
    for seed, T, K, E, dropped in cases:
        idx = _indices(seed, T, K, E, dropped)
        want = _route(lib, idx, E, static=False)
        got = _route(lib, idx, E, static=True)
        for name in want:
            assert torch.equal(got[name], want[name]), (name, T, K, E)
        # the permutation is a stable sort by expert: check it against torch directly as well
        flat = idx.flatten().cpu()
        kept = (flat >= 0).nonzero().flatten()
        order = kept[torch.sort(flat[kept], stable=True).indices]
        assert torch.equal(got["s_scatter"][: len(order)].cpu(), order.int())


def test_static_route_rejects_sizes_beyond_its_array():
    from minitrain_amd import _lib

    lib = _lib.load()
    fake = 4096
    WORKSPACE, NULL = -4, -1
    # 2^21 chunks x 1024 experts x 4 bytes is far beyond the 4 MiB array: refused on the host, nothing launched
    assert lib.mts_moe_route_static(fake, 1 << 26, 8, 1024, 64, fake, fake, fake, fake, fake, None, None, None, None) == WORKSPACE
    assert lib.mts_moe_route_static(None, 16, 2, 4, 64, fake, fake, fake, fake, fake, None, None, None, None) == NULL
