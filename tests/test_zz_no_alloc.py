"""The entry point that allocates nothing: ``dice_dispatch_static`` keeps its
histogram table in the library's own device array.  Its outputs must equal
``dice_dispatch``'s bit for bit, on two calls in a row into the same output
buffers, the second on a smaller input, and on every size class of the
dispatch (one workgroup, two launches, three launches)."""
import ctypes

import pytest
import torch

from oracle import dice_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from dice_amd import lib
    lib.load()
    return torch.device("cuda:0")


def _tables(dev, n_slots, n_experts):
    return (torch.full((n_experts,), -7, dtype=torch.int32, device=dev),
            torch.full((n_experts + 1,), -7, dtype=torch.int32, device=dev),
            torch.full((n_slots,), -7, dtype=torch.int32, device=dev),
            torch.full((n_slots,), -7, dtype=torch.int32, device=dev))


def _static_call(lib, idx, mask, n_experts, out):
    """Straight through the C ABI: no workspace, and nothing allocated between
    the argument set-up and the launch."""
    from dice_amd.lib import check, ptr, stream_ptr
    counts, offsets, perm, inv = out
    check(lib.dice_dispatch_static(ptr(idx), ptr(mask), idx.numel(), n_experts, ptr(counts), ptr(offsets),
                                   ptr(perm), ptr(inv), stream_ptr()))


@pytest.mark.parametrize("first,second,E", [
    (16384, 6000, 8),       # the DiT-XL layer's slot count, then a smaller batch (both two-launch sizes)
    (300000, 16384, 16),    # three launches, then two
    (32768, 1000, 64),      # two launches, then the one-workgroup size that uses no table at all
])
def test_static_dispatch_equals_dispatch_two_calls_in_a_row(dev, first, second, E):
    from dice_amd import ops
    from dice_amd.lib import load
    lib = load()
    g = torch.Generator().manual_seed(first + E)
    out = _tables(dev, first, E)                    # the same output buffers serve both calls
    for S in (first, second):
        idx_cpu = torch.randint(0, E, (S,), generator=g)
        idx = idx_cpu.int().to(dev)
        for mask_cpu in (None, O.skip_mask(S, "rand", None) if S % 2 == 0 else None):
            mask = None if mask_cpu is None else mask_cpu.to(dev).view(torch.uint8)
            want = ops.dispatch(idx, E, mask)                       # dice_dispatch with a workspace
            _static_call(lib, idx, mask, E, out)
            torch.cuda.synchronize()
            counts, offsets, perm, inv = out
            assert torch.equal(counts, want[0])
            assert torch.equal(offsets, want[1])
            assert torch.equal(perm[:S], want[2])
            assert torch.equal(inv[:S], want[3])
            # and both equal the oracle's stable tables
            kept = torch.arange(S) if mask_cpu is None else (~mask_cpu).nonzero().flatten()
            wc, wo, wp, _ = O.dispatch_tables(idx_cpu[kept], E)
            assert torch.equal(counts.cpu().long(), wc) and torch.equal(offsets.cpu().long(), wo)
            assert torch.equal(perm[:kept.numel()].cpu().long(), kept[wp])


def test_static_dispatch_refuses_what_its_array_cannot_hold(dev):
    from dice_amd.lib import load
    lib = load()
    limit = lib.dice_dispatch_static_scratch_bytes()
    assert limit == 1 << 20
    S, E = 1 << 20, 256                              # 2048 spans x 256 experts x 4 B = 2 MiB
    assert lib.dice_dispatch_workspace_bytes(S, E) > limit
    idx = torch.zeros(S, dtype=torch.int32, device=dev)
    out = _tables(dev, S, E)
    rc = lib.dice_dispatch_static(idx.data_ptr(), None, S, E, out[0].data_ptr(), out[1].data_ptr(),
                                  out[2].data_ptr(), out[3].data_ptr(), None)
    assert rc == -3
    assert b"static array" in lib.dice_last_error()
    torch.cuda.synchronize()
    assert int(out[1][0]) == -7                      # nothing was launched


def test_static_dispatch_allocates_nothing(dev):
    """torch's allocator statistics do not move across the call (the library
    itself calls no hipMalloc: it has no allocation call in its sources)."""
    from dice_amd.lib import load
    lib = load()
    S, E = 16384, 8
    idx = torch.randint(0, E, (S,), generator=torch.Generator().manual_seed(3)).int().to(dev)
    out = _tables(dev, S, E)
    _static_call(lib, idx, None, E, out)             # first call on the device: address look-up
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    free_before, _ = torch.cuda.mem_get_info(dev)
    _static_call(lib, idx, None, E, out)
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before
    free_after, _ = torch.cuda.mem_get_info(dev)
    assert free_after == free_before
