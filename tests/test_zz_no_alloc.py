"""The entry point that allocates nothing: cg_scan_lengths_static keeps the partial sums of the
running sum in an array that is part of the library's device image.  Called through the C ABI
and compared, bit for bit, with cg_scan_lengths (which takes its scratch from the caller) on two
calls in a row, the second with a smaller input, so that whatever the first call left in the
shared array cannot leak into the second result."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _scan_with_workspace(lib, lengths):
    from cachegen_amd import _lib
    n = lengths.numel()
    offsets = torch.full((n + 1,), -1, dtype=torch.int64, device=DEV)
    scratch = torch.empty(int(lib.cg_scan_workspace(n)), dtype=torch.uint8, device=DEV)
    _lib.check(lib.cg_scan_lengths(lengths.data_ptr(), n, offsets.data_ptr(), scratch.data_ptr(), scratch.numel(),
                                   torch.cuda.current_stream().cuda_stream))
    return offsets


def _scan_static(lib, lengths, offsets):
    from cachegen_amd import _lib
    _lib.check(lib.cg_scan_lengths_static(lengths.data_ptr(), lengths.numel(), offsets.data_ptr(),
                                          torch.cuda.current_stream().cuda_stream))


def test_static_scan_equals_the_workspace_scan_on_two_calls_in_a_row():
    from cachegen_amd import _lib
    lib = _lib.lib()
    torch.cuda.set_device(0)
    g = torch.Generator().manual_seed(5)
    big = torch.randint(0, 257, (64 * 1024 * 9 + 321,), generator=g, dtype=torch.int32).to(DEV)     # 289 tiles, ragged
    small = torch.randint(0, 257, (2048 * 3 + 7,), generator=g, dtype=torch.int32).to(DEV)          # 4 tiles
    tiny = torch.randint(0, 257, (100,), generator=g, dtype=torch.int32).to(DEV)                    # a single tile
    # more than 16384 lengths: like `big` it takes the three-launch scan that uses the built-in
    # array, of which it overwrites only the first 21 of the 290 sums `big` leaves there
    mid = torch.randint(0, 257, (2048 * 20 + 33,), generator=g, dtype=torch.int32).to(DEV)
    inputs = (big, small, tiny, mid)
    want = [_scan_with_workspace(lib, t) for t in inputs]
    # outputs exist before the calls under test: nothing is allocated between or inside them
    outs = [torch.full((t.numel() + 1,), -1, dtype=torch.int64, device=DEV) for t in inputs]
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]       # the driver's own count: a hipMalloc inside the library would show here
    _scan_static(lib, big, outs[0])
    _scan_static(lib, small, outs[1])
    _scan_static(lib, tiny, outs[2])
    _scan_static(lib, mid, outs[3])
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    for got, ref, src in zip(outs, want, inputs):
        assert torch.equal(got, ref)
        host = np.concatenate([[0], np.cumsum(src.cpu().numpy().astype(np.int64))])
        assert np.array_equal(got.cpu().numpy(), host)
    # and once more in the other order, reusing the outputs
    for o in outs:
        o.fill_(-1)
    _scan_static(lib, small, outs[1])
    _scan_static(lib, big, outs[0])
    torch.cuda.synchronize()
    assert torch.equal(outs[0], want[0]) and torch.equal(outs[1], want[1])


def test_static_scan_refuses_what_does_not_fit():
    from cachegen_amd import _lib
    lib = _lib.lib()
    x = torch.zeros(8, dtype=torch.int32, device=DEV)
    o = torch.zeros(9, dtype=torch.int64, device=DEV)
    rc = lib.cg_scan_lengths_static(x.data_ptr(), 16 * 1024 * 1024 + 1, o.data_ptr(), None)
    assert rc == -3 and b"exceed the built-in scratch" in lib.cg_last_error()
    assert lib.cg_scan_lengths_static(x.data_ptr(), 0, o.data_ptr(), None) == -1
    assert lib.cg_scan_lengths_static(None, 8, o.data_ptr(), None) == -1
