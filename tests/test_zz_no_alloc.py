"""The allocation-free column-statistics entry point against the one that takes a workspace, through the C ABI:
two calls in a row on one stream, the second on a smaller input (the shared scratch array keeps the first call's
partials), every output bit for bit."""
import pytest
import torch

from amct_amd import _lib
from util import assert_bits_equal

pytestmark = pytest.mark.gpu

_DT = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}


def _stream(dev):
    return torch.cuda.current_stream(dev).cuda_stream


def _with_workspace(x, absolute, running=None):
    lib = _lib.load()
    rows, cols = x.shape
    dev = x.device
    cmax = torch.empty(cols, dtype=torch.float32, device=dev) if running is None else running[0].clone()
    cmin = torch.empty(cols, dtype=torch.float32, device=dev) if running is None else running[1].clone()
    nbytes = lib.amct_col_minmax_workspace_bytes(rows, cols)
    ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=dev)
    _lib.check(lib.amct_col_minmax(x.data_ptr(), cmax.data_ptr(), None if absolute else cmin.data_ptr(), rows, cols,
                                   int(absolute), int(running is not None), _DT[x.dtype], ws.data_ptr(), nbytes,
                                   _stream(dev)))
    return cmax, cmin


_WARM = set()


def _warm_up(dev):
    """The first call on a device asks the runtime for the scratch array's address (which may load the library's code
    object): done once per device, before any call whose memory use is measured or that is captured in a graph."""
    if dev in _WARM:
        return
    x = torch.zeros(4, 8, dtype=torch.float32, device=dev)
    o = torch.empty(8, dtype=torch.float32, device=dev)
    _lib.check(_lib.load().amct_col_minmax_noalloc(x.data_ptr(), o.data_ptr(), o.data_ptr(), 4, 8, 0, 0, _lib.F32, _stream(dev)))
    torch.cuda.synchronize(dev)
    _WARM.add(dev)


def _no_alloc(x, cmax, cmin, absolute, accumulate):
    """Outputs are allocated by the caller beforehand: the call itself must not allocate -- neither through torch's
    caching allocator nor behind its back (the device's free memory as the runtime reports it, hipMemGetInfo)."""
    lib = _lib.load()
    rows, cols = x.shape
    _warm_up(x.device)
    before = torch.cuda.memory_stats(x.device)["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info(x.device)[0]
    _lib.check(lib.amct_col_minmax_noalloc(x.data_ptr(), cmax.data_ptr(), None if absolute else cmin.data_ptr(), rows,
                                           cols, int(absolute), int(accumulate), _DT[x.dtype], _stream(x.device)))
    assert torch.cuda.mem_get_info(x.device)[0] == free_before
    assert torch.cuda.memory_stats(x.device)["allocation.all.allocated"] == before


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_two_calls_second_smaller(dev, dtype):
    g = torch.Generator().manual_seed(11)
    big = torch.randn(2500, 4096, generator=g).to(dtype).to(dev)
    small = torch.randn(300, 520, generator=g).to(dtype).to(dev)          # fewer chunks, fewer and unaligned-count columns
    big[7, 100] = float('nan')
    outs = {}
    for name, x in (("big", big), ("small", small)):
        outs[name] = (torch.full((x.shape[1],), 7.0, dtype=torch.float32, device=dev),
                      torch.full((x.shape[1],), 7.0, dtype=torch.float32, device=dev))
    torch.cuda.synchronize()
    _no_alloc(big, *outs["big"], absolute=False, accumulate=False)
    _no_alloc(small, *outs["small"], absolute=False, accumulate=False)
    torch.cuda.synchronize()
    for name, x in (("big", big), ("small", small)):
        want_max, want_min = _with_workspace(x, False)
        assert_bits_equal(outs[name][0], want_max, name + " max")
        assert_bits_equal(outs[name][1], want_min, name + " min")
    # and against torch on the small one (NaN-free)
    assert torch.equal(outs["small"][0].cpu(), small.float().amax(dim=0).cpu())
    assert torch.equal(outs["small"][1].cpu(), small.float().amin(dim=0).cpu())


def test_running_update_and_absolute(dev):
    g = torch.Generator().manual_seed(12)
    x1 = torch.randn(700, 1024, generator=g).to(torch.bfloat16).to(dev)
    x2 = (torch.randn(90, 1024, generator=g) * 2).to(torch.bfloat16).to(dev)
    run = (torch.full((1024,), float('-inf'), dtype=torch.float32, device=dev),
           torch.full((1024,), float('inf'), dtype=torch.float32, device=dev))
    want = (run[0].clone(), run[1].clone())
    for x in (x1, x2):
        _no_alloc(x, run[0], run[1], absolute=False, accumulate=True)
        want = _with_workspace(x, False, running=want)
    assert_bits_equal(run[0], want[0], "running max")
    assert_bits_equal(run[1], want[1], "running min")
    amax = torch.empty(1024, dtype=torch.float32, device=dev)
    _no_alloc(x1, amax, amax, absolute=True, accumulate=False)
    assert_bits_equal(amax, _with_workspace(x1, True)[0], "abs max")


def test_too_wide_is_rejected(dev):
    lib = _lib.load()
    cols = _lib.COL_MINMAX_NOALLOC_MAX_COLS + 8
    x = torch.zeros(4, cols, dtype=torch.bfloat16, device=dev)
    out = torch.full((cols,), 3.0, dtype=torch.float32, device=dev)
    rc = lib.amct_col_minmax_noalloc(x.data_ptr(), out.data_ptr(), out.data_ptr(), 4, cols, 0, 0, _lib.BF16,
                                     _stream(dev))
    assert rc == -5 and b"scratch" in lib.amct_hip_strerror(rc)
    torch.cuda.synchronize()
    assert bool((out == 3.0).all())                                   # nothing was enqueued
    # the widest accepted problem
    cols = _lib.COL_MINMAX_NOALLOC_MAX_COLS
    x = torch.randn(64 * 256 + 3, cols, device=dev).to(torch.bfloat16)    # the maximum number of chunks
    cmax = torch.empty(cols, dtype=torch.float32, device=dev)
    cmin = torch.empty(cols, dtype=torch.float32, device=dev)
    _no_alloc(x, cmax, cmin, absolute=False, accumulate=False)
    want = _with_workspace(x, False)
    assert_bits_equal(cmax, want[0], "widest max")
    assert_bits_equal(cmin, want[1], "widest min")


def test_captured_in_a_graph_after_a_warm_up(dev):
    """What the entry point is for: after one eager call per device (the address look-up), the call is captured in a HIP
    graph; every replay -- with eager work and synchronisations between them, on new input values in the same buffers
    -- gives the bits of the workspace form."""
    _warm_up(dev)
    g = torch.Generator().manual_seed(13)
    x = torch.randn(1000, 2048, generator=g).to(torch.bfloat16).to(dev)
    cmax = torch.empty(2048, dtype=torch.float32, device=dev)
    cmin = torch.empty(2048, dtype=torch.float32, device=dev)
    lib = _lib.load()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _lib.check(lib.amct_col_minmax_noalloc(x.data_ptr(), cmax.data_ptr(), cmin.data_ptr(), 1000, 2048, 0, 0, _lib.BF16,
                                               _stream(dev)))
    for i in range(4):
        x.copy_(torch.randn(1000, 2048, generator=g).to(torch.bfloat16))         # eager work between the replays
        cmax.fill_(-1.0)
        cmin.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = _with_workspace(x, False)
        assert_bits_equal(cmax, want[0], "replay %d max" % i)
        assert_bits_equal(cmin, want[1], "replay %d min" % i)
