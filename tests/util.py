import torch

INT_VIEW = {torch.float32: torch.int32, torch.float16: torch.int16, torch.bfloat16: torch.int16}


def assert_bits_equal(got, want, what=""):
    """Bit-for-bit equality (distinguishes -0.0 from 0.0)."""
    got = got.detach().cpu().contiguous()
    want = want.detach().cpu().contiguous()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert got.dtype == want.dtype, (what, got.dtype, want.dtype)
    if got.dtype in INT_VIEW:
        g, w = got.view(INT_VIEW[got.dtype]), want.view(INT_VIEW[want.dtype])
    else:
        g, w = got, want
    if not torch.equal(g, w):
        bad = (g != w).nonzero()
        i = tuple(bad[0].tolist())
        raise AssertionError("{}: {} of {} differ; first at {}: got {} want {}".format(
            what, bad.shape[0], g.numel(), i, got[i].item(), want[i].item()))
