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


def load_int_quant_kat():
    """Cases of tests/golden/int_quant_kat.json as tensors: (bits, symmetric, w[1,n] f32, scale f32 scalar,
    offset int|None, codes int32[1,n], dq f32[1,n]).  Values are stored as binary32 bit patterns."""
    import json
    import os
    import numpy as np
    import torch
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "int_quant_kat.json")
    with open(path) as f:
        doc = json.load(f)

    def f32(hexes):
        return torch.from_numpy(np.array([int(h, 16) for h in hexes], dtype=np.uint32).view(np.float32).copy())

    out = []
    for c in doc["cases"]:
        out.append((c["bits"], c["symmetric"], f32(c["w"]).reshape(1, -1), f32([c["scale"]])[0], c["offset"],
                    torch.tensor(c["codes"], dtype=torch.int32).reshape(1, -1), f32(c["dq"]).reshape(1, -1)))
    return out
