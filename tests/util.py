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


def load_ref_callers():
    """tests/golden/ref_callers.pt: tensors written by the reference's CPU path (see
    tests/golden/make_ref_caller_fixtures.py).  Loaded with weights_only=True: nothing in the file is executed."""
    import os
    import torch
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_callers.pt")
    return torch.load(path, map_location="cpu", weights_only=True)


def load_int_quant_kat16():
    """Cases of tests/golden/int_quant_kat16.json as dicts of tensors: w [1,n] of the source dtype, scale f32 [G],
    offset int32 [G] | None, codes int32 [1,n], dq / awq_dq [1,n] of the source dtype; bits, symmetric, group."""
    import json
    import os
    import numpy as np
    import torch
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "int_quant_kat16.json")
    with open(path) as f:
        doc = json.load(f)
    tdt = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}

    def dec(hexes, fmt):
        v = [int(h, 16) for h in hexes]
        if fmt == "f32":
            return torch.from_numpy(np.array(v, dtype=np.uint32).view(np.float32).copy())
        return torch.from_numpy(np.array(v, dtype=np.uint16).view(np.int16).copy()).view(tdt[fmt])

    out = []
    for c in doc["cases"]:
        fmt = c["src"]
        out.append({"src": tdt[fmt], "bits": c["bits"], "symmetric": c["symmetric"], "group": c["group"],
                    "w": dec(c["w"], fmt).reshape(1, -1), "scale": dec(c["scale"], "f32"),
                    "offset": None if c["offset"] is None else torch.tensor(c["offset"], dtype=torch.int32),
                    "codes": torch.tensor(c["codes"], dtype=torch.int32).reshape(1, -1),
                    "dq": dec(c["dq"], fmt).reshape(1, -1), "awq_dq": dec(c["awq_dq"], fmt).reshape(1, -1)})
    return out
