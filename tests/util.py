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


def check_weight_only(out, x, codes_signed, scales, antioffset, group, bias, smooth, rounded, what="", exact_rel=1e-5):
    """A weight-only Linear result against the EXACT anchor (dequantised weight not rounded, fp64 contraction), with the
    bound that follows from the reading the library says it took (`rounded`: ops.gemm_w*a16_weight_rounded):

      exact reading    |err| <= exact_rel * max|row| + ulp * |y|         (fp32 accumulation, one rounding of the output)
      rounded reading  |err| <= min(hard, likely) + the same              (oracle.deploy.weight_only_error_bounds)
                       and, against the anchor with the SAME rounding of the weight, the exact reading's bound

    x may be a sample of the call's rows (then `out` holds those rows).  Returns, for the tests that state it, the
    largest deviation from the exact anchor as a fraction of the row's largest output, not counting the rounding of
    the output itself: max((|err| - ulp * |y|)+ / max|row|)."""
    import torch
    from oracle import deploy as od
    ulp = 2.0 ** -8 if x.dtype == torch.bfloat16 else 2.0 ** -11
    x2 = od.smoothed_rows(x, None if smooth is None else smooth.reshape(1, -1))
    w = od.dequant_weight(codes_signed, scales, antioffset, group, None)             # exact, fp64
    want = od.weight_quant_matmul_f64(x2, w, bias)
    rowmax = want.abs().amax(dim=1, keepdim=True)
    got = out.detach().cpu().double().reshape(want.shape)
    err = (got - want).abs()
    base = exact_rel * rowmax + want.abs() * ulp
    if not rounded:
        assert (err <= base).all(), (what, "exact reading", float((err / base).max()))
    else:
        hard, likely = od.weight_only_error_bounds(x2, w)
        tol = torch.minimum(hard, likely) + base
        assert (err <= tol).all(), (what, "rounded reading against the exact anchor", float((err / tol).max()))
        # (q - z) * s is exact in fp32 (at most 9 x 11 bits), so one rounding of the fp64 value is the kernel's rounding
        own = od.weight_quant_matmul_f64(x2, w.to(x.dtype), bias)
        err_own = (got - own).abs()
        base_own = exact_rel * own.abs().amax(dim=1, keepdim=True) + own.abs() * ulp
        assert (err_own <= base_own).all(), (what, "rounded reading against its own anchor", float((err_own / base_own).max()))
    return float(((err - want.abs() * ulp).clamp_min(0.0) / rowmax.clamp_min(1e-300)).max())
