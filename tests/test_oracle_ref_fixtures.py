"""The oracle against vectors written by the reference's own CPU path (tests/golden/ref_callers.pt, produced by
tests/golden/make_ref_caller_fixtures.py where the reference checkout exists).  Elementwise results must agree
bit for bit; the routines that run through library factorisations (GPTQ) get a stated tolerance."""
import math

import pytest
import torch

from oracle import int_quant as iq
from oracle import deploy as od
from oracle import gptq as og
from util import assert_bits_equal, load_ref_callers

DT = {"torch.float32": torch.float32, "torch.bfloat16": torch.bfloat16, "torch.float16": torch.float16}


@pytest.fixture(scope="module")
def ref():
    return load_ref_callers()


def test_fixture_file_is_complete(ref):
    assert len(ref["matrix"]) == 36 and len(ref["awq_search"]) == 4 and len(ref["smoothquant"]) == 3
    assert len(ref["gptq"]) == 4 and len(ref["weight_only_deploy"]) == 5


def test_elementwise_matrix(ref):
    """min/max, factors, fake-quant, codes and AWQ's cast-before-round fake-quant for
    {fp32,bf16,fp16} x {int8,int4} x {sym,asym} x {tensor,channel,group}: bit for bit."""
    n_awq_differs = 0
    for c in ref["matrix"]:
        w, kind, sym, strat, g = c["w"], c["kind"], c["symmetric"], c["strategy"], c["group"] or None
        tag = "{} {} sym={} {}".format(c["dtype"], kind, sym, strat)
        assert w.dtype == DT[c["dtype"]]
        mn, mx = iq.weight_min_max(w, strat, g)
        assert_bits_equal(mn, c["min"], tag + " min")
        assert_bits_equal(mx, c["max"], tag + " max")
        s, z = iq.scale_offset(mx, mn, sym, kind)
        assert_bits_equal(s, c["scale"], tag + " scale")
        if sym:
            assert z is None and c["offset"] is None
        else:
            assert z.dtype == torch.int32 and torch.equal(z, c["offset"]), tag
        assert_bits_equal(iq.fake_quant(w, kind, s, z, g), c["dq"], tag + " dq")
        codes = iq.quant_codes(w, kind, s, z, g)
        assert codes.dtype == c["codes"].dtype and codes.shape == c["codes"].shape, tag
        assert torch.equal(codes, c["codes"]), tag + " codes"
        a = iq.awq_fake_quant(w, kind, s, z, strat, g)
        assert_bits_equal(a, c["awq_dq"], tag + " awq dq")
        if not torch.equal(c["awq_dq"], c["dq"]):
            n_awq_differs += 1
    # the fixture does discriminate: on 16-bit sources the cast before the rounding changes some results
    assert n_awq_differs >= 4


def test_awq_grid_point_and_search(ref):
    for c in ref["awq_search"]:
        kind, sym, strat, g = c["kind"], c["symmetric"], c["strategy"], c["group"] or None
        for w0, w1 in zip(c["weights"], c["grid_weights"]):
            got, _, _ = iq.awq_grid_step(w0, c["grid_scale"], kind, strat, sym, g)
            assert_bits_equal(got, w1, "grid point")

        def fwd(x, ws):
            return torch.cat([torch.nn.functional.linear(x, w) for w in ws], dim=-1)

        torch.set_num_threads(1)
        best, losses = iq.awq_search_scale(c["x"], c["weights"], fwd, c["grids"], kind, strat, sym, g)
        assert len(losses) == c["grids"]
        assert_bits_equal(best, c["best_scale"], "best scale")


def test_smoothquant_statistics_and_factor(ref):
    for c in ref["smoothquant"]:
        w = c["weight"]
        dmax = torch.ones((1, w.shape[-1]), dtype=w.dtype) * torch.inf * -1
        dmin = torch.ones((1, w.shape[-1]), dtype=w.dtype) * torch.inf
        for x in c["inputs"]:
            dmax, dmin = iq.channel_min_max_update(x, dmax, dmin)
        assert_bits_equal(dmax, c["data_max"], "data_max")
        assert_bits_equal(dmin, c["data_min"], "data_min")
        act_max = torch.max(dmax.abs(), dmin.abs())
        f = iq.smooth_factor(act_max, w, c["strength"])
        assert_bits_equal(f, c["smooth"], "smooth factor")
        assert f[0, 9].item() == 1.0                    # the dead activation channel: 0 / x < eps -> 1
        ws = w * f
        s, z = iq.weight_scale_offset(ws, 'channel', True, 'int8')
        assert_bits_equal(s, c["scale_w"], "scale_w")
        # the W8A8 deploy buffers built from the calibrated module
        buf = od.w8a8_buffers(w, c["bias"], c["scale_w"], c["scale_d"], c["offset_d"], c["smooth"])
        dep = c["deploy"]
        assert torch.equal(buf["quantized_weight"], dep["quantized_weight"])
        for k in ("act_scale", "act_offset", "deq_scale", "scale_factor"):
            assert_bits_equal(buf[k], dep[k], k)
        if "pertoken_scale" in dep:
            assert_bits_equal(buf["pertoken_scale"], dep["pertoken_scale"], "pertoken_scale")
        else:
            assert buf["pertoken_scale"] is None
        want_b = c["deploy_bias"]
        assert buf["bias"].dtype == want_b.dtype and torch.equal(buf["bias"], want_b)


def test_gptq_hessian_and_optimised_weight(ref):
    """The routine runs two Cholesky factorisations and an inverse through the library, so its result depends on
    the library build: the factors (computed before any factorisation) must agree bit for bit, the optimised
    weight within a small number of quantisation steps on a small fraction of entries."""
    torch.set_num_threads(1)
    for idx, c in enumerate(ref["gptq"]):
        kind, sym, strat, g = c["kind"], c["symmetric"], c["strategy"], c["group"] or None
        w = c["weight"]
        if c["inputs"] is not None:
            h, n = None, 0
            for x in c["inputs"]:
                h, n = og.update_hessian(h, n, x, w.shape[1])
            assert torch.allclose(h, c["hessian"], rtol=1e-5, atol=1e-6)
            assert float(h[5].abs().max()) == 0.0       # the dead column
        got, s, z = og.optimize_weight(w, c["hessian"], kind, strat, sym, g)
        assert_bits_equal(s, c["scale"], "gptq scale")
        if sym:
            assert z is None and c["offset"] is None
        else:
            assert torch.equal(z, c["offset"])
        want = c["opt_weight"]
        assert got.dtype == want.dtype and got.shape == want.shape
        # same library, same thread count, same operation order: identical here; a different BLAS build may move
        # single entries across a rounding boundary, so the committed bound is "at most 0.5 % of entries differ,
        # and those by no more than two quantisation steps"
        diff = (got.float() - want.float()).abs()
        step = float(c["scale"].detach().max())
        assert (diff > 0).float().mean().item() <= 0.005, (idx, (diff > 0).float().mean().item())
        assert float(diff.max()) <= 2.0 * step + 1e-6, (idx, float(diff.max()), step)


def test_weight_only_deploy_buffers(ref):
    for c in ref["weight_only_deploy"]:
        kind, g = c["kind"], c["group"] or None
        buf = od.w4a16_buffers(c["weight"], c["bias"], c["scale_w"], c["offset_w"], kind, g)
        want = c["buffers"]
        # the fixture keeps the [K,N] codes unpacked (int8, or one int4 per int32): the packing is a torch_npu call
        qw = buf["codes_nk"].transpose(-1, -2).contiguous()
        assert qw.dtype == want["quantized_weight"].dtype and torch.equal(qw, want["quantized_weight"])
        assert_bits_equal(buf["scale_w"], want["scale_w"], "scale_w")
        if c["offset_w"] is None:
            assert "offset_w" not in want and buf["offset_w"] is None
        else:
            assert_bits_equal(buf["offset_w"], want["offset_w"], "offset_w")
        assert buf["bias"].dtype == c["dep_bias"].dtype and torch.equal(buf["bias"], c["dep_bias"])
        assert buf["group_size"] == c["dep_group_size"]


def test_cast_before_round_is_pinned_by_a_known_answer():
    """bf16 w = 3.5 with fp32 s = 1.0003: w/s = 3.49895... rounds to 3 in fp32, but narrowed to bf16 first it is
    3.5 and rounds (half to even) to 4.  AWQ's path narrows first (algorithm/awq.py:149)."""
    w = torch.tensor([[3.5, 100.0]], dtype=torch.bfloat16)
    s = torch.tensor([[1.0003]], dtype=torch.float32)
    t = (w.float() / s)[0, 0].item()
    assert 3.498 < t < 3.4995 and math.floor(t + 0.5) == 3
    assert iq.fake_quant(w, 'int8', s)[0, 0].item() == torch.tensor(3 * 1.0003).to(torch.bfloat16).item()
    a = iq.awq_fake_quant(w, 'int8', s, None, 'channel')
    assert a.dtype == torch.bfloat16
    assert a[0, 0].item() == torch.tensor(4 * 1.0003).to(torch.bfloat16).item()
    assert a[0, 0].item() != iq.fake_quant(w, 'int8', s)[0, 0].item()
    # fp16: 11 significand bits.  w = 2.5, s = 1.00001 -> 2.499975 -> fp16 2.5 -> 2 (even) both ways: no
    # difference; w = 3.5, s = 1.00001 -> 3.499965 -> fp16 3.5 -> 4 against 3
    wh = torch.tensor([[3.5, 100.0]], dtype=torch.float16)
    sh = torch.tensor([[1.00001]], dtype=torch.float32)
    assert iq.fake_quant(wh, 'int8', sh)[0, 0].item() == 3.0
    assert iq.awq_fake_quant(wh, 'int8', sh, None, 'channel')[0, 0].item() == 4.0
