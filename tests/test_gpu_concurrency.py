"""Calls on different streams, and from different host threads, are independent: the library keeps no state between
calls beyond a per-host-thread memo of the last GEMM block-shape plan, and the Python wrappers lend one scratch tensor
per device AND stream.  Everything here is compared bit for bit with the same calls made one after the other on the
default stream."""
import threading

import pytest
import torch

from amct_amd import ops

pytestmark = pytest.mark.gpu


def make_case(dev, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    K = 4096
    c = {}
    c["xq"] = {M: torch.randint(-128, 128, (M, K), generator=g, device=dev, dtype=torch.int8) for M in (16, 300, 1024, 2048)}
    c["wq"] = {N: torch.randint(-128, 128, (N, K), generator=g, device=dev, dtype=torch.int8) for N in (1536, 14336)}
    c["s_ch"] = {N: 1e-3 + 9e-3 * torch.rand(N, generator=g, device=dev) for N in (1536, 14336)}
    c["s_tok"] = {M: 0.01 + torch.rand(M, generator=g, device=dev) for M in (16, 300, 1024, 2048)}
    c["x16"] = {M: torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16) for M in (16, 64, 1100)}
    N4 = 4096
    c["packed"] = torch.randint(0, 256, (N4, K // 2), generator=g, device=dev, dtype=torch.uint8)
    c["scales"] = (1e-3 + 9e-3 * torch.rand(N4, K // 128, generator=g, device=dev)).to(torch.float16)
    c["zeros"] = torch.randint(0, 16, (N4, K // 128), generator=g, device=dev, dtype=torch.uint8)
    c["smooth"] = (0.5 + torch.rand(K, generator=g, device=dev)).to(torch.bfloat16)
    c["w"] = torch.randn(2048, K, generator=g, device=dev).to(torch.bfloat16)
    return c


def w8a8_jobs(c):
    return [lambda M=M, N=N: ops.gemm_w8a8(c["xq"][M], c["wq"][N], c["s_ch"][N], c["s_tok"][M], None)
            for M, N in ((2048, 14336), (16, 14336), (300, 1536), (1024, 14336), (16, 1536), (2048, 1536))]


def w4a16_jobs(c):
    jobs = [lambda M=M: ops.gemm_w4a16(c["x16"][M], c["packed"], c["scales"], c["zeros"], 128, c["smooth"], None) for M in (16, 64, 1100)]
    jobs.append(lambda: ops.quant_int4_group_pack(c["w"], 128)[0])
    jobs.append(lambda: ops.act_quant_per_token_int8(c["x16"][1100])[0])
    jobs.append(lambda: ops.mx_quant(c["w"], 0)[0])
    return jobs


def same(a, b):
    if a.is_floating_point():
        a, b = a.view(torch.int16), b.view(torch.int16)
    return torch.equal(a, b)


def test_two_streams_interleaved(dev):
    """The W8A8 Linear at six shapes on one stream and the W4A16 Linear (three row counts: weight streaming, tiles,
    dequantise-once), K2, K3 and K4 on another, enqueued alternately for several rounds."""
    c = make_case(dev, 3)
    ja, jb = w8a8_jobs(c), w4a16_jobs(c)
    want_a, want_b = [j() for j in ja], [j() for j in jb]
    torch.cuda.synchronize(dev)
    sa, sb = torch.cuda.Stream(dev), torch.cuda.Stream(dev)
    got_a, got_b = [], []
    for rnd in range(4):
        for i in range(6):
            with torch.cuda.stream(sa):
                got_a.append((i, ja[i]()))
            with torch.cuda.stream(sb):
                got_b.append((i, jb[i]()))
    sa.synchronize()
    sb.synchronize()
    for i, t in got_a:
        assert same(t, want_a[i]), ("stream a, job", i)
    for i, t in got_b:
        assert same(t, want_b[i]), ("stream b, job", i)


def test_two_host_threads(dev):
    """The same two job lists from two host threads at once, each on a stream of its own (ctypes releases the
    interpreter lock during a call, so the library's host code really runs concurrently: the block-shape plan memo is
    per thread, the scratch tensors per stream)."""
    c = make_case(dev, 5)
    ja, jb = w8a8_jobs(c), w4a16_jobs(c)
    want = {"a": [j() for j in ja], "b": [j() for j in jb]}
    torch.cuda.synchronize(dev)
    errors = []

    def run(name, jobs):
        try:
            torch.cuda.set_device(dev)
            s = torch.cuda.Stream(dev)
            outs = []
            with torch.cuda.stream(s):
                for rnd in range(6):
                    for i, j in enumerate(jobs):
                        outs.append((i, j()))
            s.synchronize()
            for i, t in outs:
                if not same(t, want[name][i]):
                    errors.append((name, i))
        except Exception as e:                        # noqa: BLE001 -- reported by the main thread
            errors.append((name, repr(e)))

    ta = threading.Thread(target=run, args=("a", ja))
    tb = threading.Thread(target=run, args=("b", jb))
    ta.start()
    tb.start()
    ta.join()
    tb.join()
    assert not errors, errors
