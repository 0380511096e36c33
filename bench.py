#!/usr/bin/env python3
"""Benchmark of the quantize/deploy hot path on one MI355X.

`python bench.py --gpus 1 --steps K --warmup W` prints ONE JSON line.  A step is one pass of
the headline kernel over one batch of synthetic input already resident in HBM: INT4 asymmetric
group-128 quantise + pack of a bf16 weight [14336, 4096] (benchmark configuration 2).  The line also
carries, under "kernels", the same measurement for every other kernel of the path, the roofline
of the headline kernel, and the CPU oracle timed on the host cores on a bounded sample.

Input sets rotate (>= 4 sets, > 600 MB) so that traffic reaches HBM rather than the 256 MB
last-level cache.  Launches go straight through the C ABI with preallocated outputs, so the
timed region holds kernel launches only.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PEAK_INT8_TOPS = 5000.0
PEAK_BF16_TFLOPS = 2500.0

# HBM bytes per launch as the hardware counted them (FETCH_SIZE + WRITE_SIZE, each scaled by what the same
# counter reads for the plain copy kernel of known size), with the kernel that was dispatched when they were
# counted.  A program cannot run the profiler around itself, so these are constants of each kernel at its bench
# workload; the runs they come from and their commands are kept in profiles/hbm_traffic_pmc_bench_workloads.txt.
# A kernel that was changed and not counted again has no entry (reported as null).
MEASURED_TRAFFIC = {
    "int4_group_pack": ("int4_group_pack4<2, 16, 1, false, true>", 148551685),
    "fakequant_int8": ("fq_fused<0, 256, 4, 1, false, false>", 134440825),
    "mxfp8_quant": ("mx_quant_full<2, 0, 2>", 101751472),
    "mxfp4_quant": ("mx_quant_full<2, 1, 2>", 84973719),
    "mxfp8_dequant": ("mx_dequant_full<2, 0, 8>", 101830190),
    "hif8_encode": ("hif8_encode_bf16_lut<1024, 1>", 100773601),
    "hif8_decode": ("hif8_decode_full<2, 256, 8>", 100748936),
    "act_quant_per_token": ("act_quant_token<2, 2>", 25292715),
    "col_minmax": ("col_partial_k<2, false> + col_final_k", 69345307),
    "w8a8_m2048": ("w8a8_tile_mix16<2, 0>", 255069388),
    "w8a8_m16": ("w8a8_stream<2, 4, 4, 16, 4, 0>", 59805700),
    "w8a8_linear_m16": ("w8a8_stream<2, 4, 4, 16, 8, 2>", 60417600),
    "w4a16_m2048": ("w4_dequant_rows<false> + w8a8_tile_mix16<2, 1>", 632207001),
    "w4a16_m2048_fused": ("smooth_rows + w4a16_tile_wide16<true, 2, 4, 4, 2, 2, 2, false>", 303595344),
    "w4a16_m16": ("w4a16_wave<2, true, true, 8>", 32471413),
    "w4a16_m1": ("w4a16_stream<2, 4, 1, 8, 2, true, false>", 31100571),
    "w8a16_m16": ("w8a16_stream<2, 4, 8, 8, 1, false>", 60426092),
    "w8a16_m2048": ("w8_dequant_rows<2> + w8a8_tile_mix16<2, 1>", 659261016),
    "w8a8_down_m16": ("w8a8_tile_shape<2, 2, 2, 1, 1, 4, 128> + w8a8_splitk_reduce<2>", 62957888),
    "w4a16_down_m16": ("w4a16_stream<2, 4, 4, 4, 4, false, true> + splitk_reduce16<false>", 39848448),
    "w8a16_down_m16": ("w8a16_stream<2, 4, 4, 4, 1, false> + splitk_reduce16<false>", 67237581),
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--repeats", type=int, default=5, help="timed regions of --steps launches per kernel; the median is reported")
    ap.add_argument("--only", default="", help="comma list of kernel names (default: all)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    return ap.parse_args()


class Case:
    """One kernel at one configuration: `launch(i)` enqueues one call on rotating set i."""

    def __init__(self, name, bound, work, unit_work, launch, nsets, dtype, desc):
        self.name, self.bound, self.work, self.unit_work = name, bound, work, unit_work
        self.launch, self.nsets, self.dtype, self.desc = launch, nsets, dtype, desc


def build_cases(dev, only):
    import torch
    from amct_amd import _lib, ops, workloads
    lib = _lib.load()
    st = torch.cuda.current_stream(dev).cuda_stream
    cases = []

    def want(name):
        return not only or name in only

    def sets_for(nbytes):
        return max(4, int(700e6 // nbytes) + 1)

    def dev_copies(t, n):
        base = t.to(dev)
        return [base] + [base.clone() for _ in range(n - 1)]

    # ---- streaming copy yardstick: 128 MiB read + 128 MiB write ------------------------------------------
    if want("copy"):
        nbytes = 128 << 20
        nsc = 6
        src = [torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(1) for _ in range(nsc)]
        dst = [torch.empty(nbytes, dtype=torch.uint8, device=dev) for _ in range(nsc)]

        def launch(i, src=src, dst=dst, nbytes=nbytes):
            j = i % len(src)
            rc = lib.amct_copy_bytes(src[j].data_ptr(), dst[j].data_ptr(), nbytes, st)
            assert rc == 0, rc
        cases.append(Case("copy", "hbm", 2 * nbytes, "B", launch, nsc, "u8", "plain copy of 128 MiB (yardstick)"))

    # ---- launch floor: a copy of 4 KiB, i.e. what one launch costs back to back whatever the kernel does -------------
    if want("launch_floor"):
        sf = torch.zeros(4096, dtype=torch.uint8, device=dev)
        df = torch.zeros(4096, dtype=torch.uint8, device=dev)

        def launch(i, sf=sf, df=df):
            rc = lib.amct_copy_bytes(sf.data_ptr(), df.data_ptr(), 4096, st)
            assert rc == 0, rc
        cases.append(Case("launch_floor", "hbm", 8192, "B", launch, 1, "u8",
                          "copy of 4 KiB: the time one launch takes back to back (yardstick for the launch-bound kernels)"))

    # ---- K2 (headline): int4 asym g128 quant + pack, W[14336,4096] bf16 -------------------------
    if want("int4_group_pack"):
        w = workloads.c2_weight()
        N, K = w.shape
        g = 128
        work = N * K * 2 + N * K // 2 + N * (K // g) * 2 + N * (K // g)
        ns = sets_for(work)
        ws = dev_copies(w, ns)
        packed = [torch.empty(N, K // 2, dtype=torch.uint8, device=dev) for _ in range(ns)]
        s16 = [torch.empty(N, K // g, dtype=torch.float16, device=dev) for _ in range(ns)]
        zz = [torch.empty(N, K // g, dtype=torch.uint8, device=dev) for _ in range(ns)]

        def launch(i, ws=ws, packed=packed, s16=s16, zz=zz, N=N, K=K, g=g):
            j = i % len(ws)
            rc = lib.amct_quant_int4_group_pack(ws[j].data_ptr(), packed[j].data_ptr(), s16[j].data_ptr(), _lib.F16,
                                                None, zz[j].data_ptr(), None, None, 0, N, K, g, 0, _lib.BF16, st)
            assert rc == 0, rc
        cases.append(Case("int4_group_pack", "hbm", work, "B", launch, ns, "f32",
                          "INT4 asym group-128 quantize+pack, W[14336,4096] bf16 (config 2)"))

    # ---- K1: int8 sym per-channel fake-quant, W[4096,4096] fp32 ------------------------------------
    if want("fakequant_int8"):
        w = workloads.c1_weight()
        N, K = w.shape
        work = N * K * 4 * 2 + N * 4
        ns = sets_for(work)
        ws = dev_copies(w, ns)
        dq = [torch.empty_like(ws[0]) for _ in range(ns)]
        sc = [torch.empty(N, dtype=torch.float32, device=dev) for _ in range(ns)]

        def launch(i, ws=ws, dq=dq, sc=sc, N=N, K=K):
            j = i % len(ws)
            rc = lib.amct_fakequant_int(ws[j].data_ptr(), dq[j].data_ptr(), None, 0, sc[j].data_ptr(), None, None, None, 0,
                                        N, K, 0, 8, 1, 0, -128, 127, 0, _lib.F32, st)
            assert rc == 0, rc
        cases.append(Case("fakequant_int8", "hbm", work, "B", launch, ns, "f32",
                          "INT8 sym per-channel fake-quant, W[4096,4096] fp32 (config 1)"))

    # ---- K4 / K5 on X[8192,4096] bf16 ---------------------------------------------------------------
    if any(want(n) for n in ("mxfp8_quant", "mxfp4_quant", "mxfp8_dequant", "mxfp4_dequant", "hif8_encode", "hif8_decode")):
        x = workloads.c3_activations()
        R, C = x.shape
        ns3 = sets_for(R * C * 3)
        ns = ns3
        xs = dev_copies(x, ns)
        el8 = [torch.empty(R, C, dtype=torch.uint8, device=dev) for _ in range(ns)]
        el4 = [torch.empty(R, C // 2, dtype=torch.uint8, device=dev) for _ in range(ns)]
        e8 = [torch.empty(R, C // 32, dtype=torch.uint8, device=dev) for _ in range(ns)]
        ys = [torch.empty(R, C, dtype=torch.bfloat16, device=dev) for _ in range(ns)]
        for j in range(ns):      # valid codes for the decode cases
            lib.amct_mx_quant(xs[j].data_ptr(), el8[j].data_ptr(), e8[j].data_ptr(), R, C, 0, 0, _lib.BF16, st)

        def mk_mxq(fmt, el, xs=xs, e8=e8, R=R, C=C, ns3=ns3):
            def launch(i):
                j = i % ns3
                rc = lib.amct_mx_quant(xs[j].data_ptr(), el[j].data_ptr(), e8[j].data_ptr(), R, C, fmt, 0, _lib.BF16, st)
                assert rc == 0, rc
            return launch

        def mk_mxd(fmt, el, ys=ys, e8=e8, R=R, C=C, ns3=ns3):
            def launch(i):
                j = i % ns3
                rc = lib.amct_mx_dequant(el[j].data_ptr(), e8[j].data_ptr(), ys[j].data_ptr(), R, C, fmt, _lib.BF16, st)
                assert rc == 0, rc
            return launch

        def hif_enc(i, xs=xs, el8=el8, R=R, C=C, ns3=ns3):
            j = i % ns3
            rc = lib.amct_hif8_encode(xs[j].data_ptr(), el8[j].data_ptr(), R * C, _lib.BF16, 0, st)
            assert rc == 0, rc

        def hif_dec(i, ys=ys, el8=el8, R=R, C=C, ns3=ns3):
            j = i % ns3
            rc = lib.amct_hif8_decode(el8[j].data_ptr(), ys[j].data_ptr(), R * C, _lib.BF16, st)
            assert rc == 0, rc
        if want("mxfp8_quant"):
            cases.append(Case("mxfp8_quant", "hbm", R * C * 2 + R * C + R * C // 32, "B", mk_mxq(0, el8), ns, "f32",
                              "MXFP8 E4M3 block-32 quantize, X[8192,4096] bf16 (config 3)"))
        if want("mxfp4_quant"):
            cases.append(Case("mxfp4_quant", "hbm", R * C * 2 + R * C // 2 + R * C // 32, "B", mk_mxq(1, el4), ns, "f32",
                              "MXFP4 E2M1 block-32 quantize, X[8192,4096] bf16 (config 3)"))
        if want("mxfp8_dequant"):
            cases.append(Case("mxfp8_dequant", "hbm", R * C * 2 + R * C + R * C // 32, "B", mk_mxd(0, el8), ns, "f32",
                              "MXFP8 dequantize to bf16"))
        if want("hif8_encode"):
            cases.append(Case("hif8_encode", "hbm", R * C * 3, "B", hif_enc, ns, "u8", "HiFloat8 encode, X[8192,4096] bf16 (config 3)"))
        if want("hif8_decode"):
            cases.append(Case("hif8_decode", "hbm", R * C * 3, "B", hif_dec, ns, "u8", "HiFloat8 decode to bf16"))

    # ---- K3: dynamic per-token int8, X[2048,4096] bf16 ----------------------------------------------
    if want("act_quant_per_token"):
        x4, _, _ = workloads.c4_w8a8()
        M4, K4 = x4.shape
        work = M4 * K4 * 2 + M4 * K4 + M4 * 4
        ns4 = 32
        xs4 = dev_copies(x4, ns4)
        q4 = [torch.empty(M4, K4, dtype=torch.int8, device=dev) for _ in range(ns4)]
        sc4 = [torch.empty(M4, dtype=torch.float32, device=dev) for _ in range(ns4)]

        def launch(i, xs4=xs4, q4=q4, sc4=sc4, M4=M4, K4=K4):
            j = i % len(xs4)
            rc = lib.amct_act_quant_per_token_int8(xs4[j].data_ptr(), None, q4[j].data_ptr(), sc4[j].data_ptr(), M4, K4, 0,
                                                   _lib.BF16, st)
            assert rc == 0, rc
        ns = ns4
        cases.append(Case("act_quant_per_token", "hbm", work, "B", launch, ns, "f32",
                          "dynamic per-token INT8 quantize, X[2048,4096] bf16 (config 4)"))

    # ---- column statistics over tokens (SmoothQuant calibration), X[8192,4096] bf16 ----------------------
    if want("col_minmax"):
        xc = workloads.c3_activations()
        Rc, Cc = xc.shape
        work = Rc * Cc * 2 + 2 * Cc * 4
        nsc2 = sets_for(work)
        xcs = dev_copies(xc, nsc2)
        cmx = torch.empty(Cc, dtype=torch.float32, device=dev)
        cmn = torch.empty(Cc, dtype=torch.float32, device=dev)
        wsb = lib.amct_col_minmax_workspace_bytes(Rc, Cc)
        wsc = torch.empty(wsb, dtype=torch.uint8, device=dev)

        def launch(i, xcs=xcs, cmx=cmx, cmn=cmn, wsc=wsc, wsb=wsb, Rc=Rc, Cc=Cc):
            rc = lib.amct_col_minmax(xcs[i % len(xcs)].data_ptr(), cmx.data_ptr(), cmn.data_ptr(), Rc, Cc, 0, 0, _lib.BF16,
                                     wsc.data_ptr(), wsb, st)
            assert rc == 0, rc
        cases.append(Case("col_minmax", "hbm", work, "B", launch, nsc2, "f32",
                          "per-channel max/min over tokens, X[8192,4096] bf16 (two kernels per call)"))

    # ---- GPTQ inner block: 128 columns of W[14336,4096] fp32, int4 asymmetric per-channel ----------------
    if want("gptq_block"):
        Ng, Kg, cnt = 14336, 4096, 128
        gq = torch.Generator().manual_seed(1013)
        wg = [(torch.randn(Ng, Kg, generator=gq) * 0.02).to(dev) for _ in range(2)]
        hq = torch.triu(torch.randn(cnt, cnt, generator=gq) * 0.05 + torch.eye(cnt)).to(dev).contiguous()
        sg = (torch.rand(Ng, generator=gq) * 0.01 + 0.002).to(dev)
        zg = torch.randint(-8, 8, (Ng,), generator=gq, dtype=torch.int32).to(dev)
        eg = torch.empty(Ng, cnt, dtype=torch.float32, device=dev)
        gi = torch.zeros(cnt, dtype=torch.int32, device=dev)
        work = Ng * cnt * 4 * 3 + cnt * cnt * 4

        def launch(i, wg=wg, hq=hq, sg=sg, zg=zg, eg=eg, gi=gi, Ng=Ng, Kg=Kg, cnt=cnt):
            # successive launches walk over the column blocks of two matrices: the data is not cache-resident
            wsel = wg[(i // 32) % 2]
            rc = lib.amct_gptq_block(wsel.data_ptr() + (i % 32) * cnt * 4, Kg, eg.data_ptr(), cnt, hq.data_ptr(), cnt,
                                     sg.data_ptr(), zg.data_ptr(), 1, gi.data_ptr(), Ng, cnt, -8, 7, st)
            assert rc == 0, rc
        cases.append(Case("gptq_block", "hbm", work, "B", launch, 2, "f32",
                          "GPTQ column loop of one 128-column block, W[14336,4096] fp32 (latency/ALU-bound: 128 dependent steps; bytes = block in, block and errors out)"))

    # ---- matrix-pipe yardsticks: register-only MFMA loop with pseudo-random operands, measured right before the
    # GEMMs they are the yardstick for (and behind the bandwidth-bound kernels, which they would only heat up)
    import ctypes
    for yname, bf, bound, ydesc in (("mfma_i8_yardstick", 0, "mfma_i8", "int8"), ("mfma_bf16_yardstick", 1, "mfma_bf16", "bf16")):
        if want(yname):
            sink = torch.zeros(1024, dtype=torch.int32, device=dev)
            iters = 1500 if bf else 2500
            ops_out = ctypes.c_int64(0)
            rc = lib.amct_mfma_yardstick(bf, 1, iters, sink.data_ptr(), ctypes.addressof(ops_out), st)   # also sets ops_out
            assert rc == 0, rc

            def launch(i, bf=bf, iters=iters, sink=sink, ops_out=ops_out):
                rc = lib.amct_mfma_yardstick(bf, 1, iters, sink.data_ptr(), ctypes.addressof(ops_out), st)
                assert rc == 0, rc
            cases.append(Case(yname, bound, ops_out.value, "OP", launch, 1, ydesc,
                              "register-only %s MFMA loop on every CU, pseudo-random operands (yardstick: what the "
                              "matrix pipe sustains under the power limit on such data)" % ydesc))

    # ---- the vendor library's GEMMs at the same shape (hipBLASLt through torch), as yardsticks of what tuned kernels
    # reach on this part and these operands: a plain bf16 x bf16 Linear (no dequantisation) and a plain int8 x int8
    # product (no rescale epilogue).  They are not part of the product.
    if want("lib_gemm_bf16"):
        xl = workloads.c5_w4a16(2048, 64, 4096)[0].to(dev)
        gl = torch.Generator().manual_seed(1021)
        wl = [(torch.randn(14336, 4096, generator=gl) * 0.02).to(torch.bfloat16).to(dev) for _ in range(4)]

        def launch(i, xl=xl, wl=wl):
            torch.nn.functional.linear(xl, wl[i % len(wl)])
        cases.append(Case("lib_gemm_bf16", "mfma_bf16", 2 * 2048 * 14336 * 4096, "flop", launch, 4, "bf16",
                          "torch.nn.functional.linear bf16 x bf16, M=2048 N=14336 K=4096 (vendor library yardstick)"))
    if want("lib_gemm_i8"):
        x6l, wq6l, _ = workloads.c4_w8a8()
        xql = ops.act_quant_per_token_int8(x6l.to(dev))[0]
        wql = [wq6l.to(dev).t()] + [wq6l.to(dev).clone().t() for _ in range(3)]

        def launch(i, xql=xql, wql=wql):
            torch._int_mm(xql, wql[i % len(wql)])
        cases.append(Case("lib_gemm_i8", "mfma_i8", 2 * 2048 * 14336 * 4096, "op", launch, 4, "int8",
                          "torch._int_mm int8 x int8 -> int32, M=2048 N=14336 K=4096 (vendor library yardstick)"))

    # ---- K6: W8A8 Linear, W[14336,4096] int8 ----------------------------------------------------------
    chain = {"w8a8_dynamic_m2048": 2048, "w8a8_dynamic_m16": 16}
    if want("w8a8_m2048") or want("w8a8_m16") or want("w8a8_linear_m16") or any(want(n) for n in chain):
        x6, wq6, sw6 = workloads.c4_w8a8()
        N6, K6 = wq6.shape
        nw = 6                                           # 6 x 58.7 MB of weights rotate through HBM
        wqs = dev_copies(wq6, nw)
        swd = sw6.to(dev)
        for name, M6 in (("w8a8_m2048", 2048), ("w8a8_m16", 16)):
            if not want(name):
                continue
            xq6, st6 = ops.act_quant_per_token_int8(x6[:M6].to(dev))
            outs = [torch.empty(M6, N6, dtype=torch.bfloat16, device=dev) for _ in range(nw)]

            def launch(i, xq6=xq6, st6=st6, outs=outs, M6=M6, wqs=wqs, swd=swd, N6=N6, K6=K6):
                j = i % len(wqs)
                rc = lib.amct_gemm_w8a8(xq6.data_ptr(), wqs[j].data_ptr(), st6.data_ptr(), swd.data_ptr(), None, 0,
                                        outs[j].data_ptr(), None, M6, N6, K6, _lib.BF16, st)
                assert rc == 0, rc
            if M6 >= 256:
                cases.append(Case(name, "mfma_i8", 2 * M6 * N6 * K6, "op", launch, nw, "int8",
                                  "W8A8 Linear M=%d N=14336 K=4096, per-token x per-channel rescale, bf16 out (config 4)" % M6))
            else:
                cases.append(Case(name, "hbm", N6 * K6 + M6 * K6 + M6 * N6 * 2 + N6 * 4 + M6 * 4, "B", launch, nw, "int8",
                                  "W8A8 Linear M=%d (decode): weight streaming (config 4)" % M6))

        # the deploy module's forward for 16 rows in one call: the static per-tensor quantisation of the bf16 activations
        # (npu_quantize) done inside the weight-streaming kernel while it stages them, then the Linear
        if want("w8a8_linear_m16"):
            ML = 16
            xl = x6[:ML].to(dev)
            asc = torch.full((1,), 24.0, dtype=torch.bfloat16, device=dev)
            azp = torch.zeros(1, dtype=torch.bfloat16, device=dev)
            outs_l = [torch.empty(ML, N6, dtype=torch.bfloat16, device=dev) for _ in range(nw)]

            def launch(i, xl=xl, asc=asc, azp=azp, outs_l=outs_l, ML=ML, wqs=wqs, swd=swd, N6=N6, K6=K6):
                j = i % len(wqs)
                rc = lib.amct_linear_w8a8(xl.data_ptr(), _lib.BF16, None, asc.data_ptr(), azp.data_ptr(), 1, 0, wqs[j].data_ptr(), None,
                                          swd.data_ptr(), None, 0, outs_l[j].data_ptr(), ML, N6, K6, _lib.BF16, None, 0, st)
                assert rc == 0, rc
            cases.append(Case("w8a8_linear_m16", "hbm", N6 * K6 + ML * K6 * 2 + ML * N6 * 2 + N6 * 4, "B", launch, nw, "int8",
                              "static activation quantisation + W8A8 Linear M=16 in one launch (decode, config 4): bf16 x "
                              "quantised while the weight-streaming kernel stages it"))

        # config 4 as the deployed module runs it with dynamic activation quantisation: K3 (per-token scales and codes
        # of the bf16 activations) and K6 back to back on one stream, two launches per step.  (Quantising inside the
        # GEMM would repeat K3's arithmetic in every one of the 56 / 224 blocks that share a row.)
        for name, M6 in chain.items():
            if not want(name):
                continue
            xb6 = x6[:M6].contiguous().to(dev)
            xq6 = torch.empty(M6, K6, dtype=torch.int8, device=dev)
            st6 = torch.empty(M6, dtype=torch.float32, device=dev)
            outs = [torch.empty(M6, N6, dtype=torch.bfloat16, device=dev) for _ in range(nw)]

            def launch(i, xb6=xb6, xq6=xq6, st6=st6, outs=outs, M6=M6, wqs=wqs, swd=swd, N6=N6, K6=K6):
                j = i % len(wqs)
                rc = lib.amct_act_quant_per_token_int8(xb6.data_ptr(), None, xq6.data_ptr(), st6.data_ptr(), M6, K6, 0, _lib.BF16, st)
                assert rc == 0, rc
                rc = lib.amct_gemm_w8a8(xq6.data_ptr(), wqs[j].data_ptr(), st6.data_ptr(), swd.data_ptr(), None, 0,
                                        outs[j].data_ptr(), None, M6, N6, K6, _lib.BF16, st)
                assert rc == 0, rc
            if M6 >= 256:
                cases.append(Case(name, "mfma_i8", 2 * M6 * N6 * K6, "op", launch, nw, "int8",
                                  "dynamic per-token quantise + W8A8 Linear, M=%d, two launches (config 4 as deployed)" % M6))
            else:
                cases.append(Case(name, "hbm", N6 * K6 + M6 * K6 * 2 + M6 * N6 * 2 + N6 * 4, "B", launch, nw, "int8",
                                  "dynamic per-token quantise + W8A8 Linear, M=%d (decode), two launches" % M6))

    # ---- K7: W4A16 Linear, W[14336,4096] int4 g128 ------------------------------------------------------
    if want("w4a16_m2048") or want("w4a16_m2048_fused") or want("w4a16_m16") or want("w4a16_m1"):
        x7, codes7, sc7, z7, smr7 = workloads.c5_w4a16(2048)
        N7, K7 = codes7.shape
        g7 = 128
        nw7 = 12                                         # 12 x 29.4 MB of packed weights rotate
        pk7 = dev_copies(workloads.pack_nibbles(codes7), nw7)
        scd, zd, smd = sc7.to(dev), z7.to(dev), smr7.to(dev)
        for name, M7 in (("w4a16_m2048", 2048), ("w4a16_m2048_fused", 2048), ("w4a16_m16", 16), ("w4a16_m1", 1)):
            if not want(name):
                continue
            fused = name.endswith("_fused")
            xd = x7[:M7].contiguous().to(dev)
            outs7 = [torch.empty(M7, N7, dtype=torch.bfloat16, device=dev) for _ in range(nw7)]
            # the workspace the library asks for: the smoothed activations and, from 1025 rows on, the 16-bit weight
            # (the fused form: only the smoothed activations, M * K * 2 bytes -- the library then dequantises inside every tile)
            ws7 = torch.empty(M7 * K7 * 2 if fused else max(16, lib.amct_gemm_w4a16_workspace_bytes(M7, N7, K7, g7, 1)),
                              dtype=torch.uint8, device=dev)

            def launch(i, xd=xd, outs7=outs7, M7=M7, pk7=pk7, scd=scd, zd=zd, smd=smd, N7=N7, K7=K7, g7=g7, ws7=ws7):
                j = i % len(pk7)
                rc = lib.amct_gemm_w4a16(xd.data_ptr(), smd.data_ptr(), pk7[j].data_ptr(), scd.data_ptr(), _lib.F16,
                                         zd.data_ptr(), None, outs7[j].data_ptr(), M7, N7, K7, g7, _lib.BF16,
                                         ws7.data_ptr(), ws7.numel(), st)
                assert rc == 0, rc
            wbytes = N7 * K7 // 2 + N7 * (K7 // g7) * 3
            if fused:
                cases.append(Case(name, "mfma_bf16", 2 * M7 * N7 * K7, "flop", launch, nw7, "bf16",
                                  "W4A16 Linear M=%d N=14336 K=4096, group 128, with smoothing (config 5), dequantisation FUSED into the "
                                  "GEMM's main loop (the form a call without the 117 MB weight workspace takes): smoothing pre-pass "
                                  "(smooth_rows) + w4a16_tile_wide16 on 256x256 tiles" % M7))
            elif M7 >= 256:
                cases.append(Case(name, "mfma_bf16", 2 * M7 * N7 * K7, "flop", launch, nw7, "bf16",
                                  "W4A16 Linear M=%d N=14336 K=4096, group 128, with smoothing (config 5), as ops.gemm_w4a16 runs it: two "
                                  "launches -- w4_dequant_rows (the weight dequantised once into the lent workspace, the activations "
                                  "smoothed by the same launch) + the 16-bit GEMM w8a8_tile_mix16<bf16> on 256x256 / 256x192 tiles" % M7))
            else:
                cases.append(Case(name, "hbm", wbytes + M7 * K7 * 2 + M7 * N7 * 2, "B", launch, nw7, "bf16",
                                  "W4A16 Linear M=%d (decode): weight streaming (config 5)" % M7))
    # ---- int8 weight-only Linear (W8A16), W[14336,4096] int8 per-channel, bf16 activations, M = 16 ------------------
    if want("w8a16_m16"):
        x9 = workloads.c5_w4a16(2048)[0][:16].contiguous().to(dev)
        g9 = torch.Generator().manual_seed(1033)
        N9, K9 = 14336, 4096
        w9 = dev_copies(torch.randint(-128, 128, (N9, K9), generator=g9, dtype=torch.int16).to(torch.int8), 6)
        s9 = (1e-3 + 9e-3 * torch.rand(N9, 1, generator=g9)).to(torch.bfloat16).to(dev)
        outs9 = [torch.empty(16, N9, dtype=torch.bfloat16, device=dev) for _ in range(6)]

        def launch(i, x9=x9, w9=w9, s9=s9, outs9=outs9, N9=N9, K9=K9):
            j = i % len(w9)
            rc = lib.amct_gemm_w8a16(x9.data_ptr(), None, w9[j].data_ptr(), s9.data_ptr(), _lib.BF16, None, None,
                                     outs9[j].data_ptr(), 16, N9, K9, K9, _lib.BF16, st)
            assert rc == 0, rc
        cases.append(Case("w8a16_m16", "hbm", N9 * K9 + 16 * K9 * 2 + 16 * N9 * 2 + N9 * 2, "B", launch, 6, "bf16",
                          "int8 weight-only Linear M=16 N=14336 K=4096, per-channel scales, bf16 activations (decode): weight streaming"))

    # ---- the three Linears on a down-projection shape, W[4096,14336] at M = 16: few column blocks and long rows, so the
    # tile kernels split K over blocks (partial sums in the lent workspace, a second kernel adds them)
    if want("w8a8_down_m16") or want("w4a16_down_m16") or want("w8a16_down_m16"):
        Nd, Kd, Md, gd = 4096, 14336, 16, 128
        gen = torch.Generator().manual_seed(2031)
        nwd = 8                                          # 8 x 58.7 MB (int8) / 29.4 MB (int4) of weights rotate
        xd16 = (torch.randn(Md, Kd, generator=gen) * 0.5).to(torch.bfloat16).to(dev)
        wd8 = dev_copies(torch.randint(-128, 128, (Nd, Kd), generator=gen, dtype=torch.int16).to(torch.int8), nwd)
        if want("w8a8_down_m16"):
            xqd = torch.randint(-128, 128, (Md, Kd), generator=gen, dtype=torch.int16).to(torch.int8).to(dev)
            stk = (0.01 + torch.rand(Md, generator=gen)).to(dev)
            sch = (1e-3 + 9e-3 * torch.rand(Nd, generator=gen)).to(dev)
            outs_d = [torch.empty(Md, Nd, dtype=torch.bfloat16, device=dev) for _ in range(nwd)]
            wsd = torch.empty(max(16, lib.amct_gemm_w8a8_workspace_bytes(Md, Nd, Kd)), dtype=torch.uint8, device=dev)

            def launch(i, xqd=xqd, wd8=wd8, stk=stk, sch=sch, outs_d=outs_d, wsd=wsd):
                j = i % len(wd8)
                rc = lib.amct_gemm_w8a8_ws(xqd.data_ptr(), wd8[j].data_ptr(), stk.data_ptr(), sch.data_ptr(), None, 0,
                                           outs_d[j].data_ptr(), None, Md, Nd, Kd, _lib.BF16, wsd.data_ptr(), wsd.numel(), st)
                assert rc == 0, rc
            cases.append(Case("w8a8_down_m16", "hbm", Nd * Kd + Md * Kd + Md * Nd * 2 + Nd * 4 + Md * 4, "B", launch, nwd, "int8",
                              "W8A8 Linear M=16 N=4096 K=14336 (down projection, decode): 64x64 tiles, K split over 4 blocks per tile, "
                              "int32 partial sums + reduce kernel"))
        if want("w4a16_down_m16"):
            pkd = dev_copies(torch.randint(0, 256, (Nd, Kd // 2), generator=gen, dtype=torch.int16).to(torch.uint8), nwd)
            scd4 = (1e-3 + 9e-3 * torch.rand(Nd, Kd // gd, generator=gen)).to(torch.float16).to(dev)
            zd4 = torch.randint(0, 16, (Nd, Kd // gd), generator=gen, dtype=torch.int16).to(torch.uint8).to(dev)
            outs_d4 = [torch.empty(Md, Nd, dtype=torch.bfloat16, device=dev) for _ in range(nwd)]
            wsd4 = torch.empty(max(16, lib.amct_gemm_w4a16_workspace_bytes(Md, Nd, Kd, gd, 0)), dtype=torch.uint8, device=dev)

            def launch(i, pkd=pkd, scd4=scd4, zd4=zd4, outs_d4=outs_d4, wsd4=wsd4, xd16=xd16):
                j = i % len(pkd)
                rc = lib.amct_gemm_w4a16(xd16.data_ptr(), None, pkd[j].data_ptr(), scd4.data_ptr(), _lib.F16, zd4.data_ptr(), None,
                                         outs_d4[j].data_ptr(), Md, Nd, Kd, gd, _lib.BF16, wsd4.data_ptr(), wsd4.numel(), st)
                assert rc == 0, rc
            cases.append(Case("w4a16_down_m16", "hbm", Nd * Kd // 2 + Nd * (Kd // gd) * 3 + Md * Kd * 2 + Md * Nd * 2, "B", launch, nwd, "bf16",
                              "W4A16 Linear M=16 N=4096 K=14336 (down projection, decode): weight-streaming kernel on 7 slices of 2048 "
                              "elements of K, fp32 partial sums + reduce kernel"))
        if want("w8a16_down_m16"):
            scd8 = (1e-3 + 9e-3 * torch.rand(Nd, Kd // gd, generator=gen)).to(torch.bfloat16).to(dev)
            outs_d8 = [torch.empty(Md, Nd, dtype=torch.bfloat16, device=dev) for _ in range(nwd)]
            wsd8 = torch.empty(max(16, lib.amct_gemm_w8a16_workspace_bytes(Md, Nd, Kd, gd, 0)), dtype=torch.uint8, device=dev)

            def launch(i, wd8=wd8, scd8=scd8, outs_d8=outs_d8, wsd8=wsd8, xd16=xd16):
                j = i % len(wd8)
                rc = lib.amct_gemm_w8a16_ws(xd16.data_ptr(), None, wd8[j].data_ptr(), scd8.data_ptr(), _lib.BF16, None, None,
                                            outs_d8[j].data_ptr(), Md, Nd, Kd, gd, _lib.BF16, wsd8.data_ptr(), wsd8.numel(), st)
                assert rc == 0, rc
            cases.append(Case("w8a16_down_m16", "hbm", Nd * Kd + Nd * (Kd // gd) * 2 + Md * Kd * 2 + Md * Nd * 2, "B", launch, nwd, "bf16",
                              "int8 weight-only Linear M=16 N=4096 K=14336 group 128 (down projection, decode): weight-streaming kernel on "
                              "7 slices of 2048 elements of K, fp32 partial sums + reduce kernel"))

    # ---- the same operator at M = 2048: dequantise the weight once into the lent workspace, then the 16-bit GEMM on the
    # large tiles (three launches with smoothing)
    if want("w8a16_m2048"):
        x10 = workloads.c5_w4a16(2048)[0].contiguous().to(dev)
        sm10 = workloads.c5_w4a16(2048)[4].to(dev)
        g10 = torch.Generator().manual_seed(1033)
        N10, K10 = 14336, 4096
        w10 = dev_copies(torch.randint(-128, 128, (N10, K10), generator=g10, dtype=torch.int16).to(torch.int8), 6)
        s10 = (1e-3 + 9e-3 * torch.rand(N10, K10 // 128, generator=g10)).to(torch.float16).to(dev)
        z10 = torch.randint(-128, 128, (N10, K10 // 128), generator=g10, dtype=torch.int16).to(torch.int8).to(dev)
        outs10 = [torch.empty(2048, N10, dtype=torch.bfloat16, device=dev) for _ in range(6)]
        ws10 = torch.empty(lib.amct_gemm_w8a16_workspace_bytes(2048, N10, K10, 128, 1), dtype=torch.uint8, device=dev)

        def launch(i, x10=x10, sm10=sm10, w10=w10, s10=s10, z10=z10, outs10=outs10, ws10=ws10, N10=N10, K10=K10):
            j = i % len(w10)
            rc = lib.amct_gemm_w8a16_ws(x10.data_ptr(), sm10.data_ptr(), w10[j].data_ptr(), s10.data_ptr(), _lib.F16, z10.data_ptr(),
                                        None, outs10[j].data_ptr(), 2048, N10, K10, 128, _lib.BF16, ws10.data_ptr(), ws10.numel(), st)
            assert rc == 0, rc
        cases.append(Case("w8a16_m2048", "mfma_bf16", 2 * 2048 * N10 * K10, "flop", launch, 6, "bf16",
                          "int8 weight-only Linear M=2048 N=14336 K=4096, group-128 scales and offsets, smoothing: dequantise "
                          "into the workspace + smoothing pre-pass + 16-bit GEMM on the 256x256 tiles"))

    # ---- GPTQ Hessian accumulation: H[4096,4096] fp32 <- beta H + alpha X^T X, X[2048,4096] bf16 ------------------
    # (after everything else: it heats the part like the GEMMs do).  Work = the multiply-adds of the lower triangle
    # with its diagonal, which is what a symmetric update needs; the library path beside it is the reference's
    # sequence on the device (scale H, scale x in fp32, fp32 matmul, add).
    if want("gptq_hessian_update") or want("lib_hessian_update_fp32"):
        import math
        Th, Ch = 2048, 4096
        gh = torch.Generator().manual_seed(1031)
        xh = [torch.randn(Th, Ch, generator=gh).to(torch.bfloat16).to(dev) for _ in range(4)]
        hh = [torch.zeros(Ch, Ch, dtype=torch.float32, device=dev) for _ in range(4)]
        wsh = torch.empty(lib.amct_hessian_update_workspace_bytes(Th, Ch), dtype=torch.uint8, device=dev)
        work = 2 * Th * Ch * (Ch + 1) // 2
        if want("gptq_hessian_update"):
            def launch(i, xh=xh, hh=hh, wsh=wsh, Th=Th, Ch=Ch):
                j = i % len(xh)
                rc = lib.amct_hessian_update(hh[j].data_ptr(), xh[j].data_ptr(), Th, Ch, 0.5, 2.0 / 4096, _lib.BF16,
                                             wsh.data_ptr(), wsh.numel(), st)
                assert rc == 0, rc
            cases.append(Case("gptq_hessian_update", "mfma_bf16", work, "flop", launch, 4, "bf16",
                              "GPTQ Hessian update H[4096,4096] += X^T X, X[2048,4096] bf16 (transpose + symmetric MFMA kernel; "
                              "flops of the lower triangle)"))
        if want("lib_hessian_update_fp32"):
            def launch(i, xh=xh, hh=hh):
                j = i % len(xh)
                hh[j].mul_(0.5)
                xs = math.sqrt(2.0 / 4096) * xh[j].float().t()
                hh[j].add_(xs.matmul(xs.t()))
            cases.append(Case("lib_hessian_update_fp32", "mfma_bf16", work, "flop", launch, 4, "f32",
                              "the same update as the reference writes it, on the device with library calls (fp32 matmul); "
                              "same flop count as above for comparison"))
    return cases


def spin_up(dev):
    """Bring the GPU to its sustained clocks before anything is timed (about 30 ms of copies)."""
    import torch
    from amct_amd import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream(dev).cuda_stream
    a = torch.empty(64 << 20, dtype=torch.uint8, device=dev).fill_(3)
    b = torch.empty_like(a)
    for _ in range(1500):
        lib.amct_copy_bytes(a.data_ptr(), b.data_ptr(), a.numel(), st)
    torch.cuda.synchronize(dev)


def time_case(case, steps, warmup, dev, repeats):
    """`repeats` timed regions of exactly `steps` launches each, every region between two synchronizes (device time by
    events on the launch stream, host time from the first launch until the closing event reads complete); returns the median host time of a region, the median device time per launch and the latter for every region."""
    import torch
    for i in range(warmup):
        case.launch(i)
    torch.cuda.synchronize(dev)
    walls, devs = [], []
    idx = warmup
    for _ in range(repeats):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        t0 = time.perf_counter()
        for i in range(steps):
            case.launch(idx + i)
        e1.record()
        # The host clock stops when the event behind the last launch reads complete (polled: a blocking wait adds the
        # host's wake-up latency, and torch.cuda.synchronize costs 30 - 45 us on this runtime even when nothing is
        # pending -- a tenth of a region of 20 launches); the synchronize that closes the region follows.
        while not e1.query():
            pass
        t1 = time.perf_counter()
        torch.cuda.synchronize(dev)
        walls.append(t1 - t0)
        devs.append(e0.elapsed_time(e1) / steps)
        idx += steps
    return sorted(walls)[len(walls) // 2], sorted(devs)[len(devs) // 2], devs


def _timed(run, budget_s, min_runs=3, max_runs=400):
    run()
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < min_runs or (time.perf_counter() < t_end and len(times) < max_runs):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2], len(times)


def cpu_baselines(names):
    """The oracle's restatement of the reference's CPU path for each benchmark workload, timed on the host cores
    torch gives us (capped at 16) on a bounded sample of the same synthetic input; about 25 s in total.  Returns
    {kernel name: entry}; the entry of the headline kernel is also the line's top-level cpu_baseline."""
    import torch
    from amct_amd import workloads
    from oracle import deploy as od
    from oracle import hif8
    from oracle import int_quant as iq
    from oracle import mx
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    out = {}

    def entry(name, work, unit, run, sample, budget=1.2):
        if name not in names:
            return
        med, n = _timed(run, budget)
        scale = 1e9 if unit == "GB/s" else 1e12
        out[name] = {"value": round(work / med / scale, 4), "unit": unit, "cores": cores, "kind": "port",
                     "sample": "{}; median of {} runs, {:.1f} ms each".format(sample, n, med * 1e3)}

    rows = 2048
    w2 = workloads.c2_weight(rows, 4096)

    def k2():
        s, z = iq.weight_scale_offset(w2, 'group', False, 'int4', 128)
        codes = iq.quant_codes(w2, 'int4', s, z, 128).reshape(rows, -1)
        return od.pack_nibbles_k(codes), s.squeeze(-1).to(torch.float16), (z.squeeze(-1) + 8).to(torch.uint8)
    entry("int4_group_pack", rows * 4096 * 2 + rows * 4096 // 2 + rows * 32 * 3, "GB/s", k2,
          "first 2048 of 14336 rows of the config-2 weight", 6.0)

    w1 = workloads.c1_weight(1024, 4096)

    def k1():
        s, z = iq.weight_scale_offset(w1, 'channel', True, 'int8')
        return iq.fake_quant(w1, 'int8', s, z)
    entry("fakequant_int8", 1024 * 4096 * 8 + 1024 * 4, "GB/s", k1, "first 1024 of 4096 rows of the config-1 weight")

    r3 = 512
    x3 = workloads.c3_activations(r3, 4096)
    n3 = r3 * 4096
    entry("mxfp8_quant", n3 * 3 + n3 // 32, "GB/s", lambda: mx.mx_quant(x3, mx.E4M3), "first 512 of 8192 rows of the config-3 activations")
    entry("mxfp4_quant", n3 * 2 + n3 // 2 + n3 // 32, "GB/s", lambda: mx.mx_quant(x3, mx.E2M1), "first 512 of 8192 rows of the config-3 activations")
    el, sb = mx.mx_quant(x3, mx.E4M3)
    entry("mxfp8_dequant", n3 * 3 + n3 // 32, "GB/s", lambda: mx.mx_dequant(el, sb, mx.E4M3, torch.bfloat16),
          "first 512 of 8192 rows of the config-3 activations")
    x3n = x3[:128].float().numpy()
    entry("hif8_encode", 128 * 4096 * 3, "GB/s", lambda: hif8.encode_bruteforce(x3n), "first 128 of 8192 rows of the config-3 activations (nearest-code search)")
    c3 = hif8.encode_bruteforce(x3n)
    entry("hif8_decode", 128 * 4096 * 3, "GB/s", lambda: torch.from_numpy(hif8.decode(c3)).to(torch.bfloat16),
          "first 128 of 8192 rows of the config-3 activations")
    run_max, run_min = torch.full((1, 4096), -float("inf")), torch.full((1, 4096), float("inf"))
    entry("col_minmax", n3 * 2 + 2 * 4096 * 4, "GB/s",
          lambda: iq.channel_min_max_update(x3.float(), run_max, run_min), "first 512 of 8192 rows of the config-3 activations")

    x4, wq4, sw4 = workloads.c4_w8a8(2048, 14336, 4096)
    entry("act_quant_per_token", 2048 * 4096 * 3 + 2048 * 4, "GB/s", lambda: iq.dynamic_token_quant(x4), "the config-4 activations, whole")
    xq4, st4 = iq.dynamic_token_quant(x4)
    # the GEMMs: what the reference runs on a CPU (its stand-in operators: upcast, fp32 F.linear), rows sampled
    for name, m in (("w8a8_m2048", 256), ("w8a8_m16", 16)):
        if name not in names:
            continue
        xs, ss = xq4[:m].contiguous(), st4.reshape(-1)[:m].contiguous()
        entry(name, 2 * m * 14336 * 4096, "TOP/s",
              lambda xs=xs, ss=ss: od.cpu_standin_quant_matmul_f32(xs, wq4, sw4, ss, None, torch.bfloat16),
              "{} of the rows of config 4, all 14336 output channels, fp32 F.linear as the reference's CPU stand-in".format(m))

    if any(n in names for n in ("w4a16_m2048", "w4a16_m16", "w4a16_m1")):
        x5, codes5, sc5, z5, sm5 = workloads.c5_w4a16(256, 14336, 4096)
        signed5, anti5 = codes5.to(torch.int32) - 8, -(z5.to(torch.float32) - 8)
        for name, m in (("w4a16_m2048", 256), ("w4a16_m16", 16), ("w4a16_m1", 1)):
            if name not in names:
                continue
            xs = x5[:m].contiguous()
            entry(name, 2 * m * 14336 * 4096, "TFLOP/s",
                  lambda xs=xs: od.cpu_standin_weight_quant_matmul_f32(xs, signed5, sc5, anti5, 128, None, sm5.reshape(1, -1)),
                  "{} of the rows of config 5, all 14336 output channels, fp32 dequantise + F.linear as the reference's CPU stand-in".format(m))
    if "gptq_hessian_update" in names:
        from oracle import gptq as og
        th, ch = 512, 4096
        xh = torch.randn(th, ch, generator=torch.Generator().manual_seed(1031)).to(torch.bfloat16)
        hh = [None]

        def hess():
            hh[0], _ = og.update_hessian(hh[0], 4, xh, ch)
        entry("gptq_hessian_update", 2 * th * ch * (ch + 1) // 2, "TFLOP/s", hess,
              "512 of the 2048 tokens, all 4096 columns: the reference's update (scale, fp32 matmul, add) on the host; "
              "flops of the lower triangle as for the kernel")
    if any(n in names for n in ("w8a16_m2048", "w8a16_m16")):
        g9 = torch.Generator().manual_seed(1033)
        w9 = torch.randint(-128, 128, (14336, 4096), generator=g9, dtype=torch.int16).to(torch.int32)
        s9 = (1e-3 + 9e-3 * torch.rand(14336, 32, generator=g9)).to(torch.float16)
        z9 = torch.randint(-128, 128, (14336, 32), generator=g9, dtype=torch.int16).float()
        x9 = workloads.c5_w4a16(256, 64, 4096)[0]
        for name, m in (("w8a16_m2048", 256), ("w8a16_m16", 16)):
            if name not in names:
                continue
            xs = x9[:m].contiguous()
            entry(name, 2 * m * 14336 * 4096, "TFLOP/s",
                  lambda xs=xs: od.cpu_standin_weight_quant_matmul_f32(xs, w9, s9, -z9, 128, None, None),
                  "{} rows, all 14336 output channels of an int8 weight with group-128 factors, fp32 dequantise + F.linear as the "
                  "reference's CPU stand-in".format(m))
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    only = set(x for x in args.only.split(",") if x)
    if only:
        only.add("int4_group_pack")
    try:
        line = run(args, dev, only)
    finally:
        # never leave the process with kernels still queued, whatever went wrong above
        torch.cuda.synchronize(dev)
    print(json.dumps(line))


def run(args, dev, only):
    import torch
    cases = build_cases(dev, only)
    torch.cuda.synchronize(dev)
    spin_up(dev)
    repeats = max(1, args.repeats)
    results = {}
    head = None
    for c in cases:
        wall, ms, regions = time_case(c, args.steps, args.warmup, dev, repeats)
        rate = c.work / (ms * 1e-3) / 1e9 if c.bound == "hbm" else c.work / (ms * 1e-3) / 1e12
        peak = HBM_PEAK_GBS if c.bound == "hbm" else (PEAK_INT8_TOPS if c.bound == "mfma_i8" else PEAK_BF16_TFLOPS)
        traffic = MEASURED_TRAFFIC.get(c.name)
        results[c.name] = {"desc": c.desc, "us_per_launch": round(ms * 1e3, 2),
                           "us_per_launch_by_region": [round(r * 1e3, 2) for r in regions], "achieved": round(rate, 1),
                           "unit": "GB/s" if c.bound == "hbm" else ("TOP/s" if c.bound == "mfma_i8" else "TFLOP/s"), "peak": peak,
                           "frac": round(rate / peak, 4), "work_per_launch": c.work, "sets": c.nsets, "dtype": c.dtype,
                           "traffic": traffic[1] if traffic else None, "traffic_kernel": traffic[0] if traffic else None}
        if c.name == "int4_group_pack":
            head = (c, wall, ms)
    # GEMM figures also as a fraction of what the register-only MFMA loop sustains on random operands
    for name, r in results.items():
        y = {"TOP/s": "mfma_i8_yardstick", "TFLOP/s": "mfma_bf16_yardstick"}.get(r["unit"])
        if y and y in results and name != y:
            r["frac_of_yardstick"] = round(r["achieved"] / results[y]["achieved"], 4)
        lib = {"TOP/s": "lib_gemm_i8", "TFLOP/s": "lib_gemm_bf16"}.get(r["unit"])
        if lib and lib in results and not name.startswith(("lib_gemm", "mfma_", "lib_hessian", "gptq_hessian")):
            r["vs_vendor_library"] = round(r["achieved"] / results[lib]["achieved"], 4)
    if "gptq_hessian_update" in results and "lib_hessian_update_fp32" in results:
        results["gptq_hessian_update"]["vs_vendor_library"] = round(
            results["lib_hessian_update_fp32"]["us_per_launch"] / results["gptq_hessian_update"]["us_per_launch"], 4)
        results["gptq_hessian_update"].pop("frac_of_yardstick", None)
    c, wall, ms = head
    value = c.work * args.steps / wall / 1e9
    traffic = MEASURED_TRAFFIC.get("int4_group_pack")
    line = {
        "metric": "quantize GB/s (% of HBM peak); W8A8 & W4A16 linear TOPS (% of MFMA peak)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": c.dtype, "data": "synthetic",
        "config": {"workload": c.desc, "rotating_sets": c.nsets, "input_dtype": "bf16",
                   "timing": "median of {} regions of {} launches".format(repeats, args.steps)},
        "roofline": {"bound": "hbm", "achieved": round(c.work / (ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(c.work / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": traffic[1] if traffic else None,
                     "kernel": "int4_group_pack", "bytes_per_launch": c.work},
        "kernels": results,
    }
    if not args.no_cpu:
        base = cpu_baselines(set(results) | {"int4_group_pack"})
        line["cpu_baseline"] = base["int4_group_pack"]
        for name, entry in base.items():
            if name in results:
                results[name]["cpu_baseline"] = entry
    return line


if __name__ == "__main__":
    main()
