"""Edge cases of the C ABI on the device: empty inputs enqueue nothing and succeed, malformed calls come back
with the documented error code and leave the outputs untouched, single-element and single-group shapes agree
with the oracle."""
import pytest
import torch

from amct_amd import _lib, ops
from oracle import int_quant as iq
from oracle import hif8 as oh
from util import assert_bits_equal

pytestmark = pytest.mark.gpu

E_BADARG, E_UNSUPPORTED, E_ALIGN = -1, -2, -3


def _st(dev):
    return torch.cuda.current_stream(dev).cuda_stream


def test_empty_inputs_succeed(dev):
    e = torch.empty(0, 128, device=dev)
    dq, codes, s, z = ops.fakequant_int(e, 8, False, codes_kind=ops.CODES_I8)
    assert dq.shape == (0, 128) and codes.shape == (0, 128) and s.numel() == 0 and z.numel() == 0
    packed, sc, zr, _ = ops.quant_int4_group_pack(torch.empty(0, 256, dtype=torch.bfloat16, device=dev), 128)
    assert packed.shape == (0, 128) and sc.shape == (0, 2) and zr.shape == (0, 2)
    q, st = ops.act_quant_per_token_int8(torch.empty(0, 64, dtype=torch.bfloat16, device=dev))
    assert q.shape == (0, 64) and st.numel() == 0
    el, e8 = ops.mx_quant(torch.empty(0, 64, dtype=torch.bfloat16, device=dev), ops.MX_E4M3)
    assert el.numel() == 0 and e8.numel() == 0
    assert ops.hif8_encode(torch.empty(0, dtype=torch.bfloat16, device=dev)).numel() == 0
    out = ops.gemm_w8a8(torch.empty(0, 64, dtype=torch.int8, device=dev), torch.zeros(16, 64, dtype=torch.int8, device=dev),
                        torch.ones(16, device=dev))
    assert out.shape == (0, 16)
    out = ops.gemm_w4a16(torch.empty(0, 128, dtype=torch.bfloat16, device=dev),
                         torch.zeros(16, 64, dtype=torch.uint8, device=dev),
                         torch.ones(16, 1, dtype=torch.float16, device=dev),
                         torch.zeros(16, 1, dtype=torch.uint8, device=dev), 128)
    assert out.shape == (0, 16)
    torch.cuda.synchronize(dev)


def test_error_codes_leave_outputs_untouched(dev):
    lib = _lib.load()
    st = _st(dev)
    w = torch.randn(8, 256, device=dev).to(torch.bfloat16)
    packed = torch.full((8, 128), 0xAB, dtype=torch.uint8, device=dev)
    sc = torch.zeros(8, 2, dtype=torch.float16, device=dev)
    zr = torch.zeros(8, 2, dtype=torch.uint8, device=dev)
    # cols not a multiple of the group
    rc = lib.amct_quant_int4_group_pack(w.data_ptr(), packed.data_ptr(), sc.data_ptr(), _lib.F16, None, zr.data_ptr(),
                                        None, None, 0, 8, 256, 96, 0, _lib.BF16, st)
    assert rc == E_ALIGN
    # unknown dtype enum
    rc = lib.amct_quant_int4_group_pack(w.data_ptr(), packed.data_ptr(), sc.data_ptr(), _lib.F16, None, zr.data_ptr(),
                                        None, None, 0, 8, 256, 128, 0, 7, st)
    assert rc == E_BADARG
    # MX: cols must be a multiple of 32; misaligned input pointer
    x = torch.randn(4, 96, device=dev).to(torch.bfloat16)
    el = torch.zeros(4, 96, dtype=torch.uint8, device=dev)
    e8 = torch.zeros(4, 3, dtype=torch.uint8, device=dev)
    assert lib.amct_mx_quant(x.data_ptr(), el.data_ptr(), e8.data_ptr(), 4, 80, 0, 0, _lib.BF16, st) == E_ALIGN
    assert lib.amct_mx_quant(x.data_ptr() + 2, el.data_ptr(), e8.data_ptr(), 4, 64, 0, 0, _lib.BF16, st) == E_ALIGN
    assert lib.amct_mx_quant(x.data_ptr(), el.data_ptr(), e8.data_ptr(), 4, 96, 5, 0, _lib.BF16, st) == E_BADARG
    # GEMMs: K not a multiple of the group / odd K; bad bias kind
    xa = torch.randn(4, 96, device=dev).to(torch.bfloat16)
    out = torch.zeros(4, 16, dtype=torch.bfloat16, device=dev)
    wq = torch.zeros(16, 48, dtype=torch.uint8, device=dev)
    s16 = torch.ones(16, 1, dtype=torch.float16, device=dev)
    z8 = torch.zeros(16, 1, dtype=torch.uint8, device=dev)
    rc = lib.amct_gemm_w4a16(xa.data_ptr(), None, wq.data_ptr(), s16.data_ptr(), _lib.F16, z8.data_ptr(), None,
                             out.data_ptr(), 4, 16, 96, 64, _lib.BF16, None, 0, st)
    assert rc == E_ALIGN
    xq = torch.zeros(4, 64, dtype=torch.int8, device=dev)
    w8 = torch.zeros(16, 64, dtype=torch.int8, device=dev)
    sch = torch.ones(16, device=dev)
    rc = lib.amct_gemm_w8a8(xq.data_ptr(), w8.data_ptr(), None, sch.data_ptr(), None, 3, out.data_ptr(), None,
                            4, 16, 64, _lib.BF16, st)
    assert rc == E_BADARG
    torch.cuda.synchronize(dev)
    assert bool((packed == 0xAB).all()) and bool((el == 0).all()) and bool((out == 0).all())
    assert b"align" in lib.amct_hip_strerror(E_ALIGN).lower() or len(lib.amct_hip_strerror(E_ALIGN)) > 0


def test_single_element_and_single_group(dev):
    # one element: max == min; symmetric scale = |w| / scope, code = +-scope; asymmetric clamps to zero first
    for val in (0.75, -0.75, 0.0):
        w = torch.tensor([[val]], dtype=torch.float32)
        for sym in (True, False):
            s, z = iq.weight_scale_offset(w, 'channel', sym, 'int8')
            dq, codes, gs, gz = ops.fakequant_int(w.to(dev), 8, sym, codes_kind=ops.CODES_I32)
            assert_bits_equal(gs.cpu().reshape(s.shape), s, "scale")
            if not sym:
                assert torch.equal(gz.cpu().reshape(z.shape), z)
            assert_bits_equal(dq.cpu(), iq.fake_quant(w, 'int8', s, z), "dq")
            assert torch.equal(codes.cpu(), iq.quant_codes(w, 'int8', s, z).to(torch.int32))
    # one group of 32 in one row through the packing kernel
    g = torch.Generator().manual_seed(77)
    w = (torch.randn(1, 32, generator=g) * 0.05).to(torch.bfloat16)
    packed, sc, zr, s32 = ops.quant_int4_group_pack(w.to(dev), 32, want_scales32=True)
    s, z = iq.weight_scale_offset(w, 'group', False, 'int4', 32)
    assert_bits_equal(s32.cpu().reshape(-1), s.reshape(-1), "scale32")
    codes = iq.quant_codes(w, 'int4', s, z, 32).reshape(1, 32).to(torch.int32) + 8
    lo, hi = packed.cpu().to(torch.int32) & 15, packed.cpu().to(torch.int32) >> 4
    assert torch.equal(torch.stack([lo, hi], dim=-1).reshape(1, 32), codes)
    # HiFloat8: a single scalar and the 7 elements of a ragged tail
    x = torch.tensor([3.3, -0.0, 1e-9, 7e4, float('nan'), -2.5, 0.11], dtype=torch.bfloat16)
    got = ops.hif8_encode(x.to(dev)).cpu()
    want = oh.encode_bruteforce(x.float().numpy())
    assert torch.equal(got, torch.as_tensor(want).to(torch.uint8).reshape(-1))


def test_mfma_yardstick_counts_its_operations(dev):
    """The measurement aid of bench.py: one block of 8 waves per CU, 8 MFMAs per wave and iteration; the operation count
    it reports follows from that, a zero-iteration call enqueues nothing, a null sink is refused."""
    import ctypes
    lib = _lib.load()
    sink = torch.zeros(1024, dtype=torch.int32, device=dev)
    ops_out = ctypes.c_int64(-1)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    for bf, per_mfma in ((0, 65536), (1, 32768)):
        for rnd in (0, 1):
            assert lib.amct_mfma_yardstick(bf, rnd, 3, sink.data_ptr(), ctypes.addressof(ops_out), _st(dev)) == 0
            assert ops_out.value == cus * 8 * 8 * 3 * per_mfma
    assert lib.amct_mfma_yardstick(0, 1, 0, sink.data_ptr(), ctypes.addressof(ops_out), _st(dev)) == 0 and ops_out.value == 0
    assert lib.amct_mfma_yardstick(0, 1, 3, None, ctypes.addressof(ops_out), _st(dev)) == E_BADARG
    torch.cuda.synchronize(dev)
    assert int(sink.abs().sum()) == 0                      # the sink is never written in practice
