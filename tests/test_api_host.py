"""Host-side behaviour of the reference-shaped API that needs no GPU: argument checks raise the
reference's exception types and messages before any kernel is launched."""
import pytest
import torch

from amct_amd.quantize_op import utils as qutils
from amct_amd.utils import data_utils, quant_util


def test_shape_checks_and_messages():
    w = torch.zeros(8, 64)
    with pytest.raises(RuntimeError, match=r"smooth_factor shape should be \[1, 64\] current shape is \[64\]"):
        quant_util.apply_smooth_weight(torch.ones(64), w)
    with pytest.raises(RuntimeError, match=r"AWQ params scale.shape should be \[1, 64\] current shape is \[1, 32\]"):
        quant_util.apply_awq_quantize_weight(w, torch.ones(1, 32), 32)
    with pytest.raises(ValueError, match="Not supported quant_dtype int2"):
        quant_util.convert_dtype(w, 'int2')
    with pytest.raises(ValueError, match="Not supported quant_dtype int16"):
        quant_util.quant_weight(w, 'int16', torch.ones(8, 1))
    with pytest.raises(RuntimeError, match="Linear quant only support dim from 2 to 6"):
        data_utils.check_linear_input_dim(torch.zeros(4))
    with pytest.raises(RuntimeError, match="Linear quant only support dim from 2 to 6"):
        data_utils.check_linear_input_dim(torch.zeros(1, 1, 1, 1, 1, 1, 4))
    data_utils.check_linear_input_dim(torch.zeros(2, 3, 4))
    with pytest.raises(RuntimeError, match="only support float32/float16/bfloat16"):
        data_utils.convert_precision(torch.zeros(4, 4, dtype=torch.float64), 'int8')


def test_check_scale_offset_shape():
    w = torch.zeros(8, 70)
    quant_util.check_scale_offset_shape(w, torch.ones(1))
    quant_util.check_scale_offset_shape(w, torch.ones(8, 1))
    with pytest.raises(RuntimeError, match="scale.shape should be equal to 1 or cout. current is 3"):
        quant_util.check_scale_offset_shape(w, torch.ones(3, 1))
    quant_util.check_scale_offset_shape(w, torch.ones(8, 3, 1), torch.ones(8, 3, 1), 32)
    with pytest.raises(RuntimeError, match="scale.shape should be"):
        quant_util.check_scale_offset_shape(w, torch.ones(8, 2, 1), None, 32)
    with pytest.raises(RuntimeError, match="offset_w.shape should be equal to scale_w.shape"):
        quant_util.check_scale_offset_shape(w, torch.ones(8, 3, 1), torch.ones(8, 3), 32)


def test_layout_helpers_match_oracle():
    from oracle import int_quant as iq
    w = torch.arange(3 * 40, dtype=torch.float32).reshape(3, 40)
    g = quant_util.convert_to_per_group_shape(w, 32)
    assert torch.equal(g, iq.group_view(w, 32)) and g.shape == (3, 2, 32)
    assert torch.equal(qutils.convert_to_dst_shape(g, w.shape), w)
    assert quant_util.pad_zero_by_group(w, 32).shape == (3, 64)
    assert qutils.get_int_quant_scope('int8', False) == 255
    assert qutils.get_int_quant_scope('int4', True, torch.tensor([True, False])).tolist() == [8, 7]


def test_check_scale_offset_messages():
    with pytest.raises(RuntimeError, match="Param scale has invalid value inf, nan or zeros!"):
        qutils.check_scale_offset(torch.tensor([0.0]), None)
    with pytest.raises(RuntimeError, match="Param offset has invalid value inf or nan!"):
        qutils.check_scale_offset(torch.tensor([1.0]), torch.tensor([float('inf')]))


def test_compressed_tensors_config_matches_the_fixture():
    """The quantization_config block of a converted checkpoint (experimental/.../deploy.py:171-238) against
    expected dictionaries written out by hand in tests/golden/quant_config_kat.json."""
    import json
    import os
    from amct_amd import interchange as ic
    kat = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "quant_config_kat.json")))
    assert ic.generate_ignore_item(3, 2, 1) == kat["ignore_3_2_1"]
    assert ic.generate_w4a8_quant(3, 1) == kat["w4a8_3_1"]
    assert ic.generate_quant_config(True, ["lm_head"], w4a8=True, clip=True) == kat["config_c8_w4a8_clip"]
    plain = ic.generate_quant_config(False, [])
    assert plain["kv_cache_scheme"] is None and list(plain["config_groups"]) == ["group_0"]
    assert json.loads(json.dumps(plain)) == plain          # serialisable as written


def test_operand_sizes_are_checked_before_any_launch():
    """The kernels only see pointers: every factor / bias / scale length they rely on is verified on the host and
    raises before a device is touched (so CPU tensors are enough to show it)."""
    import pytest
    import torch
    from amct_amd import ops, torch_hip
    w = torch.zeros(8, 64)
    with pytest.raises(RuntimeError, match="scale has 7 entries"):
        ops.quant_with_params(w, torch.ones(7), None, 0, -128, 127)
    with pytest.raises(RuntimeError, match="scale has 8 entries"):
        ops.quant_with_params(w, torch.ones(8), None, 32, -8, 7)
    with pytest.raises(RuntimeError, match="offset has 3 entries"):
        ops.quant_with_params(w, torch.ones(16), torch.zeros(3, dtype=torch.int32), 32, -8, 7)
    with pytest.raises(RuntimeError, match="column scale has 63 entries"):
        ops.quant_with_params(w, torch.ones(8), None, 0, -128, 127, col_scale=torch.ones(63), col_mode=ops.COL_MUL)
    with pytest.raises(RuntimeError, match="column scale has 65 entries"):
        ops.fakequant_int(w, 8, True, col_scale=torch.ones(65), col_mode=ops.COL_MUL)
    with pytest.raises(RuntimeError, match="column scale"):
        ops.quant_int4_group_pack(w, 32, col_scale=torch.ones(1), col_mode=ops.COL_MUL)
    xq = torch.zeros(6, 64, dtype=torch.int8)
    wq = torch.zeros(16, 64, dtype=torch.int8)
    with pytest.raises(RuntimeError, match="15 channel scales"):
        ops.gemm_w8a8(xq, wq, torch.ones(15))
    with pytest.raises(RuntimeError, match="4 token scales for 6 rows"):
        ops.gemm_w8a8(xq, wq, torch.ones(16), s_tok=torch.ones(4))
    with pytest.raises(RuntimeError, match="bias has 17 entries"):
        ops.gemm_w8a8(xq, wq, torch.ones(16), bias=torch.zeros(17))
    # the operator level repeats a per-token scale over leading batch dims only when it divides evenly
    with pytest.raises(RuntimeError, match="token scales"):
        torch_hip.npu_quant_matmul(xq, wq.t(), torch.ones(16), pertoken_scale=torch.ones(4))
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    wp = torch.zeros(16, 32, dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="scales have shape"):
        ops.gemm_w4a16(x, wp, torch.ones(16, 1, dtype=torch.float16), torch.zeros(16, 2, dtype=torch.uint8), 32)
    with pytest.raises(RuntimeError, match="zero-points have shape"):
        ops.gemm_w4a16(x, wp, torch.ones(16, 2, dtype=torch.float16), torch.zeros(16, 1, dtype=torch.uint8), 32)
    with pytest.raises(RuntimeError, match="smooth factor has 10 entries"):
        ops.gemm_w4a16(x, wp, torch.ones(16, 2, dtype=torch.float16), torch.zeros(16, 2, dtype=torch.uint8), 32,
                       smooth=torch.ones(10, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="bias has 3 entries"):
        ops.gemm_w4a16(x, wp, torch.ones(16, 2, dtype=torch.float16), torch.zeros(16, 2, dtype=torch.uint8), 32,
                       bias=torch.zeros(3))
    with pytest.raises(RuntimeError, match="MX elements have shape"):
        ops.mx_dequant(torch.zeros(4, 60, dtype=torch.uint8), torch.zeros(4, 2, dtype=torch.uint8), ops.MX_E4M3)
    with pytest.raises(RuntimeError, match="col_max must be"):
        ops.col_minmax(torch.zeros(4, 64), col_max=torch.zeros(63))


def test_layout_cache_hits_for_any_number_of_layers_and_dies_with_its_sources():
    """The operand cache of npu_weight_quant_batchmatmul (host logic only: CPU tensors, a counting converter): a model of
    more layers than any fixed capacity, walked in the same order twice, converts every layer once; a version bump
    converts again and replaces the old entry; freeing a source drops its entry at once; a byte cap evicts the least
    recently used entry."""
    import gc
    import torch
    from amct_amd.torch_hip import _LayoutCache
    cache = _LayoutCache()
    layers = [(torch.zeros(4, 8, dtype=torch.int8), torch.ones(1, 8), None) for _ in range(600)]
    made = []

    def walk():
        for i, t in enumerate(layers):
            cache.get(t, (0, torch.bfloat16), lambda i=i: (made.append(i), torch.zeros(8, 4))[1:])
    walk()
    walk()
    assert len(made) == 600 and cache.conversions == 600 and len(cache.entries) == 600
    # an in-place write that torch sees: converted again, the stale entry is gone
    layers[5][0].add_(1)
    walk()
    assert len(made) == 601 and made[-1] == 5 and len(cache.entries) == 600
    # the source is freed: no converted copy stays behind
    before = cache.bytes
    del layers[10:]
    gc.collect()
    assert len(cache.entries) == 10 and cache.bytes == before * 10 // 600
    # byte cap: the least recently used entry goes first
    small = _LayoutCache(max_bytes=3 * 8 * 4 * 4)
    keep = [(torch.zeros(2, 2), None, None) for _ in range(5)]
    for t in keep:
        small.get(t, 0, lambda: (torch.zeros(8, 4),))
    assert len(small.entries) == 3 and small.bytes == 3 * 128
    small.get(keep[2], 0, lambda: (torch.zeros(8, 4),))            # a hit: now the most recent
    small.get(keep[0], 0, lambda: (torch.zeros(8, 4),))            # evicts keep[3], the oldest
    assert small.conversions == 6
    n = small.conversions
    small.get(keep[2], 0, lambda: (torch.zeros(8, 4),))
    assert small.conversions == n
    small.get(keep[3], 0, lambda: (torch.zeros(8, 4),))
    assert small.conversions == n + 1


def test_weight_rounding_queries_answer_without_a_gpu():
    """amct_gemm_w4a16_weight_rounded / amct_gemm_w8a16_weight_rounded are host logic: which reading of the dequantised
    weight a call takes follows from its shape, dtype and workspace size alone."""
    from amct_amd import _lib
    lib = _lib.load()
    q4, q8 = lib.amct_gemm_w4a16_weight_rounded, lib.amct_gemm_w8a16_weight_rounded
    for dt in (_lib.BF16, _lib.F16):
        for M in (1, 2, 5, 16):
            for K in (1024, 2048, 4096):
                assert q4(M, 14336, K, 128, dt, 0) == 0                 # the weight-streaming kernels keep the integer weight
                assert q8(M, 14336, K, 128, dt, 0) == 0
                assert q8(M, 14336, K, K, dt, 0) == 0                   # per-channel factors
        for M in (17, 64, 256, 1024, 2048):
            assert q4(M, 14336, 4096, 128, dt, 1 << 30) == 1            # every tile kernel rounds it to the activation dtype
            assert q8(M, 14336, 4096, 128, dt, 1 << 30) == 1
        assert q4(16, 14336, 4096, 64, dt, 0) == 1                      # groups the streaming kernel does not take
        assert q4(16, 14336, 4000, 100, dt, 0) == 1
    # long rows walk slices whose partial sums need the lent workspace: without it another (rounding) kernel serves the call
    need = lib.amct_gemm_w4a16_workspace_bytes(16, 4096, 14336, 128, 0)
    assert need >= 7 * 16 * 4096 * 4
    assert q4(16, 4096, 14336, 128, _lib.BF16, need) == 0 and q4(16, 4096, 14336, 128, _lib.BF16, 0) == 1
    # what the GEMM entry points reject, the queries reject
    assert q4(16, 0, 4096, 128, _lib.BF16, 0) < 0 and q4(16, 64, 4096, 0, _lib.BF16, 0) < 0
    assert q4(16, 64, 4096, 128, _lib.F32, 0) < 0 and q8(16, 64, 4096, 128, _lib.F32, 0) < 0
