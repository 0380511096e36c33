"""Seeded synthetic inputs of the benchmark configurations.  Tensors are made on
the CPU with torch.Generator so the GPU kernels and any CPU checker see
identical bits; callers move them to the device."""
import torch

HOT_COLS = (7, 291, 1033, 1418, 2047, 2730, 3391, 4000)


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def c1_weight(rows=4096, cols=4096):
    """fp32 weight, N(0, 0.02)."""
    return torch.randn(rows, cols, generator=_gen(1001)) * 0.02


def c2_weight(rows=14336, cols=4096):
    """bf16 weight N(0,0.02) with 0.1 % outliers of magnitude 20 sigma."""
    w = torch.randn(rows, cols, generator=_gen(1002)) * 0.02
    mask = torch.rand(rows, cols, generator=_gen(1003)) < 0.001
    sign = torch.where(torch.rand(rows, cols, generator=_gen(1004)) < 0.5, -1.0, 1.0)
    w = torch.where(mask, sign * 0.4, w)
    return w.to(torch.bfloat16)


def c3_activations(rows=8192, cols=4096):
    """bf16 Student-t (nu=3) activations with 8 hidden channels scaled 50x."""
    g = _gen(1005)
    z = torch.randn(rows, cols, generator=g)
    c = torch.randn(3, rows, cols, generator=g)
    x = z / torch.sqrt((c * c).sum(0) / 3.0)
    for col in HOT_COLS:
        if col < cols:
            x[:, col] *= 50.0
    return x.to(torch.bfloat16)


def c4_w8a8(M=2048, N=14336, K=4096):
    """(x bf16 [M,K], wq int8 [N,K], s_w fp32 [N])."""
    x = torch.randn(M, K, generator=_gen(1006)).to(torch.bfloat16)
    wq = torch.randint(-127, 128, (N, K), generator=_gen(1007), dtype=torch.int8)
    s_w = 1e-3 + 9e-3 * torch.rand(N, generator=_gen(1008))
    return x, wq, s_w


def c5_w4a16(M=2048, N=14336, K=4096, group=128):
    """(x bf16 [M,K], u4 codes uint8 [N,K] in 0..15, scales f16 [N,K/g], zeros uint8 [N,K/g],
    smooth_recip bf16 [K]) -- SmoothQuant alpha=0.5 factors from the per-channel absmax of a
    2048-token activation batch and of the dequantised weight."""
    x_full = torch.randn(2048, K, generator=_gen(1009)).to(torch.bfloat16)
    codes = torch.randint(0, 16, (N, K), generator=_gen(1010), dtype=torch.uint8)
    scales = (1e-3 + 9e-3 * torch.rand(N, K // group, generator=_gen(1011))).half()
    zeros = torch.randint(0, 16, (N, K // group), generator=_gen(1012), dtype=torch.uint8)
    act_max = x_full.float().abs().amax(0)
    wmax = torch.zeros(K)
    step = 2048
    for n0 in range(0, N, step):                       # bounded temporary
        c = codes[n0:n0 + step].float().reshape(-1, K // group, group)
        wd = (c - zeros[n0:n0 + step].float().unsqueeze(-1)) * scales[n0:n0 + step].float().unsqueeze(-1)
        wmax = torch.maximum(wmax, wd.reshape(-1, K).abs().amax(0))
    smooth = act_max.pow(0.5) / wmax.clamp_min(1e-12).pow(0.5)
    smooth_recip = (1.0 / smooth).to(torch.bfloat16)
    x = x_full[:M] if M <= 2048 else torch.randn(M, K, generator=_gen(1013)).to(torch.bfloat16)
    return x.contiguous(), codes, scales, zeros, smooth_recip


def pack_nibbles(codes_u4):
    """uint8 [N,K] values 0..15 -> uint8 [N,K/2], even k in the low nibble."""
    return (codes_u4[:, 0::2] | (codes_u4[:, 1::2] << 4)).contiguous()
