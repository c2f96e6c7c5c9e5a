"""Seeded synthetic inputs and weight quantizers (torch, CPU or GPU).

Recipes: weights ~ N(0, 0.02) quantized with absmax scales (FP8: one f32 scale per 128x128 block,
s = amax * (1/448); NVFP4: E4M3 scale per 16 k-elements = amax/6 relative to an f32 global scale),
activations ~ N(0, 1) in BF16, router gate ~ N(0, 0.02) in BF16. The encoders are the reference's:
E4M3 round-to-nearest-even saturating at 448 (src/fp8.rs:85-121), E2M1 with its tie thresholds
(kernels/q38_contract.cuh:180-187), stored NVFP4 scale code never 0 (q38_contract.cuh:207-209).
"""
import torch

E4M3_MAX = 448.0


def generator(seed, device="cpu"):
    g = torch.Generator(device=device)
    g.manual_seed(int(seed))
    return g


def normal(shape, std, seed, device="cpu", dtype=torch.float32):
    return (torch.randn(shape, generator=generator(seed, device), device=device, dtype=torch.float32) * std).to(dtype)


def e4m3_encode(x):
    """float32 tensor already clamped to [-448, 448] -> uint8 E4M3 codes (RNE)."""
    return x.to(torch.float8_e4m3fn).view(torch.uint8)


def e4m3_decode(codes):
    return codes.view(torch.float8_e4m3fn).to(torch.float32)


def quant_fp8_block(w, block=128):
    """w [N,K] f32 -> (codes uint8 [N,K], scales f32 [ceil(N/b), ceil(K/b)])."""
    n, k = w.shape
    gn, gk = -(-n // block), -(-k // block)
    pad = torch.zeros((gn * block, gk * block), dtype=torch.float32, device=w.device)
    pad[:n, :k] = w
    blocks = pad.view(gn, block, gk, block)
    amax = blocks.abs().amax(dim=(1, 3))
    scales = amax * torch.tensor(1.0 / 448.0, dtype=torch.float32, device=w.device)
    div = scales.clamp_min(1e-12)[:, None, :, None]
    q = (blocks / div).clamp(-E4M3_MAX, E4M3_MAX)
    codes = e4m3_encode(q).view(gn * block, gk * block)[:n, :k].contiguous()
    return codes, scales.contiguous()


def quant_fp8_channel(w):
    """w [N,K] f32 -> (codes uint8 [N,K], scales bf16 [N]): one scale per output row, amax/448 rounded to BF16."""
    amax = w.abs().amax(dim=1)
    scales = (amax * torch.tensor(1.0 / 448.0, dtype=torch.float32, device=w.device)).to(torch.bfloat16)
    div = scales.to(torch.float32).clamp_min(1e-12)[:, None]
    q = (w / div).clamp(-E4M3_MAX, E4M3_MAX)
    return e4m3_encode(q).contiguous(), scales.contiguous()


def _pow2_ceil_exponent(v):
    """ceil(log2(v)) of positive float32 values, from the bit pattern (exact)."""
    bits = v.to(torch.float32).view(torch.int32)
    return ((bits >> 23) & 0xff) - 127 + ((bits & 0x7fffff) != 0).to(torch.int32)


def quant_e2m1_e8m0(w):
    """w [N,K] f32 -> (packed E2M1 codes uint8 [N,K/2], low nibble = even k; E8M0 scale codes uint8 [N,K/32]): one
    power-of-two scale per 32 elements of a row, 2^ceil(log2(amax/6))."""
    n, k = w.shape
    blocks = w.view(n, k // 32, 32)
    amax = blocks.abs().amax(dim=2).clamp_min(2.0 ** -100)
    exp = _pow2_ceil_exponent(amax / 6.0).clamp(-127, 127)
    scale = torch.pow(torch.tensor(2.0, dtype=torch.float64, device=w.device), exp.to(torch.float64)).to(torch.float32)
    q = (blocks / scale[:, :, None]).clamp(-6.0, 6.0).reshape(n, k)
    codes = e2m1_encode(q)
    packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).contiguous()
    return packed, (exp + 127).to(torch.uint8).contiguous()


def quant_e4m3_e8m0_block32(w):
    """w [N,K] f32 -> (E4M3 codes uint8 [N,K], E8M0 scale codes uint8 [ceil(N/32), K/32]): one power-of-two scale per
    32x32 block, 2^ceil(log2(amax/448))."""
    n, k = w.shape
    gn = -(-n // 32)
    pad = torch.zeros((gn * 32, k), dtype=torch.float32, device=w.device)
    pad[:n] = w
    blocks = pad.view(gn, 32, k // 32, 32)
    amax = blocks.abs().amax(dim=(1, 3)).clamp_min(2.0 ** -100)
    exp = _pow2_ceil_exponent(amax / 448.0).clamp(-127, 127)
    scale = torch.pow(torch.tensor(2.0, dtype=torch.float64, device=w.device), exp.to(torch.float64)).to(torch.float32)
    q = (blocks / scale[:, None, :, None]).clamp(-E4M3_MAX, E4M3_MAX)
    codes = e4m3_encode(q).view(gn * 32, k)[:n].contiguous()
    return codes, (exp + 127).to(torch.uint8).contiguous()


def e2m1_encode(x):
    """float32 -> 4-bit E2M1 codes (uint8), thresholds with ties toward the even code."""
    m = x.abs()
    code = torch.full_like(m, 7, dtype=torch.uint8)
    code = torch.where(m <= 5.0, torch.tensor(6, dtype=torch.uint8, device=x.device), code)
    code = torch.where(m < 3.5, torch.tensor(5, dtype=torch.uint8, device=x.device), code)
    code = torch.where(m <= 2.5, torch.tensor(4, dtype=torch.uint8, device=x.device), code)
    code = torch.where(m < 1.75, torch.tensor(3, dtype=torch.uint8, device=x.device), code)
    code = torch.where(m <= 1.25, torch.tensor(2, dtype=torch.uint8, device=x.device), code)
    code = torch.where(m < 0.75, torch.tensor(1, dtype=torch.uint8, device=x.device), code)
    code = torch.where(m <= 0.25, torch.tensor(0, dtype=torch.uint8, device=x.device), code)
    sign = (torch.signbit(x).to(torch.uint8) << 3)
    return code | sign


def quant_nvfp4(w):
    """w [N,K] f32 (K % 16 == 0) -> (codes uint8 [N,K/2], scales uint8 [N,K/16], global f32 python float)."""
    n, k = w.shape
    g = w.view(n, k // 16, 16)
    s16 = g.abs().amax(dim=2) / 6.0
    glob = s16.max() / 448.0
    if not bool(glob > 0):
        glob = torch.tensor(1.0, dtype=torch.float32, device=w.device)
    sc = e4m3_encode((s16 / glob).clamp(max=E4M3_MAX))
    sc = torch.where(sc == 0, torch.tensor(1, dtype=torch.uint8, device=w.device), sc)
    s = e4m3_decode(sc) * glob
    q = e2m1_encode(g / s[:, :, None]).view(n, k)
    codes = (q[:, 0::2] | (q[:, 1::2] << 4)).contiguous()
    return codes, sc.contiguous(), float(glob)


def zipf_popularity(experts, s, seed):
    """log-popularity offsets: popularity proportional to rank^-s under a seeded expert permutation."""
    perm = torch.randperm(experts, generator=generator(seed))
    rank = torch.empty(experts, dtype=torch.float32)
    rank[perm] = torch.arange(1, experts + 1, dtype=torch.float32)
    return (-s) * torch.log(rank)
