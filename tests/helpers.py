"""Shared builders for the GPU parity tests: seeded experts on the device and their oracle twins."""
import numpy as np
import torch

import oracle as orc
from flyingfish_amd import capi, synth
from flyingfish_amd.ops import ExpertTable


def bits(t):
    """torch BF16 tensor (any device) -> numpy uint16 bit patterns."""
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def bf16_tensor(bits_np, device="cuda"):
    return torch.from_numpy(np.ascontiguousarray(bits_np).view(np.int16)).view(torch.bfloat16).to(device)


def make_table(fmt, experts, hidden, inter, seed, device="cuda", std=0.02):
    """Seeded N(0, std) experts quantized to `fmt`; returns (table, oracle weights list).

    oracle weights[e] = (gate, up, down) BF16 effective-weight bit arrays, dequantized by the oracle
    from the very codes and scales that were uploaded.
    """
    table = ExpertTable.allocate(fmt, experts, hidden, inter, device)
    ref = []
    for e in range(experts):
        mats = [synth.normal((inter, hidden), std, seed * 1000 + e * 3 + 0), synth.normal((inter, hidden), std, seed * 1000 + e * 3 + 1),
                synth.normal((hidden, inter), std, seed * 1000 + e * 3 + 2)]
        views = table.expert_views(e)
        eff = []
        gl = []
        for i, w in enumerate(mats):
            if fmt == capi.FMT_FP8_BLOCK128:
                codes, scales = synth.quant_fp8_block(w)
                views[2 * i].copy_(codes)
                views[2 * i + 1].copy_(scales)
                eff.append(orc.dequant_fp8_block(codes.numpy(), scales.numpy()))
            elif fmt == capi.FMT_NVFP4:
                codes, scales, g = synth.quant_nvfp4(w)
                views[2 * i].copy_(codes)
                views[2 * i + 1].copy_(scales)
                gl.append(g)
                eff.append(orc.dequant_nvfp4(codes.numpy(), scales.numpy(), g))
            elif fmt == capi.FMT_FP8_CHANNEL:
                codes, scales = synth.quant_fp8_channel(w)
                views[2 * i].copy_(codes)
                views[2 * i + 1].copy_(scales)
                eff.append(orc.dequant_fp8_channel(codes.numpy(), bits(scales)))
            else:
                wb = w.to(torch.bfloat16)
                views[2 * i].copy_(wb)
                eff.append(bits(wb))
        if fmt == capi.FMT_NVFP4:
            table.global_scales[e] = torch.tensor(gl, dtype=torch.float32)
        ref.append(tuple(eff))
    return table, ref


def oracle_contributions(ref, x_bits, ids, weights_f32, rounding, limit, boundary, active=None, form=orc.LANE8):
    rows, top_k = ids.shape
    hidden = x_bits.shape[1]
    out = np.zeros((rows, top_k, hidden), dtype=np.uint16)
    for r in range(rows):
        for c in range(top_k):
            if active is not None and not active[r, c]:
                continue
            g, u, d = ref[int(ids[r, c])]
            out[r, c] = orc.expert_ffn(x_bits[r], g, u, d, float(weights_f32[r, c]), rounding, limit, boundary, form, orc.SILU_DIV)
    return out


def oracle_shared(shared_ref, x_bits, rounding, limit, form=orc.LANE8):
    g, u, d = shared_ref
    return np.stack([orc.expert_ffn(x_bits[r], g, u, d, 1.0, rounding, limit, 0, form, orc.SILU_DIV, apply_weight=False)
                     for r in range(x_bits.shape[0])])


def assert_close_bf16(got_bits, want_bits, what, max_ulp=2, rel=1e-3):
    """north-star bound: relative L2 <= 1e-3 and every element within max_ulp BF16 steps of the reference,
    the step taken at the magnitude of the reference element or, for elements far below the row's scale
    (cancelled sums), at 2^-7 of the largest reference magnitude of the row."""
    got = orc.bf16_to_f32(got_bits).astype(np.float64)
    want = orc.bf16_to_f32(want_bits).astype(np.float64)
    r = orc.rel_l2(got_bits, want_bits)
    assert r <= rel, "%s: relative L2 %.3e > %.1e" % (what, r, rel)
    want2 = want.reshape(-1, want.shape[-1])
    got2 = got.reshape(-1, got.shape[-1])
    floor = np.max(np.abs(want2), axis=1, keepdims=True) * 2.0 ** -7
    mag = np.maximum(np.abs(want2), floor)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(mag, 1e-38))) - 7)
    worst = np.max(np.abs(got2 - want2) / ulp)
    assert worst <= max_ulp, "%s: %.2f BF16 steps > %d" % (what, worst, max_ulp)
    return r, worst
