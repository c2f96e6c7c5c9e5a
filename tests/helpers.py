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


def run_parallel(fn, n, threads=1):
    """[fn(lo, hi) for contiguous pieces of range(n)], the pieces run on `threads` Python threads (the oracle's C
    functions release the GIL under ctypes), results in order."""
    threads = max(1, min(threads, n))
    cuts = [n * i // threads for i in range(threads + 1)]
    pieces = [(cuts[i], cuts[i + 1]) for i in range(threads) if cuts[i + 1] > cuts[i]]
    if len(pieces) <= 1:
        return [fn(lo, hi) for lo, hi in pieces]
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(max_workers=len(pieces)) as pool:
        return list(pool.map(lambda p: fn(*p), pieces))


def make_table_on_device(fmt, experts, hidden, inter, seed, std=0.02):
    """Seeded N(0, std) experts drawn and quantized on the GPU (full-size shapes: 44 MB per expert at 7168 x 2048).
    Returns the table; host copies come from host_expert()."""
    table = ExpertTable.allocate(fmt, experts, hidden, inter, "cuda")
    for e in range(experts):
        views = table.expert_views(e)
        gl = []
        for i, shape in enumerate([(inter, hidden), (inter, hidden), (hidden, inter)]):
            w = synth.normal(shape, std, seed * 1000 + e * 3 + i, device="cuda")
            if fmt == capi.FMT_FP8_BLOCK128:
                codes, scales = synth.quant_fp8_block(w)
            elif fmt == capi.FMT_NVFP4:
                codes, scales, g = synth.quant_nvfp4(w)
                gl.append(g)
            elif fmt == capi.FMT_FP8_CHANNEL:
                codes, scales = synth.quant_fp8_channel(w)
            elif fmt == capi.FMT_E2M1_E8M0:
                codes, scales = synth.quant_e2m1_e8m0(w)
            elif fmt == capi.FMT_E4M3_E8M0_32:
                codes, scales = synth.quant_e4m3_e8m0_block32(w)
            else:
                codes, scales = w.to(torch.bfloat16), None
            views[2 * i].copy_(codes)
            if scales is not None:
                views[2 * i + 1].copy_(scales)
        if fmt == capi.FMT_NVFP4:
            table.global_scales[e] = torch.tensor(gl, dtype=torch.float32)
    torch.cuda.synchronize()
    return table


def host_expert(table, e):
    """Raw host copies of expert e: [gate codes, gate scales, up codes, up scales, down codes, down scales] as numpy
    arrays (BF16 tensors as uint16 bit patterns, missing scales as None)."""
    out = []
    for v in table.expert_views(e):
        if v is None:
            out.append(None)
        elif v.dtype == torch.bfloat16:
            out.append(bits(v))
        else:
            out.append(v.cpu().numpy())
    return out


def effective_weights(table, e):
    """(gate, up, down) BF16 effective-weight bit arrays of expert e, dequantized by the oracle from the device's bytes."""
    m = host_expert(table, e)
    fmt = table.format
    out = []
    for i in range(3):
        codes, scales = m[2 * i], m[2 * i + 1]
        if fmt == capi.FMT_FP8_BLOCK128:
            out.append(orc.dequant_fp8_block(codes, scales))
        elif fmt == capi.FMT_NVFP4:
            out.append(orc.dequant_nvfp4(codes, scales, float(table.global_scales[e, i].item())))
        elif fmt == capi.FMT_FP8_CHANNEL:
            out.append(orc.dequant_fp8_channel(codes, scales))
        else:
            out.append(codes)
    return tuple(out)


def bf16_neighbours(bits_np):
    """The BF16 values one step below and above in magnitude (bit patterns; zero keeps zero as its lower neighbour)."""
    b = np.asarray(bits_np, dtype=np.uint16)
    mag, sign = (b & 0x7fff).astype(np.int32), b & 0x8000
    lo = np.maximum(mag - 1, 0).astype(np.uint16) | sign
    hi = np.minimum(mag + 1, 0x7f7f).astype(np.uint16) | sign
    return lo, hi


def _bf16_steps(got_bits, want_bits):
    """|got - want| in BF16 steps of the reference element (floored at 2^-7 of the row's largest reference magnitude)."""
    g, v = orc.bf16_to_f32(got_bits).astype(np.float64), orc.bf16_to_f32(want_bits).astype(np.float64)
    floor = np.max(np.abs(v), axis=-1, keepdims=True) * 2.0 ** -7
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.maximum(np.abs(v), floor), 1e-38))) - 7)
    return np.abs(g - v) / ulp


def assert_close_or_explained(got_bits, want_bits, candidates, what, max_ulp=2, rel=1e-3, rare=1e-3):
    """The north-star bar (relative L2 <= rel over the tensor, every element within max_ulp BF16 steps), where an element
    beyond max_ulp steps is accepted only if it equals one of `candidates` bit for bit (the exact results of inputs one
    BF16 step from the reference's, which the bar on the previous value allows) and such elements are rare."""
    r = orc.rel_l2(got_bits, want_bits)
    assert r <= rel, "%s: relative L2 %.3e > %.1e" % (what, r, rel)
    steps = _bf16_steps(got_bits, want_bits)
    far = steps > max_ulp
    if np.any(far):
        explained = np.zeros(got_bits.shape, dtype=bool)
        for c in candidates:
            explained |= got_bits == c
        bad = far & ~explained
        assert not np.any(bad), "%s: %d elements beyond %d steps (worst %.2f) that no input within one step explains" % (
            what, int(bad.sum()), max_ulp, float(steps[bad].max()))
        assert np.mean(far) < rare, "%s: %.2e of the elements beyond %d steps" % (what, float(np.mean(far)), max_ulp)
    return r, float(steps.max())


OUTLIER_STATS = []  # (what, relative L2, worst steps, share beyond strict, allowed share, loose) of every call, for the run's summary


def assert_close_with_rare_outliers(got_bits, want_bits, what, strict=2, loose=16, rare=1e-3, rel=1e-3):
    """A bar for values behind TWO composed stages, where the north-star bar holds per stage but an element can move
    further end to end (a BF16 step of an activation shifts every down output a little, and a cancelled output by several
    of its own steps): relative L2 <= rel over the tensor, no element beyond `loose` steps, and - what a kernel that is
    genuinely a step or two worse would fail - at most a fraction `rare` of the elements beyond `strict` steps.
    Returns (relative L2, worst steps, fraction beyond strict)."""
    r = orc.rel_l2(got_bits, want_bits)
    assert r <= rel, "%s: relative L2 %.3e > %.1e" % (what, r, rel)
    steps = _bf16_steps(got_bits, want_bits)
    worst, frac = float(steps.max()), float(np.mean(steps > strict))
    OUTLIER_STATS.append((what, r, worst, frac, rare, loose))
    assert worst <= loose, "%s: %.2f BF16 steps > %d" % (what, worst, loose)
    assert frac <= rare, "%s: %.2e of the elements beyond %d steps (allowed %.1e; worst %.1f)" % (what, frac, strict, rare, worst)
    return r, worst, frac


def assert_weighted_down_close(got_bits, down_ref_bits, weights, what, max_ulp=2, rel=1e-3):
    """Routing weight applied after the BF16 cast of the down output: c = bf16(bf16(d) * w), rows [n, H] with one weight
    each. The bar is on d: c must lie within max_ulp steps / rel of bf16(d_ref * w), and an element further away must be
    the exact weighting of a d one BF16 step from the reference's (one step of d is up to two steps of c when d sits
    just above a power of two and c just below one, plus the rounding of the product: three steps of c, none of them
    the kernel's)."""
    w = np.asarray(weights, dtype=np.float32).reshape(-1, 1)
    c = lambda d: orc.f32_to_bf16((orc.bf16_to_f32(d) * w).astype(np.float32))
    lo, hi = bf16_neighbours(down_ref_bits)
    return assert_close_or_explained(got_bits, c(down_ref_bits), [c(lo), c(hi)], what, max_ulp, rel)


def assert_swiglu_close(act_bits, gate_ref_bits, up_ref_bits, rounding, limit, kind, what, max_ulp=2, rel=1e-3):
    """Activations a = SwiGLU(bf16 gate, bf16 up) against the reference's: within max_ulp steps / rel, and an element
    further away must be the exact SwiGLU of a gate and an up value each within one BF16 step of the reference's (the
    twice-rounded product of two values one step off can sit three steps away)."""
    want = orc.silu_mul(gate_ref_bits, up_ref_bits, rounding, limit, kind)
    glo, ghi = bf16_neighbours(gate_ref_bits)
    ulo, uhi = bf16_neighbours(up_ref_bits)
    cands = [orc.silu_mul(g, u, rounding, limit, kind) for g in (glo, gate_ref_bits, ghi) for u in (ulo, up_ref_bits, uhi)]
    return assert_close_or_explained(act_bits, want, cands, what, max_ulp, rel)
