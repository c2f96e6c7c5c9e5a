"""F3: the per-channel FP8 expert format, and the reference's Lane16 / Lane8 summation orders bit for bit
(ffmoe_decode_contribute_form) against the oracle's restatement of src/cpu/expert_ffn.rs:689-776, which the CPU suite
pins against the reference's golden vectors."""
import numpy as np
import pytest
import torch

import oracle as orc
from flyingfish_amd import capi, synth
from flyingfish_amd.ops import DecodeOps
from helpers import assert_close_bf16, bits, make_table, oracle_shared

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rand_bf16(shape, std, seed):
    return synth.normal(shape, std, seed).to(torch.bfloat16)


def _case(fmt, experts, hidden, inter, rows, top_k, seed, shared):
    table, ref = make_table(fmt, experts + (1 if shared else 0), hidden, inter, seed)
    sh = table.shared_struct(experts) if shared else None
    table.experts = experts
    x = rand_bf16((rows, hidden), 1.0, seed + 7)
    g = synth.generator(seed + 8)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    wt = torch.rand((rows, top_k), generator=g) * 0.5 + 0.05
    return table, ref, sh, x, ids, wt


@pytest.mark.parametrize("rows,shared", [(1, True), (6, True), (19, False)])
def test_decode_fp8_per_channel_experts(rows, shared):
    """Streaming path (64-lane sums) on per-channel FP8 experts: the north-star tolerance against the oracle."""
    experts, hidden, inter, top_k = 6, 1024, 512, 3
    table, ref, sh, x, ids, wt = _case(capi.FMT_FP8_CHANNEL, experts, hidden, inter, rows, top_k, 171, shared)
    op = DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
    contrib, shared_out = op.contribute(x.to(DEV), ids.to(DEV), wt.to(DEV))
    torch.cuda.synchronize()
    want = np.stack([np.stack([orc.expert_ffn(bits(x)[r], *ref[int(ids[r, c])], float(wt[r, c]), orc.TWICE, 0.0, orc.AFTER_DOWN_BF16,
                                              orc.LANE8, orc.SILU_DIV) for c in range(top_k)]) for r in range(rows)])
    assert_close_bf16(bits(contrib), want, "contributions")
    assert np.all(op.done.cpu().numpy() == 1)
    if shared:
        assert_close_bf16(bits(shared_out), oracle_shared(ref[experts], bits(x), orc.TWICE, 0.0), "shared_out")


@pytest.mark.parametrize("fmt", [capi.FMT_BF16, capi.FMT_FP8_CHANNEL])
@pytest.mark.parametrize("form", [capi.FORM_LANE16, capi.FORM_LANE8])
@pytest.mark.parametrize("hidden,inter,rows,top_k,rounding,boundary", [
    (512, 256, 1, 2, capi.SWIGLU_TWICE, capi.WEIGHT_AFTER_DOWN_BF16),
    (1024, 384, 5, 3, capi.SWIGLU_ONCE, capi.WEIGHT_BEFORE_CONTRIBUTION_BF16),
    (776, 200, 3, 2, capi.SWIGLU_CLAMPED_TWICE, capi.WEIGHT_AFTER_DOWN_BF16),   # widths that are 8 mod 16: the Lane16 tail
    (512, 256, 2, 2, capi.SWIGLU_GELU_TWICE, capi.WEIGHT_BEFORE_CONTRIBUTION_BF16),
])
def test_reference_summation_orders_bit_exact(fmt, form, hidden, inter, rows, top_k, rounding, boundary):
    if fmt == capi.FMT_FP8_CHANNEL and (hidden % 16 or inter % 16):
        pytest.skip("per-channel FP8 rows are multiples of 16 codes")
    experts, limit = 5, (0.05 if rounding in (capi.SWIGLU_CLAMPED_TWICE, capi.SWIGLU_CLAMPED_ONCE) else 0.0)
    table, ref, sh, x, ids, wt = _case(fmt, experts, hidden, inter, rows, top_k, 181 + form, True)
    active = torch.ones((rows, top_k), dtype=torch.int32)
    if rows > 1:
        active[1, 0] = 0
    op = DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, rounding, limit, boundary, True)
    op.done.zero_()
    op.contributions.zero_()
    contrib, shared_out = op.contribute(x.to(DEV), ids.to(DEV), wt.to(DEV), active.to(DEV), form=form)
    torch.cuda.synchronize()
    oform = orc.LANE16 if form == capi.FORM_LANE16 else orc.LANE8
    # SiLU as the reference pairs it with the form (kernels/moe_ffn.cu:58, :201-203)
    kind = orc.SILU_RCP if (form == capi.FORM_LANE16 and rounding in (capi.SWIGLU_TWICE, capi.SWIGLU_CLAMPED_TWICE)) else orc.SILU_DIV
    xb = bits(x)
    got = bits(contrib)
    for r in range(rows):
        for c in range(top_k):
            if not active[r, c]:
                assert not got[r, c].any()
                continue
            want = orc.expert_ffn(xb[r], *ref[int(ids[r, c])], float(wt[r, c]), rounding, limit, boundary, oform, kind)
            assert np.array_equal(got[r, c], want), (r, c)
        want_sh = orc.expert_ffn(xb[r], *ref[experts], 1.0, rounding, limit, 0, oform, kind, apply_weight=False)
        assert np.array_equal(bits(shared_out)[r], want_sh), r
    assert np.array_equal(op.done.cpu().numpy(), active.numpy())


@pytest.mark.parametrize("seed", range(16))
def test_reference_summation_orders_seeded_sweep(seed):
    """Bit equality with the reference's two reduction orders at widths the fixed cases do not visit (any multiple of
    the format's granule from 64 to 1536, hence every residue of the 16- and 64-element strides), 1..9 rows, 1..6
    choices, with and without a shared expert, every rounding, both boundaries."""
    rng = np.random.default_rng(7000 + seed)
    fmt = capi.FMT_BF16 if seed % 2 == 0 else capi.FMT_FP8_CHANNEL
    form = capi.FORM_LANE16 if (seed // 2) % 2 == 0 else capi.FORM_LANE8
    gran = 8 if fmt == capi.FMT_BF16 else 16
    hidden = gran * int(rng.integers(64 // gran, 1536 // gran + 1))
    inter = gran * int(rng.integers(64 // gran, 768 // gran + 1))
    experts = int(rng.integers(2, 9))
    top_k = int(rng.integers(1, min(6, experts) + 1))
    rows = int(rng.choice([1, 2, 4, 9]))
    rounding = int(rng.integers(0, 5))
    limit = float(rng.choice([0.05, 1.0])) if rounding in (2, 3) else 0.0
    boundary = int(rng.integers(0, 2))
    shared = bool(rng.integers(0, 2))
    print("fmt=%d form=%d hidden=%d inter=%d experts=%d top_k=%d rows=%d rounding=%d limit=%g boundary=%d shared=%d" %
          (fmt, form, hidden, inter, experts, top_k, rows, rounding, limit, boundary, shared), flush=True)
    table, ref, sh, x, ids, wt = _case(fmt, experts, hidden, inter, rows, top_k, 7100 + seed, shared)
    op = DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, rounding, limit, boundary, True)
    contrib, shared_out = op.contribute(x.to(DEV), ids.to(DEV), wt.to(DEV), form=form)
    torch.cuda.synchronize()
    oform = orc.LANE16 if form == capi.FORM_LANE16 else orc.LANE8
    kind = orc.SILU_RCP if (form == capi.FORM_LANE16 and rounding in (capi.SWIGLU_TWICE, capi.SWIGLU_CLAMPED_TWICE)) else orc.SILU_DIV
    xb, got = bits(x), bits(contrib)
    for r in range(rows):
        for c in range(top_k):
            want = orc.expert_ffn(xb[r], *ref[int(ids[r, c])], float(wt[r, c]), rounding, limit, boundary, oform, kind)
            assert np.array_equal(got[r, c], want), (r, c)
        if shared:
            want_sh = orc.expert_ffn(xb[r], *ref[experts], 1.0, rounding, limit, 0, oform, kind, apply_weight=False)
            assert np.array_equal(bits(shared_out)[r], want_sh), r


@pytest.mark.parametrize("form", [capi.FORM_LANE16, capi.FORM_LANE8])
def test_reference_summation_orders_take_whole_cohorts(form):
    """A prefill cohort (600 rows x 8 choices) through the same entry, bit-equal row by row - the arithmetic of the
    reference's moe_gemm_lane16 pipeline (kernels/moe_prefill.cu:13-71: one 16-lane chain per (row, column)); here the
    assignments are sorted by expert and a group of rows shares one pass over the expert's weights."""
    experts, hidden, inter, rows, top_k = 12, 128, 64, 600, 8
    table, ref, sh, x, ids, wt = _case(capi.FMT_BF16, experts, hidden, inter, rows, top_k, 7600 + form, True)
    op = DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
    contrib, shared_out = op.contribute(x.to(DEV), ids.to(DEV), wt.to(DEV), form=form)
    torch.cuda.synchronize()
    oform = orc.LANE16 if form == capi.FORM_LANE16 else orc.LANE8
    kind = orc.SILU_RCP if form == capi.FORM_LANE16 else orc.SILU_DIV
    xb, got, got_sh = bits(x), bits(contrib), bits(shared_out)
    for r in list(range(0, rows, 37)) + [rows - 1]:
        for c in range(top_k):
            want = orc.expert_ffn(xb[r], *ref[int(ids[r, c])], float(wt[r, c]), orc.TWICE, 0.0, 0, oform, kind)
            assert np.array_equal(got[r, c], want), (r, c)
        assert np.array_equal(got_sh[r], orc.expert_ffn(xb[r], *ref[experts], 1.0, orc.TWICE, 0.0, 0, oform, kind, apply_weight=False)), r
    assert int(op.done.sum().item()) == rows * top_k


@pytest.mark.parametrize("fmt", [capi.FMT_BF16, capi.FMT_FP8_CHANNEL])
@pytest.mark.parametrize("form", [capi.FORM_LANE16, capi.FORM_LANE8])
@pytest.mark.parametrize("rows,hidden,inter", [(70, 784, 208), (9, 4608, 512), (2, 256, 128)])
def test_token_sorted_form_kernels_equal_one_block_per_choice(fmt, form, rows, hidden, inter, monkeypatch):
    """Rows of one expert share a pass over its weights (groups of 8, or as many rows as fit LDS: 4 at hidden 4608):
    contributions, shared output and done flags are the bits of the kernels that run one block per (row, choice)
    (FFMOE_FORM_GROUPED=0), with masked, invalid and out-of-range choices in the batch and widths that are 8 mod 16."""
    experts, top_k = 5, 3
    table, ref, sh, x, ids, wt = _case(fmt, experts, hidden, inter, rows, top_k, 8100 + rows + form, True)
    ids = ids.clone()
    active = (torch.rand((rows, top_k), generator=synth.generator(8200 + rows)) > 0.25).to(torch.int32)
    ids[rows - 1, 0] = experts + 2
    valid = torch.ones(experts, dtype=torch.int32)
    valid[1] = 0
    table.valid = valid.to(DEV)
    out = {}
    for grouped in ("0", "1"):
        monkeypatch.setenv("FFMOE_FORM_GROUPED", grouped)
        op = DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, capi.SWIGLU_CLAMPED_TWICE, 0.7, capi.WEIGHT_BEFORE_CONTRIBUTION_BF16, True)
        op.contributions.zero_(); op.shared_out.zero_(); op.done.zero_()
        contrib, shared_out = op.contribute(x.to(DEV), ids.to(DEV), wt.to(DEV), active.to(DEV), form=form)
        torch.cuda.synchronize()
        out[grouped] = (bits(contrib).copy(), bits(shared_out).copy(), op.done.cpu().numpy().copy())
    assert np.any(out["0"][0] != 0) and np.any(out["0"][1] != 0)
    for a, b, what in zip(out["0"], out["1"], ("contributions", "shared_out", "done")):
        assert np.array_equal(a, b), what
    live = (active.numpy() != 0) & (ids.numpy() < experts) & (ids.numpy() != 1)
    assert np.array_equal(out["1"][2].reshape(rows, top_k) != 0, live)


def test_form_entry_rejects_other_formats():
    table, _ = make_table(capi.FMT_FP8_BLOCK128, 2, 256, 128, 5)
    op = DecodeOps(table, None, 1, 1, weights_f32=True)
    x = rand_bf16((1, 256), 1.0, 1).to(DEV)
    ids = torch.zeros((1, 1), dtype=torch.int32, device=DEV)
    w = torch.ones((1, 1), device=DEV)
    with pytest.raises(capi.FfmoeError):
        op.contribute(x, ids, w, form=capi.FORM_LANE8)
