"""F4: experts of the E8M0 block-32 contract (W4A8 routed, W8A8 32x32-block shared expert) in exact arithmetic, through
the C ABI, bit-equal to the oracle's restatement of kernels/q38_contract.cuh:53-101,153-170 and
kernels/moe_ffn.cu:601-700 (pinned on the CPU against rational arithmetic and closed forms)."""
import numpy as np
import pytest
import torch

import oracle as orc
from flyingfish_amd import capi, synth
from flyingfish_amd.ops import E8m0DecodeOps, ExpertTable, PrefillOps
from helpers import assert_close_with_rare_outliers, assert_close_bf16, bits

pytestmark = pytest.mark.gpu
# Values behind two composed stages (end to end) or behind a twice-rounded product (activations of the matrix-core paths):
# the per-stage bars are 2 steps; here the relative-L2 bar holds on the tensor, no element lies beyond a loose bound, and
# the share of elements beyond 2 steps must stay below these (small shapes: a cancelled output behind one activation that
# rounded the other way moves by several of its own steps).
E2E_RARE = 5e-3
ACT_RARE = 2e-3
DEV = "cuda"


def rand_bf16(shape, std, seed):
    return synth.normal(shape, std, seed).to(torch.bfloat16)


def _tables(experts, hidden, inter, shared_inter, seed):
    routed = ExpertTable.allocate(capi.FMT_E2M1_E8M0, experts, hidden, inter, DEV)
    ref = []
    for e in range(experts):
        v = routed.expert_views(e)
        mats = []
        for i, shape in enumerate([(inter, hidden), (inter, hidden), (hidden, inter)]):
            codes, scales = synth.quant_e2m1_e8m0(synth.normal(shape, 0.05, seed * 1000 + e * 3 + i))
            v[2 * i].copy_(codes); v[2 * i + 1].copy_(scales)
            mats += [codes.numpy(), scales.numpy()]
        ref.append(mats)
    sh_table = ExpertTable.allocate(capi.FMT_E4M3_E8M0_32, 1, hidden, shared_inter, DEV)
    v = sh_table.expert_views(0)
    sh_ref = []
    for i, shape in enumerate([(shared_inter, hidden), (shared_inter, hidden), (hidden, shared_inter)]):
        codes, scales = synth.quant_e4m3_e8m0_block32(synth.normal(shape, 0.05, seed * 1000 + 900 + i))
        v[2 * i].copy_(codes); v[2 * i + 1].copy_(scales)
        sh_ref += [codes.numpy(), scales.numpy()]
    return routed, ref, sh_table, sh_ref


def test_act_quant_e8m0_bit_exact():
    x = (synth.normal((5, 256), 1.0, 3) * torch.exp(synth.normal((5, 1), 3.0, 4))).to(torch.bfloat16)
    x[2, 32:64] = 0  # an all-zero group takes the amax floor
    codes, scales = E8m0DecodeOps.act_quant(x.to(DEV))
    torch.cuda.synchronize()
    oc, os_ = orc.act_quant_e8m0(bits(x))
    assert np.array_equal(codes.cpu().numpy(), oc) and np.array_equal(scales.cpu().numpy(), os_)


@pytest.mark.parametrize("hidden,inter,shared_inter,rows,top_k", [(256, 128, 128, 1, 2), (512, 256, 384, 3, 3), (1024, 512, 512, 2, 4)])
def test_e8m0_experts_bit_exact(hidden, inter, shared_inter, rows, top_k):
    experts, limit = 6, 7.0
    routed, ref, sh_table, sh_ref = _tables(experts, hidden, inter, shared_inter, 41 + rows)
    sh = sh_table.shared_struct(0)
    x = rand_bf16((rows, hidden), 1.0, 5 + rows)
    g = synth.generator(6 + rows)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    wt = torch.rand((rows, top_k), generator=g) * 0.5 + 0.05
    active = torch.ones((rows, top_k), dtype=torch.int32)
    if rows > 1:
        active[1, 0] = 0
    op = E8m0DecodeOps(routed, sh, rows, top_k, limit)
    op.contributions.zero_()
    contrib, shared_out = op.contribute(x.to(DEV), ids.to(DEV), wt.to(DEV), active.to(DEV))
    torch.cuda.synchronize()
    got, got_sh, xb = bits(contrib), bits(shared_out), bits(x)
    for r in range(rows):
        for c in range(top_k):
            if not active[r, c]:
                assert not got[r, c].any()
                continue
            want = orc.expert_ffn_e8m0(1, xb[r], *ref[int(ids[r, c])], limit, float(wt[r, c]))
            assert np.array_equal(got[r, c], want), (r, c)
        assert np.array_equal(got_sh[r], orc.expert_ffn_e8m0(0, xb[r], *sh_ref, limit, 1.0)), r
    assert np.array_equal(op.done.cpu().numpy(), active.numpy())


@pytest.mark.parametrize("seed", range(10))
@pytest.mark.parametrize("exact", [True, False])
def test_e8m0_experts_seeded_sweep(seed, exact):
    """Bit equality at widths the fixed cases do not visit (any multiple of 32 from 64 to 1024, shared expert of another
    width, 1..5 rows, 1..6 choices, activations scaled over several binades), in the exact arithmetic and in the
    FP32-chain variant."""
    rng = np.random.default_rng(8000 + seed)
    hidden = 32 * int(rng.integers(2, 33))
    inter = 32 * int(rng.integers(2, 17))
    shared_inter = 32 * int(rng.integers(2, 17))
    experts = int(rng.integers(2, 8))
    top_k = int(rng.integers(1, min(6, experts) + 1))
    rows = int(rng.choice([1, 2, 5]))
    limit = float(rng.choice([0.5, 7.0]))
    print("hidden=%d inter=%d shared_inter=%d experts=%d top_k=%d rows=%d limit=%g exact=%d" %
          (hidden, inter, shared_inter, experts, top_k, rows, limit, exact), flush=True)
    routed, ref, sh_table, sh_ref = _tables(experts, hidden, inter, shared_inter, 8100 + seed)
    x = (synth.normal((rows, hidden), 1.0, 8200 + seed) * float(rng.choice([0.01, 1.0, 30.0]))).to(torch.bfloat16)
    g = synth.generator(8300 + seed)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    wt = torch.rand((rows, top_k), generator=g) * 0.5 + 0.05
    op = E8m0DecodeOps(routed, sh_table.shared_struct(0), rows, top_k, limit, exact=exact)
    contrib, shared_out = op.contribute(x.to(DEV), ids.to(DEV), wt.to(DEV))
    torch.cuda.synchronize()
    got, got_sh, xb = bits(contrib), bits(shared_out), bits(x)
    ffn = orc.expert_ffn_e8m0 if exact else orc.expert_ffn_e8m0_f32
    for r in range(rows):
        for c in range(top_k):
            assert np.array_equal(got[r, c], ffn(1, xb[r], *ref[int(ids[r, c])], limit, float(wt[r, c]))), (r, c)
        assert np.array_equal(got_sh[r], ffn(0, xb[r], *sh_ref, limit, 1.0)), r


def _down_exact(packed, act_bits, down, sdown):
    """The contract's down projection of one BF16 activation row: quantize per 32, exact dots, BF16."""
    hq, hs = orc.act_quant_e8m0(act_bits[None, :])
    return np.array([orc.scaled_dot_exact(packed, down[d], sdown[d] if packed else sdown[d // 32], hq[0], hs[0])[1]
                     for d in range(down.shape[0])], dtype=np.uint16)


@pytest.mark.parametrize("rows,top_k,experts,hidden,inter,shared_inter", [(40, 3, 6, 256, 128, 128), (130, 2, 3, 384, 256, 128), (5, 4, 9, 128, 128, 256)])
def test_e8m0_prefill_on_the_mx_matrix_cores(rows, top_k, experts, hidden, inter, shared_inter):
    """Cohorts of the W4A8 / W8A8 contract through ffmoe_prefill_contribute: the same quantized operands and stage
    boundaries as the exact decode entry, the dots on v_mfma_scale_f32_16x16x128_f8f6f4 (block scales applied by the
    matrix core, FP32 accumulation in its own order). Checked per stage against the exact oracle: activations, then the
    down projection of the device's own activations."""
    limit = 7.0
    routed, ref, sh_table, sh_ref = _tables(experts, hidden, inter, shared_inter, 500 + rows)
    x = rand_bf16((rows, hidden), 1.0, 510 + rows)
    g = synth.generator(520 + rows)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    wt = torch.rand((rows, top_k), generator=g) * 0.5 + 0.05
    active = torch.ones((rows, top_k), dtype=torch.int32)
    active[1, 0] = 0
    op = PrefillOps(routed, rows, top_k, swiglu=capi.SWIGLU_CLAMPED_ONCE, swiglu_limit=limit, routed_weight=capi.WEIGHT_BEFORE_DOWN_F32,
                    weights_f32=True, shared=sh_table.shared_struct(0), act_mode=capi.ACT_E4M3_E8M0_32)
    op.contributions.zero_()
    got = op.contribute(x.to(DEV), ids.to(DEV), wt.to(DEV), active=active.to(DEV))
    torch.cuda.synchronize()
    assert np.array_equal(op.done.cpu().numpy() != 0, active.numpy() != 0)
    v = op.scratch_views()
    n_live = int(active.sum())
    assert int(v["totals"][3].item()) == n_live
    perm = v["perm"].cpu().numpy()[:n_live]
    act = bits(v["act"])[:n_live]
    g2 = bits(got).reshape(rows * top_k, -1)
    xb = bits(x)
    flat_ids, flat_w = ids.reshape(-1).numpy(), wt.reshape(-1).numpy()
    want_act = np.zeros_like(act)
    want_down = np.zeros((n_live, hidden), dtype=np.uint16)
    want_full = np.zeros((n_live, hidden), dtype=np.uint16)
    for pos, a in enumerate(perm):
        m = ref[int(flat_ids[a])]
        want_full[pos], want_act[pos] = orc.expert_ffn_e8m0(1, xb[a // top_k], *m, limit, float(flat_w[a]), return_act=True)
        want_down[pos] = _down_exact(1, act[pos], m[4], m[5])
    assert_close_with_rare_outliers(act, want_act, "activations", loose=3, rare=ACT_RARE)
    assert_close_bf16(g2[perm], want_down, "down projection of the device activations")
    assert orc.rel_l2(g2[perm], want_full) <= 5e-2
    assert not g2[np.flatnonzero(active.reshape(-1).numpy() == 0)].any()
    so, sh_act = bits(op.shared_out), bits(v["sh_act"])
    want_sa = np.zeros_like(sh_act)
    want_sd = np.zeros_like(so)
    for r in range(rows):
        want_sa[r] = orc.expert_ffn_e8m0(0, xb[r], *sh_ref, limit, 1.0, return_act=True)[1]
        want_sd[r] = _down_exact(0, sh_act[r], sh_ref[4], sh_ref[5])
    assert_close_with_rare_outliers(sh_act, want_sa, "shared activations", loose=3, rare=ACT_RARE)
    assert_close_bf16(so, want_sd, "shared down projection of the device activations")


def test_e8m0_entry_checks_its_contract():
    routed, _, sh_table, _ = _tables(2, 64, 32, 32, 9)
    op = E8m0DecodeOps(routed, sh_table.shared_struct(0), 1, 1, 7.0)
    op.limit = 0.0  # the contract clamps: a limit is required
    x = rand_bf16((1, 64), 1.0, 1).to(DEV)
    ids = torch.zeros((1, 1), dtype=torch.int32, device=DEV)
    with pytest.raises(capi.FfmoeError):
        op.contribute(x, ids, torch.ones((1, 1), device=DEV))


def test_e8m0_rows_whose_scales_span_many_binades_take_the_ordered_path():
    """Block scales spread over ~100 binades: partial sums round, so only the reference's group order gives its bits."""
    experts, hidden, inter, rows, top_k, limit = 3, 256, 128, 2, 2, 7.0
    routed, ref, sh_table, sh_ref = _tables(experts, hidden, inter, inter, 77)
    g = synth.generator(78)
    for e in range(experts):
        v = routed.expert_views(e)
        for i in (1, 3, 5):
            wild = torch.randint(70, 175, v[i].shape, generator=g, dtype=torch.uint8)
            v[i].copy_(wild)
            ref[e][i] = wild.numpy()
    v = sh_table.expert_views(0)
    for i in (1, 3, 5):
        wild = torch.randint(90, 150, v[i].shape, generator=g, dtype=torch.uint8)
        v[i].copy_(wild)
        sh_ref[i] = wild.numpy()
    x = rand_bf16((rows, hidden), 1.0, 79)
    ids = torch.tensor([[0, 2], [1, 0]], dtype=torch.int32)
    wt = torch.tensor([[0.3, 0.2], [0.4, 0.1]])
    op = E8m0DecodeOps(routed, sh_table.shared_struct(0), rows, top_k, limit)
    contrib, shared_out = op.contribute(x.to(DEV), ids.to(DEV), wt.to(DEV))
    torch.cuda.synchronize()
    got, got_sh, xb = bits(contrib), bits(shared_out), bits(x)
    for r in range(rows):
        for c in range(top_k):
            assert np.array_equal(got[r, c], orc.expert_ffn_e8m0(1, xb[r], *ref[int(ids[r, c])], limit, float(wt[r, c]))), (r, c)
        assert np.array_equal(got_sh[r], orc.expert_ffn_e8m0(0, xb[r], *sh_ref, limit, 1.0)), r


@pytest.mark.parametrize("hidden,inter,shared_inter,rows,top_k", [(256, 128, 128, 1, 2), (1024, 512, 384, 3, 3)])
def test_e8m0_fp32_chain_variant_bit_exact(hidden, inter, shared_inter, rows, top_k):
    """act_mode FFMOE_ACT_E4M3_E8M0_32_F32: the reference's 32-lane FP32 kernels, reproduced lane for lane."""
    experts, limit = 5, 7.0
    routed, ref, sh_table, sh_ref = _tables(experts, hidden, inter, shared_inter, 141 + rows)
    x = rand_bf16((rows, hidden), 1.0, 15 + rows)
    g = synth.generator(16 + rows)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    wt = torch.rand((rows, top_k), generator=g) * 0.5 + 0.05
    op = E8m0DecodeOps(routed, sh_table.shared_struct(0), rows, top_k, limit, exact=False)
    contrib, shared_out = op.contribute(x.to(DEV), ids.to(DEV), wt.to(DEV))
    torch.cuda.synchronize()
    got, got_sh, xb = bits(contrib), bits(shared_out), bits(x)
    for r in range(rows):
        for c in range(top_k):
            want = orc.expert_ffn_e8m0_f32(1, xb[r], *ref[int(ids[r, c])], limit, float(wt[r, c]))
            assert np.array_equal(got[r, c], want), (r, c)
        assert np.array_equal(got_sh[r], orc.expert_ffn_e8m0_f32(0, xb[r], *sh_ref, limit, 1.0)), r
    assert np.all(op.done.cpu().numpy() == 1)
