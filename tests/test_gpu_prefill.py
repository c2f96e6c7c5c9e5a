"""GPU parity of the FP8-matrix-core path: the W8A8 block linear and the grouped prefill, through the C ABI.

Oracle: the block-F32 W8A8 arithmetic per assignment (oracle.expert_ffn_w8a8, oracle.linear_fp8_block_w8a8), both in
the reference's 32-lane order and with FP64 accumulation. The matrix cores sum each 128-block in their own order, so
BF16 outputs are compared within 2 BF16 steps / 1e-3 relative L2; grouping, permutation, scatter and done flags are
exact properties.
"""
import numpy as np
import pytest
import torch

import oracle as orc
from flyingfish_amd import capi, ops, synth
from helpers import assert_close_with_rare_outliers, assert_swiglu_close, assert_close_bf16, assert_weighted_down_close, bf16_tensor, bits

pytestmark = pytest.mark.gpu
# Values behind two composed stages (end to end) or behind a twice-rounded product (activations of the matrix-core paths):
# the per-stage bars are 2 steps; here the relative-L2 bar holds on the tensor, no element lies beyond a loose bound, and
# the share of elements beyond 2 steps must stay below these (small shapes: a cancelled output behind one activation that
# rounded the other way moves by several of its own steps).
E2E_RARE = 5e-3
ACT_RARE = 2e-3


def _fp8_matrix(n, k, seed, std=0.02):
    w = synth.normal((n, k), std, seed)
    codes, scales = synth.quant_fp8_block(w)
    return codes, scales


@pytest.mark.parametrize("m,n,k", [(1, 256, 512), (5, 384, 256), (16, 256, 1024), (17, 272, 384), (33, 512, 256), (70, 256, 384), (130, 128, 256)])
def test_linear_w8a8_matches_oracle(m, n, k):
    wc, ws = _fp8_matrix(n, k, 7 + m)
    x = synth.normal((m, k), 1.0, 99 + m, dtype=torch.bfloat16)
    xq, sx = orc.quant_act_fp8_128(bits(x))
    want, want_f32 = orc.linear_fp8_block_w8a8(wc.numpy(), ws.numpy(), xq, sx, order=0, want_f32=True)
    want64 = orc.linear_fp8_block_w8a8(wc.numpy(), ws.numpy(), xq, sx, order=1)
    y = ops.Fp8Ops.linear_w8a8(wc.cuda(), ws.cuda(), torch.from_numpy(xq).cuda(), torch.from_numpy(sx).cuda())
    torch.cuda.synchronize()
    assert_close_bf16(bits(y), want, "w8a8 linear vs 32-lane order", max_ulp=1)
    assert_close_bf16(bits(y), want64, "w8a8 linear vs FP64", max_ulp=1)


def test_linear_w8a8_device_quantizer_chain():
    """ffmoe_linear_fp8_block(act_mode = FP8_BLOCK128) = device quantizer + W8A8 linear."""
    m, n, k = 9, 256, 640
    wc, ws = _fp8_matrix(n, k, 31)
    x = synth.normal((m, k), 1.0, 32, dtype=torch.bfloat16)
    xq, sx = orc.quant_act_fp8_128(bits(x))
    want = orc.linear_fp8_block_w8a8(wc.numpy(), ws.numpy(), xq, sx, order=0)
    y = ops.Fp8Ops.linear(wc.cuda(), ws.cuda(), x.cuda(), act_mode=capi.ACT_FP8_BLOCK128)
    torch.cuda.synchronize()
    assert_close_bf16(bits(y), want, "fp8 block linear, W8A8 mode", max_ulp=1)


def test_linear_w8a8_wrong_scale_cell_is_detected():
    """Mutation control (src/backend/cuda/linear.rs:2236-2250): a swapped scale cell must leave the tolerance."""
    m, n, k = 4, 256, 512
    wc, ws = _fp8_matrix(n, k, 41)
    x = synth.normal((m, k), 1.0, 42, dtype=torch.bfloat16)
    xq, sx = orc.quant_act_fp8_128(bits(x))
    bad = ws.clone()
    bad[0, 1] = bad[0, 1] * 2.0
    want = orc.linear_fp8_block_w8a8(wc.numpy(), bad.numpy(), xq, sx, order=0)
    y = ops.Fp8Ops.linear_w8a8(wc.cuda(), ws.cuda(), torch.from_numpy(xq).cuda(), torch.from_numpy(sx).cuda())
    torch.cuda.synchronize()
    assert orc.rel_l2(bits(y)[:, :128], want[:, :128]) > 1e-2


def _make_fp8_table(experts, hidden, inter, seed):
    table = ops.ExpertTable.allocate(capi.FMT_FP8_BLOCK128, experts, hidden, inter, "cuda")
    host = []
    for e in range(experts):
        mats = []
        views = table.expert_views(e)
        for i, shape in enumerate([(inter, hidden), (inter, hidden), (hidden, inter)]):
            codes, scales = _fp8_matrix(shape[0], shape[1], seed * 1000 + e * 3 + i)
            views[2 * i].copy_(codes)
            views[2 * i + 1].copy_(scales)
            mats += [codes.numpy(), scales.numpy()]
        host.append(mats)
    return table, host


def _routing(rows, top_k, experts, seed, skew=0.0):
    rng = np.random.default_rng(seed)
    p = np.arange(1, experts + 1, dtype=np.float64) ** -skew
    p /= p.sum()
    ids = np.stack([rng.choice(experts, size=top_k, replace=False, p=p) for _ in range(rows)]).astype(np.int32)
    w = rng.uniform(0.05, 1.0, size=(rows, top_k)).astype(np.float32)
    return ids, w


def _check_prefill(op, host, x_bits, ids, w, swiglu, limit, boundary, live, got, table=None, row_step=1, threads=1):
    """Stage-wise parity: every stage is held to the 2-step / 1e-3 bar (gate and up: 1 step) on the inputs it actually saw.
      1. bookkeeping: every live assignment appears once, inside its expert's segment, in ascending order;
      2. the device's activation quantizer (codes and scales of x in the arena) equals the oracle's bit for bit;
      3. gate and up BEFORE SwiGLU, recomputed on the device from the arena's quantized rows by the standalone W8A8
         linear (the same kernel template, other tiling): each within 1 BF16 step / 1e-3 of the oracle's W8A8 linear in
         the reference's 32-lane order and of FP64 accumulation;
      4. act[pos] == two-branch SwiGLU(gate_dev, up_dev) bit for bit (the oracle's SwiGLU applied to the device's
         gate/up), so the grouped launch computed exactly those gate/up values and its epilogue is exact;
      5. contributions against the oracle's re-quantize + down + weighting of the device's own act: <= 2 BF16 steps;
      6. end to end (different stage inputs on the two sides: a gate/up value one step off moves its 128-group's
         activation scale and with it up to 128 codes, see test_w8a8_one_step_gate_differences_amplify_end_to_end):
         assignments whose act equals the oracle's bit for bit must match the full oracle within 2 steps, the whole
         tensor within 1e-2 relative L2 (measured: 2e-4 .. 3e-3, the range the CPU control gives for one-step differences).
    row_step > 1 checks every row_step-th position of each expert segment in stages 3-6 (full-size shapes; rows are
    independent of their cohort, test_prefill_rows_do_not_depend_on_their_cohort)."""
    from helpers import run_parallel
    rows, top_k = ids.shape
    v = op.scratch_views()
    n_live = int(live.sum())
    assert int(v["totals"][3].item()) == n_live
    perm = v["perm"].cpu().numpy()[:n_live]
    offsets = v["offsets"].cpu().numpy()
    flat_ids = ids.reshape(-1)
    assert sorted(perm.tolist()) == np.flatnonzero(live.reshape(-1)).tolist()
    for e in range(len(offsets) - 1):
        seg = perm[offsets[e]:offsets[e + 1]]
        assert np.all(flat_ids[seg] == e) and np.all(np.diff(seg) > 0)
    # 2. quantizer
    xq_o, sx_o = orc.quant_act_fp8_128(x_bits)
    xq_d, sx_d = v["xq"].cpu().numpy(), v["sx"].cpu().numpy()
    assert np.array_equal(xq_d, xq_o) and np.array_equal(sx_d.view(np.uint32), sx_o.view(np.uint32)), "activation quantizer"
    act = bits(v["act"])[:n_live]
    g2 = bits(got).reshape(rows * top_k, -1)
    kind = orc.SILU_SIGMOID2
    checked = []
    for e in range(len(offsets) - 1):
        pos = np.arange(offsets[e], offsets[e + 1])[::row_step]
        if pos.size == 0:
            continue
        if row_step > 1 and offsets[e + 1] - 1 not in pos:
            pos = np.append(pos, offsets[e + 1] - 1)  # the last row of the segment (tail of a short group)
        checked.append(pos)
        tok = perm[pos] // top_k
        g, sg, u, su, d, sd = host[e]
        if table is not None:
            # 3. gate / up before SwiGLU, from the device
            views = table.expert_views(e)
            xq_rows = v["xq"][torch.from_numpy(tok).cuda().long()].contiguous()
            sx_rows = v["sx"][torch.from_numpy(tok).cuda().long()].contiguous()
            g_dev = bits(ops.Fp8Ops.linear_w8a8(views[0], views[1], xq_rows, sx_rows))
            u_dev = bits(ops.Fp8Ops.linear_w8a8(views[2], views[3], xq_rows, sx_rows))
            torch.cuda.synchronize()
            for name, wc, ws, dev in (("gate", g, sg, g_dev), ("up", u, su, u_dev)):
                for order, oname in ((0, "32-lane order"), (1, "FP64")):
                    want = np.concatenate(run_parallel(lambda lo, hi: orc.linear_fp8_block_w8a8(wc, ws, xq_o[tok[lo:hi]], sx_o[tok[lo:hi]], order=order),
                                                       len(tok), threads))
                    assert_close_bf16(dev, want, "expert %d %s before SwiGLU vs %s" % (e, name, oname), max_ulp=1)
            # 4. the grouped launch's activations are exactly SwiGLU of those values
            want_act = orc.silu_mul(g_dev, u_dev, swiglu, limit, kind)
            assert np.array_equal(act[pos], want_act), "expert %d: act != SwiGLU(gate_dev, up_dev)" % e
    checked = np.concatenate(checked)
    # 5. down stage on the device's activations, 6. end to end
    def down_and_full(lo, hi):
        out = []
        for p_ in checked[lo:hi]:
            a = perm[p_]
            g, sg, u, su, d, sd = host[int(flat_ids[a])]
            wa = float(w.reshape(-1)[a])
            full, oact = orc.expert_ffn_w8a8(x_bits[a // top_k], g, sg, u, su, d, sd, wa, swiglu, limit, boundary, return_act=True)
            t_ = a // top_k
            out.append((orc.expert_down_w8a8(act[p_], d, sd, wa, boundary), full, oact, orc.expert_down_w8a8(act[p_], d, sd, apply_weight=False), wa,
                        orc.linear_fp8_block_w8a8(g, sg, xq_o[t_:t_ + 1], sx_o[t_:t_ + 1])[0], orc.linear_fp8_block_w8a8(u, su, xq_o[t_:t_ + 1], sx_o[t_:t_ + 1])[0]))
        return out
    res = [t for chunk in run_parallel(down_and_full, len(checked), threads) for t in chunk]
    want_down = np.stack([t[0] for t in res])
    want_full = np.stack([t[1] for t in res])
    want_act = np.stack([t[2] for t in res])
    a_idx = perm[checked]
    # activations against the oracle's: within 2 steps, an element further away only if it is bit for bit the SwiGLU of a
    # gate and an up value one step from the oracle's (which the gate / up bar allows) - and such elements are rare
    assert np.array_equal(want_act, orc.silu_mul(np.stack([t[5] for t in res]), np.stack([t[6] for t in res]), swiglu, limit, kind))
    assert_swiglu_close(act[checked], np.stack([t[5] for t in res]), np.stack([t[6] for t in res]), swiglu, limit, kind, "prefill activations")
    if boundary == orc.AFTER_DOWN_BF16:
        assert_weighted_down_close(g2[a_idx], np.stack([t[3] for t in res]), [t[4] for t in res], "prefill contributions from the device activations")
    else:
        assert_close_bf16(g2[a_idx], want_down, "prefill contributions from the device activations")
    same = np.array([np.array_equal(act[p_], want_act[i]) for i, p_ in enumerate(checked)])
    if same.any():
        if boundary == orc.AFTER_DOWN_BF16:  # c = bf16(bf16(d) * w): a d one step off is up to three steps of c, see the helper
            assert np.array_equal(want_full[same], want_down[same])
            assert_weighted_down_close(g2[a_idx[same]], np.stack([t[3] for t in res])[same], np.array([t[4] for t in res])[same], "prefill contributions, end to end")
        else:
            assert_close_bf16(g2[a_idx[same]], want_full[same], "prefill contributions, end to end")
    e2e = orc.rel_l2(g2[a_idx], want_full)
    print("prefill end to end: relative L2 %.2e over %d assignments (%d with oracle-identical activations)" % (e2e, len(a_idx), int(same.sum())), flush=True)
    assert e2e <= 1e-2
    return g2


@pytest.mark.parametrize("rows,top_k,experts,hidden,inter,skew", [
    (48, 4, 8, 256, 128, 0.0),     # ~24 rows per expert -> 32-row groups
    (40, 2, 16, 384, 384, 1.1),    # skewed, hidden not a multiple of the 256-column tile
    (7, 3, 32, 256, 256, 0.0),     # fewer rows than experts -> 16-row groups, empty experts
    (200, 4, 6, 256, 128, 1.1),    # > 64 rows on the popular experts -> several groups per expert
])
def test_prefill_matches_per_assignment_oracle(rows, top_k, experts, hidden, inter, skew):
    table, host = _make_fp8_table(experts, hidden, inter, 5)
    ids, w = _routing(rows, top_k, experts, 11, skew)
    x = synth.normal((rows, hidden), 1.0, 12, dtype=torch.bfloat16)
    op = ops.PrefillOps(table, rows, top_k, swiglu=capi.SWIGLU_CLAMPED_TWICE, swiglu_limit=10.0, weights_f32=True)
    got = op.contribute(x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda())
    torch.cuda.synchronize()
    assert int(op.done.sum().item()) == rows * top_k
    _check_prefill(op, host, bits(x), ids, w, orc.CLAMPED_TWICE, 10.0, orc.AFTER_DOWN_BF16, np.ones_like(ids, dtype=bool), got, table)


@pytest.mark.parametrize("seed", range(12))
def test_prefill_seeded_sweep(seed):
    """Cohorts the fixed cases do not visit: 1..300 rows, 1..8 choices, 2..40 experts, hidden and inter any multiple of
    128 from 256 to 640, uniform to heavily skewed routing (experts without rows, one expert with most of them), every
    SwiGLU rounding and both routing-weight boundaries; the configuration is a function of the seed alone."""
    rng = np.random.default_rng(6000 + seed)
    experts = int(rng.choice([2, 5, 8, 17, 40]))
    top_k = int(rng.integers(1, min(8, experts) + 1))
    rows = int(rng.choice([1, 3, 16, 17, 65, 130, 300]))
    # at least two 128-wide blocks per contraction: a single block sum leaves the matrix core with about 14 bits, which
    # for a cancelled output is not always inside two BF16 steps of the row's scale
    hidden, inter = 128 * int(rng.integers(2, 6)), 128 * int(rng.integers(2, 6))
    skew = float(rng.choice([0.0, 1.1, 3.0]))
    mode = int(rng.integers(0, 4))
    limit = float(rng.choice([0.5, 10.0])) if mode in (2, 3) else 0.0
    boundary = int(rng.integers(0, 2))
    print("rows=%d top_k=%d experts=%d hidden=%d inter=%d skew=%g mode=%d limit=%g boundary=%d" %
          (rows, top_k, experts, hidden, inter, skew, mode, limit, boundary), flush=True)
    table, host = _make_fp8_table(experts, hidden, inter, 60 + seed)
    ids, w = _routing(rows, top_k, experts, 6100 + seed, skew)
    x = synth.normal((rows, hidden), 1.0, 6200 + seed, dtype=torch.bfloat16)
    op = ops.PrefillOps(table, rows, top_k, swiglu=mode, swiglu_limit=limit, routed_weight=boundary, weights_f32=True)
    got = op.contribute(x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda())
    torch.cuda.synchronize()
    assert int(op.done.sum().item()) == rows * top_k
    _check_prefill(op, host, bits(x), ids, w, mode, limit, boundary, np.ones_like(ids, dtype=bool), got, table)


@pytest.mark.parametrize("fmt", [capi.FMT_FP8_BLOCK128, capi.FMT_NVFP4, capi.FMT_BF16, capi.FMT_FP8_CHANNEL])
@pytest.mark.parametrize("rows,top_k,experts,hidden,inter,skew,shared", [
    (40, 3, 6, 256, 128, 1.1, True),     # groups of 16..64 rows, shared expert of the same format
    (150, 2, 5, 384, 320, 3.0, False),   # one expert with most of the rows, widths that are 64 mod 128
    (3, 4, 12, 128, 192, 0.0, True),     # fewer rows than experts
])
def test_prefill_w16_matches_the_decode_oracle(fmt, rows, top_k, experts, hidden, inter, skew, shared):
    """act_mode FFMOE_ACT_BF16: the decode path's W*A16 arithmetic for whole cohorts on the BF16 matrix cores, every
    expert format. Stage-wise against the oracle of the decode path (the same effective weights; the matrix core's FP32
    accumulation against the reference's FP32 chains): activations, then the down stage on the device's activations."""
    _check_prefill_w16(fmt, rows, top_k, experts, hidden, inter, skew, shared, capi.SWIGLU_CLAMPED_TWICE, 1.0)


@pytest.mark.parametrize("fmt", [capi.FMT_BF16, capi.FMT_FP8_BLOCK128])
def test_prefill_w16_gelu_twice(fmt):
    """The tanh-GELU activation with two BF16 roundings on BF16 experts, routing weight before the contribution's
    rounding: the configuration the reference binds it to (src/backend/cuda/engine_diffusion.rs:1135-1141)."""
    _check_prefill_w16(fmt, 70, 3, 5, 256, 384, 1.5, True, capi.SWIGLU_GELU_TWICE, 0.0)


def test_prefill_w8a8_rejects_gelu_twice():
    from helpers import make_table
    table, _ = make_table(capi.FMT_FP8_BLOCK128, 2, 128, 128, 5)
    with pytest.raises(capi.FfmoeError) as e:
        op = ops.PrefillOps(table, 4, 1, swiglu=capi.SWIGLU_GELU_TWICE, weights_f32=True)
        ids = torch.zeros((4, 1), dtype=torch.int32, device="cuda")
        op.contribute(torch.zeros((4, 128), dtype=torch.bfloat16, device="cuda"), ids, torch.ones((4, 1), device="cuda"))
    assert e.value.code == capi.ERR_UNSUPPORTED


def _check_prefill_w16(fmt, rows, top_k, experts, hidden, inter, skew, shared, mode, limit):
    from helpers import make_table
    if fmt == capi.FMT_FP8_BLOCK128 and (hidden % 128 or inter % 128):
        pytest.skip("128 x 128 block scales")
    table, ref = make_table(fmt, experts + (1 if shared else 0), hidden, inter, 900 + rows)
    sh = table.shared_struct(experts) if shared else None
    table.experts = experts
    ids, w = _routing(rows, top_k, experts, 910 + rows, skew)
    active = np.ones_like(ids, dtype=np.uint32)
    if rows > 2:
        active[1, 0] = 0
    x = synth.normal((rows, hidden), 1.0, 920 + rows, dtype=torch.bfloat16)
    boundary = capi.WEIGHT_BEFORE_CONTRIBUTION_BF16
    op = ops.PrefillOps(table, rows, top_k, swiglu=mode, swiglu_limit=limit, routed_weight=boundary, weights_f32=True, shared=sh,
                        act_mode=capi.ACT_BF16)
    op.contributions.zero_()
    got = op.contribute(x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda(), active=torch.from_numpy(active).cuda())
    torch.cuda.synchronize()
    assert np.array_equal(op.done.cpu().numpy() != 0, active != 0)
    v = op.scratch_views()
    n_live = int(active.sum())
    assert int(v["totals"][3].item()) == n_live
    perm = v["perm"].cpu().numpy()[:n_live]
    act = bits(v["act"])[:n_live]
    g2 = bits(got).reshape(rows * top_k, -1)
    xb = bits(x)
    flat_ids, flat_w = ids.reshape(-1), w.reshape(-1)
    assert sorted(perm.tolist()) == np.flatnonzero(active.reshape(-1)).tolist()
    want_full = np.zeros_like(g2)
    for pos, a in enumerate(perm):
        ge, ue, de = ref[int(flat_ids[a])]
        want, want_act = orc.expert_ffn(xb[a // top_k], ge, ue, de, float(flat_w[a]), mode, limit, boundary, orc.LANE8, orc.SILU_DIV, return_act=True)
        assert_close_bf16(act[pos][None, :], want_act[None, :], "activations of assignment %d" % a)
        assert_close_bf16(g2[a][None, :], orc.expert_down(act[pos], de, float(flat_w[a]), boundary, orc.LANE8)[None, :], "down stage of assignment %d" % a)
        want_full[a] = want
    # end to end the two stages compose (a flipped BF16 step of an activation moves a cancelled down output by several of
    # its own steps at these widths): the relative-L2 bar on the whole tensor, element-wise a loose bound
    assert_close_with_rare_outliers(g2[perm], want_full[perm], "contributions, end to end", rare=E2E_RARE)
    dead = np.flatnonzero(active.reshape(-1) == 0)
    assert not g2[dead].any()
    if shared:
        ge, ue, de = ref[experts]
        so = bits(op.shared_out)
        sh_act = bits(v["sh_act"])
        want_sh = np.zeros_like(so)
        for r in range(rows):
            want, want_act = orc.expert_ffn(xb[r], ge, ue, de, 1.0, mode, limit, 0, orc.LANE8, orc.SILU_DIV, apply_weight=False, return_act=True)
            assert_close_bf16(sh_act[r][None, :], want_act[None, :], "shared activations row %d" % r)
            assert_close_bf16(so[r][None, :], orc.expert_down(sh_act[r], de, 1.0, 0, orc.LANE8, False)[None, :], "shared down row %d" % r)
            want_sh[r] = want
        assert_close_with_rare_outliers(so, want_sh, "shared_out, end to end", rare=E2E_RARE)


def test_prefill_skips_inactive_invalid_and_out_of_range():
    rows, top_k, experts, hidden, inter = 24, 4, 8, 256, 128
    table, host = _make_fp8_table(experts, hidden, inter, 6)
    ids, w = _routing(rows, top_k, experts, 21)
    ids[3, 1] = 99          # out of range
    ids[5, 0] = -1
    active = np.ones((rows, top_k), dtype=np.int32)
    active[7, 2] = 0
    active[8, :] = 0
    valid = torch.ones(experts, dtype=torch.int32)
    valid[2] = 0
    table.valid = valid.cuda()
    live = (active != 0) & (ids >= 0) & (ids < experts)
    live &= np.where((ids >= 0) & (ids < experts), ids, 0) != 2
    x = synth.normal((rows, hidden), 1.0, 22, dtype=torch.bfloat16)
    op = ops.PrefillOps(table, rows, top_k, swiglu=capi.SWIGLU_TWICE, routed_weight=capi.WEIGHT_BEFORE_CONTRIBUTION_BF16, weights_f32=True)
    sentinel = 0x7fc1
    op.contributions.view(torch.int16).fill_(sentinel)
    got = op.contribute(x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda(), active=torch.from_numpy(active).cuda())
    torch.cuda.synchronize()
    done = op.done.cpu().numpy()
    assert np.array_equal(done != 0, live)
    g = _check_prefill(op, host, bits(x), ids, w, orc.TWICE, 0.0, orc.BEFORE_CONTRIBUTION_BF16, live, got, table)
    assert np.all(g[~live.reshape(-1)] == sentinel), "a skipped assignment was written"


def test_prefill_bf16_routing_weights():
    rows, top_k, experts, hidden, inter = 20, 2, 4, 256, 128
    table, host = _make_fp8_table(experts, hidden, inter, 8)
    ids, w = _routing(rows, top_k, experts, 31)
    wb = torch.from_numpy(w).to(torch.bfloat16)
    x = synth.normal((rows, hidden), 1.0, 33, dtype=torch.bfloat16)
    op = ops.PrefillOps(table, rows, top_k, weights_f32=False)
    got = op.contribute(x.cuda(), torch.from_numpy(ids).cuda(), wb.cuda())
    torch.cuda.synchronize()
    _check_prefill(op, host, bits(x), ids, wb.float().numpy(), orc.TWICE, 0.0, orc.AFTER_DOWN_BF16, np.ones_like(ids, dtype=bool), got, table)


def test_prefill_rows_do_not_depend_on_their_cohort():
    """Per-row arithmetic: a row gives bit-identical contributions whether it is run with 300 other rows (64-row
    groups), in a cohort of 9 (16-row groups) or alone."""
    rows, top_k, experts, hidden, inter = 300, 4, 8, 512, 256
    table, _ = _make_fp8_table(experts, hidden, inter, 9)
    ids, w = _routing(rows, top_k, experts, 41, 1.1)
    x = synth.normal((rows, hidden), 1.0, 42, dtype=torch.bfloat16).cuda()
    ids_d, w_d = torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    full = ops.PrefillOps(table, rows, top_k)
    ref = bits(full.contribute(x, ids_d, w_d)).copy()
    for lo, n in [(0, 9), (123, 1), (290, 10)]:
        part = ops.PrefillOps(table, n, top_k)
        got = bits(part.contribute(x[lo:lo + n].contiguous(), ids_d[lo:lo + n].contiguous(), w_d[lo:lo + n].contiguous()))
        assert np.array_equal(got, ref[lo:lo + n]), "rows %d..%d differ between cohorts" % (lo, lo + n)


@pytest.mark.gpu
@pytest.mark.parametrize("act_mode", [capi.ACT_FP8_BLOCK128, capi.ACT_BF16])
def test_prefill_grouping_switches_leave_every_bit_alone(act_mode, monkeypatch):
    """Rows per group (FFMOE_PREFILL_MF) and the order of the unit list (FFMOE_PREFILL_RGB, FFMOE_PREFILL_TGB) decide which block computes
    what, not what is computed: every setting gives the default run's contributions bit for bit. 700 rows over 6 skewed
    experts give groups of every length and experts with more row groups than the smallest blockings hold; a group
    size a path has no kernel for (8 on the BF16 matrix cores) falls back to its largest, an unknown value is ignored."""
    rows, top_k, experts, hidden, inter = 700, 3, 6, 512, 384
    table, _ = _make_fp8_table(experts, hidden, inter, 19)
    ids, w = _routing(rows, top_k, experts, 43, 1.3)
    x = synth.normal((rows, hidden), 1.0, 44, dtype=torch.bfloat16).cuda()
    ids_d, w_d = torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    op = ops.PrefillOps(table, rows, top_k, act_mode=act_mode)
    monkeypatch.delenv("FFMOE_PREFILL_MF", raising=False)
    monkeypatch.delenv("FFMOE_PREFILL_RGB", raising=False)
    monkeypatch.delenv("FFMOE_PREFILL_TGB", raising=False)
    ref = bits(op.contribute(x, ids_d, w_d)).copy()
    assert np.any(ref != 0)
    for wide in ("0", "1"):   # 64-row groups on the FP8 path: four or eight waves per block
        monkeypatch.setenv("FFMOE_PREFILL_MF", "4")
        monkeypatch.setenv("FFMOE_PREFILL_WIDE", wide)
        op.contributions.zero_()
        assert np.array_equal(bits(op.contribute(x, ids_d, w_d)), ref), "FFMOE_PREFILL_WIDE=%s changes the result" % wide
    monkeypatch.delenv("FFMOE_PREFILL_WIDE")
    for mf, rgb, tgb in [("1", "1", "1"), ("1", "5", "2"), ("2", "3", "1000000"), ("4", "2", "3"), ("4", "1000000", "1"), ("8", "1", "4"),
                         ("8", "4", "2"), ("3", "0", "0"), ("4", "32", "4"), ("4", "16", "5")]:
        monkeypatch.setenv("FFMOE_PREFILL_MF", mf)
        monkeypatch.setenv("FFMOE_PREFILL_RGB", rgb)
        monkeypatch.setenv("FFMOE_PREFILL_TGB", tgb)
        op.contributions.zero_()
        got = bits(op.contribute(x, ids_d, w_d))
        assert np.array_equal(got, ref), "FFMOE_PREFILL_MF=%s FFMOE_PREFILL_RGB=%s FFMOE_PREFILL_TGB=%s changes the result" % (mf, rgb, tgb)


@pytest.mark.parametrize("fmt", [capi.FMT_FP8_BLOCK128, capi.FMT_NVFP4, capi.FMT_BF16, capi.FMT_FP8_CHANNEL])
@pytest.mark.parametrize("rows,mf", [(70, "1"), (70, "4"), (9, "2"), (150, "2")])
def test_prefill_shared_expert_rides_in_the_routed_launches_bitwise(fmt, rows, mf, monkeypatch):
    """W*A16 cohorts: a shared expert of the routed experts' format and width is appended to the routed launches as
    row groups of its own. Its outputs, its activations and the routed contributions are the bits of the separate
    launches (FFMOE_PREFILL_SHARED_RIDE=0), whatever the group size and with rows that do not fill the last group."""
    from helpers import make_table
    top_k, experts, hidden, inter = 3, 5, 256, 384
    table, _ = make_table(fmt, experts + 1, hidden, inter, 300 + rows)
    sh = table.shared_struct(experts)
    table.experts = experts
    ids, w = _routing(rows, top_k, experts, 310 + rows, 1.2)
    x = synth.normal((rows, hidden), 1.0, 320 + rows, dtype=torch.bfloat16).cuda()
    ids_d, w_d = torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    monkeypatch.setenv("FFMOE_PREFILL_MF", mf)
    out = {}
    for ride in ("0", "1"):
        monkeypatch.setenv("FFMOE_PREFILL_SHARED_RIDE", ride)
        op = ops.PrefillOps(table, rows, top_k, swiglu=capi.SWIGLU_TWICE, routed_weight=capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True,
                            shared=sh, act_mode=capi.ACT_BF16)
        op.contributions.zero_(); op.shared_out.zero_(); op.scratch.zero_()
        got = op.contribute(x, ids_d, w_d)
        torch.cuda.synchronize()
        v = op.scratch_views()
        out[ride] = (bits(got).copy(), bits(op.shared_out).copy(), bits(v["sh_act"]).copy(), op.done.cpu().numpy().copy())
    assert np.any(out["0"][1] != 0) and np.any(out["0"][2] != 0)
    for a, b, what in zip(out["0"], out["1"], ("contributions", "shared_out", "shared activations", "done")):
        assert np.array_equal(a, b), what


@pytest.mark.parametrize("fmt", [capi.FMT_FP8_BLOCK128, capi.FMT_BF16])
@pytest.mark.parametrize("rows", [9, 24, 40, 70])
def test_prefill_shared_expert_on_one_wave_blocks_bitwise(fmt, rows, monkeypatch):
    """W*A16 cohorts: a shared expert in launches of its own whose four-wave tiles would not fill the CUs runs on one-wave
    blocks over a quarter of the columns each. Every output element sees the same matrix instructions in the same order:
    shared_out and the shared activations are the bits of the four-wave launches (FFMOE_PREFILL_SHARED_NARROW=0)."""
    from helpers import make_table
    top_k, experts, hidden, inter = 2, 4, 256, 384
    table, _ = make_table(fmt, experts + 1, hidden, inter, 900 + rows)
    sh = table.shared_struct(experts)
    table.experts = experts
    ids, w = _routing(rows, top_k, experts, 910 + rows, 0.5)
    x = synth.normal((rows, hidden), 1.0, 920 + rows, dtype=torch.bfloat16).cuda()
    ids_d, w_d = torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    monkeypatch.setenv("FFMOE_PREFILL_SHARED_RIDE", "0")
    monkeypatch.setenv("FFMOE_SHARED_SPLITK", "0")  # the grouped kernels, also where the split-contraction kernel would take a BF16 expert
    out = {}
    for narrow in ("0", "1"):
        monkeypatch.setenv("FFMOE_PREFILL_SHARED_NARROW", narrow)
        op = ops.PrefillOps(table, rows, top_k, swiglu=capi.SWIGLU_TWICE, routed_weight=capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True,
                            shared=sh, act_mode=capi.ACT_BF16)
        op.contributions.zero_(); op.shared_out.zero_(); op.scratch.zero_()
        print("fmt=%d rows=%d narrow=%s" % (fmt, rows, narrow), flush=True)
        got = op.contribute(x, ids_d, w_d)
        torch.cuda.synchronize()
        v = op.scratch_views()
        out[narrow] = (bits(got).copy(), bits(op.shared_out).copy(), bits(v["sh_act"]).copy())
    assert np.any(out["0"][1] != 0) and np.any(out["0"][2] != 0)
    for a, b, what in zip(out["0"], out["1"], ("contributions", "shared_out", "shared activations")):
        assert np.array_equal(a, b), what


@pytest.mark.parametrize("rows,hidden,inter", [(9, 256, 256), (25, 512, 256), (32, 1792, 512), (33, 256, 768), (64, 768, 256), (65, 512, 512), (130, 256, 256)])
@pytest.mark.parametrize("mode,limit", [(capi.SWIGLU_TWICE, 0.0), (capi.SWIGLU_CLAMPED_ONCE, 3.0), (capi.SWIGLU_GELU_TWICE, 0.0)])
def test_prefill_bf16_shared_expert_on_the_split_contraction_kernel(rows, hidden, inter, mode, limit, monkeypatch):
    """A BF16 shared expert over so few rows that the grouped kernels would give it fewer tiles than CUs runs on blocks whose
    eight waves split the contraction (hidden and intermediate size multiples of 256). Per stage against the oracle at the
    north-star bar: activations from x, the down rows from the kernel's own activations; end to end at the composed bar,
    and next to the grouped kernels' results (FFMOE_SHARED_SPLITK=0)."""
    from helpers import make_table
    top_k, experts = 2, 3
    table, ref = make_table(capi.FMT_BF16, experts + 1, hidden, inter, 930 + rows)
    sh = table.shared_struct(experts)
    table.experts = experts
    ids, w = _routing(rows, top_k, experts, 940 + rows, 0.5)
    x = synth.normal((rows, hidden), 1.0, 950 + rows, dtype=torch.bfloat16)
    monkeypatch.setenv("FFMOE_PREFILL_SHARED_RIDE", "0")
    out = {}
    for split in ("0", "1"):
        monkeypatch.setenv("FFMOE_SHARED_SPLITK", split)
        op = ops.PrefillOps(table, rows, top_k, swiglu=mode, swiglu_limit=limit, routed_weight=capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True,
                            shared=sh, act_mode=capi.ACT_BF16)
        op.contributions.zero_(); op.shared_out.zero_(); op.scratch.zero_()
        print("rows=%d hidden=%d inter=%d mode=%d split=%s" % (rows, hidden, inter, mode, split), flush=True)
        got = op.contribute(x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda())
        torch.cuda.synchronize()
        v = op.scratch_views()
        out[split] = (bits(got).copy(), bits(op.shared_out).copy(), bits(v["sh_act"]).copy())
    assert np.array_equal(out["0"][0], out["1"][0]), "the routed choices do not depend on the shared expert's kernel"
    so, sh_act = out["1"][1], out["1"][2]
    ge, ue, de = ref[experts]
    xb = bits(x)
    want_sh = np.zeros_like(so)
    for r in range(rows):
        want, want_act = orc.expert_ffn(xb[r], ge, ue, de, 1.0, mode, limit, 0, orc.LANE8, orc.SILU_DIV, apply_weight=False, return_act=True)
        assert_close_bf16(sh_act[r][None, :], want_act[None, :], "shared activations row %d" % r)
        assert_close_bf16(so[r][None, :], orc.expert_down(sh_act[r], de, 1.0, 0, orc.LANE8, False)[None, :], "shared down row %d" % r)
        want_sh[r] = want
    assert_close_with_rare_outliers(so, want_sh, "shared_out, end to end", rare=E2E_RARE)
    # (the two kernels' FP32 sums differ in order only, which moves a BF16 result about once in 2^15 elements: no bitwise
    # difference can be demanded of shapes this small)
    assert_close_bf16(sh_act, out["0"][2], "shared activations against the grouped kernels", max_ulp=4)


@pytest.mark.parametrize("rows,hidden,inter", [(4, 1024, 1024), (17, 2048, 1024), (32, 3072, 2048), (25, 1024, 2048), (32, 7168, 2048)])
def test_prefill_split_contraction_kernel_with_the_token_panel_in_lds_bitwise(rows, hidden, inter, monkeypatch):
    """Up to 32 rows, contractions that are multiples of 1024: the split-contraction kernel moves its token panel through LDS
    with row-contiguous requests instead of requesting it in the matrix instruction's lane order. Same operands into the same
    instructions in the same order: activations and shared output are the bits of the lane-order kernel
    (FFMOE_SPLITK_LDS=0), whose parity test_prefill_bf16_shared_expert_on_the_split_contraction_kernel holds; the first
    rows are also checked against the oracle here, since no shape of that test takes this path."""
    from helpers import make_table
    top_k, experts = 2, 3
    table, ref = make_table(capi.FMT_BF16, experts + 1, hidden, inter, 1930 + rows)
    sh = table.shared_struct(experts)
    table.experts = experts
    ids, w = _routing(rows, top_k, experts, 1940 + rows, 0.5)
    x = synth.normal((rows, hidden), 1.0, 1950 + rows, dtype=torch.bfloat16)
    monkeypatch.setenv("FFMOE_PREFILL_SHARED_RIDE", "0")
    monkeypatch.setenv("FFMOE_SHARED_SPLITK", "1")
    out = {}
    for lds in ("0", "1"):
        monkeypatch.setenv("FFMOE_SPLITK_LDS", lds)
        op = ops.PrefillOps(table, rows, top_k, swiglu=capi.SWIGLU_TWICE, swiglu_limit=0.0, routed_weight=capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True,
                            shared=sh, act_mode=capi.ACT_BF16)
        op.contributions.zero_(); op.shared_out.zero_(); op.scratch.zero_()
        print("split contraction rows=%d hidden=%d inter=%d token panel in LDS=%s" % (rows, hidden, inter, lds), flush=True)
        op.contribute(x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda())
        torch.cuda.synchronize()
        out[lds] = (bits(op.shared_out).copy(), bits(op.scratch_views()["sh_act"]).copy())
    assert np.array_equal(out["0"][1], out["1"][1]), "shared activations"
    assert np.array_equal(out["0"][0], out["1"][0]), "shared output"
    assert np.any(out["1"][0] != 0)
    ge, ue, de = ref[experts]
    xb = bits(x)
    for r in sorted({0, rows // 2, rows - 1}):
        _, want_act = orc.expert_ffn(xb[r], ge, ue, de, 1.0, capi.SWIGLU_TWICE, 0.0, 0, orc.LANE8, orc.SILU_DIV, apply_weight=False, return_act=True)
        assert_close_bf16(out["1"][1][r][None, :], want_act[None, :], "shared activations row %d" % r)
        assert_close_bf16(out["1"][0][r][None, :], orc.expert_down(out["1"][1][r], de, 1.0, 0, orc.LANE8, False)[None, :], "shared down row %d" % r)


@pytest.mark.parametrize("fmt,switch", [(capi.FMT_NVFP4, "FFMOE_PREFILL_NVFP4_LINES"), (capi.FMT_FP8_BLOCK128, "FFMOE_PREFILL_FP8_LINES")])
@pytest.mark.parametrize("rows,mf,hidden,inter", [(70, "1", 512, 256), (70, "4", 256, 768), (9, "2", 1024, 256), (150, "2", 256, 512), (200, "wide", 768, 512),
                                                  (33, "1", 384, 640)])
def test_prefill_line_kernels_equal_the_k_block_kernel_bitwise(fmt, switch, rows, mf, hidden, inter, monkeypatch):
    """NVFP4 experts whose rows are whole 128-byte code lines (K a multiple of 256) and block-FP8 experts (K a multiple of
    128) go through kernels that move whole lines, several K blocks at a time and two sets ahead. Same operands into the
    same matrix instructions in the same order: contributions, activations and the riding shared expert's outputs are the
    bits of the per-K-block kernel (the switch = 0), for every group size, one set per contraction, odd numbers of sets
    and rows that do not fill the last group."""
    if fmt == capi.FMT_NVFP4 and (hidden % 256 or inter % 256):
        pytest.skip("the per-K-block kernel serves these contractions either way")
    from helpers import make_table
    top_k, experts = 3, 5
    table, _ = make_table(fmt, experts + 1, hidden, inter, 700 + rows)
    sh = table.shared_struct(experts)
    table.experts = experts
    ids, w = _routing(rows, top_k, experts, 710 + rows, 1.2)
    x = synth.normal((rows, hidden), 1.0, 720 + rows, dtype=torch.bfloat16).cuda()
    ids_d, w_d = torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    if mf == "wide":
        monkeypatch.setenv("FFMOE_PREFILL_MF", "4")
    else:
        monkeypatch.setenv("FFMOE_PREFILL_MF", mf)
        monkeypatch.setenv("FFMOE_PREFILL_WIDE", "0")
    out = {}
    for lines in ("0", "1"):
        monkeypatch.setenv(switch, lines)
        op = ops.PrefillOps(table, rows, top_k, swiglu=capi.SWIGLU_TWICE, routed_weight=capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True,
                            shared=sh, act_mode=capi.ACT_BF16)
        op.contributions.zero_(); op.shared_out.zero_(); op.scratch.zero_()
        print("fmt=%d rows=%d mf=%s hidden=%d inter=%d lines=%s" % (fmt, rows, mf, hidden, inter, lines), flush=True)
        got = op.contribute(x, ids_d, w_d)
        torch.cuda.synchronize()
        v = op.scratch_views()
        out[lines] = (bits(got).copy(), bits(op.shared_out).copy(), bits(v["act"]).copy(), op.done.cpu().numpy().copy())
    assert np.any(out["0"][0] != 0) and np.any(out["0"][1] != 0) and int(out["0"][3].sum()) == rows * top_k
    for a, b, what in zip(out["0"], out["1"], ("contributions", "shared_out", "activations", "done")):
        assert np.array_equal(a, b), what


@pytest.mark.parametrize("rows", [8, 16, 64, 65])
@pytest.mark.parametrize("shared_inter", [256, 512])
def test_decode_nvfp4_cohort_with_a_bf16_shared_expert(rows, shared_inter, monkeypatch):
    """ffmoe_decode_contribute, NVFP4 experts with whole code lines and a BF16 shared expert, 8 rows and more: the routed
    choices run on the line-wise cohort kernel (the bits of ffmoe_prefill_contribute in the W*A16 arithmetic); the shared
    expert stays on the streaming kernels in an arena of its own behind the cohort's (the bits of the all-streaming
    dispatch) up to 24 rows and moves to the matrix cores beyond - in one call and issued stage by stage."""
    from helpers import make_table
    top_k, experts, hidden, inter = 3, 6, 256, 512
    table, _ = make_table(capi.FMT_NVFP4, experts, hidden, inter, 800 + rows)
    sh_table, _ = make_table(capi.FMT_BF16, 1, hidden, shared_inter, 801 + rows)
    sh = sh_table.shared_struct(0)
    ids, w = _routing(rows, top_k, experts, 810 + rows, 1.0)
    x = synth.normal((rows, hidden), 1.0, 820 + rows, dtype=torch.bfloat16).cuda()
    ids_d, w_d = torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    for name in ("FFMOE_DECODE_COHORT_ROWS", "FFMOE_DECODE_SHARED_STREAM_ROWS", "FFMOE_PREFILL_SHARED_RIDE", "FFMOE_SHARED_SPLITK"):
        monkeypatch.delenv(name, raising=False)

    def run(stagewise):
        op = ops.DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True)
        op.contributions.zero_(); op.shared_out.zero_(); op.scratch.zero_()
        if stagewise:
            op.contribute(x, ids_d, w_d, stage=0)
            c, so = op.contribute(x, ids_d, w_d, stage=1)
        else:
            c, so = op.contribute(x, ids_d, w_d)
        torch.cuda.synchronize()
        return bits(c).copy(), bits(so).copy()
    print("rows=%d shared_inter=%d" % (rows, shared_inter), flush=True)
    got_c, got_s = run(False)
    st_c, st_s = run(True)
    assert np.array_equal(got_c, st_c) and np.array_equal(got_s, st_s), "stage by stage = one call"
    monkeypatch.setenv("FFMOE_DECODE_COHORT_ROWS", "0")
    str_c, str_s = run(False)
    monkeypatch.delenv("FFMOE_DECODE_COHORT_ROWS")
    assert np.any(got_c != str_c), "the routed choices did not move to the cohort kernels"
    pre = ops.PrefillOps(table, rows, top_k, swiglu=capi.SWIGLU_TWICE, routed_weight=capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True,
                         act_mode=capi.ACT_BF16)
    want = pre.contribute(x, ids_d, w_d)
    torch.cuda.synchronize()
    assert np.array_equal(got_c, bits(want)), "routed choices: the cohort kernels' bits"
    # and inside the end-to-end bar of the matrix-core path against the streaming kernels
    assert_close_with_rare_outliers(got_c.reshape(rows * top_k, hidden), str_c.reshape(rows * top_k, hidden), "cohort vs streaming contributions", rare=E2E_RARE)
    # the BF16 shared expert (hidden and width multiples of 256): blocks that split the contraction at every cohort size
    assert_close_with_rare_outliers(got_s, str_s, "shared expert on the matrix cores vs streaming", rare=E2E_RARE)
    # without that kernel it stays on the streaming kernels up to 24 rows (their bits) and moves to the grouped kernels beyond
    monkeypatch.setenv("FFMOE_SHARED_SPLITK", "0")
    _, old_s = run(False)
    monkeypatch.delenv("FFMOE_SHARED_SPLITK")
    if rows <= 24:
        assert np.array_equal(old_s, str_s), "shared expert: the streaming kernels' bits"
    else:
        assert_close_with_rare_outliers(old_s, str_s, "shared expert on the grouped kernels vs streaming", rare=E2E_RARE)


@pytest.mark.parametrize("rows,top_k,experts", [(1, 1, 3), (37, 4, 9), (128, 8, 70), (341, 3, 5)])
def test_prefill_single_launch_bookkeeping_equals_the_four_launches(rows, top_k, experts, monkeypatch):
    """Small cohorts (by default up to 256 assignments, here forced up to the kernel's 1024) are counted, planned and listed
    by one block in one launch. Segment offsets,
    the stable permutation, group descriptors, both unit lists and the totals are those of the count / plan / fill
    launches (FFMOE_PREFILL_BOOK_SMALL=0), with inactive, invalid and out-of-range assignments in the input."""
    hidden, inter = 128, 128
    table, _ = _make_fp8_table(experts, hidden, inter, 77)
    ids, w = _routing(rows, top_k, experts, 500 + rows, 1.4)
    ids = ids.copy()
    active = (np.random.default_rng(rows).random(ids.shape) > 0.2).astype(np.uint32)
    if rows > 1:
        ids[rows // 2, 0] = experts + 3   # out of range: skipped
        ids[rows - 1, top_k - 1] = -1
    valid = torch.ones(experts, dtype=torch.int32)
    valid[experts // 2] = 0
    table.valid = valid.cuda()
    x = synth.normal((rows, hidden), 1.0, 510 + rows, dtype=torch.bfloat16).cuda()
    ids_d, w_d, act_d = torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda(), torch.from_numpy(active).cuda()
    seen = {}
    for small in ("0", "1024"):
        monkeypatch.setenv("FFMOE_PREFILL_BOOK_SMALL", small)
        op = ops.PrefillOps(table, rows, top_k, weights_f32=True)
        op.scratch.zero_(); op.contributions.zero_()
        got = op.contribute(x, ids_d, w_d, active=act_d)
        torch.cuda.synchronize()
        v = op.scratch_views()
        live = int(v["totals"][3].item())
        seen[small] = dict(totals=v["totals"].cpu().numpy().copy(), counts=v["counts"].cpu().numpy().copy(), offsets=v["offsets"].cpu().numpy().copy(),
                           gbase=v["gbase"].cpu().numpy().copy(), perm=v["perm"].cpu().numpy()[:live].copy(), out=bits(got).copy(),
                           done=op.done.cpu().numpy().copy())
    for k in seen["0"]:
        assert np.array_equal(seen["0"][k], seen["1024"][k]), k
    flat = ids.reshape(-1)
    keep = (active.reshape(-1) != 0) & (flat >= 0) & (flat < experts) & (flat != experts // 2)
    want = sorted(np.flatnonzero(keep).tolist(), key=lambda a: (flat[a], a))
    assert seen["1024"]["perm"].tolist() == want


def test_prefill_then_combine_layer():
    """contribute -> ordered combine equals the oracle's combine over the oracle's contributions within BF16 noise."""
    rows, top_k, experts, hidden, inter = 32, 4, 8, 256, 128
    table, host = _make_fp8_table(experts, hidden, inter, 10)
    ids, w = _routing(rows, top_k, experts, 51)
    x = synth.normal((rows, hidden), 1.0, 52, dtype=torch.bfloat16)
    op = ops.PrefillOps(table, rows, top_k)
    ids_d = torch.from_numpy(ids).cuda()
    c = op.contribute(x.cuda(), ids_d, torch.from_numpy(w).cuda())
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    y = ops.CombineOps.combine(c, None, ids_d, capi.COMBINE_ROUTED, done=op.done, status=status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    want = orc.combine(bits(c), None, None, ids, None, capi.COMBINE_ROUTED)
    assert np.array_equal(bits(y), want)


def _oracle_shared_w8a8(mats, x_bits, swiglu, limit):
    """(shared_out, activation) of the always-on expert per row: the W8A8 FFN without a routing weight."""
    g, sg, u, su, d, sd = mats
    return [orc.expert_ffn_w8a8(x_bits[r], g, sg, u, su, d, sd, 1.0, swiglu, limit, orc.AFTER_DOWN_BF16, apply_weight=False, return_act=True)
            for r in range(x_bits.shape[0])]


@pytest.mark.parametrize("rows", [1, 5, 40])
def test_prefill_shared_expert(rows):
    """The always-on expert as one dense group through the same kernels: activations within 3 BF16 steps of the oracle,
    shared_out within 2 steps of the oracle's down stage applied to the device activations."""
    top_k, experts, hidden, inter = 2, 6, 256, 384
    table, host = _make_fp8_table(experts + 1, hidden, inter, 12)
    shared = table.shared_struct(experts)
    table.experts = experts
    ids, w = _routing(rows, top_k, experts, 61)
    x = synth.normal((rows, hidden), 1.0, 62, dtype=torch.bfloat16)
    op = ops.PrefillOps(table, rows, top_k, shared=shared)
    got = op.contribute(x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda())
    torch.cuda.synchronize()
    _check_prefill(op, host, bits(x), ids, w, orc.TWICE, 0.0, orc.AFTER_DOWN_BF16, np.ones_like(ids, dtype=bool), got, table)
    # shared expert: scratch regions follow the routed ones (see PrefillOps.scratch_views)
    sh_act = bits(op.scratch_views()["sh_act"])
    g, sg, u, su, d, sd = host[experts]
    want = _oracle_shared_w8a8(host[experts], bits(x), orc.TWICE, 0.0)
    want_act = np.stack([a for _, a in want])
    assert_close_with_rare_outliers(sh_act, want_act, "shared activations", loose=3, rare=ACT_RARE)
    want_out = np.stack([orc.expert_down_w8a8(sh_act[r], d, sd, apply_weight=False) for r in range(rows)])
    assert_close_bf16(bits(op.shared_out), want_out, "shared_out from the device activations")


@pytest.mark.parametrize("rows,top_k", [(1, 4), (3, 2)])
def test_decode_w8a8_act_mode_runs_the_same_arithmetic(rows, top_k):
    """ffmoe_decode_contribute with FFMOE_ACT_FP8_BLOCK128 = the grouped W8A8 path: bit-identical to PrefillOps."""
    experts, hidden, inter = 6, 256, 256
    table, _ = _make_fp8_table(experts + 1, hidden, inter, 13)
    shared = table.shared_struct(experts)
    table.experts = experts
    ids, w = _routing(rows, top_k, experts, 71)
    x = synth.normal((rows, hidden), 1.0, 72, dtype=torch.bfloat16).cuda()
    ids_d, w_d = torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    pre = ops.PrefillOps(table, rows, top_k, shared=shared)
    pre.contribute(x, ids_d, w_d)
    dec = ops.DecodeOps(table, shared, rows, top_k, act_mode=capi.ACT_FP8_BLOCK128, weights_f32=True)
    dec.done.zero_()
    c, s = dec.contribute(x, ids_d, w_d)
    torch.cuda.synchronize()
    assert np.array_equal(bits(c), bits(pre.contributions)) and np.array_equal(bits(s), bits(pre.shared_out))
    assert int(dec.done.sum().item()) == rows * top_k


def test_prefill_token_order_reversal_reverses_outputs_bitwise():
    """Row-permutation invariance (src/backend/cuda/moe/prefill_tests.rs:424-484): feeding the tokens in reverse order
    gives the reversed contributions bit for bit."""
    rows, top_k, experts, hidden, inter = 90, 4, 8, 256, 256
    table, _ = _make_fp8_table(experts, hidden, inter, 14)
    ids, w = _routing(rows, top_k, experts, 81, 1.1)
    x = synth.normal((rows, hidden), 1.0, 82, dtype=torch.bfloat16).cuda()
    ids_d, w_d = torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    op = ops.PrefillOps(table, rows, top_k)
    fwd = bits(op.contribute(x, ids_d, w_d)).copy()
    rev = bits(op.contribute(x.flip(0).contiguous(), ids_d.flip(0).contiguous(), w_d.flip(0).contiguous())).copy()
    assert np.array_equal(rev[::-1], fwd)


def test_prefill_mutation_controls_change_the_output():
    """Swapping two experts' codes, or their scales, must change the contributions that used them
    (src/backend/cuda/moe/prefill_tests.rs:485-535)."""
    rows, top_k, experts, hidden, inter = 40, 2, 4, 256, 128
    table, _ = _make_fp8_table(experts, hidden, inter, 15)
    ids, w = _routing(rows, top_k, experts, 91)
    x = synth.normal((rows, hidden), 1.0, 92, dtype=torch.bfloat16).cuda()
    ids_d, w_d = torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    op = ops.PrefillOps(table, rows, top_k)
    base = bits(op.contribute(x, ids_d, w_d)).copy()
    uses = (ids == 0) | (ids == 1)
    assert uses.any() and (~uses).any()
    for which in (0, 1):  # 0: gate codes, 1: gate scales
        a, b = table.expert_views(0)[which], table.expert_views(1)[which]
        ta = a.clone(); a.copy_(b); b.copy_(ta)
        got = bits(op.contribute(x, ids_d, w_d)).copy()
        changed = np.any(got != base, axis=2)
        assert np.all(changed[uses]) and not np.any(changed[~uses]), "mutation %d" % which
        tb = a.clone(); a.copy_(b); b.copy_(tb)  # swap back
    assert np.array_equal(bits(op.contribute(x, ids_d, w_d)), base)


def test_prefill_graph_replay_equals_eager():
    """Eager-vs-graph bit equality (src/backend/cuda/moe/testing.rs:8-31): the whole call is capturable (no host
    read-back, no memset nodes); three replays with eager work in between all reproduce the eager result."""
    rows, top_k, experts, hidden, inter = 70, 4, 8, 256, 256
    table, _ = _make_fp8_table(experts + 1, hidden, inter, 16)
    shared = table.shared_struct(experts)
    table.experts = experts
    ids, w = _routing(rows, top_k, experts, 95)
    x = synth.normal((rows, hidden), 1.0, 96, dtype=torch.bfloat16).cuda()
    ids_d, w_d = torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    op = ops.PrefillOps(table, rows, top_k, shared=shared)
    eager_c = bits(op.contribute(x, ids_d, w_d)).copy()
    eager_s = bits(op.shared_out).copy()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            op.contribute(x, ids_d, w_d)
    torch.cuda.current_stream().wait_stream(side)
    for it in range(3):
        op.contributions.zero_(); op.shared_out.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(bits(op.contributions), eager_c) and np.array_equal(bits(op.shared_out), eager_s), "replay %d" % it


def _e4m3_pow2(p, negative=False):
    assert -6 <= p <= 8
    return ((p + 7) << 3) | (0x80 if negative else 0)


@pytest.mark.parametrize("big,lost", [((0, 1), 6), ((0, 127), 14), ((5, 70), 14), ((31, 32), 14), ((40, 47), 6)])
def test_matrix_core_block_sum_keeps_13_bits_below_the_largest_product_of_a_group_of_8(big, lost):
    """What bounds the W8A8 kernels' agreement with an FP32 chain, pinned on constructed 128-term blocks: the FP8 matrix
    instruction adds the products of 8 consecutive k exactly down to 2^-13 of the largest product among them and drops
    what lies below; across groups of 8 it keeps FP32's bits. Block: +2^16 and -2^16 at the two `big` positions (they
    cancel), 126 products of 2^(16-d) elsewhere, unit scales. For d <= 13 the sum is exact; for d = 14 .. 26 exactly
    the small products sharing a group of 8 with a big one vanish: 6 of them when both big ones share a group, 14
    otherwise. A 128-term block sum of like-sized products is therefore good to about 2^-13 relative to its largest
    products, against 2^-24 for the reference's FP32 chain: BF16 roundings of gate / up (8 bits) flip in a few percent
    of the positions, never by more than one step."""
    n, k = 16, 128
    ones = torch.ones((1, 1), dtype=torch.float32, device="cuda")
    for d in list(range(0, 14)) + [14, 15, 20, 26]:
        tot = 16 - d
        a = min(8, max(-6, tot // 2))
        b = tot - a
        w = np.full((n, k), _e4m3_pow2(a), dtype=np.uint8)
        x = np.full((1, k), _e4m3_pow2(b), dtype=np.uint8)
        w[:, big[0]] = _e4m3_pow2(8); x[0, big[0]] = _e4m3_pow2(8)
        w[:, big[1]] = _e4m3_pow2(8, True); x[0, big[1]] = _e4m3_pow2(8)
        y = ops.Fp8Ops.linear_w8a8(torch.from_numpy(w).cuda(), ones, torch.from_numpy(x).cuda(), ones)
        torch.cuda.synchronize()
        got = y.float().cpu().numpy()
        kept = 126 if d <= 13 else 126 - lost
        assert np.all(got == kept * 2.0 ** tot), "d=%d: got %r, expected %d x 2^%d" % (d, got[0, :2], kept, tot)


def _nvfp4_table_and_its_fp8_derivation(experts, hidden, inter, seed, small_scales=True):
    """An NVFP4 expert table, the host copies of its experts re-rounded to E4M3 as the W4A8 mode defines it (oracle), and a
    block-FP8 table on the device filled with exactly those derived codes and scales."""
    nv = ops.ExpertTable.allocate(capi.FMT_NVFP4, experts, hidden, inter, "cuda")
    derived = ops.ExpertTable.allocate(capi.FMT_FP8_BLOCK128, experts, hidden, inter, "cuda")
    host = []
    rng = np.random.default_rng(seed)
    for e in range(experts):
        nv_views, fp8_views, entry, gl = nv.expert_views(e), derived.expert_views(e), [], []
        for i, shape in enumerate([(inter, hidden), (inter, hidden), (hidden, inter)]):
            codes, scales, g = synth.quant_nvfp4(synth.normal(shape, 0.02, seed * 1000 + e * 3 + i))
            scales = scales.numpy().copy()
            if small_scales:  # some groups far below the matrix's largest: their re-rounded weights are E4M3 subnormals
                pick = rng.random(scales.shape) < 0.06
                scales[pick] = rng.integers(1, 0x28, size=int(pick.sum()), dtype=np.uint8)
            nv_views[2 * i].copy_(codes)
            nv_views[2 * i + 1].copy_(torch.from_numpy(scales))
            gl.append(g)
            c8, s8 = orc.nvfp4_to_fp8_block(codes.numpy(), scales, g)
            fp8_views[2 * i].copy_(torch.from_numpy(c8))
            fp8_views[2 * i + 1].copy_(torch.from_numpy(s8))
            entry += [c8, s8]
        nv.global_scales[e] = torch.tensor(gl, dtype=torch.float32)
        host.append(tuple(entry))
    return nv, derived, host


@pytest.mark.parametrize("rows,top_k,experts,hidden,inter,skew", [
    (48, 4, 8, 256, 128, 0.0),
    (200, 3, 5, 384, 256, 1.1),    # several 64-row groups per popular expert, hidden not a multiple of the column tile
    (7, 2, 16, 256, 384, 0.0),     # fewer rows than experts
])
def test_prefill_w4a8_nvfp4_experts_on_the_fp8_matrix_cores(rows, top_k, experts, hidden, inter, skew):
    """FP8 activations on NVFP4 experts (act_mode FFMOE_ACT_FP8_BLOCK128 with an NVFP4 table): every weight is rounded to
    E4M3 inside the kernel, on its way through LDS. The cohort must equal, bit for bit, the block-FP8 cohort of a table
    that holds the oracle's derivation of those weights - which proves the in-kernel conversion code for code - and that
    cohort is checked stage by stage against the W8A8 oracle on the derived weights."""
    nv, derived, host = _nvfp4_table_and_its_fp8_derivation(experts, hidden, inter, 31)
    ids, w = _routing(rows, top_k, experts, 32, skew)
    x = synth.normal((rows, hidden), 1.0, 33, dtype=torch.bfloat16)
    x_d, ids_d, w_d = x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    op = ops.PrefillOps(nv, rows, top_k, swiglu=capi.SWIGLU_TWICE, weights_f32=True, act_mode=capi.ACT_FP8_BLOCK128)
    got = op.contribute(x_d, ids_d, w_d)
    torch.cuda.synchronize()
    assert int(op.done.sum().item()) == rows * top_k
    ref_op = ops.PrefillOps(derived, rows, top_k, swiglu=capi.SWIGLU_TWICE, weights_f32=True, act_mode=capi.ACT_FP8_BLOCK128)
    want = ref_op.contribute(x_d, ids_d, w_d)
    torch.cuda.synchronize()
    assert np.array_equal(bits(op.scratch_views()["act"])[:rows * top_k], bits(ref_op.scratch_views()["act"])[:rows * top_k]), "activations"
    assert np.array_equal(bits(got), bits(want)), "contributions differ from the block-FP8 cohort on the derived weights"
    _check_prefill(op, host, bits(x), ids, w, orc.TWICE, 0.0, orc.AFTER_DOWN_BF16, np.ones_like(ids, dtype=bool), got, derived)


def test_decode_w4a8_with_an_nvfp4_shared_expert():
    """ffmoe_decode_contribute(act_mode = FFMOE_ACT_FP8_BLOCK128) on NVFP4 experts with an NVFP4 shared expert: the routed
    choices and the shared expert both through the in-kernel conversion, bit-identical to the derived block-FP8 table."""
    experts, hidden, inter, rows, top_k = 5, 256, 256, 9, 3
    nv, derived, _ = _nvfp4_table_and_its_fp8_derivation(experts + 1, hidden, inter, 41)
    sh_nv, sh_fp8 = nv.shared_struct(experts), derived.shared_struct(experts)
    nv.experts = derived.experts = experts
    ids, w = _routing(rows, top_k, experts, 42)
    x = synth.normal((rows, hidden), 1.0, 43, dtype=torch.bfloat16).cuda()
    ids_d, w_d = torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    out = []
    for table, sh in ((nv, sh_nv), (derived, sh_fp8)):
        dec = ops.DecodeOps(table, sh, rows, top_k, act_mode=capi.ACT_FP8_BLOCK128, weights_f32=True)
        dec.done.zero_()
        c, s = dec.contribute(x, ids_d, w_d)
        torch.cuda.synchronize()
        assert int(dec.done.sum().item()) == rows * top_k
        out.append((bits(c).copy(), bits(s).copy()))
    assert np.array_equal(out[0][0], out[1][0]), "contributions"
    assert np.array_equal(out[0][1], out[1][1]), "shared_out"
    assert out[0][0].any() and out[0][1].any()
