"""GPU parity at the benchmarked dimensions (hidden 7168, intermediate 2048): the steady state of the hand-waited K loops
of the grouped matrix-core kernels (56 and 16 K blocks of 128, 64-row groups, every rows-per-group variant), batched
decode beyond the LDS row budget, and one whole DeepSeek-V3-shape token through NativeMoe with 256 experts in 8 groups.
A handful of experts is materialised (44 MB each); the oracle checks a subset of rows per expert where a full check would
take minutes (rows are independent of their cohort, which tests at small shapes establish bit for bit).
Reference analogues: src/backend/cuda/moe/decode_tests.rs:201-623, src/backend/cuda/moe/reference.rs:613-678."""
import os

import numpy as np
import pytest
import torch

import oracle as orc
from flyingfish_amd import capi, ops, synth
from helpers import assert_close_bf16, assert_close_with_rare_outliers, assert_swiglu_close, assert_weighted_down_close, bits, effective_weights, host_expert, make_table_on_device, run_parallel
from test_gpu_prefill import _check_prefill, _routing

pytestmark = pytest.mark.gpu
H, I = 7168, 2048
THREADS = 12
# end to end through both stages on the matrix-core paths: the largest share of elements further than two BF16 steps from
# the scalar oracle (measured 0 .. 2e-3 at these shapes; cancelled outputs behind activations that rounded the other way)
E2E_RARE = 5e-3
# activations of the MX cohort path against the exact oracle's: a twice-rounded product of gate / up values one step off
# can sit three steps away; such elements must stay rare
ACT_RARE = 2e-3


def test_prefill_w8a8_full_width_every_group_size(monkeypatch):
    """C5 dimensions, 3 experts, 110 rows x top-2 with skewed routing (one expert beyond 64 rows: a full 64-row group and
    a tail group): gate/up runs 56 K blocks, down 16. The default grouping is checked stage by stage against the oracle
    on every 9th row of each expert; every other rows-per-group variant (other kernels, other prefetch depth) must
    reproduce it bit for bit."""
    experts, rows, top_k = 3, 110, 2
    monkeypatch.delenv("FFMOE_PREFILL_MF", raising=False)
    monkeypatch.delenv("FFMOE_PREFILL_RGB", raising=False)
    table = make_table_on_device(capi.FMT_FP8_BLOCK128, experts, H, I, 71)
    host = [host_expert(table, e) for e in range(experts)]
    ids, w = _routing(rows, top_k, experts, 72, 1.2)
    counts = np.bincount(ids.reshape(-1), minlength=experts)
    assert counts.max() > 64 and counts.min() >= 1, counts
    x = synth.normal((rows, H), 1.0, 73, dtype=torch.bfloat16)
    op = ops.PrefillOps(table, rows, top_k, swiglu=capi.SWIGLU_TWICE, weights_f32=True)
    x_d, ids_d, w_d = x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    print("full-width W8A8 cohort, default grouping, rows per expert", counts.tolist(), flush=True)
    got = op.contribute(x_d, ids_d, w_d)
    torch.cuda.synchronize()
    ref = bits(got).copy()
    assert int(op.done.sum().item()) == rows * top_k
    _check_prefill(op, host, bits(x), ids, w, orc.TWICE, 0.0, orc.AFTER_DOWN_BF16, np.ones_like(ids, dtype=bool), got, table,
                   row_step=9, threads=THREADS)
    for mf in ("1", "2", "4", "8"):
        monkeypatch.setenv("FFMOE_PREFILL_MF", mf)
        print("full-width W8A8 cohort, FFMOE_PREFILL_MF=" + mf, flush=True)
        op.contributions.zero_()
        again = bits(op.contribute(x_d, ids_d, w_d))
        assert np.array_equal(again, ref), "FFMOE_PREFILL_MF=%s changes the result at 56 / 16 K blocks" % mf
    monkeypatch.delenv("FFMOE_PREFILL_MF")
    monkeypatch.setenv("FFMOE_PREFILL_WIDE", "0")   # 64-row groups with four waves per block instead of eight
    op.contributions.zero_()
    assert np.array_equal(bits(op.contribute(x_d, ids_d, w_d)), ref), "FFMOE_PREFILL_WIDE=0 changes the result"


def test_prefill_w8a8_cohort_beyond_64_k_blocks(monkeypatch):
    """A contraction of 66 K blocks (hidden 8448) through the grouped kernels: the block scales are held 64 K blocks at a
    time and re-armed inside the K loop. Stage-wise against the oracle on every 11th row, and every kernel variant bit for
    bit against the default one."""
    experts, rows, top_k, hidden, inter = 2, 150, 1, 8448, 256
    for k in ("FFMOE_PREFILL_MF", "FFMOE_PREFILL_RGB", "FFMOE_PREFILL_WIDE"):
        monkeypatch.delenv(k, raising=False)
    table = make_table_on_device(capi.FMT_FP8_BLOCK128, experts, hidden, inter, 171)
    host = [host_expert(table, e) for e in range(experts)]
    ids, w = _routing(rows, top_k, experts, 172, 0.5)
    x = synth.normal((rows, hidden), 1.0, 173, dtype=torch.bfloat16)
    op = ops.PrefillOps(table, rows, top_k, swiglu=capi.SWIGLU_TWICE, weights_f32=True)
    x_d, ids_d, w_d = x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    print("W8A8 cohort at 66 K blocks, default grouping", flush=True)
    got = op.contribute(x_d, ids_d, w_d)
    torch.cuda.synchronize()
    ref = bits(got).copy()
    _check_prefill(op, host, bits(x), ids, w, orc.TWICE, 0.0, orc.AFTER_DOWN_BF16, np.ones_like(ids, dtype=bool), got, table,
                   row_step=11, threads=THREADS)
    for mf, wide in (("4", "0"), ("1", "1"), ("2", "1"), ("8", "1")):
        monkeypatch.setenv("FFMOE_PREFILL_MF", mf)
        monkeypatch.setenv("FFMOE_PREFILL_WIDE", wide)
        print("W8A8 cohort at 66 K blocks, FFMOE_PREFILL_MF=%s FFMOE_PREFILL_WIDE=%s" % (mf, wide), flush=True)
        op.contributions.zero_()
        assert np.array_equal(bits(op.contribute(x_d, ids_d, w_d)), ref), (mf, wide)


@pytest.mark.parametrize("m", [3, 40, 70, 130])
def test_linear_w8a8_more_than_64_k_blocks(m):
    """K = 8448 = 66 K blocks: the block-scale registers are re-armed after 64 blocks; every rows-per-group kernel."""
    n, k = 256, 8448
    w = synth.normal((n, k), 0.02, 81)
    wc, ws = synth.quant_fp8_block(w)
    x = synth.normal((m, k), 1.0, 82 + m, dtype=torch.bfloat16)
    xq, sx = orc.quant_act_fp8_128(bits(x))
    print("W8A8 linear m=%d n=%d k=%d" % (m, n, k), flush=True)
    y = ops.Fp8Ops.linear_w8a8(wc.cuda(), ws.cuda(), torch.from_numpy(xq).cuda(), torch.from_numpy(sx).cuda())
    torch.cuda.synchronize()
    for order in (0, 1):
        want = np.concatenate(run_parallel(lambda lo, hi: orc.linear_fp8_block_w8a8(wc.numpy(), ws.numpy(), xq[lo:hi], sx[lo:hi], order=order), m, THREADS))
        assert_close_bf16(bits(y), want, "w8a8 linear, 66 K blocks, order %d" % order, max_ulp=1)


@pytest.mark.parametrize("fmt", [capi.FMT_FP8_BLOCK128, capi.FMT_NVFP4, capi.FMT_BF16, capi.FMT_FP8_CHANNEL])
def test_prefill_w16_full_width(fmt, monkeypatch):
    """The W*A16 cohort kernels (BF16 matrix cores) at 7168 / 2048: 112 and 32 K blocks of 64, 64-row groups and a tail,
    shared expert as a dense group. Stage-wise against the decode oracle on a subset of rows; the other rows-per-group
    variants reproduce the default bit for bit."""
    experts, rows, top_k = 2, 90, 2
    monkeypatch.delenv("FFMOE_PREFILL_MF", raising=False)
    table = make_table_on_device(fmt, experts + 1, H, I, 91 + fmt)
    sh = table.shared_struct(experts)
    table.experts = experts
    ref = [effective_weights(table, e) for e in range(experts + 1)]
    ids = np.stack([np.array([0, 1], dtype=np.int32) for _ in range(rows)])  # every row on both experts: 90 rows each
    w = np.random.default_rng(92).uniform(0.05, 1.0, size=(rows, top_k)).astype(np.float32)
    x = synth.normal((rows, H), 1.0, 93, dtype=torch.bfloat16)
    mode, limit, boundary = capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16
    op = ops.PrefillOps(table, rows, top_k, swiglu=mode, swiglu_limit=limit, routed_weight=boundary, weights_f32=True, shared=sh, act_mode=capi.ACT_BF16)
    x_d, ids_d, w_d = x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda()
    print("full-width W*A16 cohort fmt=%d" % fmt, flush=True)
    got = op.contribute(x_d, ids_d, w_d)
    torch.cuda.synchronize()
    g2 = bits(got).reshape(rows * top_k, -1).copy()
    so = bits(op.shared_out).copy()
    v = op.scratch_views()
    perm = v["perm"].cpu().numpy()[:rows * top_k]
    act = bits(v["act"])[:rows * top_k]
    sh_act = bits(v["sh_act"])
    xb = bits(x)
    check = list(range(0, rows * top_k, 13)) + [rows - 1, rows, rows * top_k - 1]  # positions in expert order, incl. both tails

    def one(lo, hi):
        out = []
        for pos in check[lo:hi]:
            a = int(perm[pos])
            ge, ue, de = ref[int(ids.reshape(-1)[a])]
            want = orc.expert_ffn(xb[a // top_k], ge, ue, de, float(w.reshape(-1)[a]), mode, limit, boundary, orc.LANE8, orc.SILU_DIV)
            xr = xb[a // top_k][None, :]
            out.append((pos, a, want, orc.linear_skinny(ge, xr, 2)[0], orc.linear_skinny(ue, xr, 2)[0], orc.expert_down(act[pos], de, 1.0, boundary, orc.LANE8, False)))
        return out
    e2e_got, e2e_want, acts, g_refs, u_refs, downs, wts_ = [], [], [], [], [], [], []
    for chunk in run_parallel(one, len(check), THREADS):
        for pos, a, want, g_ref, u_ref, down_ref in chunk:
            acts.append(act[pos]); g_refs.append(g_ref); u_refs.append(u_ref); downs.append(down_ref); wts_.append(float(w.reshape(-1)[a]))
            e2e_got.append(g2[a]); e2e_want.append(want)
    # each stage at the bar on its own inputs: activations within 2 steps of SwiGLU(gate, up) from FP64 accumulation, an
    # element further away only if a gate / up one step off explains it bit for bit
    assert_swiglu_close(np.stack(acts), np.stack(g_refs), np.stack(u_refs), mode, limit, orc.SILU_DIV, "activations vs SwiGLU of the FP64-accumulated gate / up")
    assert_weighted_down_close(np.stack(e2e_got), np.stack(downs), wts_, "down stage on the device activations")
    # end to end the two stages compose (a flipped BF16 step of an activation moves every down output a little): the
    # relative-L2 bar on the checked tensor, few elements beyond two steps, none beyond a loose bound
    r_, worst_, frac_ = assert_close_with_rare_outliers(np.stack(e2e_got), np.stack(e2e_want), "contributions, end to end", rare=E2E_RARE)
    print("end to end: relative L2 %.2e, worst %.1f steps, %.2e beyond 2 steps" % (r_, worst_, frac_), flush=True)
    ge, ue, de = ref[experts]
    rows_sh = [0, 15, 16, 63, 64, rows - 1]

    def shared_rows(lo, hi):
        return [(r, orc.expert_ffn(xb[r], ge, ue, de, 1.0, mode, limit, 0, orc.LANE8, orc.SILU_DIV, apply_weight=False, return_act=True),
                 orc.expert_down(sh_act[r], de, 1.0, 0, orc.LANE8, False)) for r in rows_sh[lo:hi]]
    for chunk in run_parallel(shared_rows, len(rows_sh), THREADS):
        for r, (want, want_act), want_down in chunk:
            assert_close_bf16(sh_act[r][None, :], want_act[None, :], "shared activations row %d" % r)
            assert_close_bf16(so[r][None, :], want_down[None, :], "shared down row %d" % r)
    for mf in ("1", "2"):
        monkeypatch.setenv("FFMOE_PREFILL_MF", mf)
        print("full-width W*A16 cohort fmt=%d FFMOE_PREFILL_MF=%s" % (fmt, mf), flush=True)
        op.contributions.zero_()
        again = bits(op.contribute(x_d, ids_d, w_d)).reshape(rows * top_k, -1)
        assert np.array_equal(again, g2), "FFMOE_PREFILL_MF=%s changes the result" % mf


def test_prefill_mx_full_width(monkeypatch):
    """The E2M1/E8M0 cohort kernel (MX matrix cores) at 7168 / 2048, 56 and 16 K blocks, 64-row group plus tail, with the
    E4M3/E8M0 shared expert: stage-wise against the exact oracle on a subset of rows, other group sizes bit for bit."""
    from test_gpu_e8m0 import _down_exact
    experts, rows, top_k, limit = 2, 80, 2, 7.0
    monkeypatch.delenv("FFMOE_PREFILL_MF", raising=False)
    routed = make_table_on_device(capi.FMT_E2M1_E8M0, experts, H, I, 101, std=0.05)
    sh_table = make_table_on_device(capi.FMT_E4M3_E8M0_32, 1, H, I, 102, std=0.05)
    ref = [host_expert(routed, e) for e in range(experts)]
    sh_ref = host_expert(sh_table, 0)
    ids = np.stack([np.array([0, 1], dtype=np.int32) for _ in range(rows)])
    wt = np.random.default_rng(103).uniform(0.05, 0.55, size=(rows, top_k)).astype(np.float32)
    x = synth.normal((rows, H), 1.0, 104, dtype=torch.bfloat16)
    op = ops.PrefillOps(routed, rows, top_k, swiglu=capi.SWIGLU_CLAMPED_ONCE, swiglu_limit=limit, routed_weight=capi.WEIGHT_BEFORE_DOWN_F32,
                        weights_f32=True, shared=sh_table.shared_struct(0), act_mode=capi.ACT_E4M3_E8M0_32)
    x_d, ids_d, w_d = x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(wt).cuda()
    print("full-width MX cohort", flush=True)
    got = op.contribute(x_d, ids_d, w_d)
    torch.cuda.synchronize()
    g2 = bits(got).reshape(rows * top_k, -1).copy()
    so = bits(op.shared_out).copy()
    v = op.scratch_views()
    perm = v["perm"].cpu().numpy()[:rows * top_k]
    act = bits(v["act"])[:rows * top_k]
    sh_act = bits(v["sh_act"])
    xb = bits(x)
    check = [0, 17, 63, 64, rows - 1, rows, rows + 40, rows * top_k - 1]

    def one(lo, hi):
        out = []
        for pos in check[lo:hi]:
            a = int(perm[pos])
            m = ref[int(ids.reshape(-1)[a])]
            full, want_act = orc.expert_ffn_e8m0(1, xb[a // top_k], *m, limit, float(wt.reshape(-1)[a]), return_act=True)
            out.append((pos, a, full, want_act, _down_exact(1, act[pos], m[4], m[5])))
        return out
    for chunk in run_parallel(one, len(check), THREADS):
        for pos, a, full, want_act, want_down in chunk:
            assert_close_with_rare_outliers(act[pos][None, :], want_act[None, :], "activations of assignment %d" % a, loose=3, rare=ACT_RARE)
            assert_close_bf16(g2[a][None, :], want_down[None, :], "down projection of the device activations, assignment %d" % a)
    rows_sh = [0, 33, rows - 1]

    def shared_rows(lo, hi):
        return [(r, orc.expert_ffn_e8m0(0, xb[r], *sh_ref, limit, 1.0, return_act=True)[1], _down_exact(0, sh_act[r], sh_ref[4], sh_ref[5])) for r in rows_sh[lo:hi]]
    for chunk in run_parallel(shared_rows, len(rows_sh), THREADS):
        for r, want_act, want_down in chunk:
            assert_close_with_rare_outliers(sh_act[r][None, :], want_act[None, :], "shared activations row %d" % r, loose=3, rare=ACT_RARE)
            assert_close_bf16(so[r][None, :], want_down[None, :], "shared down projection row %d" % r)
    for mf in ("1", "2"):
        monkeypatch.setenv("FFMOE_PREFILL_MF", mf)
        print("full-width MX cohort FFMOE_PREFILL_MF=" + mf, flush=True)
        op.contributions.zero_()
        again = bits(op.contribute(x_d, ids_d, w_d)).reshape(rows * top_k, -1)
        assert np.array_equal(again, g2), "FFMOE_PREFILL_MF=%s changes the result" % mf


def _cpubase_contributions(table, x_bits, ids, wts, shared_e, boundary):
    """Contributions [rows, top_k, H], shared_out [rows, H] and activations from the multithreaded CPU port (bit-equal to
    the scalar oracle in Lane16 / reciprocal-SiLU form, tests/test_host_contract.py)."""
    rows, top_k = ids.shape
    cache = {}

    def host(e):
        if e not in cache:
            cache[e] = tuple(host_expert(table, e))
        return cache[e]
    experts, rws, w, ap = [], [], [], []
    for r in range(rows):
        for c in range(top_k):
            experts.append(host(int(ids[r, c]))); rws.append(r); w.append(float(wts[r, c])); ap.append(1)
    for r in range(rows):
        experts.append(host(shared_e)); rws.append(r); w.append(1.0); ap.append(0)
    job = orc.CpuDecodeJob(x_bits, rws, experts, w, ap, boundary)
    out = job.run(THREADS)
    A = rows * top_k
    return out[:A].reshape(rows, top_k, -1), out[A:], job.act


@pytest.mark.parametrize("rows", [8, 33])
def test_decode_fp8_full_width_beyond_the_lds_row_budget(rows, monkeypatch):
    """Hidden 7168 with 8 and 33 rows on the streaming kernels: a block's LDS holds 4 token rows at this width, so the
    shared expert is served in several row groups and a popular expert in more than one. Every contribution and shared
    row against the CPU port (Lane16), three of them also against the scalar oracle. (The rule that hands the shared
    expert of larger batches to the matrix-core kernels is switched off here and checked end to end below.)"""
    experts, top_k = 6, 4
    monkeypatch.setenv("FFMOE_DECODE_COHORT_ROWS", "0")
    monkeypatch.setenv("FFMOE_DECODE_SHARED_COHORT_ROWS", "0")
    table = make_table_on_device(capi.FMT_FP8_BLOCK128, experts + 1, H, I, 111)
    sh = table.shared_struct(experts)
    table.experts = experts
    g = synth.generator(112 + rows)
    x = synth.normal((rows, H), 1.0, 113 + rows).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    wt = torch.rand((rows, top_k), generator=g) * 0.5 + 0.05
    op = ops.DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True)
    op.contributions.zero_()
    print("full-width decode rows=%d" % rows, flush=True)
    contrib, shared_out = op.contribute(x.cuda(), ids.cuda(), wt.cuda())
    torch.cuda.synchronize()
    assert int(op.done.sum().item()) == rows * top_k
    want_c, want_s, want_act = _cpubase_contributions(table, bits(x), ids.numpy(), wt.numpy(), experts, orc.AFTER_DOWN_BF16)
    A = rows * top_k
    got_c, got_s = bits(contrib), bits(shared_out)
    # each launch on its own inputs: activations against the CPU port's, the down stage against the oracle's down stage on
    # the device's activations; end to end the relative-L2 bar and four steps (one flipped BF16 step of an activation
    # moves a cancelled down output by more than two of its own steps)
    h = bits(op.scratch[: (A + rows) * I * 2].view(torch.bfloat16).view(A + rows, I))
    eff = [effective_weights(table, e) for e in range(experts + 1)]
    jobs = [(r, c) for r in range(rows) for c in range(top_k)] + [(r, -1) for r in range(rows)]
    xb = bits(x)

    def stages(lo, hi):
        out = []
        for r, c in jobs[lo:hi]:
            ge, ue, de = eff[int(ids[r, c])] if c >= 0 else eff[experts]
            a = r * top_k + c if c >= 0 else A + r
            out.append((orc.linear_skinny(ge, xb[r][None, :], 2)[0], orc.linear_skinny(ue, xb[r][None, :], 2)[0],
                        orc.expert_down(h[a], de, 1.0, 0, orc.LANE8, False)))
        return out
    res = [t for chunk in run_parallel(stages, len(jobs), THREADS) for t in chunk]
    assert_swiglu_close(h, np.stack([t[0] for t in res]), np.stack([t[1] for t in res]), orc.TWICE, 0.0, orc.SILU_DIV,
                        "activations vs SwiGLU of the FP64-accumulated gate / up")
    d_ref = np.stack([t[2] for t in res])
    assert_weighted_down_close(got_c.reshape(A, -1), d_ref[:A], wt.numpy().reshape(-1), "down stage on the device activations")
    assert_close_bf16(got_s, d_ref[A:], "shared down stage on the device activations")
    r_, worst_ = assert_close_bf16(got_c, want_c, "contributions vs the CPU port, end to end", max_ulp=4)
    print("contributions end to end: relative L2 %.2e, worst %.1f steps" % (r_, worst_), flush=True)
    assert_close_bf16(got_s, want_s, "shared_out vs the CPU port, end to end", max_ulp=4)
    for r, c in [(0, 0), (rows // 2, 1), (rows - 1, top_k - 1)]:
        ge, ue, de = effective_weights(table, int(ids[r, c]))
        want = orc.expert_ffn(xb[r], ge, ue, de, float(wt[r, c]), orc.TWICE, 0.0, orc.AFTER_DOWN_BF16, orc.LANE8, orc.SILU_DIV)
        assert_close_bf16(got_c[r, c][None, :], want[None, :], "contribution (%d, %d) vs the scalar oracle" % (r, c), max_ulp=4)
    # the default dispatch of the same batch (from 4 rows the whole batch on the matrix cores, the shared expert riding in
    # the routed launches): same bars end to end
    monkeypatch.delenv("FFMOE_DECODE_COHORT_ROWS")
    monkeypatch.delenv("FFMOE_DECODE_SHARED_COHORT_ROWS")
    op.contributions.zero_(); op.shared_out.zero_()
    c2, s2 = op.contribute(x.cuda(), ids.cuda(), wt.cuda())
    torch.cuda.synchronize()
    if rows < 4:
        assert np.array_equal(bits(c2), got_c) and np.array_equal(bits(s2), got_s), "small batches stay on the streaming kernels"
    # on the matrix cores the two stages compose as in test_prefill_w16_full_width (each stage inside its bar there): the
    # relative-L2 bar on the tensor, element-wise a loose bound for cancelled outputs
    if rows >= 4:
        # stage by stage as above: the cohort launches leave their activations in the prefill arena
        v = ops.PrefillOps.arena_views(op.scratch, table, rows, top_k, sh)
        perm2 = v["perm"].cpu().numpy()[:A]
        act2 = np.empty((A + rows, I), dtype=np.uint16)
        act2[perm2] = bits(v["act"])[:A]
        act2[A:] = bits(v["sh_act"])
        assert_swiglu_close(act2, np.stack([t[0] for t in res]), np.stack([t[1] for t in res]), orc.TWICE, 0.0, orc.SILU_DIV,
                            "cohort path: activations vs SwiGLU of the FP64-accumulated gate / up")

        def downs(lo, hi):
            return [orc.expert_down(act2[r * top_k + c if c >= 0 else A + r], eff[int(ids[r, c])][2] if c >= 0 else eff[experts][2], 1.0, 0, orc.LANE8, False)
                    for r, c in jobs[lo:hi]]
        d2 = np.stack([t for chunk in run_parallel(downs, len(jobs), THREADS) for t in chunk])
        assert_weighted_down_close(bits(c2).reshape(A, -1), d2[:A], wt.numpy().reshape(-1), "cohort path: down stage on the device activations")
        assert_close_bf16(bits(s2), d2[A:], "cohort path: shared down stage on the device activations")
    for name, got_, want_ in (("contributions", bits(c2), want_c), ("shared_out", bits(s2), want_s)):
        r_, worst_, frac_ = assert_close_with_rare_outliers(got_, want_, name + " of the default dispatch vs the CPU port, end to end",
                                                            loose=16 if rows >= 4 else 4, rare=E2E_RARE)
        print("default dispatch, %s end to end: relative L2 %.2e, worst %.1f steps, %.2e beyond 2 steps" % (name, r_, worst_, frac_), flush=True)


def test_decode_nvfp4_full_width_batched():
    """C4 dimensions, 9 rows: NVFP4 routed experts with a BF16 shared expert (a cohort pass and a streaming pass, an arena
    each) at hidden 7168."""
    experts, top_k, rows = 4, 3, 9
    table = make_table_on_device(capi.FMT_NVFP4, experts, H, I, 121)
    sh_table = make_table_on_device(capi.FMT_BF16, 1, H, I, 122)
    sh = sh_table.shared_struct(0)
    g = synth.generator(123)
    x = synth.normal((rows, H), 1.0, 124).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    wt = torch.rand((rows, top_k), generator=g) * 0.5 + 0.05
    op = ops.DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True)
    print("full-width NVFP4 decode rows=%d" % rows, flush=True)
    contrib, shared_out = op.contribute(x.cuda(), ids.cuda(), wt.cuda())
    torch.cuda.synchronize()
    ref = [effective_weights(table, e) for e in range(experts)]
    sref = effective_weights(sh_table, 0)
    xb, got, got_s = bits(x), bits(contrib), bits(shared_out)
    jobs = [(r, c) for r in range(rows) for c in range(top_k)] + [(r, -1) for r in range(rows)]

    def one(lo, hi):
        out = []
        for r, c in jobs[lo:hi]:
            if c >= 0:
                ge, ue, de = ref[int(ids[r, c])]
                out.append(orc.expert_ffn(xb[r], ge, ue, de, float(wt[r, c]), orc.TWICE, 0.0, orc.AFTER_DOWN_BF16, orc.LANE8, orc.SILU_DIV))
            else:
                out.append(orc.expert_ffn(xb[r], *sref, 1.0, orc.TWICE, 0.0, 0, orc.LANE8, orc.SILU_DIV, apply_weight=False))
        return out
    res = [t for chunk in run_parallel(one, len(jobs), THREADS) for t in chunk]
    # 9 rows: the routed choices run on the line-wise cohort kernel (both stages on the matrix cores compose as in
    # test_prefill_w16_full_width: the relative-L2 bar on the row, element-wise a loose bound for cancelled outputs), the
    # shared expert on the streaming kernels
    for (r, c), want in zip(jobs, res):
        if c >= 0:
            assert_close_with_rare_outliers(got[r, c][None, :], want[None, :], "contribution (%d, %d)" % (r, c), rare=E2E_RARE)
        else:
            assert_close_bf16(got_s[r][None, :], want[None, :], "shared_out row %d" % r)


def _sparse_c3_table(hit, seed):
    """A 256-expert table at the C3 dimensions in which only the experts in `hit` (and the shared expert) are
    materialised; every other slot points at one spare expert, so a wrong selection still reads valid memory."""
    store = make_table_on_device(capi.FMT_FP8_BLOCK128, len(hit) + 2, H, I, seed)
    rows = store.slots.cpu()
    slots = rows[len(hit) + 1].repeat(256, 1)
    for i, e in enumerate(hit):
        slots[e] = rows[i]
    table = ops.ExpertTable(capi.FMT_FP8_BLOCK128, 256, H, I, store.storage, slots.cuda())
    return table, store, store.shared_struct(len(hit))


def test_c3_token_through_native_moe_256_experts_8_groups():
    """One DeepSeek-V3-shape token end to end: FP32 router logits over 256 experts, sigmoid grouped top-8 (8 groups, keep
    4) x 2.5, FP8 experts + shared expert, ungated combine. ids and weights bit for bit against the oracle, the 8
    contributions and the shared row against the oracle's FFN, y bit for bit against the oracle's combine of the device's
    contributions and within the layer bound of the oracle's own pipeline; all launch variants give the same bits."""
    E, K = 256, 8
    router = synth.normal((E, H), 0.02, 131).to(torch.bfloat16)
    bias = synth.normal((E,), 0.01, 132)
    x = synth.normal((1, H), 1.0, 133).to(torch.bfloat16)
    lg = orc.route_logits_f32(bits(x), bits(router))
    oi, ow = orc.route_topk_noaux(lg, bias.numpy()[None, :], K, 0, 2.5, 8, 4)
    hit = [int(e) for e in oi[0]]
    table, store, shared = _sparse_c3_table(hit, 134)
    layer = ops.NativeMoe(table, shared, router.cuda(), bias.cuda(), 1, K, 2.5, 8, 4, swiglu=capi.SWIGLU_TWICE,
                          routed_weight=capi.WEIGHT_AFTER_DOWN_BF16, combine_mode=capi.COMBINE_UNGATED)
    layer.two_launch = False  # the separate launches first: they write contributions and shared_out
    print("C3 token through NativeMoe, experts hit", hit, flush=True)
    y = bits(layer.run(x.cuda())).copy()
    torch.cuda.synchronize()
    assert int(layer.status.item()) == 0
    assert np.array_equal(layer.ids.cpu().numpy(), oi), "router ids"
    assert np.array_equal(layer.weights.cpu().numpy().view(np.uint32), ow.view(np.uint32)), "router weights"
    want_c, want_s, _ = _cpubase_contributions(store, bits(x), np.arange(K, dtype=np.int32)[None, :], ow, K, orc.AFTER_DOWN_BF16)
    got_c, got_s = bits(layer.decode.contributions), bits(layer.decode.shared_out)
    assert_close_bf16(got_c, want_c, "contributions")
    assert_close_bf16(got_s, want_s, "shared expert")
    assert np.array_equal(y, orc.combine(got_c, got_s, None, oi, None, orc.COMBINE_UNGATED)), "combine of the device contributions"
    want_y = orc.combine(want_c, want_s, None, oi, None, orc.COMBINE_UNGATED)
    terms = np.concatenate([orc.bf16_to_f32(want_c), orc.bf16_to_f32(want_s)[:, None, :], orc.bf16_to_f32(want_y)[:, None, :]], axis=1)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.max(np.abs(terms), axis=1).astype(np.float64), 1e-30))) - 7)
    err = np.abs(orc.bf16_to_f32(y).astype(np.float64) - orc.bf16_to_f32(want_y).astype(np.float64))
    assert np.all(err <= 3 * (K + 1) * ulp), float(np.max(err / ulp))
    assert orc.rel_l2(y, want_y) <= 4e-3
    # the other launch variants of the same layer: bit-identical y
    for name, setup in (("two launches after the logits (default)", dict()), ("separate top-k launch", dict(two_launch=False, inline_select=False)),
                        ("fused finish", dict(two_launch=False, inline_select=False, fused_finish=True)), ("one resident launch", dict(one_launch=True))):
        other = ops.NativeMoe(table, shared, router.cuda(), bias.cuda(), 1, K, 2.5, 8, 4, swiglu=capi.SWIGLU_TWICE,
                              routed_weight=capi.WEIGHT_AFTER_DOWN_BF16, combine_mode=capi.COMBINE_UNGATED)
        for k_, v_ in setup.items():
            setattr(other, k_, v_)
        print("C3 token,", name, flush=True)
        y2 = bits(other.run(x.cuda())).copy()
        torch.cuda.synchronize()
        assert np.array_equal(other.ids.cpu().numpy(), oi)
        assert np.array_equal(y2, y), name


def test_decode_fp8_full_width_64_rows_on_the_cohort_path(monkeypatch):
    """64 rows at hidden 7168: ffmoe_decode_contribute hands the whole batch to the matrix-core cohort kernels (every expert
    streamed once, the shared expert as one 64-row group). Same effective weights and BF16 boundaries as the streaming
    kernels: contributions and shared rows against the CPU port end to end, and bit-identical rows whether 64 or 48 rows
    are in the batch (rows do not depend on their cohort on this path either)."""
    experts, top_k, rows = 6, 4, 64
    monkeypatch.delenv("FFMOE_DECODE_COHORT_ROWS", raising=False)
    monkeypatch.delenv("FFMOE_DECODE_SHARED_COHORT_ROWS", raising=False)
    monkeypatch.delenv("FFMOE_PREFILL_MF", raising=False)
    table = make_table_on_device(capi.FMT_FP8_BLOCK128, experts + 1, H, I, 141)
    sh = table.shared_struct(experts)
    table.experts = experts
    g = synth.generator(142)
    x = synth.normal((rows, H), 1.0, 143).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    wt = torch.rand((rows, top_k), generator=g) * 0.5 + 0.05
    op = ops.DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True)
    op.contributions.zero_()
    print("full-width decode rows=64 (cohort path)", flush=True)
    contrib, shared_out = op.contribute(x.cuda(), ids.cuda(), wt.cuda())
    torch.cuda.synchronize()
    assert int(op.done.sum().item()) == rows * top_k
    got_c, got_s = bits(contrib).copy(), bits(shared_out).copy()
    want_c, want_s, _ = _cpubase_contributions(table, bits(x), ids.numpy(), wt.numpy(), experts, orc.AFTER_DOWN_BF16)
    # the stages of this path are held to their bars in test_prefill_w16_full_width; end to end the relative-L2 bar on the
    # tensor and a loose element-wise bound for cancelled outputs, as there
    r_, worst_, frac_ = assert_close_with_rare_outliers(got_c, want_c, "contributions vs the CPU port, end to end", rare=E2E_RARE)
    print("contributions end to end: relative L2 %.2e, worst %.1f steps, %.2e beyond 2 steps" % (r_, worst_, frac_), flush=True)
    assert_close_with_rare_outliers(got_s, want_s, "shared_out vs the CPU port, end to end", rare=E2E_RARE)
    part = ops.DecodeOps(table, sh, 48, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True)
    c2, s2 = part.contribute(x[8:56].contiguous().cuda(), ids[8:56].contiguous().cuda(), wt[8:56].contiguous().cuda())
    torch.cuda.synchronize()
    assert np.array_equal(bits(c2), got_c[8:56]) and np.array_equal(bits(s2), got_s[8:56]), "rows depend on their cohort"
    # the streaming kernels on the same batch (rules switched off): within the same bars of the cohort path's result
    monkeypatch.setenv("FFMOE_DECODE_COHORT_ROWS", "0")
    monkeypatch.setenv("FFMOE_DECODE_SHARED_COHORT_ROWS", "0")
    c3, s3 = op.contribute(x.cuda(), ids.cuda(), wt.cuda())
    torch.cuda.synchronize()
    assert_close_with_rare_outliers(bits(c3), want_c, "streaming kernels vs the CPU port, end to end", rare=E2E_RARE)
    assert_close_with_rare_outliers(bits(s3), want_s, "streaming kernels, shared_out", rare=E2E_RARE)


def test_prefill_c5_full_scale_bookkeeping_and_sampled_assignments():
    """BASELINE config 5 at its real size: 4096 tokens x top-8 over 256 experts with Zipf(s = 1.1) popularity - 32,768
    assignments through the multi-block count / plan / unit-list / stable-fill launches and both grouped GEMMs. The
    bookkeeping is checked exactly (every assignment once, inside its expert's segment, ascending within it - the
    invariants of kernels/moe_prefill.cu:495-499 and src/backend/cuda/moe/prefill_tests.rs:652-700 - counts, offsets,
    totals, every done flag set once); 16 assignments at the start, middle and end of the segments of the most popular,
    mid-popular and least popular experts are checked stage by stage against the oracle. Only the six experts those
    assignments hit are materialised (44 MB each); every other slot points at a spare expert, so all 32,768 rows still
    stream real weights."""
    E, K, R = 256, 8, 4096
    rng = np.random.default_rng(20251)
    pop = np.empty(E)
    pop[rng.permutation(E)] = np.arange(1, E + 1, dtype=np.float64) ** -1.1
    logits = np.log(pop)[None, :] - np.log(-np.log(rng.uniform(1e-12, 1.0 - 1e-12, size=(R, E))))   # Gumbel: a draw without replacement
    ids = np.argsort(-logits, axis=1, kind="stable")[:, :K].astype(np.int32)
    w = rng.uniform(0.05, 1.0, size=(R, K)).astype(np.float32)
    counts = np.bincount(ids.reshape(-1), minlength=E)
    order = np.argsort(-counts, kind="stable")
    live = [int(e) for e in order if counts[e] > 0]
    assert counts.max() > 2000 and counts.min() < 64 and len(live) >= 250, (counts.max(), counts.min(), len(live))
    hit = [live[0], live[1], live[len(live) // 2], live[len(live) // 2 + 1], live[-2], live[-1]]
    table, store, _ = _sparse_c3_table(hit, 151)
    host = {e: host_expert(store, i) for i, e in enumerate(hit)}
    x = synth.normal((R, H), 1.0, 152, dtype=torch.bfloat16)
    op = ops.PrefillOps(table, R, K, swiglu=capi.SWIGLU_TWICE, weights_f32=True)
    print("C5 full scale: %d assignments, rows per expert max %d min %d, %d experts touched" % (R * K, counts.max(), counts.min(), len(live)), flush=True)
    got = op.contribute(x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda())
    torch.cuda.synchronize()
    # bookkeeping, exactly
    v = op.scratch_views()
    A = R * K
    assert v["totals"].cpu().numpy()[3] == A
    assert np.array_equal(v["counts"].cpu().numpy(), counts)
    offsets = v["offsets"].cpu().numpy()
    assert np.array_equal(offsets, np.concatenate([[0], np.cumsum(counts)]))
    perm = v["perm"].cpu().numpy()[:A]
    assert np.array_equal(np.sort(perm), np.arange(A)), "every assignment exactly once"
    flat_ids = ids.reshape(-1)
    assert np.array_equal(flat_ids[perm], np.repeat(np.arange(E), counts)), "every position inside its expert's segment"
    inner = np.ones(A, dtype=bool)
    inner[offsets[1:-1][offsets[1:-1] < A]] = False
    inner[0] = False
    assert np.all((np.diff(perm) > 0)[inner[1:]]), "ascending assignment index within a segment"
    assert np.array_equal(op.done.cpu().numpy(), np.ones((R, K), dtype=np.int32)), "done set once per assignment"
    # sampled assignments, stage by stage
    picks = []
    for e in hit:
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        picks += sorted({lo, (lo + hi) // 2, hi - 1})
    picks = picks[:16]
    xb = bits(x)
    xq, sx = orc.quant_act_fp8_128(xb)
    assert np.array_equal(v["xq"].cpu().numpy(), xq) and np.array_equal(v["sx"].cpu().numpy().view(np.uint32), sx.view(np.uint32)), "activation quantizer"
    act = bits(v["act"][torch.tensor(picks, device="cuda")])
    g2 = bits(got.reshape(A, H)[torch.from_numpy(perm[picks]).cuda().long()])
    flat_w = w.reshape(-1)

    def one(lo, hi):
        out = []
        for i in range(lo, hi):
            a = int(perm[picks[i]])
            m, t = host[int(flat_ids[a])], a // K
            out.append((orc.linear_fp8_block_w8a8(m[0], m[1], xq[t:t + 1], sx[t:t + 1])[0], orc.linear_fp8_block_w8a8(m[2], m[3], xq[t:t + 1], sx[t:t + 1])[0],
                        orc.expert_down_w8a8(act[i], m[4], m[5], apply_weight=False), float(flat_w[a])))
        return out
    res = [t for chunk in run_parallel(one, len(picks), THREADS) for t in chunk]
    assert_swiglu_close(act, np.stack([t[0] for t in res]), np.stack([t[1] for t in res]), orc.TWICE, 0.0, orc.SILU_SIGMOID2,
                        "activations of the sampled assignments")
    assert_weighted_down_close(g2, np.stack([t[2] for t in res]), [t[3] for t in res], "down stage of the sampled assignments on the device activations")
    # a second cohort through the same arena after clearing done: same bits (nothing in the arena has to start at zero)
    first = bits(got.reshape(A, H)[torch.from_numpy(perm[picks]).cuda().long()]).copy()
    op.done.zero_()
    again = op.contribute(x.cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda())
    torch.cuda.synchronize()
    assert np.array_equal(bits(again.reshape(A, H)[torch.from_numpy(perm[picks]).cuda().long()]), first)
