"""One token, the expert part of the layer in one resident launch (ffmoe_decode_token_layer) against the separate
launches (selection, gate/up, down, combine), whose oracle parity test_gpu_parity.py covers: ids, weights and y must be
bit-identical."""
import numpy as np
import pytest
import torch

from flyingfish_amd import capi, synth
from flyingfish_amd.ops import CombineOps, DecodeOps, ExpertTable, NativeMoe
from helpers import bits, make_table

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rand_bf16(shape, std, seed):
    return synth.normal(shape, std, seed).to(torch.bfloat16)


@pytest.mark.parametrize("fmt,hidden,inter,top_k,shared", [
    (capi.FMT_FP8_BLOCK128, 1024, 512, 8, True),     # 9 groups, one step per row
    (capi.FMT_FP8_BLOCK128, 512, 2048, 3, True),     # two steps per down row
    (capi.FMT_FP8_BLOCK128, 1024, 384, 4, False),    # routed only
    (capi.FMT_NVFP4, 1024, 512, 6, True),
    (capi.FMT_BF16, 1024, 256, 2, True),
])
def test_token_layer_equals_separate_launches_given_ids(fmt, hidden, inter, top_k, shared):
    """ids / weights given: every combine mode, with and without inactive choices."""
    experts, seed = 10, 197
    table, _ = make_table(fmt, experts + (1 if shared else 0), hidden, inter, seed)
    sh = table.shared_struct(experts) if shared else None
    table.experts = experts
    x = rand_bf16((1, hidden), 1.0, seed + 7).to(DEV)
    g = synth.generator(seed + 8)
    ids = torch.randperm(experts, generator=g)[:top_k].to(torch.int32).view(1, top_k).to(DEV)
    wt = (torch.rand((1, top_k), generator=g) * 0.5 + 0.05).to(DEV)
    scale = rand_bf16((1,), 0.5, seed + 9).to(DEV)
    modes = [capi.COMBINE_ROUTED] if not shared else [capi.COMBINE_GATED, capi.COMBINE_UNGATED, capi.COMBINE_BF16,
                                                      capi.COMBINE_ACCUM_FP32, capi.COMBINE_ACCUM_BF16]
    for boundary in (capi.WEIGHT_AFTER_DOWN_BF16, capi.WEIGHT_BEFORE_CONTRIBUTION_BF16):
        for with_active in (False, True):
            active = None
            if with_active:
                a = torch.ones((1, top_k), dtype=torch.int32)
                a[0, 0] = 0
                a[0, top_k - 1] = 0 if top_k > 2 else 1
                active = a.to(DEV)
            op = DecodeOps(table, sh, 1, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, boundary, True)
            op.done.zero_()
            op.contributions.zero_()  # the accumulate modes add every slot, live or not: skipped slots must read as zero
            contrib, shared_out = op.contribute(x, ids, wt, active)
            for mode in modes:
                want = CombineOps.combine(contrib, shared_out, ids, mode, scale=scale, done=op.done, final_active=active)
                y = torch.full((1, hidden), 7.0, dtype=torch.bfloat16, device=DEV)
                status = torch.zeros(1, dtype=torch.int32, device=DEV)
                assert op.token_layer(x, ids, wt, mode, y, status=status, scale=scale, active=active)
                torch.cuda.synchronize()
                assert int(status.item()) == 0
                assert np.array_equal(bits(y), bits(want)), "mode %d active %s boundary %d" % (mode, with_active, boundary)


@pytest.mark.parametrize("fmt", [capi.FMT_FP8_BLOCK128, capi.FMT_NVFP4])
@pytest.mark.parametrize("experts,n_group,topk_group", [(64, 1, 1), (256, 8, 4)])
def test_token_layer_selects_like_the_separate_launch(fmt, experts, n_group, topk_group):
    hidden, inter, top_k = 512, 256, 6
    table, _ = make_table(fmt, experts + 1, hidden, inter, 61)
    sh = table.shared_struct(experts)
    table.experts = experts
    router = rand_bf16((experts, hidden), 0.05, 62).to(DEV)
    bias = (torch.randn(experts, generator=torch.Generator().manual_seed(63)) * 0.1).to(DEV)
    got = {}
    for one_launch in (False, True):
        layer = NativeMoe(table, sh, router, bias, 1, top_k, routed_scaling=2.5, n_group=n_group, topk_group=topk_group)
        layer.one_launch = one_launch
        layer.inline_select = False
        layer.two_launch = False
        outs = []
        for step in range(4):  # consecutive launches on one scratch arena: each must see only its own activations
            x = rand_bf16((1, hidden), 1.0, 64 + step).to(DEV)
            y = bits(layer.run(x)).copy()
            outs.append((layer.ids.cpu().numpy().copy(), layer.weights.cpu().numpy().copy(), y))
            assert int(layer.status.item()) == 0
        assert layer.one_launch == one_launch
        got[one_launch] = outs
    for a, b in zip(got[False], got[True]):
        for name, u, v in zip(("ids", "weights", "y"), a, b):
            assert np.array_equal(u, v), name
    assert len({o[2].tobytes() for o in got[True]}) == 4  # four different tokens, four different outputs


def test_token_layer_at_dsv3_width_many_launches():
    """hidden 7168 / inter 2048 (3.5 output rows per wave, one gate/up row pair per wave and group), 8 of 16 experts +
    shared; 40 launches alternating over 4 tokens on one arena must reproduce the separate launches every time."""
    hidden, inter, experts, top_k = 7168, 2048, 16, 8
    table = ExpertTable.allocate(capi.FMT_FP8_BLOCK128, experts + 1, hidden, inter, DEV)
    g = torch.Generator(device="cpu").manual_seed(5)
    for e in range(experts + 1):
        v = table.expert_views(e)
        for i in range(3):
            v[2 * i].copy_(torch.randint(0, 120, v[2 * i].shape, generator=g, dtype=torch.uint8).to(DEV))
            v[2 * i + 1].copy_((torch.rand(v[2 * i + 1].shape, generator=g) * 2e-3 + 1e-3).to(DEV))
    sh = table.shared_struct(experts)
    table.experts = experts
    router = rand_bf16((64, hidden), 0.05, 6).to(DEV)[:experts].contiguous()
    xs = [rand_bf16((1, hidden), 1.0, 70 + i).to(DEV) for i in range(4)]
    op = DecodeOps(table, sh, 1, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
    want, idl, wl = [], [], []
    for i, x in enumerate(xs):
        gi = synth.generator(80 + i)
        ids = torch.randperm(experts, generator=gi)[:top_k].to(torch.int32).view(1, top_k).to(DEV)
        wt = (torch.rand((1, top_k), generator=gi) * 0.5 + 0.05).to(DEV)
        op.done.zero_()
        c, s = op.contribute(x, ids, wt)
        want.append(bits(CombineOps.combine(c, s, ids, capi.COMBINE_UNGATED, done=op.done)).copy())
        idl.append(ids); wl.append(wt)
    y = torch.zeros((1, hidden), dtype=torch.bfloat16, device=DEV)
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    for it in range(40):
        i = it % 4
        assert op.token_layer(xs[i], idl[i], wl[i], capi.COMBINE_UNGATED, y, status=status)
        if it % 8 == 7 or it < 4:
            torch.cuda.synchronize()
            assert np.array_equal(bits(y), want[i]), it
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), want[39 % 4]) and int(status.item()) == 0
    # every launch hands its arena back zero-filled, so no launch can meet a word of an earlier one
    assert int(op.token_scratch.view(torch.int32).count_nonzero().item()) == 0


def test_token_layer_shapes_may_alternate_on_one_arena():
    """Two layers of different shape (top_k, widths, with and without a shared expert) take turns on ONE arena: each
    launch must reproduce its separate launches, which holds only because the arena is clean between launches."""
    cases = []
    arena = None
    for n, (hidden, inter, experts, top_k, shared) in enumerate([(1024, 512, 8, 6, True), (512, 1024, 6, 2, False)]):
        table, _ = make_table(capi.FMT_FP8_BLOCK128, experts + (1 if shared else 0), hidden, inter, 300 + n)
        sh = table.shared_struct(experts) if shared else None
        table.experts = experts
        op = DecodeOps(table, sh, 1, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
        x = rand_bf16((1, hidden), 1.0, 310 + n).to(DEV)
        gi = synth.generator(320 + n)
        ids = torch.randperm(experts, generator=gi)[:top_k].to(torch.int32).view(1, top_k).to(DEV)
        wt = (torch.rand((1, top_k), generator=gi) * 0.5 + 0.05).to(DEV)
        mode = capi.COMBINE_UNGATED if shared else capi.COMBINE_ROUTED
        op.done.zero_()
        c, s = op.contribute(x, ids, wt)
        want = bits(CombineOps.combine(c, s, ids, mode, done=op.done)).copy()
        cases.append((op, x, ids, wt, mode, want, torch.zeros((1, hidden), dtype=torch.bfloat16, device=DEV)))
    size = max(c[0].scratch.numel() for c in cases)
    arena = torch.zeros(size, dtype=torch.uint8, device=DEV)
    for op, *_ in cases:
        op.token_scratch = arena[: op.scratch.numel()]
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    for it in range(12):
        op, x, ids, wt, mode, want, y = cases[it % 2]
        assert op.token_layer(x, ids, wt, mode, y, status=status)
        torch.cuda.synchronize()
        assert np.array_equal(bits(y), want), it
    assert int(status.item()) == 0 and int(arena.view(torch.int32).count_nonzero().item()) == 0


def test_token_layer_flags_bad_expert_and_declines_batches():
    table, _ = make_table(capi.FMT_FP8_BLOCK128, 5, 512, 256, 5)
    sh = table.shared_struct(4)
    table.experts = 4
    x = rand_bf16((1, 512), 1.0, 3).to(DEV)
    ids = torch.tensor([[1, 9, 2]], dtype=torch.int32, device=DEV)  # 9 is out of range
    wt = torch.full((1, 3), 0.25, device=DEV)
    op = DecodeOps(table, sh, 1, 3, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
    y = torch.zeros((1, 512), dtype=torch.bfloat16, device=DEV)
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    assert op.token_layer(x, ids, wt, capi.COMBINE_UNGATED, y, status=status)
    torch.cuda.synchronize()
    assert int(status.item()) == 1
    good = torch.tensor([[1, 2]], dtype=torch.int32, device=DEV)
    op2 = DecodeOps(table, sh, 1, 2, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
    c2, s2 = op2.contribute(x, good, wt[:, :2].contiguous())
    want = CombineOps.combine(c2, s2, good, capi.COMBINE_UNGATED)
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), bits(want))
    op3 = DecodeOps(table, sh, 2, 2, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
    x2 = rand_bf16((2, 512), 1.0, 4).to(DEV)
    ids2 = torch.tensor([[0, 1], [2, 3]], dtype=torch.int32, device=DEV)
    y2 = torch.zeros((2, 512), dtype=torch.bfloat16, device=DEV)
    assert not op3.token_layer(x2, ids2, torch.full((2, 2), 0.5, device=DEV), capi.COMBINE_UNGATED, y2)


def test_token_layer_graph_replay_equals_eager():
    table, _ = make_table(capi.FMT_FP8_BLOCK128, 9, 1024, 512, 23)
    sh = table.shared_struct(8)
    table.experts = 8
    router = rand_bf16((64, 1024), 0.02, 24).to(DEV)
    table64, _ = make_table(capi.FMT_FP8_BLOCK128, 65, 1024, 512, 29)
    sh64 = table64.shared_struct(64)
    table64.experts = 64
    bias = torch.zeros(64, device=DEV)
    layer = NativeMoe(table64, sh64, router, bias, 1, 3, routed_scaling=2.5, combine_mode=capi.COMBINE_UNGATED,
                      routed_weight=capi.WEIGHT_AFTER_DOWN_BF16)
    xs = [rand_bf16((1, 1024), 1.0, 25 + i).to(DEV) for i in range(3)]
    layer.one_launch = False
    layer.two_launch = False
    eager = [bits(layer.run(x)).copy() for x in xs]
    layer.one_launch = True
    x_in = xs[0].clone()
    layer.run(x_in)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            layer.run(x_in)
    torch.cuda.current_stream().wait_stream(side)
    assert layer.one_launch
    for it in range(6):
        x_in.copy_(xs[it % 3])
        layer.y.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(bits(layer.y), eager[it % 3]), "replay %d" % it
    assert int(layer.status.item()) == 0


def test_token_layer_bounded_wait_gives_up_and_the_next_launch_recovers(monkeypatch):
    """The grid-wide hand-over of the one-launch layer is a bounded wait: with FFMOE_TOKEN_SPIN_LIMIT=0 (read at every call) a
    block that finds activations of other blocks missing on its first look gives up, sets bit 1 of the status word and
    still leaves the kernel; the last block out hands the arena and the claim counters back clean. Whether any block has
    to give up is a matter of timing, so both outcomes are accepted for the forced call - status 0 with the right y, or
    status 2 - and the launches that follow (default limit, same arena, same stream) must give the separate launches' bits."""
    experts, hidden, inter, top_k, seed = 12, 2048, 1024, 8, 211
    table, _ = make_table(capi.FMT_FP8_BLOCK128, experts + 1, hidden, inter, seed)
    sh = table.shared_struct(experts)
    table.experts = experts
    op = DecodeOps(table, sh, 1, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
    g = synth.generator(seed + 1)
    gave_up = 0
    for trial in range(6):
        x = rand_bf16((1, hidden), 1.0, seed + 10 + trial).to(DEV)
        ids = torch.randperm(experts, generator=g)[:top_k].to(torch.int32).view(1, top_k).to(DEV)
        wt = (torch.rand((1, top_k), generator=g) * 0.5 + 0.05).to(DEV)
        op.done.zero_()
        contrib, shared_out = op.contribute(x, ids, wt)
        want = bits(CombineOps.combine(contrib, shared_out, ids, capi.COMBINE_UNGATED, done=op.done)).copy()
        y = torch.full((1, hidden), 7.0, dtype=torch.bfloat16, device=DEV)
        status = torch.zeros(1, dtype=torch.int32, device=DEV)
        monkeypatch.setenv("FFMOE_TOKEN_SPIN_LIMIT", "0")
        print("one-launch layer, spin limit 0, trial %d" % trial, flush=True)
        assert op.token_layer(x, ids, wt, capi.COMBINE_UNGATED, y, status=status)
        torch.cuda.synchronize()
        st = int(status.item())
        assert st in (0, 2), st
        if st == 0:
            assert np.array_equal(bits(y), want), "no block gave up, so y must be right"
        gave_up += st == 2
        monkeypatch.delenv("FFMOE_TOKEN_SPIN_LIMIT")
        for again in range(2):
            y.fill_(7.0)
            status.zero_()
            assert op.token_layer(x, ids, wt, capi.COMBINE_UNGATED, y, status=status)
            torch.cuda.synchronize()
            assert int(status.item()) == 0
            assert np.array_equal(bits(y), want), "launch %d after a forced give-up" % again
    print("forced give-ups: %d of 6 launches" % gave_up, flush=True)
