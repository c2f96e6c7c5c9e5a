"""ffmoe_decode_contribute_static: the decode contribution with the library's built-in per-GPU scratch array, for callers
that cannot allocate. It must give ffmoe_decode_contribute's results bit for bit (the same kernels run), also on a
second call with a smaller input that finds the first call's bytes in the shared array, and it must reject a shape that
does not fit the array without launching anything."""
import ctypes

import numpy as np
import pytest
import torch

from flyingfish_amd import capi, synth
from flyingfish_amd.ops import DecodeOps
from helpers import bits, make_table

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _case(table, sh, fmt, experts, hidden, rows, top_k, seed, act_mode=capi.ACT_BF16):
    g = synth.generator(seed)
    x = synth.normal((rows, hidden), 1.0, seed + 1).to(torch.bfloat16).to(DEV)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32).to(DEV)
    wt = (torch.rand((rows, top_k), generator=g) * 0.5 + 0.05).to(DEV)
    active = (torch.rand((rows, top_k), generator=g) > 0.2).to(torch.int32).to(DEV)
    out = []
    for static in (False, True):
        op = DecodeOps(table, sh, rows, top_k, act_mode, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True)
        op.contributions.zero_()
        op.shared_out.zero_()
        print("no-alloc case fmt=%d rows=%d top_k=%d seed=%d static=%d act_mode=%d" % (fmt, rows, top_k, seed, static, act_mode), flush=True)
        if static:
            op.contribute_static(x, ids, wt, active)
        else:
            op.contribute(x, ids, wt, active)
        torch.cuda.synchronize()
        out.append((bits(op.contributions).copy(), bits(op.shared_out).copy(), op.done.cpu().numpy().copy()))
    (c0, s0, d0), (c1, s1, d1) = out
    assert np.array_equal(d0, d1) and np.array_equal(d0 != 0, active.cpu().numpy() != 0)
    assert np.array_equal(c0, c1), "contributions differ from ffmoe_decode_contribute"
    assert np.array_equal(s0, s1), "shared_out differs from ffmoe_decode_contribute"
    assert c0.any() and s0.any()


@pytest.mark.parametrize("fmt", [capi.FMT_FP8_BLOCK128, capi.FMT_NVFP4])
def test_static_scratch_matches_caller_scratch_twice(fmt):
    experts, hidden, inter = 8, 1024, 512
    table, _ = make_table(fmt, experts + 1, hidden, inter, 901)
    sh = table.shared_struct(experts)
    table.experts = experts
    # two calls in a row on the same GPU array: 19 rows x 4 choices (grouped path), then one row x 3 choices
    _case(table, sh, fmt, experts, hidden, 19, 4, 910)
    _case(table, sh, fmt, experts, hidden, 1, 3, 920)
    # and a larger one again, so stale descriptors of the small call would show
    _case(table, sh, fmt, experts, hidden, 6, 2, 930)


def test_static_scratch_w8a8_mode():
    experts, hidden, inter = 6, 512, 384
    table, _ = make_table(capi.FMT_FP8_BLOCK128, experts + 1, hidden, inter, 941)
    sh = table.shared_struct(experts)
    table.experts = experts
    _case(table, sh, capi.FMT_FP8_BLOCK128, experts, hidden, 9, 3, 950, act_mode=capi.ACT_FP8_BLOCK128)
    _case(table, sh, capi.FMT_FP8_BLOCK128, experts, hidden, 2, 2, 960, act_mode=capi.ACT_FP8_BLOCK128)


def test_static_scratch_rejects_oversize_and_reports_its_size():
    L = capi.lib()
    cap = L.ffmoe_decode_static_scratch_bytes()
    assert cap == 8 << 20
    experts, hidden, inter = 4, 1024, 512
    table, _ = make_table(capi.FMT_FP8_BLOCK128, experts, hidden, inter, 971)
    rows, top_k = 4096, 1  # (rows * top_k + rows) * inter * 2 bytes of activations alone exceed the array
    assert L.ffmoe_decode_scratch_bytes(rows, top_k, experts, hidden, inter, 0) > cap
    x = torch.zeros((rows, hidden), dtype=torch.bfloat16, device=DEV)
    ids = torch.zeros((rows, top_k), dtype=torch.int32, device=DEV)
    wt = torch.ones((rows, top_k), dtype=torch.float32, device=DEV)
    contrib = torch.full((rows, top_k, hidden), 7.0, dtype=torch.bfloat16, device=DEV)
    d = capi.Decode(rows, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, 1, x.data_ptr(), ids.data_ptr(), None,
                    wt.data_ptr(), contrib.data_ptr(), None, None, None, 0, None)
    tc = table.c_struct()
    rc = L.ffmoe_decode_contribute_static(ctypes.byref(tc), None, ctypes.byref(d), None)
    assert rc == capi.ERR_SCRATCH and "built-in arena" in capi.last_error()
    torch.cuda.synchronize()
    assert bool((contrib == 7.0).all()), "a rejected call must not launch anything"


@pytest.mark.parametrize("rows,top_k", [(1, 4), (9, 3)])
def test_static_scratch_call_replays_from_a_hip_graph(rows, top_k):
    """The caller this entry point is for: one ffmoe_decode_contribute_static call captured into a HIP graph (after a first
    call outside capture, which looks the array's address up) and replayed with new inputs in the same buffers. Every
    replay, with eager work and synchronisations in between, must give the eager ffmoe_decode_contribute bits."""
    experts, hidden, inter = 8, 1024, 512
    table, _ = make_table(capi.FMT_FP8_BLOCK128, experts + 1, hidden, inter, 981)
    sh = table.shared_struct(experts)
    table.experts = experts
    g = synth.generator(982)
    x = synth.normal((rows, hidden), 1.0, 983).to(torch.bfloat16).to(DEV)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32).to(DEV)
    wt = (torch.rand((rows, top_k), generator=g) * 0.5 + 0.05).to(DEV)
    eager = DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True)
    op = DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True)
    op.contribute_static(x, ids, wt)   # first call on this GPU outside capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    print("capturing ffmoe_decode_contribute_static rows=%d top_k=%d" % (rows, top_k), flush=True)
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            op.contribute_static(x, ids, wt)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for replay in range(4):
        x.copy_(synth.normal((rows, hidden), 1.0, 990 + replay).to(torch.bfloat16))
        ids.copy_(torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32))
        op.contributions.zero_(); op.shared_out.zero_(); op.done.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        c, s = eager.contribute(x, ids, wt)
        torch.cuda.synchronize()
        assert np.array_equal(bits(op.contributions), bits(c)) and np.array_equal(bits(op.shared_out), bits(s)), "replay %d" % replay
        assert bool((op.done != 0).all())
