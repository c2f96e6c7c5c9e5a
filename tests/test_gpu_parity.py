"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs."""
import json
import os

import numpy as np
import pytest
import torch

import oracle as orc
from flyingfish_amd import capi, synth
from flyingfish_amd.ops import CombineOps, DecodeOps, ExpertTable, Fp8Ops, NativeMoe, NvFp4Ops, RouteOps, gemm_skinny_bf16, swiglu
from helpers import assert_close_bf16, bf16_tensor, bits, make_table, oracle_contributions, oracle_shared

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "shared-ops.json")
DEV = "cuda"


def rand_bf16(shape, std, seed):
    return synth.normal(shape, std, seed).to(torch.bfloat16)


@pytest.fixture(autouse=True)
def _streaming_decode_kernels(monkeypatch):
    """The decode tests of this module check the streaming kernels stage by stage (they read the activations out of that
    path's arena): block-FP8 batches of 8 rows and more, which the library would hand to the matrix-core cohort kernels,
    stay on them here. The cohort dispatch has its own tests (test_gpu_prefill.py, test_gpu_fullsize.py)."""
    monkeypatch.setenv("FFMOE_DECODE_COHORT_ROWS", "0")


# ------------------------------------------------------------------------------------------------
# codecs through the product path
def test_device_e4m3_decode_all_codes():
    # W[n, 0] = code n with unit scale, x = e_0  =>  y[n] = bf16(decode(n)); E4M3 values are exact in BF16
    n, k = 256, 128
    codes = torch.zeros((n, k), dtype=torch.uint8)
    codes[:, 0] = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    codes[0x7F, 0] = 0
    codes[0xFF, 0] = 0
    scales = torch.ones((2, 1), dtype=torch.float32)
    x = torch.zeros((1, k), dtype=torch.bfloat16)
    x[0, 0] = 1.0
    y = Fp8Ops.linear(codes.to(DEV), scales.to(DEV), x.to(DEV))
    L = orc.lib()
    want = np.array([0.0 if c in (0x7F, 0xFF) else L.orc_decode_e4m3(c) for c in range(256)], dtype=np.float32)
    assert np.array_equal(y.float().cpu().numpy()[0], want)


def test_device_effective_weight_rounding_matches_oracle():
    # every code against awkward f32 scales: y[n] = bf16(decode(code) * scale) must equal the oracle bit for bit
    n, k = 256, 128
    codes = torch.zeros((n, k), dtype=torch.uint8)
    col = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    col[0x7F] = 0
    col[0xFF] = 0
    codes[:, 0] = col
    x = torch.zeros((1, k), dtype=torch.bfloat16)
    x[0, 0] = 1.0
    L = orc.lib()
    for s0, s1 in [(1.0078125, 0.0123456), (3.3e-5, 7.77e-3), (1.9999999, 0.33333334)]:
        scales = torch.tensor([[s0], [s1]], dtype=torch.float32)
        y = bits(Fp8Ops.linear(codes.to(DEV), scales.to(DEV), x.to(DEV)))[0]
        want = np.array([L.orc_effective_weight(int(col[c]), float(np.float32(s0 if c < 128 else s1))) for c in range(256)], dtype=np.uint16)
        assert np.array_equal(y & 0x7FFF, want & 0x7FFF) and np.array_equal(y[want & 0x7FFF != 0], want[want & 0x7FFF != 0])


def test_device_activation_quantizer_bits():
    m, k = 7, 7168
    x = rand_bf16((m, k), 1.0, 101)
    x[3] = 0
    x[4, :128] *= 1e-20
    codes, scales = Fp8Ops.quantize(x.to(DEV))
    wc, ws = orc.quant_act_fp8_128(bits(x))
    assert np.array_equal(scales.cpu().numpy().view(np.uint32), ws.view(np.uint32))
    assert np.array_equal(codes.cpu().numpy(), wc)
    # reference fixture (src/backend/cuda/linear.rs:2320-2338), k with a ragged last group
    m, k = 5, 264
    i = np.arange(m * k, dtype=np.int64)
    vals = orc.f32_to_bf16((((i * 19 + 3) % 251).astype(np.float32) / np.float32(32) - np.float32(4))).reshape(m, k)
    codes, scales = Fp8Ops.quantize(bf16_tensor(vals))
    wc, ws = orc.quant_act_fp8_128(vals)
    assert np.array_equal(codes.cpu().numpy(), wc) and np.array_equal(scales.cpu().numpy().view(np.uint32), ws.view(np.uint32))
    # every finite BF16 value up to 2^20 in magnitude, in two orders (sorted: groups of like-sized values, quotients near the
    # top of the grid; shuffled: every group holds large values, quotients down to the subnormal codes and zero): the codes come
    # from the hardware conversion, the oracle's from the reference's software encoder
    pats = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = (pats.astype(np.uint32) << 16).view(np.float32)
    keep = pats[np.isfinite(f) & (np.abs(f) <= 2.0 ** 20)]
    keep = keep[: (keep.size // 1024) * 1024]
    rng = np.random.default_rng(77)
    for order in (keep, rng.permutation(keep)):
        vals = order.reshape(-1, 1024)
        codes, scales = Fp8Ops.quantize(bf16_tensor(vals))
        wc, ws = orc.quant_act_fp8_128(vals)
        assert np.array_equal(scales.cpu().numpy().view(np.uint32), ws.view(np.uint32))
        assert np.array_equal(codes.cpu().numpy(), wc)
        assert len(np.unique(wc)) >= 250  # (nearly) the whole code space is exercised


def test_device_swiglu_golden_bits():
    with open(GOLDEN) as f:
        fx = json.load(f)["swiglu"]
    n = len(fx["gate"])
    g = np.zeros(16, np.float32); g[:n] = fx["gate"]
    u = np.zeros(16, np.float32); u[:n] = fx["up"]
    gt, ut = torch.from_numpy(g).to(torch.bfloat16).view(1, 16).to(DEV), torch.from_numpy(u).to(torch.bfloat16).view(1, 16).to(DEV)
    assert bits(swiglu(gt, ut, capi.SWIGLU_CLAMPED_TWICE, fx["limit"]))[0, :n].tolist() == fx["twice"]
    assert bits(swiglu(gt, ut, capi.SWIGLU_CLAMPED_ONCE, fx["limit"]))[0, :n].tolist() == fx["once"]
    # dense random sweep against the oracle for all five modes
    gg, uu = rand_bf16((8, 4096), 3.0, 5), rand_bf16((8, 4096), 3.0, 6)
    for mode in range(5):
        got = bits(swiglu(gg.to(DEV), uu.to(DEV), mode, 2.5))
        want = orc.silu_mul(bits(gg), bits(uu), mode, 2.5, orc.SILU_DIV)
        assert np.array_equal(got, want), mode


def test_device_gelu_twice_every_gate_value():
    """tanh-GELU with two roundings: every BF16 gate pattern (NaNs aside) against the oracle, bit for bit."""
    gate = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    keep = np.isfinite(orc.bf16_to_f32(gate))
    gate = gate[keep][: (int(keep.sum()) // 8) * 8]
    for seed, scale in ((1, 1.0), (2, 40.0)):
        up = bits(rand_bf16((1, gate.size), scale, seed))[0]
        gt = torch.from_numpy(gate.view(np.int16)).view(torch.bfloat16).view(1, -1).to(DEV)
        ut = torch.from_numpy(up.view(np.int16)).view(torch.bfloat16).view(1, -1).to(DEV)
        got = bits(swiglu(gt, ut, capi.SWIGLU_GELU_TWICE, 0.0))[0]
        assert np.array_equal(got, orc.silu_mul(gate, up, orc.GELU_TWICE, 0.0, orc.SILU_DIV))


# ------------------------------------------------------------------------------------------------
# router
@pytest.mark.parametrize("rows,experts,hidden", [(1, 64, 2048), (3, 256, 512), (2, 100, 264)])
def test_route_logits_bf16_bit_exact(rows, experts, hidden):
    x, w = rand_bf16((rows, hidden), 1.0, 11), rand_bf16((experts, hidden), 0.02, 12)
    got = bits(RouteOps.logits_bf16(x.to(DEV), w.to(DEV)))
    assert np.array_equal(got, orc.route_logits_bf16(bits(x), bits(w)))


def test_route_logits_bf16_bit_exact_with_zero_subnormal_and_underflowing_products():
    """The kernel chains FP32 products of the BF16 values; a product that is zero or below the normal range sends its chunk
    of 256 columns through fmas on the values themselves. Planted: exact zeros in the token and in the router, products in
    the subnormal range, products that underflow to zero, and huge values next to them - bit for bit against the oracle."""
    rows, experts, hidden = 2, 70, 1032
    x, w = rand_bf16((rows, hidden), 1.0, 13), rand_bf16((experts, hidden), 0.02, 14)
    x[0, 5] = 0.0                       # an exact zero in the token: chunk 0 of row 0
    w[3, 300] = 0.0                     # an exact zero in the router: chunk 1, both rows
    x[1, 600], w[:, 600] = 2.0 ** -70, (torch.arange(experts, dtype=torch.float32) + 1.0).to(torch.bfloat16) * 2.0 ** -62  # subnormal products
    x[1, 601], w[:, 601] = 2.0 ** -100, 2.0 ** -90                                                      # underflow to zero
    x[1, 602], w[:, 602] = -(2.0 ** -120), 2.0 ** -20                                                   # tiny, sign
    x[0, 800], w[:, 800] = 3.0e38, 1.0e-38                                                              # huge times tiny: normal
    x[1, 1031], w[7, 1031] = 2.0 ** -64, -(2.0 ** -64)                                                  # last column of the ragged last chunk
    got = bits(RouteOps.logits_bf16(x.to(DEV), w.to(DEV)))
    assert np.array_equal(got, orc.route_logits_bf16(bits(x), bits(w)))
    # and a token row of zeros
    z = torch.zeros((1, hidden), dtype=torch.bfloat16)
    assert np.array_equal(bits(RouteOps.logits_bf16(z.to(DEV), w.to(DEV))), orc.route_logits_bf16(bits(z), bits(w)))


@pytest.mark.parametrize("rows,experts,hidden", [(1, 256, 7168), (9, 64, 2048), (5, 33, 520),
                                                 # from 96 rows on: the kernel that keeps a tile of router rows in LDS
                                                 (300, 256, 7168), (96, 8, 2048), (97, 33, 520), (203, 50, 4104), (1000, 9, 8), (128, 256, 7168)])
def test_route_logits_f32_bit_exact_and_close_to_f64(rows, experts, hidden):
    x, w = rand_bf16((rows, hidden), 1.0, 13), rand_bf16((experts, hidden), 0.02, 14)
    got = RouteOps.logits_f32(x.to(DEV), w.to(DEV)).cpu().numpy()
    want = orc.route_logits_f32(bits(x), bits(w))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    f64 = x.double().numpy() @ w.double().numpy().T
    assert np.max(np.abs(got - f64)) <= 16 * 2.0 ** -24 * np.max(np.abs(x.double().numpy()) @ np.abs(w.double().numpy()).T)


@pytest.mark.parametrize("score", [capi.SCORE_SOFTMAX, capi.SCORE_SIGMOID])
@pytest.mark.parametrize("rows,experts,top_k", [(4, 64, 4), (3, 256, 8), (2, 1000, 32), (5, 48, 6)])
def test_route_topk_bit_exact(score, rows, experts, top_k):
    lg = rand_bf16((rows, experts), 1.5, 15 + experts)
    lg[0, 1] = lg[0, experts - 1] = 6.0          # planted exact tie inside the top-k
    lg[1, 7] = lg[1, 3]                           # planted tie somewhere
    ids, w = RouteOps.topk(lg.to(DEV), top_k, score)
    fn = orc.route_topk_softmax if score == capi.SCORE_SOFTMAX else orc.route_topk_sigmoid
    wi, ww = fn(bits(lg), top_k)
    assert np.array_equal(ids.cpu().numpy(), wi)
    assert np.array_equal(bits(w), ww)
    assert ids[0, 0] == 1 and ids[0, 1] == experts - 1


def test_route_noaux_golden_and_random():
    with open(GOLDEN) as f:
        routers = json.load(f)["routers"]
    for fx in routers:
        mode = {"sigmoid": 0, "sqrtsoftplus": 1}[fx["mode"]]
        lg = torch.tensor([fx["logits"]], dtype=torch.float32, device=DEV)
        b = torch.tensor([fx["bias"]], dtype=torch.float32, device=DEV)
        ids, w = RouteOps.topk_noaux(lg, b, fx["top_k"], mode, fx["scale"])
        assert ids[0].tolist() == fx["ids"]
        want = np.array(fx["weights"], dtype=np.float32)
        assert np.all(np.abs(w[0].cpu().numpy() - want) <= 2e-6 * np.maximum(1, np.abs(want)))
        oi, ow = orc.route_topk_noaux(lg.cpu().numpy(), b.cpu().numpy(), fx["top_k"], mode, fx["scale"])
        assert np.array_equal(w.cpu().numpy().view(np.uint32), ow.view(np.uint32))
    rng = np.random.default_rng(3)
    for rows, experts, top_k, ng, kg in [(16, 256, 8, 1, 1), (16, 256, 8, 8, 4), (7, 64, 6, 4, 2), (3, 384, 6, 1, 1)]:
        lg = rng.normal(size=(rows, experts)).astype(np.float32)
        b = rng.normal(scale=0.2, size=(experts,)).astype(np.float32)
        lg[0, 5] = lg[0, 9]
        for mode in (0, 1):
            for wf32 in (True, False):
                ids, w = RouteOps.topk_noaux(torch.from_numpy(lg).to(DEV), torch.from_numpy(b).to(DEV), top_k, mode, 2.5, ng, kg, wf32)
                oi, ow = orc.route_topk_noaux(lg, b[None, :], top_k, mode, 2.5, ng, kg)
                assert np.array_equal(ids.cpu().numpy(), oi), (rows, experts, mode)
                if wf32:
                    assert np.array_equal(w.cpu().numpy().view(np.uint32), ow.view(np.uint32))
                else:
                    assert np.array_equal(bits(w), orc.f32_to_bf16(ow))


@pytest.mark.parametrize("seed", range(24))
def test_route_seeded_sweep_bit_exact(seed):
    """Router shapes the fixed cases do not visit: expert counts that are not powers of two, top_k from 1 to 32, rows
    1..40, grouped selection with every divisor pair, planted ties, both score functions, both weight types. Ids and
    weights are compared bit for bit."""
    rng = np.random.default_rng(2000 + seed)
    experts = int(rng.choice([8, 33, 48, 64, 100, 160, 256, 384, 1000]))
    top_k = int(rng.integers(1, min(32, experts - 1) + 1))
    rows = int(rng.choice([1, 2, 5, 17, 40]))
    lg = rng.normal(size=(rows, experts)).astype(np.float32) * float(rng.choice([0.5, 2.0, 6.0]))
    for r in range(rows):  # planted exact ties: the lower id must win
        a, b = rng.choice(experts, 2, replace=False)
        lg[r, a] = lg[r, b]
    b = rng.normal(scale=0.2, size=(experts,)).astype(np.float32)
    # noaux with the group filter where the shape allows one
    groupings = [(1, 1)]
    for ng in (2, 4, 8):
        if experts % ng == 0:
            for kg in range(1, ng + 1):
                if kg * (experts // ng) >= top_k:
                    groupings.append((ng, kg))
    ng, kg = groupings[int(rng.integers(0, len(groupings)))]
    mode = int(rng.integers(0, 2))
    scaling = float(rng.choice([1.0, 1.5, 2.5]))
    print("experts=%d top_k=%d rows=%d groups=%d/%d mode=%d scaling=%g" % (experts, top_k, rows, ng, kg, mode, scaling), flush=True)
    try:
        ids, w = RouteOps.topk_noaux(torch.from_numpy(lg).to(DEV), torch.from_numpy(b).to(DEV), top_k, mode, scaling, ng, kg, True)
    except capi.FfmoeError as e:
        assert e.code == capi.ERR_UNSUPPORTED and ng > 1, e  # a group width the wave selection does not take
        ng, kg = 1, 1
        ids, w = RouteOps.topk_noaux(torch.from_numpy(lg).to(DEV), torch.from_numpy(b).to(DEV), top_k, mode, scaling, ng, kg, True)
    oi, ow = orc.route_topk_noaux(lg, b[None, :], top_k, mode, scaling, ng, kg)
    assert np.array_equal(ids.cpu().numpy(), oi)
    assert np.array_equal(w.cpu().numpy().view(np.uint32), ow.view(np.uint32))
    # softmax / sigmoid top-k on BF16 logits
    lb = torch.from_numpy(lg).to(torch.bfloat16)
    for score, fn in ((capi.SCORE_SOFTMAX, orc.route_topk_softmax), (capi.SCORE_SIGMOID, orc.route_topk_sigmoid)):
        i2, w2 = RouteOps.topk(lb.to(DEV), top_k, score)
        wi, ww = fn(bits(lb), top_k)
        assert np.array_equal(i2.cpu().numpy(), wi) and np.array_equal(bits(w2), ww)


@pytest.mark.parametrize("rows,experts,hidden,top_k,ng,kg", [(1, 256, 7168, 8, 8, 4), (5, 64, 1024, 6, 1, 1), (3, 100, 520, 4, 4, 2), (2, 1000, 256, 32, 1, 1)])
def test_route_noaux_decode_equals_two_step_and_oracle(rows, experts, hidden, top_k, ng, kg):
    x, w = rand_bf16((rows, hidden), 1.0, 31), rand_bf16((experts, hidden), 0.02, 32)
    w[3] = w[7]                                   # two experts with identical logits: the tie goes to the lower id
    bias = synth.normal((experts,), 0.05, 33)
    bias[3] = bias[7]
    logits = torch.empty((rows, experts), dtype=torch.float32, device=DEV)
    ids = torch.empty((rows, top_k), dtype=torch.int32, device=DEV)
    wts = torch.empty((rows, top_k), dtype=torch.float32, device=DEV)
    done = torch.ones((rows, top_k), dtype=torch.int32, device=DEV)
    for _ in range(2):
        RouteOps.route_noaux(x.to(DEV), w.to(DEV), bias.to(DEV), top_k, logits, ids, wts, done=done,
                             routed_scaling=2.5, n_group=ng, topk_group=kg)
        torch.cuda.synchronize()
        assert int(done.abs().sum().item()) == 0
        ol = orc.route_logits_f32(bits(x), bits(w))
        oi, ow = orc.route_topk_noaux(ol, bias.numpy()[None, :], top_k, 0, 2.5, ng, kg)
        assert np.array_equal(logits.cpu().numpy().view(np.uint32), ol.view(np.uint32))
        assert np.array_equal(ids.cpu().numpy(), oi)
        assert np.array_equal(wts.cpu().numpy().view(np.uint32), ow.view(np.uint32))
        done.fill_(1)
    i2, w2 = RouteOps.topk_noaux(RouteOps.logits_f32(x.to(DEV), w.to(DEV)), bias.to(DEV), top_k, 0, 2.5, ng, kg, True)
    assert torch.equal(i2, ids) and torch.equal(w2.view(torch.int32), wts.view(torch.int32))


def test_route_decode_fused_c1_shape():
    x, w = rand_bf16((1, 2048), 1.0, 21), rand_bf16((64, 2048), 0.02, 22)
    ids, wt, logits = RouteOps.route(x.to(DEV), w.to(DEV), 4, capi.SCORE_SOFTMAX)
    ol = orc.route_logits_bf16(bits(x), bits(w))
    oi, ow = orc.route_topk_softmax(ol, 4)
    assert np.array_equal(bits(logits), ol) and np.array_equal(ids.cpu().numpy(), oi) and np.array_equal(bits(wt), ow)


@pytest.mark.parametrize("score", [capi.SCORE_SOFTMAX, capi.SCORE_SIGMOID])
@pytest.mark.parametrize("rows,experts,hidden,top_k", [(1, 64, 2048, 4), (3, 64, 520, 6), (5, 33, 264, 8), (2, 8, 4104, 3), (1, 128, 512, 4)])
def test_route_decode_one_launch_equals_the_two_launches_and_the_oracle(score, rows, experts, hidden, top_k):
    """ffmoe_route_decode: up to 64 experts the wave that runs a row's logit chains also selects (one launch); beyond, logits
    and selection are two launches. Logits, ids and weights bit for bit against the oracle and against the separate calls,
    with exact ties planted among the router rows (equal rows give equal logits: the lower id wins)."""
    x, w = rand_bf16((rows, hidden), 1.0, 121 + rows), rand_bf16((experts, hidden), 0.05, 122 + experts)
    w[experts - 1] = w[1]
    w[5] = w[2]
    print("route decode rows=%d experts=%d hidden=%d top_k=%d score=%d" % (rows, experts, hidden, top_k, score), flush=True)
    ids, wt, logits = RouteOps.route(x.to(DEV), w.to(DEV), top_k, score)
    torch.cuda.synchronize()
    ol = orc.route_logits_bf16(bits(x), bits(w))
    fn = orc.route_topk_softmax if score == capi.SCORE_SOFTMAX else orc.route_topk_sigmoid
    oi, ow = fn(ol, top_k)
    assert np.array_equal(bits(logits), ol)
    assert np.array_equal(ids.cpu().numpy(), oi)
    assert np.array_equal(bits(wt), ow)
    l2 = RouteOps.logits_bf16(x.to(DEV), w.to(DEV))
    i2, w2 = RouteOps.topk(l2, top_k, score)
    assert torch.equal(l2.view(torch.int16), logits.view(torch.int16)) and torch.equal(i2, ids) and torch.equal(w2.view(torch.int16), wt.view(torch.int16))


# ------------------------------------------------------------------------------------------------
# decode contributions
def _run_decode(fmt, experts, hidden, inter, rows, top_k, seed, shared, swiglu_mode=capi.SWIGLU_TWICE, limit=0.0,
                boundary=capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=False, with_active=False):
    table, ref = make_table(fmt, experts + (1 if shared else 0), hidden, inter, seed)
    sh = table.shared_struct(experts) if shared else None
    table.experts = experts
    x = rand_bf16((rows, hidden), 1.0, seed + 7)
    g = synth.generator(seed + 8)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    wt = torch.rand((rows, top_k), generator=g) * 0.5 + 0.05
    wdev = wt.to(DEV) if weights_f32 else wt.to(torch.bfloat16).to(DEV)
    wref = wt.numpy() if weights_f32 else wt.to(torch.bfloat16).float().numpy()
    active = None
    if with_active:
        active = (torch.rand((rows, top_k), generator=g) > 0.3).to(torch.int32)
    op = DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, swiglu_mode, limit, boundary, weights_f32)
    op.contributions.zero_()
    contrib, shared_out = op.contribute(x.to(DEV), ids.to(DEV), wdev, active.to(DEV) if active is not None else None)
    torch.cuda.synchronize()
    want = oracle_contributions(ref, bits(x), ids.numpy(), wref, swiglu_mode, limit, boundary, active.numpy() if active is not None else None)
    got = bits(contrib)
    stats = assert_close_bf16(got, want, "contributions")
    done = op.done.cpu().numpy()
    assert np.array_equal(done != 0, np.ones_like(done, bool) if active is None else active.numpy() != 0)
    if shared:
        assert_close_bf16(bits(shared_out), oracle_shared(ref[experts], bits(x), swiglu_mode, limit), "shared_out")
    return stats


def test_decode_fp8_c1_shape_single_token():
    # BASELINE config 1: hidden 2048, 64 experts, top-4, inter 1408, FP8 128x128 (weights for 8 experts are enough
    # for one token; ids are drawn from them)
    r, worst = _run_decode(capi.FMT_FP8_BLOCK128, 8, 2048, 1408, 1, 4, 31, shared=False)
    print("C1 rel_l2=%.2e worst_ulp=%.2f" % (r, worst))


@pytest.mark.parametrize("rows,top_k,shared", [(1, 8, True), (2, 4, True), (5, 3, False), (8, 4, True), (19, 2, True)])
def test_decode_fp8_batched_rows_group_by_expert(rows, top_k, shared):
    _run_decode(capi.FMT_FP8_BLOCK128, 8, 1024, 512, rows, top_k, 40 + rows, shared)


def test_decode_fp8_modes_and_active_mask():
    _run_decode(capi.FMT_FP8_BLOCK128, 6, 512, 384, 4, 3, 51, True, capi.SWIGLU_CLAMPED_TWICE, 0.05, capi.WEIGHT_BEFORE_CONTRIBUTION_BF16, True, True)
    _run_decode(capi.FMT_FP8_BLOCK128, 6, 512, 384, 1, 3, 52, False, capi.SWIGLU_ONCE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, False, True)
    _run_decode(capi.FMT_FP8_BLOCK128, 6, 512, 384, 3, 2, 53, True, capi.SWIGLU_CLAMPED_ONCE, 0.1, capi.WEIGHT_AFTER_DOWN_BF16, True, False)


@pytest.mark.parametrize("fmt", [capi.FMT_BF16, capi.FMT_FP8_BLOCK128, capi.FMT_NVFP4, capi.FMT_FP8_CHANNEL])
@pytest.mark.parametrize("rows", [1, 5])
def test_decode_gelu_twice(fmt, rows):
    """SwigluRounding::GeluTwice of the reference (src/cpu/expert_ffn.rs:65,87-91,110-113) on the streaming decode kernels."""
    _run_decode(fmt, 6, 512, 384, rows, 3, 58 + rows, True, capi.SWIGLU_GELU_TWICE, 0.0, capi.WEIGHT_BEFORE_CONTRIBUTION_BF16, True, False)


@pytest.mark.parametrize("rows", [1, 6])
def test_decode_nvfp4(rows):
    _run_decode(capi.FMT_NVFP4, 6, 1024, 512, rows, 3, 61, True)


@pytest.mark.parametrize("rows", [1, 6])
def test_decode_bf16_experts(rows):
    _run_decode(capi.FMT_BF16, 5, 1024, 256, rows, 2, 71, True)


@pytest.mark.parametrize("seed", range(32))
def test_decode_seeded_shape_sweep(seed):
    """Shapes the fixed cases do not visit: every format at odd multiples of its granule (row tails, partial slabs,
    hidden < inter and the reverse), 1..17 rows, 1..8 choices, with and without a shared expert, an active mask, every
    SwiGLU rounding and both routing-weight boundaries; the configuration is a function of the seed alone.

    Each launch is held to the bar on its own inputs: the activations against the oracle's, the down stage against the
    oracle's down stage on the activations the device produced. End to end the two stages compose: one flipped BF16
    step of an activation can move a cancelled down output by more than two of its own steps at these small shapes, so
    that comparison keeps the relative-L2 bar and allows four steps."""
    rng = np.random.default_rng(1000 + seed)
    fmt = [capi.FMT_FP8_BLOCK128, capi.FMT_NVFP4, capi.FMT_BF16, capi.FMT_FP8_CHANNEL][seed % 4]
    gran = {capi.FMT_FP8_BLOCK128: 128, capi.FMT_NVFP4: 32, capi.FMT_BF16: 8, capi.FMT_FP8_CHANNEL: 16}[fmt]
    hidden = gran * int(rng.integers(128 // gran, 1536 // gran + 1))
    inter = gran * int(rng.integers(128 // gran, 1024 // gran + 1))
    experts = int(rng.integers(2, 13))
    top_k = int(rng.integers(1, min(8, experts) + 1))
    rows = int(rng.choice([1, 1, 2, 3, 4, 7, 9, 17]))
    mode = int(rng.integers(0, 5))
    limit = float(rng.choice([0.03, 0.1, 1.0])) if mode in (2, 3) else 0.0
    boundary = int(rng.integers(0, 2))
    shared, weights_f32, with_active = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    print("fmt=%d hidden=%d inter=%d experts=%d top_k=%d rows=%d mode=%d limit=%g boundary=%d shared=%d f32=%d mask=%d" %
          (fmt, hidden, inter, experts, top_k, rows, mode, limit, boundary, shared, weights_f32, with_active), flush=True)
    table, ref = make_table(fmt, experts + (1 if shared else 0), hidden, inter, 3000 + seed)
    sh = table.shared_struct(experts) if shared else None
    table.experts = experts
    x = rand_bf16((rows, hidden), 1.0, 3007 + seed)
    g = synth.generator(3008 + seed)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    wt = torch.rand((rows, top_k), generator=g) * 0.5 + 0.05
    wdev = wt.to(DEV) if weights_f32 else wt.to(torch.bfloat16).to(DEV)
    wref = wt.numpy() if weights_f32 else wt.to(torch.bfloat16).float().numpy()
    active = (torch.rand((rows, top_k), generator=g) > 0.3).to(torch.int32) if with_active else torch.ones((rows, top_k), dtype=torch.int32)
    op = DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, mode, limit, boundary, weights_f32)
    op.contributions.zero_()
    contrib, shared_out = op.contribute(x.to(DEV), ids.to(DEV), wdev, active.to(DEV) if with_active else None)
    torch.cuda.synchronize()
    got = bits(contrib)
    A = rows * top_k
    h = bits(op.scratch[: (A + rows) * inter * 2].view(torch.bfloat16).view(A + rows, inter))  # slot a, then A + row for the shared expert
    done = op.done.cpu().numpy()
    assert np.array_equal(done != 0, active.numpy() != 0)
    xb = bits(x)
    for r in range(rows):
        for c in range(top_k):
            if not active[r, c]:
                assert not got[r, c].any()
                continue
            ge, ue, de = ref[int(ids[r, c])]
            want, act = orc.expert_ffn(xb[r], ge, ue, de, float(wref[r, c]), mode, limit, boundary, orc.LANE8, orc.SILU_DIV, return_act=True)
            assert_close_bf16(h[r * top_k + c][None, :], act[None, :], "activations row %d choice %d" % (r, c))
            assert_close_bf16(got[r, c][None, :], orc.expert_down(h[r * top_k + c], de, float(wref[r, c]), boundary, orc.LANE8)[None, :],
                              "down stage row %d choice %d" % (r, c))
            assert_close_bf16(got[r, c][None, :], want[None, :], "contribution row %d choice %d" % (r, c), max_ulp=4)
        if shared:
            ge, ue, de = ref[experts]
            want, act = orc.expert_ffn(xb[r], ge, ue, de, 1.0, mode, limit, 0, orc.LANE8, orc.SILU_DIV, apply_weight=False, return_act=True)
            so = bits(shared_out)[r]
            assert_close_bf16(h[A + r][None, :], act[None, :], "shared activations row %d" % r)
            assert_close_bf16(so[None, :], orc.expert_down(h[A + r], de, 1.0, 0, orc.LANE8, False)[None, :], "shared down stage row %d" % r)
            assert_close_bf16(so[None, :], want[None, :], "shared_out row %d" % r, max_ulp=4)


@pytest.mark.parametrize("rows,routed_fmt,shared_fmt,shared_extra", [(1, capi.FMT_NVFP4, capi.FMT_BF16, 0), (6, capi.FMT_NVFP4, capi.FMT_BF16, 0),
                                                                     (3, capi.FMT_FP8_BLOCK128, capi.FMT_BF16, 0), (9, capi.FMT_NVFP4, capi.FMT_BF16, 8),
                                                                     (5, capi.FMT_FP8_BLOCK128, capi.FMT_NVFP4, 32), (4, capi.FMT_NVFP4, capi.FMT_BF16, -64)])
def test_decode_shared_expert_in_another_format(rows, routed_fmt, shared_fmt, shared_extra):
    """BASELINE config 4: NVFP4 routed experts next to a BF16 shared expert (two passes over one scratch arena). With a
    shared expert slightly wider (or narrower) than the routed ones both passes must still agree on the arena's row
    stride and on where the grouping tables sit, also when the stages are issued one by one."""
    experts, hidden, inter, top_k, seed = 6, 1024, 512, 3, 91
    table, ref = make_table(routed_fmt, experts, hidden, inter, seed)
    stable, sref = make_table(shared_fmt, 1, hidden, inter + shared_extra, seed + 1)
    sh = stable.shared_struct(0)
    x = rand_bf16((rows, hidden), 1.0, seed + 7)
    g = synth.generator(seed + 8)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    wt = (torch.rand((rows, top_k), generator=g) * 0.5 + 0.05).to(torch.bfloat16)
    op = DecodeOps(table, sh, rows, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, False)
    contrib, shared_out = op.contribute(x.to(DEV), ids.to(DEV), wt.to(DEV))
    torch.cuda.synchronize()
    want = oracle_contributions(ref, bits(x), ids.numpy(), wt.float().numpy(), capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16)
    assert_close_bf16(bits(contrib), want, "contributions")
    assert_close_bf16(bits(shared_out), oracle_shared(sref[0], bits(x), capi.SWIGLU_TWICE, 0.0), "shared_out")
    assert np.all(op.done.cpu().numpy() != 0)
    # the two stages may also be issued one by one
    c0 = bits(contrib).copy()
    s0 = bits(shared_out).copy()
    op.contributions.zero_(); op.shared_out.zero_()
    op.contribute(x.to(DEV), ids.to(DEV), wt.to(DEV), stage=0)
    op.contribute(x.to(DEV), ids.to(DEV), wt.to(DEV), stage=1)
    torch.cuda.synchronize()
    assert np.array_equal(bits(op.contributions), c0) and np.array_equal(bits(op.shared_out), s0)


@pytest.mark.parametrize("fmt,hidden,inter,top_k,shared", [
    (capi.FMT_FP8_BLOCK128, 1024, 512, 8, True),     # 9 groups, one step per row
    (capi.FMT_FP8_BLOCK128, 512, 2048, 3, True),     # 4 groups, two steps per row
    (capi.FMT_FP8_BLOCK128, 1024, 384, 4, False),    # routed only
    (capi.FMT_NVFP4, 1024, 512, 6, True),
    (capi.FMT_BF16, 1024, 256, 2, True),
    (capi.FMT_FP8_BLOCK128, 9216, 256, 2, True),     # 36 columns per block on 256 CUs: 9 shared units for 8 waves
    (capi.FMT_FP8_BLOCK128, 16384, 128, 1, True),    # 64 columns per block: 16 shared units
])
def test_decode_finish_equals_down_plus_combine(fmt, hidden, inter, top_k, shared):
    """One-token finish (one launch) against the separate down and combine launches: bit-identical y in every
    combine mode, with and without inactive choices; oracle parity of the separate path is covered above."""
    experts, seed = 10, 97
    table, ref = make_table(fmt, experts + (1 if shared else 0), hidden, inter, seed)
    sh = table.shared_struct(experts) if shared else None
    table.experts = experts
    x = rand_bf16((1, hidden), 1.0, seed + 7).to(DEV)
    g = synth.generator(seed + 8)
    ids = torch.randperm(experts, generator=g)[:top_k].to(torch.int32).view(1, top_k).to(DEV)
    wt = (torch.rand((1, top_k), generator=g) * 0.5 + 0.05).to(DEV)
    scale = rand_bf16((1,), 0.5, seed + 9).to(DEV)
    modes = [capi.COMBINE_ROUTED] if not shared else [capi.COMBINE_GATED, capi.COMBINE_UNGATED, capi.COMBINE_BF16,
                                                      capi.COMBINE_ACCUM_FP32, capi.COMBINE_ACCUM_BF16]
    for with_active in (False, True):
        active = None
        if with_active:
            a = torch.ones((1, top_k), dtype=torch.int32)
            a[0, 0] = 0
            a[0, top_k - 1] = 0 if top_k > 2 else 1
            active = a.to(DEV)
        op = DecodeOps(table, sh, 1, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
        op.done.zero_()
        op.contributions.zero_()  # the accumulate modes add every slot, live or not: skipped slots must read as zero
        contrib, shared_out = op.contribute(x, ids, wt, active)
        for mode in modes:
            want = CombineOps.combine(contrib, shared_out, ids, mode, scale=scale, done=op.done, final_active=active)
            y = torch.full((1, hidden), 7.0, dtype=torch.bfloat16, device=DEV)
            status = torch.zeros(1, dtype=torch.int32, device=DEV)
            op.contribute(x, ids, wt, active, stage=0)
            assert op.finish(x, ids, wt, mode, y, status=status, scale=scale, active=active)
            torch.cuda.synchronize()
            assert int(status.item()) == 0
            assert np.array_equal(bits(y), bits(want)), "mode %d active %s" % (mode, with_active)


@pytest.mark.parametrize("shape", ["16,8", "128,8", "7,12", "3,16"])
def test_decode_finish_shape_override_keeps_the_bits(shape, monkeypatch):
    """FFMOE_FINISH_SHAPE = "blocks,waves" changes the launch shape only: also where a block holds more shared-expert
    units than it has waves (16 blocks of 64 columns = 16 units on 8 waves), y stays what the separate launches give."""
    experts, hidden, inter, top_k, seed = 6, 1024, 256, 3, 131
    table, _ = make_table(capi.FMT_FP8_BLOCK128, experts + 1, hidden, inter, seed)
    sh = table.shared_struct(experts)
    table.experts = experts
    x = rand_bf16((1, hidden), 1.0, seed + 1).to(DEV)
    ids = torch.tensor([[4, 0, 3]], dtype=torch.int32, device=DEV)
    wt = torch.tensor([[0.4, 0.25, 0.35]], device=DEV)
    op = DecodeOps(table, sh, 1, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
    contrib, shared_out = op.contribute(x, ids, wt)
    want = CombineOps.combine(contrib, shared_out, ids, capi.COMBINE_UNGATED, done=op.done)
    monkeypatch.setenv("FFMOE_FINISH_SHAPE", shape)
    y = torch.full((1, hidden), 7.0, dtype=torch.bfloat16, device=DEV)
    op.contribute(x, ids, wt, stage=0)
    assert op.finish(x, ids, wt, capi.COMBINE_UNGATED, y)
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), bits(want))


def test_decode_finish_flags_bad_expert_and_declines_unsupported_shapes():
    table, _ = make_table(capi.FMT_FP8_BLOCK128, 5, 512, 256, 5)
    sh = table.shared_struct(4)
    table.experts = 4
    x = rand_bf16((1, 512), 1.0, 3).to(DEV)
    ids = torch.tensor([[1, 9, 2]], dtype=torch.int32, device=DEV)  # 9 is out of range
    wt = torch.full((1, 3), 0.25, device=DEV)
    op = DecodeOps(table, sh, 1, 3, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
    op.contribute(x, ids, wt, stage=0)
    y = torch.zeros((1, 512), dtype=torch.bfloat16, device=DEV)
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    assert op.finish(x, ids, wt, capi.COMBINE_UNGATED, y, status=status)
    torch.cuda.synchronize()
    assert int(status.item()) == 1
    # the two good choices and the shared expert still add up
    good = torch.tensor([[1, 2]], dtype=torch.int32, device=DEV)
    op2 = DecodeOps(table, sh, 1, 2, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
    c2, s2 = op2.contribute(x, good, wt[:, :2].contiguous())
    want = CombineOps.combine(c2, s2, good, capi.COMBINE_UNGATED)
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), bits(want))
    # two rows: outside the fast path, nothing launched
    op3 = DecodeOps(table, sh, 2, 2, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
    x2 = rand_bf16((2, 512), 1.0, 4).to(DEV)
    ids2 = torch.tensor([[0, 1], [2, 3]], dtype=torch.int32, device=DEV)
    y2 = torch.zeros((2, 512), dtype=torch.bfloat16, device=DEV)
    assert not op3.finish(x2, ids2, torch.full((2, 2), 0.5, device=DEV), capi.COMBINE_UNGATED, y2)


def test_decode_dsv3_width_single_token():
    # hidden 7168 / inter 2048 at DeepSeek-V3 width, 3 routed experts + shared, one token
    _run_decode(capi.FMT_FP8_BLOCK128, 3, 7168, 2048, 1, 3, 81, True)


def test_decode_row_count_invariance_bitwise():
    # rows batched == each row run alone, bit for bit (src/backend/cuda/moe/decode_tests.rs:347-399)
    experts, hidden, inter, rows, top_k = 8, 1024, 512, 6, 4
    table, _ = make_table(capi.FMT_FP8_BLOCK128, experts, hidden, inter, 91)
    x = rand_bf16((rows, hidden), 1.0, 92).to(DEV)
    g = synth.generator(93)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32).to(DEV)
    wt = (torch.rand((rows, top_k), generator=g) + 0.1).to(torch.bfloat16).to(DEV)
    batched = DecodeOps(table, None, rows, top_k)
    full = batched.contribute(x, ids, wt)[0].clone()
    single = DecodeOps(table, None, 1, top_k)
    for r in range(rows):
        one = single.contribute(x[r:r + 1].contiguous(), ids[r:r + 1].contiguous(), wt[r:r + 1].contiguous())[0]
        assert torch.equal(one[0].view(torch.int16), full[r].view(torch.int16)), r


def test_decode_mutation_controls():
    # swapping two experts' codes or changing one scale must change the output (prefill_tests.rs:485-535)
    experts, hidden, inter = 4, 512, 256
    table, _ = make_table(capi.FMT_FP8_BLOCK128, experts, hidden, inter, 95)
    x = rand_bf16((1, hidden), 1.0, 96).to(DEV)
    ids = torch.tensor([[0, 1]], dtype=torch.int32, device=DEV)
    wt = torch.tensor([[0.5, 0.25]], dtype=torch.bfloat16, device=DEV)
    op = DecodeOps(table, None, 1, 2)
    base = op.contribute(x, ids, wt)[0].clone()
    v0, v1 = table.expert_views(0), table.expert_views(1)
    tmp = v0[0].clone(); v0[0].copy_(v1[0]); v1[0].copy_(tmp)
    swapped = op.contribute(x, ids, wt)[0].clone()
    assert not torch.equal(base.view(torch.int16), swapped.view(torch.int16))
    v1[0].copy_(v0[0]); v0[0].copy_(tmp)
    assert torch.equal(op.contribute(x, ids, wt)[0].view(torch.int16), base.view(torch.int16))
    v0[5][0, 0] *= 1.5
    assert not torch.equal(op.contribute(x, ids, wt)[0].view(torch.int16), base.view(torch.int16))


# ------------------------------------------------------------------------------------------------
# standalone linears (BASELINE config 2 at reduced N so the oracle stays fast)
@pytest.mark.parametrize("m", [1, 4, 16])
@pytest.mark.parametrize("k,n", [(7168, 256), (2048, 384)])
def test_linear_fp8_block_w8a16(m, k, n):
    w = synth.normal((n, k), 0.02, 200 + m)
    codes, scales = synth.quant_fp8_block(w)
    x = rand_bf16((m, k), 1.0, 300 + m)
    y = bits(Fp8Ops.linear(codes.to(DEV), scales.to(DEV), x.to(DEV)))
    eff = orc.dequant_fp8_block(codes.numpy(), scales.numpy())
    want = np.stack([[orc.f32_to_bf16(np.float32(orc.dot(orc.bf16_to_f32(bits(x)[r]), eff[c], orc.LANE8))) for c in range(n)] for r in range(m)]).astype(np.uint16).reshape(m, n)
    assert_close_bf16(y, want, "fp8 linear")
    f64 = orc.linear_skinny(eff, bits(x), 2)
    assert_close_bf16(y, f64, "fp8 linear vs f64")


@pytest.mark.parametrize("m,k,n", [
    (5, 7168, 64),     # two x panels, 8-row tiles
    (16, 3648, 48),    # 57 column units: a second panel of one unit, waves without work
    (33, 256, 4096),   # a block per 16 weight rows, three passes of 16 / 16 / 1 rows
    (9, 192, 32),      # three units for eight waves
])
def test_linear_fp8_block_matrix_core_path(m, k, n):
    """More than 4 rows go through the BF16 matrix cores: the same effective weights, FP32 accumulation in the
    instruction's order; against the reference's Lane8 order and the FP64 sum, and against the streaming kernel."""
    import os
    w = synth.normal((n, k), 0.02, 700 + m)
    codes, scales = synth.quant_fp8_block(w)
    x = rand_bf16((m, k), 1.0, 710 + m)
    y = bits(Fp8Ops.linear(codes.to(DEV), scales.to(DEV), x.to(DEV)))
    eff = orc.dequant_fp8_block(codes.numpy(), scales.numpy())
    assert_close_bf16(y, orc.linear_skinny(eff, bits(x), 2), "fp8 linear (matrix cores) vs f64")
    os.environ["FFMOE_LINEAR_NO_MFMA"] = "1"
    try:
        y2 = bits(Fp8Ops.linear(codes.to(DEV), scales.to(DEV), x.to(DEV)))
    finally:
        del os.environ["FFMOE_LINEAR_NO_MFMA"]
    assert_close_bf16(y, y2, "fp8 linear: matrix cores vs streaming kernel")
    # rows are independent: a row computed alone (streaming kernel) and inside the 16-row panel agree to the bar, and
    # the panel's padding rows leave nothing behind
    assert orc.rel_l2(y, y2) < 1e-3


@pytest.mark.parametrize("m,k,n", [(40, 2048, 192), (17, 3712, 48), (21, 128, 4096)])
def test_linear_nvfp4_and_bf16_matrix_core_path(m, k, n):
    """NVFP4 beyond 16 rows (the reference switches to its MMA kernel there, nvfp4_linear.cu:262-573, bounded by
    max_abs 0.03125 / rmse 0.004 in its tests; here the usual bar against the FP64 sum) and BF16 weights beyond 4."""
    w = synth.normal((n, k), 0.02, 800 + m)
    codes, scales, g = synth.quant_nvfp4(w)
    x = rand_bf16((m, k), 1.0, 801 + m)
    gs = torch.tensor([g], dtype=torch.float32, device=DEV)
    y = bits(NvFp4Ops.gemm(codes.to(DEV), scales.to(DEV), gs, x.to(DEV)))
    eff = orc.dequant_nvfp4(codes.numpy(), scales.numpy(), g)
    want = orc.linear_skinny(eff, bits(x), 2)
    assert_close_bf16(y, want, "nvfp4 linear (matrix cores) vs f64")
    d = orc.bf16_to_f32(y).astype(np.float64) - orc.bf16_to_f32(want).astype(np.float64)
    assert np.abs(d).max() <= 0.03125 and np.sqrt((d * d).mean()) <= 0.004
    wb = w.to(torch.bfloat16)
    yb = bits(gemm_skinny_bf16(wb.to(DEV), x.to(DEV)))
    assert_close_bf16(yb, orc.linear_skinny(bits(wb), bits(x), 2), "bf16 skinny (matrix cores)")


@pytest.mark.parametrize("m", [1, 3, 16])
def test_linear_nvfp4_and_bf16(m):
    n, k = 192, 2048
    w = synth.normal((n, k), 0.02, 400)
    codes, scales, g = synth.quant_nvfp4(w)
    x = rand_bf16((m, k), 1.0, 401 + m)
    gs = torch.tensor([g], dtype=torch.float32, device=DEV)
    y = bits(NvFp4Ops.gemm(codes.to(DEV), scales.to(DEV), gs, x.to(DEV)))
    eff = orc.dequant_nvfp4(codes.numpy(), scales.numpy(), g)
    assert_close_bf16(y, orc.linear_skinny(eff, bits(x), 1), "nvfp4 linear (reference skinny order)")
    wb = w.to(torch.bfloat16)
    yb = bits(gemm_skinny_bf16(wb.to(DEV), x.to(DEV)))
    assert_close_bf16(yb, orc.linear_skinny(bits(wb), bits(x), 2), "bf16 skinny")
    # nibble-swap control (src/backend/cuda/linear.rs:4737)
    sw = ((codes << 4) | (codes >> 4)).to(torch.uint8)
    y2 = bits(NvFp4Ops.gemm(sw.to(DEV), scales.to(DEV), gs, x.to(DEV)))
    assert not np.array_equal(y, y2)


# ------------------------------------------------------------------------------------------------
# combine
def test_combine_modes_bit_exact():
    rows, top_k, hidden = 5, 8, 1024
    c = rand_bf16((rows, top_k, hidden), 1.0, 500)
    sh = rand_bf16((rows, hidden), 1.0, 501)
    g = synth.generator(502)
    ids = torch.stack([torch.randperm(64, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    act = (torch.rand((rows, top_k), generator=g) > 0.25).to(torch.int32)
    x = rand_bf16((rows, hidden), 1.0, 503)
    seg = rand_bf16((hidden,), 0.05, 504)
    scale = CombineOps.shared_scale(x.to(DEV), seg.to(DEV))
    assert np.array_equal(bits(scale), orc.shared_scale(bits(x), bits(seg)))
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    for mode in range(6):
        y = CombineOps.combine(c.to(DEV), sh.to(DEV), ids.to(DEV), mode, scale=scale, done=act.to(DEV), final_active=act.to(DEV), status=status)
        want = orc.combine(bits(c), bits(sh), bits(scale), ids.numpy(), act.numpy().astype(np.uint32), mode)
        assert np.array_equal(bits(y), want), mode
    assert int(status.item()) == 0
    # a slot whose done flag disagrees with final_active raises the status bit (the reference traps here)
    bad = act.clone(); bad[2, 1] ^= 1
    CombineOps.combine(c.to(DEV), sh.to(DEV), ids.to(DEV), capi.COMBINE_BF16, done=bad.to(DEV), final_active=act.to(DEV), status=status)
    assert int(status.item()) == 1


@pytest.mark.parametrize("seed", range(12))
def test_combine_seeded_sweep_bit_exact(seed):
    """Combine shapes the fixed case does not visit (1..33 rows, 1..8 choices, hidden any multiple of 8 up to 2048,
    rows with no active choice at all), every mode, bit for bit."""
    rng = np.random.default_rng(4000 + seed)
    rows, top_k = int(rng.choice([1, 2, 7, 33])), int(rng.integers(1, 9))
    hidden = 8 * int(rng.integers(16, 257))
    experts = int(rng.integers(top_k, 65)) + 1
    c = rand_bf16((rows, top_k, hidden), 1.0, 4100 + seed)
    sh = rand_bf16((rows, hidden), 1.0, 4200 + seed)
    g = synth.generator(4300 + seed)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    act = (torch.rand((rows, top_k), generator=g) > 0.3).to(torch.int32)
    act[0] = 0  # a row whose choices are all inactive
    scale = rand_bf16((rows,), 0.5, 4400 + seed).to(DEV)
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    print("rows=%d top_k=%d hidden=%d experts=%d" % (rows, top_k, hidden, experts), flush=True)
    for mode in range(6):
        y = CombineOps.combine(c.to(DEV), sh.to(DEV), ids.to(DEV), mode, scale=scale, done=act.to(DEV), final_active=act.to(DEV), status=status)
        want = orc.combine(bits(c), bits(sh), bits(scale), ids.numpy(), act.numpy().astype(np.uint32), mode)
        assert np.array_equal(bits(y), want), mode
    assert int(status.item()) == 0


def test_combine_residual_and_peer_join_bit_exact():
    """combine + residual add in one launch, gated and ungated, in place and to y_out, and the form that takes a routed
    sum computed elsewhere (kernels/moe_combine.cu:246-533), against the oracle's combine + BF16 adds."""
    rows, top_k, hidden = 3, 6, 2304   # 2304 = 9 x 256: the last block of a row is partly empty
    c = rand_bf16((rows, top_k, hidden), 1.0, 510)
    sh = rand_bf16((rows, hidden), 1.0, 511)
    g = synth.generator(512)
    ids = torch.stack([torch.randperm(32, generator=g)[:top_k] for _ in range(rows)]).to(torch.int32)
    act = (torch.rand((rows, top_k), generator=g) > 0.25).to(torch.int32)
    xw = rand_bf16((rows, hidden + 64), 1.0, 513)       # x rows live inside wider rows (x_stride > hidden)
    x = xw[:, :hidden]
    seg = rand_bf16((hidden,), 0.05, 514)
    res0 = rand_bf16((rows, hidden), 1.0, 515)
    scale = orc.shared_scale(bits(x.contiguous()), bits(seg))
    actn = act.numpy().astype(np.uint32)

    def bf16_add(a_bits, b_bits):
        return orc.f32_to_bf16(orc.bf16_to_f32(a_bits) + orc.bf16_to_f32(b_bits))
    xd = xw.to(DEV)[:, :hidden]
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    for gated in (True, False):
        ff = orc.combine(bits(c), bits(sh), scale, ids.numpy(), actn, capi.COMBINE_GATED if gated else capi.COMBINE_UNGATED)
        kw = dict(seg=seg.to(DEV), x=xd) if gated else {}
        y = torch.empty((rows, hidden), dtype=torch.bfloat16, device=DEV)
        CombineOps.combine_residual(sh.to(DEV), y_out=y, contributions=c.to(DEV), ids=ids.to(DEV), done=act.to(DEV),
                                    final_active=act.to(DEV), status=status, **kw)
        assert np.array_equal(bits(y), ff), "y_out gated=%s" % gated
        res = res0.clone().to(DEV)
        CombineOps.combine_residual(sh.to(DEV), residual=res, contributions=c.to(DEV), ids=ids.to(DEV), done=act.to(DEV),
                                    final_active=act.to(DEV), status=status, **kw)
        assert np.array_equal(bits(res), bf16_add(bits(res0), ff)), "residual gated=%s" % gated
        # peer join: the routed sum arrives as BF16
        routed = orc.combine(bits(c), None, None, ids.numpy(), actn, capi.COMBINE_ROUTED)
        res = res0.clone().to(DEV)
        CombineOps.combine_residual(sh.to(DEV), residual=res, routed_in=bf16_tensor(routed), **kw)
        assert np.array_equal(bits(res), bf16_add(bits(res0), ff)), "join gated=%s" % gated
    assert int(status.item()) == 0


def test_residency_protocol_publish_mask_and_stale_choices():
    """Slot publication, routing mask and the epoch check (kernels/moe_route.cu:650-681, kernels/moe_ffn.cu:140-154):
    a choice routed against an epoch that has since been replaced contributes nothing and leaves done = 0, which the
    combine reports through its status word (the reference traps)."""
    from flyingfish_amd.ops import Residency
    experts, hidden, inter, rows, top_k = 6, 512, 256, 2, 3
    table, ref = make_table(capi.FMT_FP8_BLOCK128, experts, hidden, inter, 700)
    addresses = table.slots.cpu().clone()
    # start with an empty table and publish experts 0..4 at epochs 1..5; expert 5 stays out
    table.slots.zero_()
    table.valid = torch.zeros(experts, dtype=torch.int32, device=DEV)
    table.generation = torch.zeros(experts, dtype=torch.int64, device=DEV)
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    for e in range(5):
        Residency.publish(table, e, addresses[e].tolist(), epoch=e + 1, status=status)
    torch.cuda.synchronize()
    assert table.valid.cpu().tolist() == [1, 1, 1, 1, 1, 0] and table.generation.cpu().tolist() == [1, 2, 3, 4, 5, 0]
    assert torch.equal(table.slots.cpu()[:5], addresses[:5]) and int(status.item()) == 0
    ids = torch.tensor([[0, 5, 2], [4, 1, 3]], dtype=torch.int32, device=DEV)
    active, gen = Residency.mask(table, ids, status=status)
    torch.cuda.synchronize()
    assert active.cpu().tolist() == [[1, 0, 1], [1, 1, 1]] and gen.cpu().tolist() == [[1, 0, 3], [5, 2, 4]] and int(status.item()) == 0
    x = rand_bf16((rows, hidden), 1.0, 701).to(DEV)
    wt = torch.full((rows, top_k), 0.5, device=DEV)
    op = DecodeOps(table, None, rows, top_k, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, True)
    op.done.zero_()
    op.contribute(x, ids, wt, active, assignment_gen=gen)
    torch.cuda.synchronize()
    assert op.done.cpu().tolist() == [[1, 0, 1], [1, 1, 1]]
    first = bits(op.contributions).copy()
    # expert 2 is replaced (same weights, new epoch 9; expert 5 comes in over victim 1): choices routed earlier against
    # epochs 3 and 2 are now stale
    Residency.publish(table, 2, addresses[2].tolist(), epoch=9, status=status)
    Residency.publish(table, 5, addresses[5].tolist(), epoch=10, victim=1, status=status)
    op.done.zero_()
    op.contributions.zero_()
    op.contribute(x, ids, wt, active, assignment_gen=gen)
    torch.cuda.synchronize()
    assert op.done.cpu().tolist() == [[1, 0, 0], [1, 0, 1]]
    second = bits(op.contributions)
    assert np.array_equal(second[0, 0], first[0, 0]) and np.array_equal(second[1, 2], first[1, 2]) and not second[0, 2].any() and not second[1, 1].any()
    CombineOps.combine(op.contributions, None, ids, capi.COMBINE_ROUTED, done=op.done, final_active=active, status=status)
    torch.cuda.synchronize()
    assert int(status.item()) == 1
    # an epoch may only move forward; out-of-range ids are flagged by the mask
    status.zero_()
    Residency.publish(table, 0, addresses[0].tolist(), epoch=1, status=status)
    torch.cuda.synchronize()
    assert int(status.item()) == 1
    status.zero_()
    Residency.mask(table, torch.tensor([[0, 77, 2]], dtype=torch.int32, device=DEV), status=status)
    torch.cuda.synchronize()
    assert int(status.item()) == 1


# ------------------------------------------------------------------------------------------------
# whole layer
def test_native_moe_layer_matches_oracle_pipeline():
    experts, hidden, inter, rows, top_k = 16, 1024, 512, 4, 4
    table, ref = make_table(capi.FMT_FP8_BLOCK128, experts + 1, hidden, inter, 600)
    shared = table.shared_struct(experts)
    table.experts = experts
    router = rand_bf16((experts, hidden), 0.02, 601)
    bias = synth.normal((experts,), 0.01, 602)
    x = rand_bf16((rows, hidden), 1.0, 603)
    layer = NativeMoe(table, shared, router.to(DEV), bias.to(DEV), rows, top_k, 2.5, 4, 2)
    y = layer.run(x.to(DEV))
    torch.cuda.synchronize()
    assert int(layer.status.item()) == 0
    lg = orc.route_logits_f32(bits(x), bits(router))
    oi, ow = orc.route_topk_noaux(lg, bias.numpy()[None, :], top_k, 0, 2.5, 4, 2)
    assert np.array_equal(layer.ids.cpu().numpy(), oi)
    assert np.array_equal(layer.weights.cpu().numpy().view(np.uint32), ow.view(np.uint32))
    contrib = oracle_contributions(ref, bits(x), oi, ow, orc.TWICE, 0.0, orc.BEFORE_CONTRIBUTION_BF16)
    sh = oracle_shared(ref[experts], bits(x), orc.TWICE, 0.0)
    want = orc.combine(contrib, sh, None, oi, None, orc.COMBINE_BF16)
    # Every contribution may sit 2 BF16 steps from the oracle's and the BF16 running sum rounds once per term, so the
    # bound per element is 3 steps per term at the largest term's magnitude (the reference bounds its own GPU layer
    # by measured combine-order spread + 1 ulp at the largest output, src/backend/cuda/moe/reference.rs:613-678).
    terms = np.concatenate([orc.bf16_to_f32(contrib), orc.bf16_to_f32(sh)[:, None, :], orc.bf16_to_f32(want)[:, None, :]], axis=1)
    mag = np.max(np.abs(terms), axis=1).astype(np.float64)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(mag, 1e-30))) - 7)
    err = np.abs(orc.bf16_to_f32(bits(y)).astype(np.float64) - orc.bf16_to_f32(want).astype(np.float64))
    assert np.all(err <= 3 * (top_k + 1) * ulp), float(np.max(err / ulp))
    assert orc.rel_l2(bits(y), want) <= 4e-3


def test_decode_layer_graph_replay_equals_eager():
    """Eager-vs-graph bit equality of the whole decode layer (route, contribute, combine), several replays."""
    table, _ = make_table(capi.FMT_FP8_BLOCK128, 9, 1024, 512, 23)
    sh = table.shared_struct(8)
    table.experts = 8
    router = rand_bf16((8, 1024), 0.02, 24).to(DEV)
    bias = torch.zeros(8, device=DEV)
    for rows in (1, 4):
        layer = NativeMoe(table, sh, router, bias, rows, 3, routed_scaling=2.5, combine_mode=capi.COMBINE_UNGATED,
                          routed_weight=capi.WEIGHT_AFTER_DOWN_BF16)
        x = rand_bf16((rows, 1024), 1.0, 25 + rows).to(DEV)
        eager = bits(layer.run(x)).copy()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                layer.run(x)
        torch.cuda.current_stream().wait_stream(side)
        for it in range(3):
            layer.y.zero_()
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            assert np.array_equal(bits(layer.y), eager), "rows %d replay %d" % (rows, it)
        assert int(layer.status.item()) == 0


@pytest.mark.parametrize("fmt", [capi.FMT_FP8_BLOCK128, capi.FMT_NVFP4])
@pytest.mark.parametrize("experts,n_group,topk_group", [(64, 1, 1), (256, 8, 4)])
def test_one_token_selection_inside_gate_up_launch(fmt, experts, n_group, topk_group):
    """ffmoe_decode_contribute_from_logits: ids, weights, contributions and y equal the separate top-k launch bit for bit."""
    hidden, inter, top_k = 512, 256, 6
    table, _ = make_table(fmt, experts + 1, hidden, inter, 61)
    sh = table.shared_struct(experts)
    table.experts = experts
    router = rand_bf16((experts, hidden), 0.05, 62).to(DEV)
    bias = (torch.randn(experts, generator=torch.Generator().manual_seed(63)) * 0.1).to(DEV)
    x = rand_bf16((1, hidden), 1.0, 64).to(DEV)
    got = {}
    for inline in (False, True):
        layer = NativeMoe(table, sh, router, bias, 1, top_k, routed_scaling=2.5, n_group=n_group, topk_group=topk_group)
        layer.inline_select = inline
        layer.two_launch = False  # this test reads contributions and done, which the two-launch path does not write
        layer.decode.done.fill_(7)  # stale flags: both paths must clear them
        y = bits(layer.run(x)).copy()
        assert layer.inline_select == inline
        got[inline] = (layer.ids.cpu().numpy().copy(), layer.weights.cpu().numpy().copy(), bits(layer.decode.contributions).copy(), y,
                       layer.decode.done.cpu().numpy().copy())
        assert int(layer.status.item()) == 0
    for name, a, b in zip(("ids", "weights", "contributions", "y", "done"), got[False], got[True]):
        assert np.array_equal(a, b), name
    assert got[True][4].ravel().tolist() == [1] * top_k
    # and against the oracle's selection
    ids, w = orc.route_topk_noaux(orc.route_logits_f32(bits(x), bits(router)), bias.cpu().numpy()[None, :], top_k, 0, 2.5, n_group, topk_group)
    assert np.array_equal(ids, got[True][0]) and np.array_equal(w.view(np.uint32), got[True][1].view(np.uint32))


def test_selection_inside_gate_up_launch_rejects_batches():
    table, _ = make_table(capi.FMT_FP8_BLOCK128, 64, 256, 128, 71)
    ops = DecodeOps(table, None, 2, 2, capi.ACT_BF16, weights_f32=True)
    x = rand_bf16((2, 256), 1.0, 72).to(DEV)
    logits = torch.zeros((2, 64), device=DEV)
    ids = torch.zeros((2, 2), dtype=torch.int32, device=DEV)
    w = torch.zeros((2, 2), device=DEV)
    assert ops.contribute_from_logits(x, logits, None, ids, w) is None


@pytest.mark.parametrize("fmt,hidden,inter", [(capi.FMT_FP8_BLOCK128, 512, 256), (capi.FMT_FP8_BLOCK128, 1280, 2048), (capi.FMT_NVFP4, 512, 256),
                                              (capi.FMT_FP8_CHANNEL, 256, 512), (capi.FMT_BF16, 512, 256)])
@pytest.mark.parametrize("experts,n_group,topk_group,top_k", [(64, 1, 1, 3), (256, 8, 4, 8), (128, 4, 2, 5)])
def test_token_forward_two_launches_equal_the_separate_launches(fmt, hidden, inter, experts, n_group, topk_group, top_k):
    """ffmoe_decode_token_forward (selection behind the shared expert's rows in the gate/up launch, then down + weight +
    combine in one launch): ids, weights and y equal the separate launches bit for bit, for every combine mode, with and
    without a shared expert, over consecutive tokens on one arena."""
    table = make_table(fmt, 4 + 1, hidden, inter, 161)[0]
    # experts beyond the four materialised ones reuse their slots (only the arithmetic per slot matters here)
    slots = table.slots[:4].repeat((experts + 3) // 4, 1)[:experts].contiguous()
    big = ExpertTable(fmt, experts, hidden, inter, table.storage, slots,
                      table.global_scales[:4].repeat((experts + 3) // 4, 1)[:experts].contiguous() if table.global_scales is not None else None)
    sh = table.shared_struct(4)
    router = rand_bf16((experts, hidden), 0.05, 162).to(DEV)
    bias = (torch.randn(experts, generator=torch.Generator().manual_seed(163)) * 0.1).to(DEV)
    for mode, shared in ((capi.COMBINE_BF16, True), (capi.COMBINE_UNGATED, True), (capi.COMBINE_ACCUM_FP32, True), (capi.COMBINE_ROUTED, False)):
        got = {}
        for two in (False, True):
            layer = NativeMoe(big, sh if shared else None, router, bias, 1, top_k, routed_scaling=2.5, n_group=n_group, topk_group=topk_group,
                              combine_mode=mode)
            layer.two_launch = two
            layer.inline_select = False
            outs = []
            for step in range(3):
                x = rand_bf16((1, hidden), 1.0, 165 + step).to(DEV)
                print("token forward fmt=%d hidden=%d inter=%d experts=%d top_k=%d mode=%d two_launch=%d step=%d" % (fmt, hidden, inter, experts, top_k, mode, two, step), flush=True)
                y = bits(layer.run(x)).copy()
                outs.append((layer.ids.cpu().numpy().copy(), layer.weights.cpu().numpy().copy(), y))
                assert int(layer.status.item()) == 0
            assert layer.two_launch == two
            got[two] = outs
        for a, b in zip(got[False], got[True]):
            for name, u, v in zip(("ids", "weights", "y"), a, b):
                assert np.array_equal(u, v), "%s, combine mode %d" % (name, mode)


@pytest.mark.parametrize("fmt,shared_fmt,hidden,inter,shared_inter", [(capi.FMT_NVFP4, capi.FMT_BF16, 512, 256, 256), (capi.FMT_NVFP4, capi.FMT_BF16, 256, 512, 128),
                                                                     (capi.FMT_NVFP4, capi.FMT_BF16, 2048, 256, 384), (capi.FMT_NVFP4, capi.FMT_BF16, 4096, 128, 128),
                                                                     (capi.FMT_NVFP4, capi.FMT_BF16, 2048, 1024, 1024), (capi.FMT_NVFP4, capi.FMT_BF16, 4096, 2048, 2048),
                                                                     (capi.FMT_NVFP4, capi.FMT_BF16, 2048, 1536, 1536),
                                                                     (capi.FMT_FP8_BLOCK128, capi.FMT_BF16, 256, 256, 384), (capi.FMT_FP8_BLOCK128, capi.FMT_FP8_BLOCK128, 256, 256, 512)])
@pytest.mark.parametrize("experts,n_group,topk_group,top_k", [(64, 1, 1, 3), (256, 8, 4, 8)])
def test_token_forward_with_a_shared_expert_of_another_format_or_width(fmt, shared_fmt, hidden, inter, shared_inter, experts, n_group, topk_group, top_k):
    """ffmoe_decode_token_forward next to a shared expert that cannot share the routed launches (BF16 next to NVFP4 experts,
    or another width): the shared expert's own two launches leave its BF16 row in shared_out and the finish adds that row;
    at hidden 2048 and 4096 a BF16 shared expert's gate/up rows run inside the NVFP4 gate/up launch, in BF16, and where its
    width is the experts' (128, 1024 and 2048 columns here: one, two and four steps per BF16 row; 1536 is three, which keeps
    the down launch) its down rows run inside the finish launch.
    ids, weights and y equal the separate launches bit for bit, for every combine mode, over consecutive tokens."""
    table = make_table(fmt, 4, hidden, inter, 171)[0]
    slots = table.slots[:4].repeat((experts + 3) // 4, 1)[:experts].contiguous()
    big = ExpertTable(fmt, experts, hidden, inter, table.storage, slots,
                      table.global_scales[:4].repeat((experts + 3) // 4, 1)[:experts].contiguous() if table.global_scales is not None else None)
    sh_table = make_table(shared_fmt, 1, hidden, shared_inter, 172)[0]
    sh = sh_table.shared_struct(0)
    router = rand_bf16((experts, hidden), 0.05, 173).to(DEV)
    bias = (torch.randn(experts, generator=torch.Generator().manual_seed(174)) * 0.1).to(DEV)
    for mode in (capi.COMBINE_BF16, capi.COMBINE_UNGATED, capi.COMBINE_ACCUM_FP32, capi.COMBINE_ACCUM_BF16):
        got = {}
        for two in (False, True):
            layer = NativeMoe(big, sh, router, bias, 1, top_k, routed_scaling=2.5, n_group=n_group, topk_group=topk_group, combine_mode=mode)
            layer.two_launch = two
            layer.inline_select = False
            outs = []
            for step in range(3):
                x = rand_bf16((1, hidden), 1.0, 175 + step).to(DEV)
                print("token forward fmt=%d shared fmt=%d hidden=%d inter=%d shared inter=%d experts=%d top_k=%d mode=%d two_launch=%d step=%d"
                      % (fmt, shared_fmt, hidden, inter, shared_inter, experts, top_k, mode, two, step), flush=True)
                y = bits(layer.run(x)).copy()
                outs.append((layer.ids.cpu().numpy().copy(), layer.weights.cpu().numpy().copy(), y))
                assert int(layer.status.item()) == 0
            assert layer.two_launch == two, "the two-launch path refused the layer"
            got[two] = outs
        for a, b in zip(got[False], got[True]):
            for name, u, v in zip(("ids", "weights", "y"), a, b):
                assert np.array_equal(u, v), "%s, combine mode %d" % (name, mode)
        assert np.any(got[True][0][2] != 0)


@pytest.mark.parametrize("m", [1, 3, 4])
@pytest.mark.parametrize("k,n,count", [(7168, 200, 5), (2048, 384, 3), (640, 72, 9)])
def test_linear_fp8_block_batch_equals_single_calls(m, k, n, count):
    """ffmoe_linear_fp8_block_batch: several linears of one shape in one launch, every item bit-identical to its own
    ffmoe_linear_fp8_block call (whose parity with the oracle test_linear_fp8_block_w8a16 holds)."""
    weights, xs, ys, want = [], [], [], []
    for i in range(count):
        c, sc = synth.quant_fp8_block(synth.normal((n, k), 0.02, 700 + 10 * i + m))
        weights.append((c.to(DEV), sc.to(DEV)))
        xs.append(rand_bf16((m, k), 1.0, 800 + 10 * i + m).to(DEV))
        ys.append(torch.zeros((m, n), dtype=torch.bfloat16, device=DEV))
        want.append(bits(Fp8Ops.linear(weights[-1][0], weights[-1][1], xs[-1])).copy())
    items = Fp8Ops.linear_batch_items(weights, xs, ys)
    print("batched linear m=%d k=%d n=%d count=%d" % (m, k, n, count), flush=True)
    Fp8Ops.linear_batch(items, m, n, k)
    torch.cuda.synchronize()
    for i in range(count):
        assert np.array_equal(bits(ys[i]), want[i]), "item %d differs from its single call" % i
    with pytest.raises(capi.FfmoeError):
        Fp8Ops.linear_batch(items, 5, n, k)  # more than 4 rows per item: single calls (matrix-core path)
