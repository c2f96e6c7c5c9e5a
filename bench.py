#!/usr/bin/env python3
"""Benchmark of the quantized MoE expert-FFN hot path on one MI355X.

Workload (BASELINE config 3, the one the metric is quoted on): DeepSeek-V3-shape FP8 MoE decode layer,
hidden 7168, 256 routed experts + 1 shared, expert intermediate 2048, sigmoid grouped top-8 (8 groups, keep 4),
renormalised weights x 2.5, E4M3 weights with 128x128 f32 block scales, batch 1 by default.
A step = one layer call (router logits -> top-k -> expert contributions -> combine) on one token batch
already resident in HBM. Successive steps use different seeded tokens from a ring, so the selected experts
change every step and their weights come from HBM, not from the 256 MB Infinity Cache.

Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# HBM bytes per gate/up launch, not read in the run: FETCH_SIZE and WRITE_SIZE of rocprofv3 --pmc runs of this script, each
# scaled by what the same counter reads for a 256 MiB plain copy (--calibrate-copy); keyed by (batch, experts). Source of
# the figure, with the commands: profiles/decode_layer_fp8_c3_batch1.hbm_traffic.txt. Other workloads report null.
GATE_UP_TRAFFIC_BYTES = {(1, 256): 265451800}
TRAFFIC_SOURCE = "profiles/decode_layer_fp8_c3_batch1.hbm_traffic.txt"
# W8A8 gate/up launch of the default prefill cohort (4096 tokens, 256 experts, seed 20251): FETCH_SIZE x 1.99977 + WRITE_SIZE
PREFILL_GATE_UP_TRAFFIC_BYTES = 9190000000 + 135000000
PREFILL_TRAFFIC_SOURCE = "profiles/prefill_fp8_c5_4096tok.kernel_stats.txt"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", choices=["decode", "prefill", "widening", "linear", "c1"], default="decode",
                    help="decode = BASELINE config 3 (the headline line); prefill = config 5 (4096 tokens, Zipf s=1.1, FP8 matrix cores); "
                         "widening = the formats and fused steps next to the path (per-channel FP8 / BF16 experts, Lane16 / Lane8 orders, "
                         "combine + residual); linear = config 2 (standalone FP8 block skinny linear, M = 1, 4, 16, 64); "
                         "c1 = config 1 (hidden 2048, 64 experts, softmax top-4, intermediate 1408, one token)")
    ap.add_argument("--no-parity-gate", action="store_true", help="skip the oracle check of one ring slot that precedes the timing")
    ap.add_argument("--batch", type=int, default=None, help="tokens per step (decode: 1, 8, 64; prefill: 4096)")
    ap.add_argument("--format", choices=["fp8", "nvfp4", "e2m1"], default="fp8",
                    help="routed-expert format: fp8 = config 3 (shared expert FP8 too); nvfp4 = config 4 (NVFP4 routed experts, "
                         "BF16 shared expert, quoted at --batch 32)")
    ap.add_argument("--experts", type=int, default=256)
    ap.add_argument("--ring", type=int, default=64, help="distinct token batches cycled through")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--prefill-act", choices=["auto", "fp8", "bf16"], default="auto", help="prefill: fp8 = FP8 activations on the FP8 matrix "
                    "cores (W8A8 for block-FP8 experts; W4A8 for --format nvfp4, whose weights are rounded to E4M3 inside the kernel); "
                    "bf16 = the decode path's W*A16 arithmetic on the BF16 matrix cores (any --format); auto = fp8 for --format fp8, bf16 for nvfp4")
    ap.add_argument("--one-launch", action="store_true", help="one token: selection, gate/up, down and combine in the one resident "
                    "launch (ffmoe_decode_token_layer) instead of launches of their own")
    ap.add_argument("--separate-topk", action="store_true", help="one token: run the top-k selection as a launch of its own "
                    "instead of in the prologue of the gate/up launch")
    ap.add_argument("--graph", action="store_true", help="replay one HIP graph per ring slot instead of launching eagerly "
                    "(eager is faster here: launches run ahead of the GPU, a graph replay adds a few microseconds per step)")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="also run one plain device copy of this many MiB (a known-size kernel that scales the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    ap.add_argument("--no-secondary", action="store_true", help="headline run: skip the other configurations (config 3 at 8 and 64 tokens, "
                    "config 4, config 5) that the default line carries under `secondary`")
    ap.add_argument("--seed", type=int, default=20251)
    return ap.parse_args()


def build_layer(args, torch, capi, ops, synth, make_tokens=True, prebuilt=None):
    """The expert table of --format (seeded weights, quantized on the device) and, for decode, the layer and its token ring.
    prebuilt = (table, shared) of an earlier call with the same format, experts and seed: the weights are not drawn again."""
    H, I, E, K = 7168, 2048, args.experts, 8
    dev = "cuda"
    nvfp4 = args.format == "nvfp4"
    if prebuilt is not None:
        table, shared = prebuilt
        return (table, None, None, (H, I, E, K)) if not make_tokens else _layer_and_ring(args, torch, capi, ops, synth, table, shared, (H, I, E, K))
    if args.format == "e2m1":  # E2M1 codes with one E8M0 scale per 32 columns (the W4A8 contract); prefill cohorts only
        assert not make_tokens, "--format e2m1 is a prefill workload"
        table = ops.ExpertTable.allocate(capi.FMT_E2M1_E8M0, E, H, I, dev)
        for e in range(E):
            v = table.expert_views(e)
            for i, shape in enumerate([(I, H), (I, H), (H, I)]):
                codes, scales = synth.quant_e2m1_e8m0(synth.normal(shape, 0.02, args.seed * 100003 + e * 3 + i, device=dev))
                v[2 * i].copy_(codes)
                v[2 * i + 1].copy_(scales)
        return table, None, None, (H, I, E, K)
    if nvfp4:
        table = ops.ExpertTable.allocate(capi.FMT_NVFP4, E, H, I, dev)
        shared_table = ops.ExpertTable.allocate(capi.FMT_BF16, 1, H, I, dev)
    else:
        table = ops.ExpertTable.allocate(capi.FMT_FP8_BLOCK128, E + 1, H, I, dev)
        shared_table = None
    for e in range(E + 1):
        routed = e < E
        v = table.expert_views(e) if (routed or not nvfp4) else shared_table.expert_views(0)
        gl = []
        for i, shape in enumerate([(I, H), (I, H), (H, I)]):
            w = synth.normal(shape, 0.02, args.seed * 100003 + e * 3 + i, device=dev)
            if nvfp4 and routed:
                codes, scales, g = synth.quant_nvfp4(w)
                v[2 * i].copy_(codes)
                v[2 * i + 1].copy_(scales)
                gl.append(g)
            elif nvfp4:
                v[2 * i].copy_(w.to(torch.bfloat16))
            else:
                codes, scales = synth.quant_fp8_block(w)
                v[2 * i].copy_(codes)
                v[2 * i + 1].copy_(scales)
        if nvfp4 and routed:
            table.global_scales[e] = torch.tensor(gl, dtype=torch.float32)
    if nvfp4:
        shared = shared_table.shared_struct(0)
        table.shared_table = shared_table  # keep the storage alive
        table.shared_bytes = shared_table.weight_bytes_per_expert()
    else:
        shared = table.shared_struct(E)
        table.experts = E
        table.shared_bytes = table.weight_bytes_per_expert()
    table.shared_struct_kept = shared
    if not make_tokens:
        return table, None, None, (H, I, E, K)
    return _layer_and_ring(args, torch, capi, ops, synth, table, shared, (H, I, E, K))


def _layer_and_ring(args, torch, capi, ops, synth, table, shared, dims):
    H, I, E, K = dims
    dev = "cuda"
    router = synth.normal((E, H), 0.02, args.seed + 1, device=dev, dtype=torch.bfloat16)
    bias = torch.zeros(E, dtype=torch.float32, device=dev)
    layer = ops.NativeMoe(table, shared, router, bias, args.batch, K, routed_scaling=2.5, n_group=8, topk_group=4,
                          swiglu=capi.SWIGLU_TWICE, routed_weight=capi.WEIGHT_AFTER_DOWN_BF16, combine_mode=capi.COMBINE_UNGATED)
    layer.inline_select = not args.separate_topk
    layer.one_launch = args.one_launch
    xs = [synth.normal((args.batch, H), 1.0, args.seed + 1000 + i, device=dev, dtype=torch.bfloat16) for i in range(args.ring)]
    return table, layer, xs, dims


def layer_bytes(table, distinct, rows, dims):
    H, I, E, K = dims
    per = table.weight_bytes_per_expert()
    return distinct * per + table.shared_bytes + E * H * 2 + rows * H * 2 * (2 + K)


def gate_up_bytes(table, distinct, rows, dims):
    """Algorithmic bytes of one gate/up launch: gate+up codes and scales of every expert touched (routed distinct
    + shared), the token rows read and the activations written. Gate and up are two thirds of an expert's bytes in
    every format."""
    H, I, E, K = dims
    return (distinct * table.weight_bytes_per_expert() + table.shared_bytes) * 2 // 3 + rows * H * 2 + rows * (K + 1) * I * 2


def _checkers():
    """The oracle and the comparison helpers of the test-suite: the checker, never the thing measured."""
    tests = os.path.join(ROOT, "tests")
    if tests not in sys.path:
        sys.path.insert(0, tests)
    import numpy as np
    import oracle as orc
    import helpers
    return np, orc, helpers


def rewarm(torch, step, seconds=0.1):
    """Untimed: run `step` back to back for about `seconds`, so that what follows does not start on idle clocks."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            step()
        torch.cuda.synchronize()


def parity_gate_decode(args, torch, capi, ops, table, layer, x, dims):
    """Oracle check of one ring slot, outside the timed region; raises SystemExit when the layer the timing is about to
    measure does not match the CPU restatement: router ids and weights bit for bit, every contribution and the shared
    row end to end through both stages (relative L2 <= 1e-3 over the tensor; element-wise at most 5e-3 of the elements
    beyond 2 BF16 steps and none beyond 16, the bound the test-suite uses where a flipped BF16 step of an activation moves
    a cancelled down output: the per-stage bars of 2 steps are held by tests/test_gpu_fullsize.py on the same shapes), y of
    the timed launch sequence bit-identical to the separate launches and inside the layer bound of the oracle pipeline."""
    np, orc, hp = _checkers()
    H, I, E, K = dims
    rows = min(args.batch, 2)
    y_timed = hp.bits(layer.run(x)).copy()
    ids_t, w_t = layer.ids.cpu().numpy().copy(), layer.weights.cpu().numpy().copy()
    saved = (layer.two_launch, layer.one_launch)
    layer.two_launch = layer.one_launch = False   # the separate launches write contributions and shared_out
    y_sep = hp.bits(layer.run(x)).copy()
    layer.two_launch, layer.one_launch = saved
    torch.cuda.synchronize()
    fail = []
    if not (np.array_equal(y_timed, y_sep) and np.array_equal(ids_t, layer.ids.cpu().numpy())):
        fail.append("the timed launch sequence and the separate launches disagree")
    xb = hp.bits(x)
    lg = orc.route_logits_f32(xb, hp.bits(layer.router))
    bias = layer.bias.cpu().numpy()
    oi, ow = orc.route_topk_noaux(lg, bias[None, :] if bias.ndim == 1 else bias, K, 0, 2.5, 8, 4)
    if not np.array_equal(ids_t, oi):
        fail.append("router ids differ from the oracle")
    if not np.array_equal(w_t.view(np.uint32), ow.view(np.uint32)):
        fail.append("router weights differ from the oracle")
    got_c, got_s = hp.bits(layer.decode.contributions), hp.bits(layer.decode.shared_out)
    shared_table = getattr(table, "shared_table", None)
    eff = {}

    def weights_of(e):
        if e not in eff:
            eff[e] = hp.effective_weights(shared_table, 0) if (e == E and shared_table is not None) else hp.effective_weights(table, e)
        return eff[e]
    jobs = [(r, c) for r in range(rows) for c in range(K)] + [(r, -1) for r in range(rows)]
    for e in sorted({int(oi[r, c]) for r in range(rows) for c in range(K)} | {E}):
        weights_of(e)

    def one(lo, hi):
        out = []
        for r, c in jobs[lo:hi]:
            g, u, d = weights_of(int(oi[r, c]) if c >= 0 else E)
            out.append(orc.expert_ffn(xb[r], g, u, d, float(ow[r, c]) if c >= 0 else 1.0, orc.TWICE, 0.0, orc.AFTER_DOWN_BF16, orc.LANE8, orc.SILU_DIV,
                                      apply_weight=c >= 0))
        return out
    res = [t for chunk in hp.run_parallel(one, len(jobs), min(16, len(os.sched_getaffinity(0)))) for t in chunk]
    want_c = np.stack(res[:rows * K]).reshape(rows, K, H)
    want_s = np.stack(res[rows * K:])
    stats = {}
    try:
        stats["contributions"] = hp.assert_close_with_rare_outliers(got_c[:rows], want_c, "contributions", loose=16, rare=5e-3)
        stats["shared_out"] = hp.assert_close_with_rare_outliers(got_s[:rows], want_s, "shared expert", loose=16, rare=5e-3)
    except AssertionError as exc:
        fail.append(str(exc))
    want_y = orc.combine(want_c, want_s, None, oi[:rows], None, orc.COMBINE_UNGATED)
    terms = np.concatenate([orc.bf16_to_f32(want_c), orc.bf16_to_f32(want_s)[:, None, :], orc.bf16_to_f32(want_y)[:, None, :]], axis=1)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.max(np.abs(terms), axis=1).astype(np.float64), 1e-30))) - 7)
    err = np.abs(orc.bf16_to_f32(y_timed[:rows]).astype(np.float64) - orc.bf16_to_f32(want_y).astype(np.float64))
    y_rel = orc.rel_l2(y_timed[:rows], want_y)
    if not (np.all(err <= 3 * (K + 1) * ulp) and y_rel <= 4e-3):
        fail.append("y: %.1f steps of the largest term, relative L2 %.2e" % (float(np.max(err / ulp)), y_rel))
    if fail:
        print("bench.py parity gate FAILED: " + "; ".join(fail), file=sys.stderr)
        sys.exit(3)
    return {"checked": "ring slot 0, %d token row(s): ids and weights bit-exact, %d contributions + shared rows, y" % (rows, rows * K),
            "contributions_rel_l2": stats["contributions"][0], "contributions_worst_bf16_steps": stats["contributions"][1],
            "contributions_share_beyond_2_steps": stats["contributions"][2],
            "y_rel_l2": y_rel, "oracle": "oracle/ffmoe_oracle.cpp (scalar, Lane8 form)"}


def parity_gate_prefill(args, torch, capi, ops, table, pre, x, ids, wts, dims, a16):
    """Oracle check of a sample of the cohort, outside the timed region: the assignments at the start, the middle and the
    end of the segments of the most popular expert, a mid-popular and the least popular one, each stage on the inputs it
    saw (activations against the oracle's, the down stage against the oracle's down stage on the device's activations)."""
    np, orc, hp = _checkers()
    H, I, E, K = dims
    pre.done.zero_()
    got = pre.contribute(x, ids, wts)
    torch.cuda.synchronize()
    v = pre.scratch_views()
    n_live = int(v["totals"][3].item())
    perm = v["perm"].cpu().numpy()[:n_live]
    offsets = v["offsets"].cpu().numpy()
    counts = np.diff(offsets)
    order = np.argsort(-counts, kind="stable")
    live = [int(e) for e in order if counts[e] > 0]
    picks = []
    for e in (live[0], live[len(live) // 2], live[-1]):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        picks += sorted({lo, (lo + hi) // 2, hi - 1})
    xb = hp.bits(x)
    xq, sx = (None, None) if a16 else orc.quant_act_fp8_128(xb)
    flat_ids, flat_w = ids.cpu().numpy().reshape(-1), wts.cpu().numpy().reshape(-1)
    act = hp.bits(v["act"][torch.tensor(picks, device="cuda")])
    g2 = hp.bits(got.reshape(pre.rows * K, H)[torch.from_numpy(perm[picks]).cuda().long()])
    host = {}
    for e in sorted({int(flat_ids[perm[p]]) for p in picks}):
        host[e] = hp.effective_weights(table, e) if a16 else hp.host_expert(table, e)
        if not a16 and table.format == capi.FMT_NVFP4:  # W4A8: the oracle's E4M3 derivation of the NVFP4 weights, then W8A8
            m, d8 = host[e], []
            for i in range(3):
                d8 += list(orc.nvfp4_to_fp8_block(m[2 * i], m[2 * i + 1], float(table.global_scales[e, i].item())))
            host[e] = d8

    def one(lo, hi):
        out = []
        for i in range(lo, hi):
            a = int(perm[picks[i]])
            m, wa = host[int(flat_ids[a])], float(flat_w[a])
            t = a // K
            if a16:
                g_ref, u_ref = orc.linear_skinny(m[0], xb[t:t + 1], 2)[0], orc.linear_skinny(m[1], xb[t:t + 1], 2)[0]
                d_ref = orc.expert_down(act[i], m[2], 1.0, 0, orc.LANE8, False)
            else:
                g_ref = orc.linear_fp8_block_w8a8(m[0], m[1], xq[t:t + 1], sx[t:t + 1])[0]
                u_ref = orc.linear_fp8_block_w8a8(m[2], m[3], xq[t:t + 1], sx[t:t + 1])[0]
                d_ref = orc.expert_down_w8a8(act[i], m[4], m[5], apply_weight=False)
            out.append((g_ref, u_ref, d_ref, wa))
        return out
    res = [t for chunk in hp.run_parallel(one, len(picks), min(16, len(os.sched_getaffinity(0)))) for t in chunk]
    try:
        # activations: within 2 steps of SwiGLU(gate, up) of the oracle, further only where a gate / up one step off explains it
        a_stats = hp.assert_swiglu_close(act, np.stack([t[0] for t in res]), np.stack([t[1] for t in res]), orc.TWICE, 0.0,
                                         orc.SILU_DIV if a16 else orc.SILU_SIGMOID2, "activations")
        d_stats = hp.assert_weighted_down_close(g2, np.stack([t[2] for t in res]), [t[3] for t in res], "down stage on the device activations")
    except AssertionError as exc:
        print("bench.py parity gate FAILED: " + str(exc), file=sys.stderr)
        sys.exit(3)
    return {"checked": "%d assignments (first, middle, last of the segments of the most, a mid and the least popular expert), per stage" % len(picks),
            "activations_rel_l2": a_stats[0], "activations_worst_bf16_steps": a_stats[1], "down_rel_l2": d_stats[0], "down_worst_bf16_steps": d_stats[1],
            "oracle": "oracle/ffmoe_oracle.cpp (%s)" % ("W*A16, Lane8 form" if a16 else "W8A8 block-128, 32-lane order")}


def cpu_baseline(args, torch, table, layer, xs, dims):
    """The reference's CPU expert path (multithreaded port in oracle/cpu_baseline.cpp) on a bounded sample of the
    same workload: the routed + shared experts of a few ring slots, weights copied to host, cold between trials."""
    import numpy as np
    import oracle as orc
    H, I, E, K = dims
    threads = min(orc.cpubase().cpubase_max_threads(), len(os.sched_getaffinity(0)))
    slots = list(range(min(6, len(xs))))  # 1 warm-up + 5 timed trials (src/cpu/expert_ffn.rs:3000-3034)
    jobs = []
    for s in slots:
        layer.run(xs[s])
        torch.cuda.synchronize()
        ids = layer.ids.cpu().numpy()
        wts = layer.weights.cpu().numpy()
        rows = min(args.batch, 4)  # bounded sample: at most 4 token rows of the batch
        experts, rws, w, ap = [], [], [], []
        cache = {}

        def host(e):
            if e not in cache:
                cache[e] = tuple(v.cpu().numpy() for v in table.expert_views(e))
            return cache[e]
        for r in range(rows):
            for c in range(K):
                experts.append(host(int(ids[r, c]))); rws.append(r); w.append(float(wts[r, c])); ap.append(1)
            experts.append(host(E)); rws.append(r); w.append(1.0); ap.append(0)
        x_bits = xs[s].view(torch.int16).cpu().numpy().view(np.uint16)
        jobs.append((orc.CpuDecodeJob(x_bits, rws, experts, w, ap), rows))
    times = []
    for i, (job, rows) in enumerate(jobs):
        t0 = time.perf_counter()
        job.run(threads)
        dt = time.perf_counter() - t0
        if i > 0:
            times.append(dt / rows)
    times.sort()
    med = times[len(times) // 2]
    rows = jobs[0][1]
    return {"value": med * 1e6, "unit": "us/layer per token row", "cores": threads, "kind": "port",
            "isa": orc.cpubase().cpubase_isa().decode(),
            "sample": "%d ring slots x %d token row(s), %d expert FFNs per row (top-%d + shared), weights cold per trial, "
                      "1 warm-up + %d timed, median" % (len(jobs), rows, K + 1, K, len(times)),
            "tokens_per_s": 1.0 / med}


MFMA_FP8_PEAK_TFLOPS = 5000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0


def prefill_main(args, torch, capi, ops, synth, prebuilt=None):
    """BASELINE config 5: R tokens routed top-8 over 256 experts with Zipf(s=1.1) popularity (seeded router logits =
    log popularity under a seeded expert permutation + Gumbel noise, so the top-8 is a draw without replacement),
    grouped W8A8 GEMMs on the FP8 matrix cores, routed-only ordered combine. A step = top-k selection from the logits
    + prefill contribute + combine on inputs resident in HBM."""
    import math
    R = args.batch
    table, layer, _, dims = build_layer(args, torch, capi, ops, synth, make_tokens=False, prebuilt=prebuilt)
    H, I, E, K = dims
    dev = "cuda"
    g = torch.Generator(device="cpu").manual_seed(args.seed + 77)
    order = torch.randperm(E, generator=g)
    pop = torch.empty(E, dtype=torch.float64)
    pop[order] = torch.arange(1, E + 1, dtype=torch.float64) ** -1.1
    u = torch.rand((R, E), generator=g, dtype=torch.float64).clamp_(1e-12, 1.0 - 1e-12)
    logits = (pop.log()[None, :] - (-u.log()).log()).to(torch.float32).to(dev)
    x = synth.normal((R, H), 1.0, args.seed + 5000, device=dev, dtype=torch.bfloat16)
    bias = torch.zeros(E, dtype=torch.float32, device=dev)
    mx = args.format == "e2m1"
    a16 = not mx and (args.prefill_act == "bf16" or (args.format == "nvfp4" and args.prefill_act != "fp8"))
    w4a8 = not mx and not a16 and args.format == "nvfp4"
    default_cohort = not mx and not a16 and args.format == "fp8" and R == 4096 and E == 256 and args.seed == 20251  # the cohort the committed profile measured
    if mx:
        pre = ops.PrefillOps(table, R, K, swiglu=capi.SWIGLU_CLAMPED_ONCE, swiglu_limit=7.0, routed_weight=capi.WEIGHT_BEFORE_DOWN_F32,
                             weights_f32=True, act_mode=capi.ACT_E4M3_E8M0_32)
    else:
        pre = ops.PrefillOps(table, R, K, swiglu=capi.SWIGLU_TWICE, weights_f32=True, act_mode=capi.ACT_BF16 if a16 else capi.ACT_FP8_BLOCK128)
    peak = MFMA_BF16_PEAK_TFLOPS if a16 else MFMA_FP8_PEAK_TFLOPS  # an E2M1 x E4M3 instruction runs at the 8-bit rate
    ids = torch.empty((R, K), dtype=torch.int32, device=dev)
    wts = torch.empty((R, K), dtype=torch.float32, device=dev)
    y = torch.empty((R, H), dtype=torch.bfloat16, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)

    def step():
        ops.RouteOps.topk_noaux(logits, bias, K, score_mode=capi.NOAUX_SIGMOID, routed_scaling=2.5, weights_f32=True, out=(ids, wts))
        pre.done.zero_()
        c = pre.contribute(x, ids, wts)
        ops.CombineOps.combine(c, None, ids, capi.COMBINE_ROUTED, done=pre.done, status=status, out=y)

    step()
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    parity = None
    if not args.no_parity_gate and not mx:
        parity = parity_gate_prefill(args, torch, capi, ops, table, pre, x, ids, wts, dims, a16)
    # the gate keeps the host busy for seconds while the GPU idles: bring it back to its working clocks (untimed), then the
    # W warm-up steps, then exactly K timed steps
    rewarm(torch, step)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    counts = torch.bincount(ids.reshape(-1).long(), minlength=E).cpu()
    touched = int((counts > 0).sum())
    A = R * K
    flop_total = A * 6.0 * H * I
    # dominant kernel: the gate/up grouped GEMM, timed alone with events on the launch stream
    nb = max(3, min(args.steps, 20))
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(nb)]
    ev2 = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(nb)]
    for a, b in ev:
        a.record(); pre.contribute(x, ids, wts, stage=1); b.record()
    for a, b in ev2:
        a.record(); pre.contribute(x, ids, wts, stage=3); b.record()
    torch.cuda.synchronize()
    k0 = sorted(a.elapsed_time(b) for a, b in ev)
    k1 = sorted(a.elapsed_time(b) for a, b in ev2)
    k0_avg, k1_avg = sum(k0) / len(k0), sum(k1) / len(k1)
    flop0 = A * 4.0 * H * I
    per = table.weight_bytes_per_expert()
    # side pass in front of the cohort, reported apart from it: the FP32 router logits of all R rows (the cohort itself
    # starts from seeded logits), R x E x H multiply-adds on the vector ALUs in the oracle's summation order
    router = synth.normal((E, H), 0.02, args.seed + 1, device=dev, dtype=torch.bfloat16)
    lg_out = torch.empty((R, E), dtype=torch.float32, device=dev)
    for _ in range(2):
        ops.RouteOps.logits_f32(x, router, out=lg_out)
    evl = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(5)]
    for a, b in evl:
        a.record(); ops.RouteOps.logits_f32(x, router, out=lg_out); b.record()
    torch.cuda.synchronize()
    lg_ms = sorted(a.elapsed_time(b) for a, b in evl)[len(evl) // 2]
    lg_parity = None
    if not args.no_parity_gate:
        _, orc_, hp_ = _checkers()
        sample = [0, R // 2, R - 1]
        want_lg = orc_.route_logits_f32(hp_.bits(x[sample]), hp_.bits(router))
        if not (lg_out[sample].cpu().numpy().view("uint32") == want_lg.view("uint32")).all():
            print("bench.py parity gate FAILED: router logits differ from the oracle", file=sys.stderr)
            sys.exit(3)
        lg_parity = "rows %s bit-exact against the oracle" % sample
    out = {
        "metric": "moe_prefill_ms", "value": ms, "unit": "ms/cohort", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": ("%s weights dequantized to bf16 x bf16 activations, f32 accumulate" % args.format) if a16 else
                 "nvfp4 weights rounded to fp8_e4m3 in the kernel x fp8_e4m3 activations (per-128 f32 scales), f32 accumulate" if w4a8 else
                 "fp4_e2m1 weights x fp8_e4m3 activations, e8m0 scales per 32 applied by the matrix core, f32 accumulate" if mx else
                 "fp8_e4m3 weights x fp8_e4m3 activations (per-128 f32 scales), f32 accumulate", "data": "synthetic",
        "config": {"workload": ("DeepSeek-V3-shape %s MoE prefill, %d tokens, Zipf s=1.1" % (args.format.upper(), R)) if (a16 or mx or w4a8) else
                               "DeepSeek-V3-shape FP8 MoE prefill (BASELINE config 5), %d tokens, Zipf s=1.1" % R,
                   "hidden": H, "intermediate": I, "experts": E, "top_k": K,
                   "act_mode": "FFMOE_ACT_BF16 (W*A16 on the BF16 matrix cores)" if a16 else
                               "FFMOE_ACT_E4M3_E8M0_32 (W4A8 on the MX matrix cores)" if mx else
                               "FFMOE_ACT_FP8_BLOCK128 on NVFP4 experts (W4A8 on the FP8 matrix cores)" if w4a8 else "FFMOE_ACT_FP8_BLOCK128 (W8A8)",
                   "tokens": R, "experts_touched": touched, "max_rows_per_expert": int(counts.max()), "min_rows_per_expert": int(counts.min())},
        "tokens_per_s": R / (ms * 1e-3),
        "routed_tflop": flop_total / 1e12,
        "cohort_tflops": flop_total / (ms * 1e-3) / 1e12,
        "cohort_mfma_frac": flop_total / (ms * 1e-3) / 1e12 / peak,
        "weight_bytes_once": touched * per,
        "cohort_weight_gbps": touched * per / (ms * 1e-3) / 1e9,
        "roofline": {"kernel": ("ffmoe::k_w16_grouped<F, MF, 0, P>" if a16 else "ffmoe::k_mx_grouped<MF, 0, 1, P>" if mx else "ffmoe::k_w8a8_grouped<MF, 0, P>") + " (gate/up grouped GEMM + SwiGLU)", "bound": "mfma",
                     "achieved": flop0 / (k0_avg * 1e-3) / 1e12, "peak": peak, "unit": "TFLOP/s",
                     "frac": flop0 / (k0_avg * 1e-3) / 1e12 / peak,
                     "traffic": PREFILL_GATE_UP_TRAFFIC_BYTES if default_cohort else None,
                     "traffic_source": PREFILL_TRAFFIC_SOURCE if default_cohort else None,
                     "flop_per_launch": flop0, "avg_ms": k0_avg, "min_ms": k0[0],
                     "weight_bytes_once": touched * per * 2 // 3, "weight_gbps": touched * per * 2 / 3 / (k0_avg * 1e-3) / 1e9},
        "down_kernel": {"kernel": "ffmoe::k_w16_grouped<F, MF, 1, P>" if a16 else "ffmoe::k_mx_grouped<MF, 1, 1, P>" if mx else "ffmoe::k_w8a8_grouped<MF, 1, P>", "avg_ms": k1_avg, "min_ms": k1[0],
                        "tflops": A * 2.0 * H * I / (k1_avg * 1e-3) / 1e12},
    }
    out["router_logits"] = {"kernel": "ffmoe::k_route_logits_f32_rows (FP32 logits of all token rows, vector ALUs, the oracle's summation order)",
                            "ms": lg_ms, "flop": 2.0 * R * E * H, "tflops": 2.0 * R * E * H / (lg_ms * 1e-3) / 1e12,
                            "frac_of_fp32_vector_peak": 2.0 * R * E * H / (lg_ms * 1e-3) / 1e12 / 157.3,
                            "frac_of_unpacked_fp32_rate": 2.0 * R * E * H / (lg_ms * 1e-3) / 1e12 / 78.65, "parity": lg_parity,
                            "note": "side pass, not part of `value`: the cohort starts from seeded logits (BASELINE config 5). The published 157.3 "
                                    "TFLOP/s counts two fmas per lane and instruction (packed FP32), which this build is compiled without; one "
                                    "v_fma_f32 per lane and instruction is half of it"}
    out["parity"] = parity if parity is not None else ("not gated in bench.py for this format (tests/test_gpu_e8m0.py, tests/test_gpu_fullsize.py)" if mx else None)
    if not args.no_cpu_baseline and args.format == "fp8":
        out["cpu_baseline"] = cpu_baseline_prefill(args, torch, table, x, ids, wts, dims)
    return out


def cpu_baseline_prefill(args, torch, table, x, ids, wts, dims):
    """The reference's CPU expert path (W8A16 contract, multithreaded port in oracle/cpu_baseline.cpp) on a bounded
    sample of the cohort: the assignments of the first 24 token rows (192 expert FFNs), 1 warm-up + 3 timed, median,
    scaled to the whole cohort by the assignment count."""
    import numpy as np
    import oracle as orc
    H, I, E, K = dims
    threads = min(orc.cpubase().cpubase_max_threads(), len(os.sched_getaffinity(0)))
    rows = min(24, x.shape[0])
    ids_h, w_h = ids[:rows].cpu().numpy(), wts[:rows].cpu().numpy()
    cache = {}

    def host(e):
        if e not in cache:
            cache[e] = tuple(v.cpu().numpy() for v in table.expert_views(e))
        return cache[e]
    experts, rws, w, ap = [], [], [], []
    for r in range(rows):
        for c in range(K):
            experts.append(host(int(ids_h[r, c]))); rws.append(r); w.append(float(w_h[r, c])); ap.append(1)
    x_bits = x[:rows].view(torch.int16).cpu().numpy().view(np.uint16)
    job = orc.CpuDecodeJob(x_bits, rws, experts, w, ap)
    times = []
    for i in range(4):
        t0 = time.perf_counter()
        job.run(threads)
        if i > 0:
            times.append(time.perf_counter() - t0)
    times.sort()
    per = times[len(times) // 2] / (rows * K)
    total = x.shape[0] * K
    return {"value": per * total * 1e3, "unit": "ms/cohort", "cores": threads, "kind": "port", "isa": orc.cpubase().cpubase_isa().decode(),
            "sample": "%d expert FFNs (all %d choices of the first %d token rows), 1 warm-up + %d timed, median, scaled by %d / %d assignments; "
                      "W8A16 arithmetic of the CPU expert path" % (rows * K, K, rows, len(times), total, rows * K),
            "tokens_per_s": x.shape[0] / (per * total)}


def c1_main(args, torch, capi, ops, synth):
    """BASELINE config 1: one MoE decode step at the shape of the reference's own CPU-runnable case: 1 token, hidden 2048,
    64 routed experts (no shared expert), softmax top-4 over BF16 logits, intermediate 1408, FP8 E4M3 experts with
    128 x 128 f32 block scales. A step = fused BF16-logit route + gate/up + down + routed-only combine on a token from a
    ring, inputs resident in HBM."""
    import numpy as np
    H, I, E, K = 2048, 1408, 64, 4
    dev = "cuda"
    table = ops.ExpertTable.allocate(capi.FMT_FP8_BLOCK128, E, H, I, dev)
    for e in range(E):
        v = table.expert_views(e)
        for i, shape in enumerate([(I, H), (I, H), (H, I)]):
            c, sc = synth.quant_fp8_block(synth.normal(shape, 0.02, args.seed * 100003 + e * 3 + i, device=dev))
            v[2 * i].copy_(c); v[2 * i + 1].copy_(sc)
    router = synth.normal((E, H), 0.02, args.seed + 1, device=dev, dtype=torch.bfloat16)
    xs = [synth.normal((1, H), 1.0, args.seed + 1000 + i, device=dev, dtype=torch.bfloat16) for i in range(args.ring)]
    dec = ops.DecodeOps(table, None, 1, K, capi.ACT_BF16, capi.SWIGLU_TWICE, 0.0, capi.WEIGHT_AFTER_DOWN_BF16, False)
    y = torch.empty((1, H), dtype=torch.bfloat16, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    logits = torch.empty((1, E), dtype=torch.bfloat16, device=dev)
    ids = torch.empty((1, K), dtype=torch.int32, device=dev)
    wts = torch.empty((1, K), dtype=torch.bfloat16, device=dev)

    def step_separate(i):
        x = xs[i % len(xs)]
        ops.RouteOps.route(x, router, K, capi.SCORE_SOFTMAX, logits=logits, ids=ids, weights=wts)
        dec.done.zero_()
        c, _ = dec.contribute(x, ids, wts)
        return ops.CombineOps.combine(c, None, ids, capi.COMBINE_ROUTED, done=dec.done, status=status, out=y)

    fused = [True]  # down + routing weight + ordered combine in one launch (ffmoe_decode_finish) where the shape allows it

    def step(i):
        if not fused[0]:
            return step_separate(i)
        x = xs[i % len(xs)]
        ops.RouteOps.route(x, router, K, capi.SCORE_SOFTMAX, logits=logits, ids=ids, weights=wts)
        dec.contribute(x, ids, wts, stage=0)
        if dec.finish(x, ids, wts, capi.COMBINE_ROUTED, y, status=status):
            return y
        fused[0] = False
        return step_separate(i)

    step(0)
    torch.cuda.synchronize()
    parity = None
    if not args.no_parity_gate:
        np_, orc, hp = _checkers()
        y_fused = hp.bits(step(0)).copy()
        torch.cuda.synchronize()
        got_y = hp.bits(step_separate(0)).copy()
        torch.cuda.synchronize()
        if not np.array_equal(y_fused, got_y):
            print("bench.py parity gate FAILED: the fused down + combine launch differs from the separate launches", file=sys.stderr)
            sys.exit(3)
        xb = hp.bits(xs[0])
        ol = orc.route_logits_bf16(xb, hp.bits(router))
        oi, ow = orc.route_topk_softmax(ol, K)
        ok = np.array_equal(hp.bits(logits), ol) and np.array_equal(ids.cpu().numpy(), oi) and np.array_equal(hp.bits(wts), ow)
        want_c = np.stack([orc.expert_ffn(xb[0], *hp.effective_weights(table, int(oi[0, c])), float(orc.bf16_to_f32(ow)[0, c]), orc.TWICE, 0.0,
                                          orc.AFTER_DOWN_BF16, orc.LANE8, orc.SILU_DIV) for c in range(K)])[None]
        try:
            st = hp.assert_close_bf16(hp.bits(dec.contributions), want_c, "contributions", max_ulp=4)
            assert ok, "router logits, ids or weights differ from the oracle"
            assert np.array_equal(got_y, orc.combine(hp.bits(dec.contributions), None, None, oi, None, orc.COMBINE_ROUTED)), "combine"
        except AssertionError as exc:
            print("bench.py parity gate FAILED: " + str(exc), file=sys.stderr)
            sys.exit(3)
        parity = {"checked": "ring slot 0: BF16 logits, ids and weights bit-exact, 4 contributions, combine bit-exact on the device contributions",
                  "contributions_rel_l2": st[0], "contributions_worst_bf16_steps": st[1]}
        rewarm(torch, lambda: step(0))
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(args.warmup + i)
    torch.cuda.synchronize()
    us = (time.perf_counter() - t0) / args.steps * 1e6
    per = table.weight_bytes_per_expert()
    nbytes = K * per + E * H * 2 + H * 2 * (2 + K)
    # the streaming launches alone (gate/up, then down) with events on the launch stream
    def timed(stage):
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(8)]
        for a, b in ev:
            a.record()
            for i in range(16):
                dec.contribute(xs[i % len(xs)], ids, wts, stage=stage)
            b.record()
        torch.cuda.synchronize()
        return sum(a.elapsed_time(b) for a, b in ev) * 1e3 / (8 * 16)
    k0, k1 = timed(0), timed(1)
    b0 = K * per * 2 // 3 + H * 2 + K * I * 2
    out = {"metric": "moe_layer_decode_us", "value": us, "unit": "us/layer", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": us / 1e3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
           "dtype": "fp8_e4m3 weights, bf16 activations, f32 accumulate", "data": "synthetic",
           "config": {"workload": "MoE decode step at the reference's CPU-runnable shape (BASELINE config 1), batch 1", "hidden": H, "intermediate": I,
                      "experts": E, "shared_experts": 0, "top_k": K, "routing": "softmax top-4 over BF16 logits", "ring": len(xs),
                      "launches_per_layer": "fused BF16-logit route; gate/up; down + combine" if fused[0] else
                                            "fused BF16-logit route; gate/up; down; combine (+ a done-flag fill)"},
           "tokens_per_s": 1e6 / us, "layer_bytes": nbytes, "layer_hbm_gbps": nbytes / us / 1e3, "layer_hbm_frac": nbytes / us / 1e3 / HBM_PEAK_GBPS,
           "roofline": {"kernel": "ffmoe::k_decode_stage<FmtFp8, S, 0, 1, NR> (gate/up + SwiGLU)", "bound": "hbm", "achieved": b0 / k0 / 1e3,
                        "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": b0 / k0 / 1e3 / HBM_PEAK_GBPS, "traffic": None, "bytes_per_launch": b0,
                        "avg_us": k0, "launches_timed": 128, "note": "the same 4 experts every launch (34 MB: cache-resident), latency-bound"},
           "down_kernel": {"avg_us": k1}, "parity": parity}
    return out


def linear_main(args, torch, capi, ops, synth):
    """BASELINE config 2: the standalone FP8 128x128-block skinny linear, bf16 in and out, M in {1, 4, 16} (and 64) at
    (K, N) = (7168, 2048) and (2048, 7168), over a ring of 24 weight sets (353 MB, beyond the caches). One JSON line;
    value = M = 16 at K 7168, the case the matrix-core path was built for."""
    dev = "cuda"
    rows = {}
    for k, n in ((7168, 2048), (2048, 7168)):
        ring = 24
        ws = []
        for i in range(ring):
            w = synth.normal((n, k), 0.02, args.seed + 31 * i + k, device=dev)
            ws.append(synth.quant_fp8_block(w))
        for m in (1, 4, 16, 64):
            x = synth.normal((m, k), 1.0, args.seed + m, device=dev, dtype=torch.bfloat16)
            y = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
            for c, sc in ws:
                ops.Fp8Ops.linear(c, sc, x, out=y)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            reps = max(1, args.steps // ring)
            e0.record()
            for _ in range(reps):
                for c, sc in ws:
                    ops.Fp8Ops.linear(c, sc, x, out=y)
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / (reps * ring)
            nbytes = n * k + 4 * ((n + 127) // 128) * ((k + 127) // 128) + 2 * m * (k + n)
            rows["k%d_n%d_m%d" % (k, n, m)] = {"us": us, "gbps": nbytes / us / 1e3, "hbm_frac": nbytes / us / 1e3 / HBM_PEAK_GBPS}
        # steady state of M = 1: eight linears of the ring per launch (ffmoe_linear_fp8_block_batch), the start-up of a
        # launch paid once per batch; the ring is walked in three batches per repetition
        for m in (1, 4):
            x = synth.normal((m, k), 1.0, args.seed + m, device=dev, dtype=torch.bfloat16)
            ys = [torch.empty((m, n), dtype=torch.bfloat16, device=dev) for _ in range(ring)]
            batches = [ops.Fp8Ops.linear_batch_items(ws[b:b + 8], [x] * 8, ys[b:b + 8]) for b in range(0, ring, 8)]
            for it in batches:
                ops.Fp8Ops.linear_batch(it, m, n, k)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            reps = max(1, args.steps // ring)
            e0.record()
            for _ in range(reps):
                for it in batches:
                    ops.Fp8Ops.linear_batch(it, m, n, k)
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / (reps * ring)
            nbytes = n * k + 4 * ((n + 127) // 128) * ((k + 127) // 128) + 2 * m * (k + n)
            rows["k%d_n%d_m%d_batch8" % (k, n, m)] = {"us_per_linear": us, "gbps": nbytes / us / 1e3, "hbm_frac": nbytes / us / 1e3 / HBM_PEAK_GBPS}
    head = rows["k7168_n2048_m16"]
    out = {"metric": "fp8_block_linear_us", "value": head["us"], "unit": "us/call", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": head["us"] * 1e-3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
           "dtype": "fp8_e4m3 weights (f32 128x128 block scales), bf16 activations, f32 accumulate", "data": "synthetic",
           "config": {"workload": "standalone FP8 block-scaled skinny linear (BASELINE config 2), M = 16, K = 7168, N = 2048"},
           "roofline": {"kernel": "ffmoe::k_linear_mfma<FmtFp8, TR> (more than 4 rows) / ffmoe::k_linear<FmtFp8, S, RG>", "bound": "hbm",
                        "achieved": head["gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": head["hbm_frac"], "traffic": None},
           "cases": rows}
    return out


def widening_main(args, torch, capi, ops, synth):
    """The rows next to the headline path, timed at the DeepSeek-V3 layer shape with one token (8 of 16 experts +
    shared expert, weights = random codes, resident): per-channel FP8 and BF16 experts on the streaming decode path,
    the same experts in the reference's Lane16 / Lane8 summation orders (ffmoe_decode_contribute_form), and the fused
    combine + shared gate + residual add. One JSON line; value = the per-channel FP8 streaming contribution."""
    H, I, E, K = 7168, 2048, 16, 8
    dev = "cuda"
    g = torch.Generator(device="cpu").manual_seed(args.seed)
    xs = [synth.normal((1, H), 1.0, args.seed + 1000 + i, device=dev, dtype=torch.bfloat16) for i in range(8)]
    idl = [torch.randperm(E, generator=g)[:K].reshape(1, K).to(torch.int32).to(dev) for _ in range(8)]
    w = (torch.rand((1, K), generator=g) * 0.5 + 0.05).to(dev)

    def timed(fn, n):
        for i in range(5):
            fn(i)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(n):
            fn(i)
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / n

    rows = {}
    for name, fmt in (("fp8_per_channel", capi.FMT_FP8_CHANNEL), ("bf16", capi.FMT_BF16)):
        table = ops.ExpertTable.allocate(fmt, E + 1, H, I, dev)
        for e in range(E + 1):
            v = table.expert_views(e)
            for i in range(3):
                if fmt == capi.FMT_FP8_CHANNEL:
                    v[2 * i].random_(0, 120)
                    v[2 * i + 1].fill_(0.001)
                else:
                    v[2 * i].normal_(0.0, 0.02)
        shared = table.shared_struct(E)
        table.experts = E
        dec = ops.DecodeOps(table, shared, 1, K, weights_f32=True)
        nbytes = (K + 1) * table.weight_bytes_per_expert()
        us = timed(lambda i: dec.contribute(xs[i % 8], idl[i % 8], w), args.steps)
        rows[name] = {"streaming_us": us, "weight_bytes": nbytes, "streaming_gbps": nbytes / (us * 1e-6) / 1e9,
                      "streaming_hbm_frac": nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS}
        for fname, form in (("lane16", capi.FORM_LANE16), ("lane8", capi.FORM_LANE8)):
            us_f = timed(lambda i: dec.contribute(xs[i % 8], idl[i % 8], w, form=form), max(4, args.steps // 8))
            rows[name][fname + "_us"] = us_f
            rows[name][fname + "_gbps"] = nbytes / (us_f * 1e-6) / 1e9
        del dec, table
    # E8M0 block-32 contract: W4A8 routed experts + W8A8 32x32-block shared expert, exact integer dots
    table = ops.ExpertTable.allocate(capi.FMT_E2M1_E8M0, E, H, I, dev)
    sh_table = ops.ExpertTable.allocate(capi.FMT_E4M3_E8M0_32, 1, H, I, dev)
    for t, n in ((table, E), (sh_table, 1)):
        for e in range(n):
            v = t.expert_views(e)
            for i in range(3):
                v[2 * i].random_(0, 256)
                if t is sh_table:
                    v[2 * i].bitwise_and_(0x77)  # no E4M3 NaN codes
                v[2 * i + 1].random_(118, 124)
    e8 = ops.E8m0DecodeOps(table, sh_table.shared_struct(0), 1, K, 10.0)
    nbytes = K * table.weight_bytes_per_expert() + sh_table.weight_bytes_per_expert()
    us = timed(lambda i: e8.contribute(xs[i % 8], idl[i % 8], w), max(4, args.steps // 4))
    rows["e8m0_w4a8_routed_w8a8_shared_exact"] = {"us": us, "weight_bytes": nbytes, "gbps": nbytes / (us * 1e-6) / 1e9,
                                                  "hbm_frac": nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS}
    e8f = ops.E8m0DecodeOps(table, sh_table.shared_struct(0), 1, K, 10.0, exact=False)
    us = timed(lambda i: e8f.contribute(xs[i % 8], idl[i % 8], w), max(4, args.steps // 4))
    rows["e8m0_w4a8_routed_w8a8_shared_fp32_chain"] = {"us": us, "weight_bytes": nbytes, "gbps": nbytes / (us * 1e-6) / 1e9,
                                                       "hbm_frac": nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS}
    del e8, e8f, table, sh_table
    # fused combine + shared gate + residual (one token and 64 tokens)
    for R in (1, 64):
        contrib = synth.normal((R, K, H), 0.05, 3, device=dev, dtype=torch.bfloat16)
        shared_out = synth.normal((R, H), 0.05, 4, device=dev, dtype=torch.bfloat16)
        x = synth.normal((R, H), 1.0, 5, device=dev, dtype=torch.bfloat16)
        resid = synth.normal((R, H), 1.0, 6, device=dev, dtype=torch.bfloat16)
        seg = synth.normal((H,), 0.02, 7, device=dev, dtype=torch.bfloat16)
        ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(R)]).to(torch.int32).to(dev)
        us = timed(lambda i: ops.CombineOps.combine_residual(shared_out, residual=resid, contributions=contrib, ids=ids, seg=seg, x=x), args.steps)
        rows["combine_residual_rows_%d" % R] = {"us": us, "bytes": R * H * 2 * (K + 4), "gbps": R * H * 2 * (K + 4) / (us * 1e-6) / 1e9}
    out = {"metric": "moe_decode_contribution_us", "value": rows["fp8_per_channel"]["streaming_us"], "unit": "us/call", "n_gpus": 1,
           "steps": args.steps, "warmup": 5, "ms_per_step": rows["fp8_per_channel"]["streaming_us"] / 1e3, "higher_is_better": False,
           "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3 (per-channel bf16 scales) / bf16 weights, bf16 activations, f32 accumulate",
           "data": "synthetic",
           "config": {"workload": "rows next to the headline path at the DeepSeek-V3 layer shape, one token: per-channel FP8 and BF16 "
                                  "experts (streaming and Lane16 / Lane8 orders), fused combine + residual",
                      "hidden": H, "intermediate": I, "experts_resident": E + 1, "top_k": K, "shared_experts": 1},
           "rows": rows}
    return out


def decode_main(args, torch, capi, ops, synth, prebuilt=None):
    """BASELINE configs 3 and 4: the decode layer at --batch tokens. Returns the line and the table it drew."""
    table, layer, xs, dims = build_layer(args, torch, capi, ops, synth, prebuilt=prebuilt)
    H, I, E, K = dims
    torch.cuda.synchronize()

    if args.calibrate_copy:
        src = torch.full((args.calibrate_copy << 20,), 3, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)  # reads and writes exactly calibrate_copy MiB
        torch.cuda.synchronize()
        del src, dst
    # distinct experts per ring slot (measured from the ids)
    distinct = []
    for x in xs:
        layer.run(x)
        torch.cuda.synchronize()
        distinct.append(int(torch.unique(layer.ids).numel()))
    assert int(layer.status.item()) == 0, "combine saw a (row, choice) slot that was not contributed exactly once"
    parity = None if args.no_parity_gate else parity_gate_decode(args, torch, capi, ops, table, layer, xs[0], dims)

    graphs = None
    if args.graph and args.one_launch:
        # the one-launch layer tells its activations from an earlier launch's by a per-launch tag that is a kernel argument:
        # a captured launch would replay one tag for ever
        print("bench.py: --graph cannot be combined with --one-launch (ffmoe_decode_token_layer must not be captured)", file=sys.stderr)
        sys.exit(2)
    if args.graph:
        graphs = []
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for x in xs:
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=side):
                    layer.run(x)
                graphs.append(g)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()

    def step(i):
        if graphs is not None:
            graphs[i % len(graphs)].replay()
        else:
            layer.run(xs[i % len(xs)])

    rewarm(torch, lambda: step(0))  # untimed: the parity gate left the GPU idle for seconds
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(args.warmup + i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    us_per_layer = elapsed / args.steps * 1e6
    used = [distinct[(args.warmup + i) % len(xs)] for i in range(args.steps)]
    mean_distinct = sum(used) / len(used)
    bytes_layer = layer_bytes(table, mean_distinct, args.batch, dims)

    # dominant kernel: the gate/up + SwiGLU launch, timed as the layer issues it. One token: the launch with the top-k
    # selection in its prologue (stage 0 of ffmoe_decode_token_forward) from each ring slot's logits; batches: the plain
    # gate/up launch from each ring slot's ids. 8 batches of 16 back-to-back launches over the ring with events on the
    # launch stream (a batch per event pair, so the event overhead is amortised and the figure is the kernel's own
    # duration; weights stay cold because consecutive launches read different experts), whatever --steps is.
    dec = layer.decode
    routed = []
    for x in xs:
        layer.run(x)
        routed.append((layer.ids.clone(), layer.weights.clone(), layer.logits.clone()))
    torch.cuda.synchronize()
    token_path = args.batch == 1 and layer.two_launch and not args.one_launch
    bias1 = layer.bias if layer.bias.dim() == 1 else layer.bias[0]

    def launch(stage, s_):
        # the second launch alone would not be the launch the layer issues (one token: it starts from the record of the live
        # choices that the gate/up launch of the same call leaves; batches: from that call's grouping): time both launches
        # and subtract the first
        if token_path:
            ok = dec.token_forward(xs[s_], layer.ids, layer.weights, layer.combine_mode, layer.y, routed[s_][2], bias=bias1, status=layer.status,
                                   routed_scaling=2.5, n_group=8, topk_group=4, stage=0 if stage == 0 else None)
            assert ok
        else:
            dec.contribute(xs[s_], routed[s_][0], routed[s_][1], stage=0 if stage == 0 else None)

    def time_stage(stage):
        batch, nb = 16, 8
        for i in range(batch):
            launch(stage, i % len(xs))
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(nb)]
        for b_ in range(nb):
            ev[b_][0].record()
            for i in range(batch):
                launch(stage, (b_ * batch + i) % len(xs))
            ev[b_][1].record()
        torch.cuda.synchronize()
        return sorted(a.elapsed_time(b) * 1e3 / batch for a, b in ev), nb * batch  # us per launch

    kt, launches_timed = time_stage(0)
    k_avg = sum(kt) / len(kt)
    mean_distinct_k = sum(distinct) / len(distinct)
    k_bytes = gate_up_bytes(table, mean_distinct_k, args.batch, dims)
    # one token, NVFP4 experts next to a BF16 shared expert: the shared expert's rows ride in both launches in BF16 (gate/up
    # rows as every block's first slice, down rows as every wave's first units of the finish), so the bytes split as for one
    # format. With that switched off by the environment the shared expert's down launch is its own, in front of the routed
    # gate/up, and its down matrix and output row count in stage 0.
    mixed_token = token_path and args.format == "nvfp4"
    own_down = mixed_token and (os.environ.get("FFMOE_DECODE_MIXED_FINISH") == "0" or os.environ.get("FFMOE_DECODE_MIXED_GATE_UP") == "0")
    shared_down = table.shared_bytes // 3 + I * 2 + H * 2 if own_down else 0
    k_bytes += shared_down
    achieved = k_bytes / (k_avg * 1e-6) / 1e9
    # second streaming launch: down (+ routing weight; one token: + ordered combine)
    dt, _ = time_stage(1)
    dt = sorted(max(t - k_avg, 0.0) for t in dt)
    d_avg = sum(dt) / len(dt)
    d_bytes = (mean_distinct_k * table.weight_bytes_per_expert() + table.shared_bytes) // 3 + args.batch * (K + 1) * I * 2 + \
        (args.batch * H * 2 if token_path else args.batch * (K + 1) * H * 2) - (shared_down - 2 * H * 2 if own_down else 0)  # own down launch: the finish reads the shared row instead of a down matrix

    fname = "FmtFp8" if args.format == "fp8" else "FmtNvfp4"
    cohort = not token_path and args.batch >= 4 and not os.environ.get("FFMOE_DECODE_COHORT_ROWS")  # the library's default hand-over to the matrix cores
    if mixed_token:
        gate_up_kernel = ("ffmoe::k_decode_stage<FmtNvfp4, S, 0, 1, NR, FmtBf16, SSH> (gate/up + SwiGLU launch: the BF16 shared expert's rows as every "
                          "block's first slice next to the top-k selection, then the NVFP4 rows%s)" % (
                              "; with the shared expert's own BF16 down launch behind it" if own_down else ""))
        down_kernel = ("ffmoe::k_decode_finish<FmtNvfp4, S, NR> (routed down + routing weight + ordered combine with the shared row)" if own_down else
                       "ffmoe::k_decode_finish<FmtNvfp4, S, NR, 512, FmtBf16, SSH> (down of the BF16 shared expert and of the NVFP4 choices + routing weight + "
                       "ordered combine)")
    elif token_path:
        gate_up_kernel = "ffmoe::k_decode_stage<%s, S, 0, 1, NR> (gate/up + SwiGLU launch, top-k selection in its prologue, as the layer issues it)" % fname
        down_kernel = "ffmoe::k_decode_finish<%s, S, NR> (down + routing weight + ordered combine)" % fname
    elif cohort:
        lines = "k_w16_fp8_lines" if args.format == "fp8" else "k_w16_nvfp4_lines"
        gate_up_kernel = ("ffmoe::%s<MF, 0, P, NW> (gate/up + SwiGLU of the token cohort on the BF16 matrix cores, each chosen expert's weights streamed "
                          "once%s)" % (lines, "; the BF16 shared expert's gate/up launch rides in the figure" if args.format != "fp8" else ""))
        down_kernel = "ffmoe::%s<MF, 1, P, NW> (down + routing weight of the cohort%s)" % (
            lines, "; with the BF16 shared expert's down launch" if args.format != "fp8" else "")
    else:
        gate_up_kernel = "ffmoe::k_decode_stage<%s, S, 0, RG, NR> (gate/up + SwiGLU launch)" % fname
        down_kernel = "ffmoe::k_decode_stage<%s, S, 1, RG, NR> (down + routing weight)" % fname

    out = {
        "metric": "moe_layer_decode_us", "value": us_per_layer, "unit": "us/layer", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": us_per_layer / 1e3,
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": ("fp8_e4m3" if args.format == "fp8" else "nvfp4 (e2m1 + e4m3 group scales)") + " weights, bf16 activations, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": ("DeepSeek-V3-shape FP8 MoE decode layer (BASELINE config 3), batch %d" % args.batch) if args.format == "fp8" else
                               ("DeepSeek-V3-shape MoE decode layer, NVFP4 routed experts + BF16 shared expert (BASELINE config 4), batch %d" % args.batch),
                   "hidden": H, "intermediate": I, "experts": E, "shared_experts": 1, "top_k": K,
                   "routing": "sigmoid grouped top-8 (8 groups, keep 4), renormalised x2.5",
                   "weights": "E4M3 + f32 128x128 block scales" if args.format == "fp8" else "E2M1 pairs + E4M3 scale per 16 + f32 global",
                   "act_mode": "FFMOE_ACT_BF16 (W8A16)" if args.format == "fp8" else "BF16 activations (W4A16)",
                   "batch": args.batch, "ring": len(xs), "launch": "eager" if graphs is None else "hip graph per ring slot",
                   "launches_per_layer": ("router logits; gate/up with the top-k selection in its prologue (BF16 shared rows first); shared expert down; "
                                          "routed down + weight + combine with the shared row") if own_down else
                                         "router logits; gate/up with the top-k selection in its prologue; down + weight + combine" if token_path else
                                         "router logits; top-k; grouping; gate/up; down; combine"},
        "tokens_per_s": args.batch / (us_per_layer * 1e-6),
        "distinct_routed_experts": mean_distinct,
        "layer_bytes": bytes_layer,
        "layer_hbm_gbps": bytes_layer / (us_per_layer * 1e-6) / 1e9,
        "layer_hbm_frac": bytes_layer / (us_per_layer * 1e-6) / 1e9 / HBM_PEAK_GBPS,
        "roofline": {"kernel": gate_up_kernel,
                     "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": GATE_UP_TRAFFIC_BYTES.get((args.batch, args.experts)) if args.format == "fp8" else None,
                     "traffic_source": TRAFFIC_SOURCE if (args.format == "fp8" and (args.batch, args.experts) in GATE_UP_TRAFFIC_BYTES) else None,
                     "bytes_per_launch": k_bytes, "avg_us": k_avg, "min_us": kt[0], "median_us": kt[len(kt) // 2],
                     "launches_timed": launches_timed},
        "down_kernel": {"kernel": down_kernel,
                        "bytes_per_launch": d_bytes, "avg_us": d_avg, "min_us": dt[0], "median_us": dt[len(dt) // 2],
                        "achieved": d_bytes / (d_avg * 1e-6) / 1e9, "frac": d_bytes / (d_avg * 1e-6) / 1e9 / HBM_PEAK_GBPS},
        "parity": parity,
    }
    if not args.no_cpu_baseline and args.format == "fp8":
        out["cpu_baseline"] = cpu_baseline(args, torch, table, layer, xs, dims)
    return out, table


def _brief_decode(out):
    """The figures of a decode line that the one-line summary of the other configurations keeps."""
    return {"workload": out["config"]["workload"], "us": out["value"], "steps": out["steps"], "distinct_routed_experts": out["distinct_routed_experts"],
            "bytes": out["layer_bytes"], "gbps": out["layer_hbm_gbps"], "frac": out["layer_hbm_frac"], "bound": "hbm",
            "gate_up": {"kernel": out["roofline"]["kernel"], "us": out["roofline"]["avg_us"], "bytes": out["roofline"]["bytes_per_launch"],
                        "frac": out["roofline"]["frac"]},
            "down": {"kernel": out["down_kernel"]["kernel"], "us": out["down_kernel"]["avg_us"], "bytes": out["down_kernel"]["bytes_per_launch"],
                     "frac": out["down_kernel"]["frac"]},
            "parity": out["parity"]}


def secondary(args, torch, capi, ops, synth, fp8_table):
    """The other configurations the metric names, measured after the headline's timed region in the same process and each
    behind its own oracle gate: config 3 at 8 and 64 tokens, config 5 (prefill on the FP8 matrix cores, with its CPU
    baseline sample) on the headline's expert table, config 4 (NVFP4 routed experts + BF16 shared expert) at 32 tokens and
    one token on a table of its own. Fewer steps than the stand-alone runs of the same workloads (--batch, --format,
    --workload prefill), the same measurement otherwise."""
    import copy
    sec = {}
    fp8 = (fp8_table, fp8_table.shared_struct_kept)
    for batch, steps in ((8, 60), (64, 32)):
        a = copy.copy(args)
        a.batch, a.ring, a.steps, a.warmup, a.calibrate_copy, a.no_cpu_baseline = batch, 16, steps, 4, 0, True
        out, _ = decode_main(a, torch, capi, ops, synth, prebuilt=fp8)
        sec["c3_fp8_batch%d" % batch] = _brief_decode(out)
    a = copy.copy(args)
    a.workload, a.batch, a.steps, a.warmup, a.prefill_act = "prefill", 4096, 6, 2, "auto"
    out = prefill_main(a, torch, capi, ops, synth, prebuilt=fp8)
    sec["c5_fp8_prefill_4096"] = {
        "workload": out["config"]["workload"], "ms": out["value"], "steps": out["steps"], "flop": out["routed_tflop"] * 1e12, "tflops": out["cohort_tflops"],
        "frac": out["cohort_mfma_frac"], "bound": "mfma", "peak_tflops": MFMA_FP8_PEAK_TFLOPS, "weight_gbps_once": out["cohort_weight_gbps"],
        "experts_touched": out["config"]["experts_touched"], "max_rows_per_expert": out["config"]["max_rows_per_expert"],
        "gate_up": {"kernel": out["roofline"]["kernel"], "ms": out["roofline"]["avg_ms"], "flop": out["roofline"]["flop_per_launch"], "frac": out["roofline"]["frac"]},
        "down": {"kernel": out["down_kernel"]["kernel"], "ms": out["down_kernel"]["avg_ms"], "tflops": out["down_kernel"]["tflops"],
                 "frac": out["down_kernel"]["tflops"] / MFMA_FP8_PEAK_TFLOPS},
        "parity": out["parity"], "cpu_baseline": out.get("cpu_baseline")}
    del out
    nv = None
    for batch, steps, ring in ((32, 48, 16), (1, 100, 64)):
        a = copy.copy(args)
        a.format, a.batch, a.ring, a.steps, a.warmup, a.calibrate_copy, a.no_cpu_baseline = "nvfp4", batch, ring, steps, 4, 0, True
        out, t = decode_main(a, torch, capi, ops, synth, prebuilt=nv)
        nv = (t, t.shared_struct_kept)
        sec["c4_nvfp4_batch%d" % batch] = _brief_decode(out)
    return sec


def main():
    args = parse()
    if args.batch is None:
        args.batch = 1 if args.workload == "decode" else 4096
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path; "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from flyingfish_amd import capi, ops, synth
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    capi.lib()  # fail loudly when the HIP library is missing
    if args.workload == "prefill":
        if args.steps == 200 and args.warmup == 20:
            args.steps, args.warmup = 10, 2
        out = prefill_main(args, torch, capi, ops, synth)
    elif args.workload == "widening":
        out = widening_main(args, torch, capi, ops, synth)
    elif args.workload == "linear":
        out = linear_main(args, torch, capi, ops, synth)
    elif args.workload == "c1":
        out = c1_main(args, torch, capi, ops, synth)
    else:
        out, table = decode_main(args, torch, capi, ops, synth)
        # the headline line (config 3, one token) also carries the rest of the metric, measured after its own timed region
        headline = args.format == "fp8" and args.batch == 1 and args.experts == 256 and not (args.one_launch or args.separate_topk or args.graph)
        if headline and not args.no_secondary:
            out["secondary"] = secondary(args, torch, capi, ops, synth, table)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
