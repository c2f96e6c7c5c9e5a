"""ctypes front-end of the CPU oracle (test infrastructure only).

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import
this package. The shipped library never does.

All BF16 tensors cross this boundary as ``numpy.uint16`` bit patterns.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libffmoe_oracle.so")
_BASE_PATH = os.path.join(_HERE, "libffmoe_cpubase.so")

TWICE, ONCE, CLAMPED_TWICE, CLAMPED_ONCE, GELU_TWICE = 0, 1, 2, 3, 4
AFTER_DOWN_BF16, BEFORE_CONTRIBUTION_BF16 = 0, 1
LANE16, LANE8, F64 = 0, 1, 2
SILU_DIV, SILU_RCP, SILU_SIGMOID2 = 0, 1, 2


def build(force=False):
    """Compile the oracle and the CPU baseline with g++ (see oracle/Makefile)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE, "all"], stdout=subprocess.DEVNULL)


def _load(path):
    if not os.path.exists(path):
        build()
    return ctypes.CDLL(path)


_lib = None
_base = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load(_LIB_PATH)
        L = _lib
        L.orc_decode_e4m3.restype = ctypes.c_float
        L.orc_decode_e4m3.argtypes = [ctypes.c_uint8]
        L.orc_encode_e4m3.restype = ctypes.c_uint8
        L.orc_encode_e4m3.argtypes = [ctypes.c_float]
        L.orc_decode_e2m1.restype = ctypes.c_float
        L.orc_decode_e2m1.argtypes = [ctypes.c_uint8]
        L.orc_encode_e2m1.restype = ctypes.c_uint8
        L.orc_encode_e2m1.argtypes = [ctypes.c_float]
        L.orc_bf16_rne.restype = ctypes.c_uint16
        L.orc_bf16_rne.argtypes = [ctypes.c_float]
        L.orc_expf.restype = ctypes.c_float
        L.orc_expf.argtypes = [ctypes.c_float]
        L.orc_log1pf_unit.restype = ctypes.c_float
        L.orc_log1pf_unit.argtypes = [ctypes.c_float]
        L.orc_effective_weight.restype = ctypes.c_uint16
        L.orc_effective_weight.argtypes = [ctypes.c_uint8, ctypes.c_float]
        L.orc_nvfp4_effective_weight.restype = ctypes.c_uint16
        L.orc_nvfp4_effective_weight.argtypes = [ctypes.c_uint8, ctypes.c_uint8, ctypes.c_float]
        L.orc_silu_mul.restype = ctypes.c_uint16
        L.orc_silu_mul.argtypes = [ctypes.c_uint16, ctypes.c_uint16, ctypes.c_int, ctypes.c_float, ctypes.c_int]
        L.orc_dot.restype = ctypes.c_float
        L.orc_fixture_unit.restype = ctypes.c_float
        L.orc_fixture_unit.argtypes = [ctypes.c_uint64] * 4
        L.orc_fixture_seed.restype = ctypes.c_uint64
        L.orc_fixture_seed.argtypes = [ctypes.c_uint32, ctypes.c_uint64]
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


# ------------------------------------------------------------------------------------------------
# numpy helpers that do not need the C library
def bf16_to_f32(bits):
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(x):
    """Round-to-nearest-even float32 -> bfloat16 bit patterns."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_bf16_rne_array(_p(x), _p(out), ctypes.c_long(x.size))
    return out


def expf(x):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().orc_expf_array(_p(x), _p(out), ctypes.c_long(x.size))
    return out


def tanhf(x):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().orc_tanhf_array(_p(x), _p(out), ctypes.c_long(x.size))
    return out


def gelu_tanh(x):
    """0.5 g (1 + tanh(0.7978846 (g + 0.044715 g^3))) in FP32, one rounding per operation."""
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().orc_gelu_tanh_array(_p(x), _p(out), ctypes.c_long(x.size))
    return out


# ------------------------------------------------------------------------------------------------
def dequant_fp8_block(codes, scales, bn=128, bk=128):
    codes = _c(codes, np.uint8)
    scales = _c(scales, np.float32)
    n, k = codes.shape
    out = np.empty((n, k), dtype=np.uint16)
    lib().orc_dequant_fp8_block(_p(codes), _p(scales), n, k, bn, bk, _p(out))
    return out


def dequant_fp8_channel(codes, scales_bf16):
    codes = _c(codes, np.uint8)
    scales_bf16 = _c(scales_bf16, np.uint16)
    n, k = codes.shape
    out = np.empty((n, k), dtype=np.uint16)
    lib().orc_dequant_fp8_channel(_p(codes), _p(scales_bf16), n, k, _p(out))
    return out


def dequant_nvfp4(codes, scales, global_scale):
    codes = _c(codes, np.uint8)
    scales = _c(scales, np.uint8)
    n, kh = codes.shape
    k = kh * 2
    out = np.empty((n, k), dtype=np.uint16)
    lib().orc_dequant_nvfp4(_p(codes), _p(scales), ctypes.c_float(global_scale), n, k, _p(out))
    return out


def nvfp4_to_fp8_block(codes, scales, global_scale):
    """NVFP4 matrix -> (E4M3 codes [n, k], f32 block scales [n / 128, k / 128]) of the W4A8 mode: every weight rounded to
    E4M3 as e2m1 x e4m3(scale) / 8, every 128 x 128 block scaled by 8 x global."""
    c = _c(codes, np.uint8)
    s = _c(scales, np.uint8)
    n, k2 = c.shape
    k = k2 * 2
    out = np.empty((n, k), dtype=np.uint8)
    lib().orc_nvfp4_to_e4m3(_p(c), _p(s), n, k, _p(out))
    return out, np.full(((n + 127) // 128, (k + 127) // 128), np.float32(global_scale) * np.float32(8.0), dtype=np.float32)


def quant_weight_fp8_block(w, bn=128, bk=128):
    w = _c(w, np.float32)
    n, k = w.shape
    codes = np.empty((n, k), dtype=np.uint8)
    scales = np.empty((-(-n // bn), -(-k // bk)), dtype=np.float32)
    lib().orc_quant_weight_fp8_block(_p(w), n, k, bn, bk, _p(codes), _p(scales))
    return codes, scales


def quant_weight_nvfp4(w):
    w = _c(w, np.float32)
    n, k = w.shape
    assert k % 16 == 0
    codes = np.empty((n, k // 2), dtype=np.uint8)
    scales = np.empty((n, k // 16), dtype=np.uint8)
    g = ctypes.c_float(0)
    lib().orc_quant_weight_nvfp4(_p(w), n, k, _p(codes), _p(scales), ctypes.byref(g))
    return codes, scales, float(np.float32(g.value))


def quant_act_fp8_128(x_bf16):
    x = _c(x_bf16, np.uint16)
    m, k = x.shape
    codes = np.empty((m, k), dtype=np.uint8)
    scales = np.empty((m, -(-k // 128)), dtype=np.float32)
    lib().orc_quant_act_fp8_128(_p(x), m, k, _p(codes), _p(scales))
    return codes, scales


# ------------------------------------------------------------------------------------------------
def route_logits_bf16(x, w):
    x = _c(x, np.uint16)
    w = _c(w, np.uint16)
    rows, hidden = x.shape
    experts = w.shape[0]
    out = np.empty((rows, experts), dtype=np.uint16)
    lib().orc_route_logits_bf16(_p(x), _p(w), _p(out), rows, experts, hidden)
    return out


def route_logits_f32(x, w):
    x = _c(x, np.uint16)
    w = _c(w, np.uint16)
    rows, hidden = x.shape
    experts = w.shape[0]
    out = np.empty((rows, experts), dtype=np.float32)
    lib().orc_route_logits_f32(_p(x), _p(w), _p(out), rows, experts, hidden)
    return out


def route_topk_softmax(logits_bf16, top_k):
    lg = _c(logits_bf16, np.uint16)
    rows, experts = lg.shape
    ids = np.empty((rows, top_k), dtype=np.int32)
    w = np.empty((rows, top_k), dtype=np.uint16)
    lib().orc_route_topk_softmax(_p(lg), _p(ids), _p(w), rows, experts, top_k)
    return ids, w


def route_topk_sigmoid(logits_bf16, top_k):
    lg = _c(logits_bf16, np.uint16)
    rows, experts = lg.shape
    ids = np.empty((rows, top_k), dtype=np.int32)
    w = np.empty((rows, top_k), dtype=np.uint16)
    lib().orc_route_topk_sigmoid(_p(lg), _p(ids), _p(w), rows, experts, top_k)
    return ids, w


def route_topk_noaux(logits, bias, top_k, score_mode=0, routed_scaling=1.0, n_group=1, topk_group=1):
    lg = _c(logits, np.float32)
    rows, experts = lg.shape
    b = None if bias is None else _c(np.broadcast_to(bias, lg.shape), np.float32)
    ids = np.empty((rows, top_k), dtype=np.int32)
    w = np.empty((rows, top_k), dtype=np.float32)
    lib().orc_route_topk_noaux(_p(lg), _p(b), _p(ids), _p(w), rows, experts, top_k, score_mode,
                               ctypes.c_float(routed_scaling), n_group, topk_group)
    return ids, w


def topk_ids(scores, k):
    s = _c(scores, np.float32)
    ids = np.empty(k, dtype=np.int32)
    lib().orc_topk_ids(_p(s), s.size, k, _p(ids))
    return ids


# ------------------------------------------------------------------------------------------------
def silu_mul(gate_bf16, up_bf16, rounding, limit=0.0, kind=SILU_DIV):
    g = _c(gate_bf16, np.uint16)
    u = _c(up_bf16, np.uint16)
    out = np.empty(g.shape, dtype=np.uint16)
    lib().orc_silu_mul_array(_p(g), _p(u), _p(out), ctypes.c_long(g.size), rounding, ctypes.c_float(limit), kind)
    return out


def dot(x_f32, w_bf16, form):
    x = _c(x_f32, np.float32)
    w = _c(w_bf16, np.uint16)
    return float(lib().orc_dot(_p(x), _p(w), x.size, form))


def expert_ffn(x, gate, up, down, routing=1.0, rounding=TWICE, limit=0.0, boundary=AFTER_DOWN_BF16,
               form=LANE8, silu_kind=SILU_DIV, apply_weight=True, return_act=False):
    """One (row, choice) contribution over BF16 effective weights. x [H], gate/up [I,H], down [H,I]."""
    x = _c(x, np.uint16)
    gate = _c(gate, np.uint16)
    up = _c(up, np.uint16)
    down = _c(down, np.uint16)
    I, H = gate.shape
    assert x.shape == (H,) and up.shape == (I, H) and down.shape == (H, I)
    out = np.empty(H, dtype=np.uint16)
    act = np.empty(I, dtype=np.uint16)
    lib().orc_expert_ffn(_p(x), _p(gate), _p(up), _p(down), H, I, ctypes.c_float(routing), rounding,
                         ctypes.c_float(limit), boundary, form, silu_kind, int(bool(apply_weight)), _p(out), _p(act))
    return (out, act) if return_act else out


def expert_down(act, down, routing=1.0, boundary=AFTER_DOWN_BF16, form=LANE8, apply_weight=True):
    """Second half of expert_ffn from a given BF16 activation [I]: down [H, I], routing weight at `boundary`."""
    act = _c(act, np.uint16)
    down = _c(down, np.uint16)
    H, I = down.shape
    assert act.shape == (I,)
    out = np.empty(H, dtype=np.uint16)
    lib().orc_expert_down(_p(act), _p(down), H, I, ctypes.c_float(routing), boundary, form, int(bool(apply_weight)), _p(out))
    return out


def linear_fp8_block_w8a8(w_codes, w_scales, x_codes, x_scales, order=0, want_f32=False):
    w = _c(w_codes, np.uint8)
    sw = _c(w_scales, np.float32)
    xq = _c(x_codes, np.uint8)
    sx = _c(x_scales, np.float32)
    n, k = w.shape
    m = xq.shape[0]
    y = np.empty((m, n), dtype=np.uint16)
    yf = np.empty((m, n), dtype=np.float32)
    lib().orc_linear_fp8_block_w8a8(_p(w), _p(sw), _p(xq), _p(sx), m, n, k, order, _p(y), _p(yf))
    return (y, yf) if want_f32 else y


def expert_ffn_w8a8(x, gate, sgate, up, sup, down, sdown, routing=1.0, rounding=TWICE, limit=0.0, boundary=AFTER_DOWN_BF16,
                    order=0, silu_kind=SILU_SIGMOID2, apply_weight=True, return_act=False):
    """One (row, choice) contribution on the block-F32 W8A8 path. x [H] bf16 bits; gate/up codes [I,H]; down [H,I]."""
    x = _c(x, np.uint16)
    gate, up, down = _c(gate, np.uint8), _c(up, np.uint8), _c(down, np.uint8)
    sgate, sup, sdown = _c(sgate, np.float32), _c(sup, np.float32), _c(sdown, np.float32)
    I, H = gate.shape
    assert x.shape == (H,) and up.shape == (I, H) and down.shape == (H, I)
    out = np.empty(H, dtype=np.uint16)
    act = np.empty(I, dtype=np.uint16)
    lib().orc_expert_ffn_w8a8(_p(x), _p(gate), _p(sgate), _p(up), _p(sup), _p(down), _p(sdown), H, I, ctypes.c_float(routing),
                              rounding, ctypes.c_float(limit), boundary, order, silu_kind, int(bool(apply_weight)), _p(out), _p(act))
    return (out, act) if return_act else out


def expert_down_w8a8(act, down, sdown, routing=1.0, boundary=AFTER_DOWN_BF16, order=0, apply_weight=True):
    """Second half of expert_ffn_w8a8 from a given BF16 activation [I]: re-quantize, down, routing weight."""
    act = _c(act, np.uint16).reshape(1, -1)
    aq, sa = quant_act_fp8_128(act)
    d, lin = linear_fp8_block_w8a8(down, sdown, aq, sa, order=order, want_f32=True)
    if not apply_weight:
        return d[0]
    w = np.float32(routing)
    v = bf16_to_f32(d[0]) * w if boundary == AFTER_DOWN_BF16 else lin[0] * w
    return f32_to_bf16(v.astype(np.float32))


def act_quant_e8m0(x_bf16):
    """rows of BF16 bits [rows, k] -> (E4M3 codes [rows, k], E8M0 scale codes [rows, k / 32])."""
    x = _c(x_bf16, np.uint16)
    rows, k = x.shape
    codes = np.empty((rows, k), dtype=np.uint8)
    scales = np.empty((rows, k // 32), dtype=np.uint8)
    if lib().orc_act_quant_e8m0(_p(x), rows, k, _p(codes), _p(scales)) != 0:
        raise ValueError("activation scale exponent out of range")
    return codes, scales


def scaled_dot_exact(packed, w, sw, x_codes, x_scales):
    """One exact dot of the E8M0 contract -> (FP64 total, BF16 bits)."""
    w, sw, xc, xs = _c(w, np.uint8), _c(sw, np.uint8), _c(x_codes, np.uint8), _c(x_scales, np.uint8)
    total = ctypes.c_double()
    rounded = ctypes.c_uint16()
    if lib().orc_scaled_dot_exact(int(packed), _p(w), _p(sw), _p(xc), _p(xs), xc.size, ctypes.byref(total), ctypes.byref(rounded)) != 0:
        raise ValueError("NaN code or 0xff scale")
    return total.value, rounded.value


def expert_ffn_e8m0(packed, x, gate, sgate, up, sup, down, sdown, limit, route_weight=1.0, return_act=False):
    """One expert on one token in the exact E8M0 contract; see orc_expert_ffn_e8m0."""
    x = _c(x, np.uint16)
    H = x.size
    down = _c(down, np.uint8)
    I = down.shape[1] * (2 if packed else 1)
    out = np.empty(H, dtype=np.uint16)
    act = np.empty(I, dtype=np.uint16)
    rc = lib().orc_expert_ffn_e8m0(int(packed), _p(x), _p(_c(gate, np.uint8)), _p(_c(sgate, np.uint8)), _p(_c(up, np.uint8)),
                                   _p(_c(sup, np.uint8)), _p(down), _p(_c(sdown, np.uint8)), H, I, ctypes.c_float(limit),
                                   ctypes.c_float(route_weight), _p(out), _p(act))
    if rc != 0:
        raise ValueError("orc_expert_ffn_e8m0 failed (%d)" % rc)
    return (out, act) if return_act else out


def e8m0_dot_f32(packed, w, sw, x_codes, x_scales):
    """One dot of the FP32-chain variant of the E8M0 contract (32-lane order of the reference's kernels)."""
    w, sw, xc, xs = _c(w, np.uint8), _c(sw, np.uint8), _c(x_codes, np.uint8), _c(x_scales, np.uint8)
    lib().orc_e8m0_dot_f32.restype = ctypes.c_float
    return float(lib().orc_e8m0_dot_f32(int(packed), _p(w), _p(sw), _p(xc), _p(xs), xc.size))


def expert_ffn_e8m0_f32(packed, x, gate, sgate, up, sup, down, sdown, limit, route_weight=1.0):
    """One expert on one token, FP32-chain variant; see orc_expert_ffn_e8m0_f32."""
    x = _c(x, np.uint16)
    H = x.size
    down = _c(down, np.uint8)
    I = down.shape[1] * (2 if packed else 1)
    out = np.empty(H, dtype=np.uint16)
    rc = lib().orc_expert_ffn_e8m0_f32(int(packed), _p(x), _p(_c(gate, np.uint8)), _p(_c(sgate, np.uint8)), _p(_c(up, np.uint8)),
                                       _p(_c(sup, np.uint8)), _p(down), _p(_c(sdown, np.uint8)), H, I, ctypes.c_float(limit),
                                       ctypes.c_float(route_weight), _p(out), None)
    if rc != 0:
        raise ValueError("orc_expert_ffn_e8m0_f32 failed (%d)" % rc)
    return out


def linear_skinny(weight_bf16, x_bf16, kind=0):
    w = _c(weight_bf16, np.uint16)
    x = _c(x_bf16, np.uint16)
    n, k = w.shape
    m = x.shape[0]
    y = np.empty((m, n), dtype=np.uint16)
    lib().orc_linear_skinny(_p(w), _p(x), m, n, k, kind, _p(y))
    return y


def shared_scale(x_bf16, seg_bf16):
    x = _c(x_bf16, np.uint16)
    seg = _c(seg_bf16, np.uint16)
    rows, hidden = x.shape
    out = np.empty(rows, dtype=np.uint16)
    lib().orc_shared_scale(_p(x), _p(seg), _p(out), rows, hidden)
    return out


COMBINE_GATED, COMBINE_UNGATED, COMBINE_BF16, COMBINE_ACCUM_FP32, COMBINE_ACCUM_BF16, COMBINE_ROUTED = 0, 1, 2, 3, 4, 5
COMBINE_DESC_BF16_GATED, COMBINE_ASC_BF16_GATED = 6, 7


def combine(contributions, shared, scale, ids, active, mode):
    c = _c(contributions, np.uint16)
    rows, top_k, hidden = c.shape
    sh = None if shared is None else _c(shared, np.uint16)
    sc = None if scale is None else _c(scale, np.uint16)
    ii = None if ids is None else _c(ids, np.int32)
    ac = None if active is None else _c(active, np.uint32)
    y = np.empty((rows, hidden), dtype=np.uint16)
    lib().orc_combine(_p(c), _p(sh), _p(sc), _p(ii), _p(ac), _p(y), rows, top_k, hidden, mode)
    return y


def weight_f32(down_bf16, w_f32):
    d = _c(down_bf16, np.uint16)
    w = _c(w_f32, np.float32).reshape(-1)
    a, h = d.shape
    out = np.empty((a, h), dtype=np.uint16)
    lib().orc_weight_f32(_p(d), _p(w), _p(out), a, h)
    return out


def fixture_fill(variant, slot, a0, n0, n1, n2, scale):
    salt = lib().orc_fixture_seed(variant, slot)
    out = np.empty((n0, n1, n2), dtype=np.uint16)
    lib().orc_fixture_fill(ctypes.c_uint64(salt), ctypes.c_uint64(a0), n0, n1, n2, ctypes.c_float(scale), _p(out))
    return out


def pattern_fill(seed0, phase, n):
    out = np.empty(n, dtype=np.uint16)
    lib().orc_pattern_fill(ctypes.c_uint64(seed0), ctypes.c_double(phase), ctypes.c_long(n), _p(out))
    return out


# ------------------------------------------------------------------------------------------------
# metrics of src/verify.rs:568-576 (rel_rmse) and :605-638 (ordered-bits BF16 distance)
def rel_l2(actual_bf16, ref_bf16):
    a = bf16_to_f32(actual_bf16).astype(np.float64).ravel()
    r = bf16_to_f32(ref_bf16).astype(np.float64).ravel()
    den = np.sqrt(np.sum(r * r))
    return float(np.sqrt(np.sum((a - r) ** 2)) / den) if den > 0 else float(np.sqrt(np.sum((a - r) ** 2)))


def bf16_order_key(bits):
    b = np.asarray(bits, dtype=np.uint16).astype(np.int64)
    return np.where(b & 0x8000, (~b) & 0xFFFF, b | 0x8000)


def bf16_ulp_max(actual_bf16, ref_bf16):
    return int(np.max(np.abs(bf16_order_key(actual_bf16) - bf16_order_key(ref_bf16)))) if np.size(actual_bf16) else 0


# ------------------------------------------------------------------------------------------------
# multithreaded CPU baseline (cpu_baseline.cpp): port of the reference's two-phase CPU expert pool
def cpubase():
    global _base
    if _base is None:
        _base = _load(_BASE_PATH)
        _base.cpubase_max_threads.restype = ctypes.c_int
        _base.cpubase_isa.restype = ctypes.c_char_p
    return _base


class CpuDecodeJob:
    """Host copies of the experts a decode batch touches, laid out for cpubase_moe_decode.

    experts: list of (gate_codes, gate_scales, up_codes, up_scales, down_codes, down_scales) numpy arrays,
    one entry per assignment (repeat the entry when two assignments share an expert).
    """

    def __init__(self, x_bf16, rows, experts, weights, apply_w, boundary=AFTER_DOWN_BF16):
        self.x = _c(x_bf16, np.uint16)
        self.rows = _c(rows, np.int32)
        self.keep = [tuple(_c(a, a.dtype) for a in ex) for ex in experts]
        self.ptrs = np.array([[a.ctypes.data for a in ex] for ex in self.keep], dtype=np.uint64)
        self.w = _c(weights, np.float32)
        self.apply = _c(apply_w, np.int32)
        self.n = len(experts)
        self.I, self.H = self.keep[0][0].shape
        self.boundary = boundary
        self.xf = np.empty((self.n, self.H), dtype=np.float32)
        self.act = np.empty((self.n, self.I), dtype=np.uint16)
        self.out = np.empty((self.n, self.H), dtype=np.uint16)

    def run(self, threads):
        rc = cpubase().cpubase_moe_decode(_p(self.x), _p(self.rows), _p(self.ptrs), _p(self.w), _p(self.apply), self.n, self.H,
                                          self.I, self.boundary, int(threads), _p(self.xf), _p(self.act), _p(self.out))
        if rc != 0:
            raise RuntimeError("cpubase_moe_decode rejected the shapes")
        return self.out
