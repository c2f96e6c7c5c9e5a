"""Host-side checks that need no GPU: the C-ABI library loads, exports every declared symbol, and rejects
contract violations before touching the device; the synthetic quantizers equal the oracle's; the CPU baseline
equals the scalar oracle bit for bit."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import oracle as orc
from flyingfish_amd import capi, synth
from flyingfish_amd.ops import ExpertTable

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "ffmoe.h")).read()
    declared = set(re.findall(r"\b(ffmoe_[a-z0-9_]+)\s*\(", header))
    lib = capi.lib()
    for name in sorted(declared):
        assert hasattr(lib, name), name
    assert declared == set(capi.EXPORTS)
    assert lib.ffmoe_version() == 1


def test_route_contract_violations_are_reported_before_launch():
    L = capi.lib()
    assert L.ffmoe_route_topk(None, 16, 16, 1, 64, 4, 0, None) == capi.ERR_NULL and "NULL" in capi.last_error()
    assert L.ffmoe_route_topk(24, 16, 32, 1, 64, 4, 0, None) == capi.ERR_ALIGN
    assert L.ffmoe_route_topk(4096, 8192, 12288, 1, 64, 64, 0, None) == capi.ERR_SHAPE      # top_k > 32
    assert L.ffmoe_route_topk(4096, 8192, 12288, 1, 2048, 4, 0, None) == capi.ERR_SHAPE     # experts > 1024
    assert L.ffmoe_route_topk(4096, 8192, 12288, 1, 4, 4, 0, None) == capi.ERR_SHAPE        # top_k == experts
    assert L.ffmoe_route_topk(4096, 4096, 12288, 1, 64, 4, 0, None) == capi.ERR_OVERLAP
    assert L.ffmoe_route_logits_bf16(4096, 1 << 20, 1 << 21, 1, 64, 100, None) == capi.ERR_SHAPE  # hidden % 8
    assert L.ffmoe_route_topk_noaux(4096, None, 0, 8192, 12288, 1, 1, 256, 8, 0, ctypes.c_float(-1.0), 1, 1, None) == capi.ERR_SHAPE
    assert L.ffmoe_route_topk_noaux(4096, None, 0, 8192, 12288, 1, 1, 256, 8, 0, ctypes.c_float(2.5), 7, 4, None) == capi.ERR_SHAPE
    assert L.ffmoe_route_topk_noaux(4096, None, 0, 8192, 12288, 1, 1, 256, 8, 3, ctypes.c_float(2.5), 1, 1, None) == capi.ERR_UNSUPPORTED


def _decode_args(**kw):
    d = dict(rows=1, top_k=4, act_mode=0, swiglu=0, swiglu_limit=0.0, routed_weight=0, weights_f32=0, x=1 << 20, ids=2 << 20,
             active=None, weights=3 << 20, contributions=4 << 20, shared_out=None, done=None, scratch=8 << 20, scratch_bytes=1 << 20)
    d.update(kw)
    return capi.Decode(d["rows"], d["top_k"], d["act_mode"], d["swiglu"], d["swiglu_limit"], d["routed_weight"], d["weights_f32"],
                       d["x"], d["ids"], d["active"], d["weights"], d["contributions"], d["shared_out"], d["done"], d["scratch"],
                       d["scratch_bytes"])


def test_decode_contract_violations_are_reported_before_launch():
    L = capi.lib()
    table = capi.ExpertTable(capi.FMT_FP8_BLOCK128, 64, 2048, 1408, 16 << 20, None, None)

    def call(t=table, **kw):
        a = _decode_args(**kw)
        return L.ffmoe_decode_contribute(ctypes.byref(t), None, ctypes.byref(a), None)
    assert call(x=None) == capi.ERR_NULL
    assert call(x=(1 << 20) + 8) == capi.ERR_ALIGN
    assert call(top_k=40) == capi.ERR_SHAPE
    # block-FP8 batches of 32 rows and more go to the cohort kernels, which take any row count (here: too small an arena);
    # the streaming kernels of the other formats keep their limit of 4096 assignments per call
    assert call(rows=4096) == capi.ERR_SCRATCH
    nv_rows = capi.ExpertTable(capi.FMT_NVFP4, 64, 2048, 1408, 16 << 20, None, 32 << 20)
    assert call(t=nv_rows, rows=4096, scratch_bytes=1 << 30, contributions=1 << 40) == capi.ERR_SHAPE and "prefill" in capi.last_error()
    assert call(scratch_bytes=16) == capi.ERR_SCRATCH
    assert call(contributions=1 << 20) == capi.ERR_OVERLAP
    assert call(act_mode=2) == capi.ERR_UNSUPPORTED
    nv = capi.ExpertTable(capi.FMT_NVFP4, 64, 2048, 1408, 16 << 20, None, 32 << 20)
    # FP8 activations run on block-FP8 experts (W8A8) and NVFP4 experts (W4A8, which needs the global scales), not on BF16 ones
    bf = capi.ExpertTable(capi.FMT_BF16, 64, 2048, 1408, 16 << 20, None, None)
    assert call(t=bf, act_mode=1) == capi.ERR_UNSUPPORTED
    nv_no_globals = capi.ExpertTable(capi.FMT_NVFP4, 64, 2048, 1408, 16 << 20, None, None)
    assert call(t=nv_no_globals, act_mode=1) == capi.ERR_NULL
    assert call(swiglu=2, swiglu_limit=0.0) == capi.ERR_SHAPE
    assert call(swiglu=7) == capi.ERR_UNSUPPORTED
    bad = capi.ExpertTable(capi.FMT_FP8_BLOCK128, 64, 2000, 1408, 16 << 20, None, None)
    assert call(t=bad) == capi.ERR_SHAPE
    assert L.ffmoe_decode_contribute_stage(ctypes.byref(table), None, ctypes.byref(_decode_args()), 2, None) == capi.ERR_SHAPE
    assert L.ffmoe_decode_scratch_bytes(1, 8, 256, 7168, 2048, 2048) >= 9 * 2048 * 2


def test_linear_and_combine_contract_violations():
    L = capi.lib()
    assert L.ffmoe_linear_fp8_block(1 << 20, 2 << 20, 3 << 20, 4 << 20, 1, 256, 100, 0, None, 0, None) == capi.ERR_SHAPE
    assert L.ffmoe_linear_fp8_block(1 << 20, 2 << 20, 3 << 20, 3 << 20, 1, 256, 128, 0, None, 0, None) == capi.ERR_OVERLAP
    assert L.ffmoe_linear_fp8_block(1 << 20, 2 << 20, 3 << 20, 4 << 20, 1, 256, 128, 1, None, 0, None) == capi.ERR_NULL  # scratch
    assert L.ffmoe_linear_nvfp4(1 << 20, 2 << 20, None, 3 << 20, 4 << 20, 1, 256, 128, None) == capi.ERR_NULL
    assert L.ffmoe_combine(1 << 20, 2 << 20, None, 3 << 20, None, None, 4 << 20, None, 1, 8, 100, 2, None) == capi.ERR_SHAPE
    assert L.ffmoe_combine(1 << 20, 2 << 20, None, 3 << 20, None, None, 4 << 20, None, 1, 8, 128, 0, None) == capi.ERR_NULL  # gated needs scale
    assert L.ffmoe_combine(1 << 20, 2 << 20, None, 3 << 20, None, None, 4 << 20, None, 1, 8, 128, 9, None) == capi.ERR_UNSUPPORTED
    assert L.ffmoe_swiglu(1 << 20, 2 << 20, 3 << 20, 1, 12, 0, ctypes.c_float(0), None) == capi.ERR_SHAPE
    assert L.ffmoe_quant_fp8_f32_128(1 << 20, 1 << 20, 2 << 20, 1, 128, None) == capi.ERR_OVERLAP


def _prefill_args(**kw):
    d = dict(rows=64, top_k=4, act_mode=capi.ACT_FP8_BLOCK128, swiglu=0, swiglu_limit=0.0, routed_weight=0, weights_f32=1, x=1 << 20,
             ids=2 << 20, active=None, weights=3 << 20, contributions=64 << 20, done=None, scratch=256 << 20, scratch_bytes=1 << 30,
             shared=None, shared_out=None, assignment_gen=None)
    d.update(kw)
    return capi.Prefill(d["rows"], d["top_k"], d["act_mode"], d["swiglu"], d["swiglu_limit"], d["routed_weight"], d["weights_f32"],
                        d["x"], d["ids"], d["active"], d["weights"], d["contributions"], d["done"], d["scratch"], d["scratch_bytes"],
                        d["shared"], d["shared_out"], d["assignment_gen"])


def test_prefill_contract_violations_are_reported_before_launch():
    L = capi.lib()
    table = capi.ExpertTable(capi.FMT_FP8_BLOCK128, 64, 2048, 1408 - 1408 % 128, 16 << 20, None, None)

    def call(t=table, **kw):
        a = _prefill_args(**kw)
        return L.ffmoe_prefill_contribute(ctypes.byref(t), ctypes.byref(a), None)
    assert L.ffmoe_prefill_contribute(None, None, None) == capi.ERR_NULL
    assert call(act_mode=capi.ACT_E4M3_E8M0_32) == capi.ERR_UNSUPPORTED
    nv = capi.ExpertTable(capi.FMT_NVFP4, 64, 2048, 1280, 16 << 20, None, 32 << 20)
    bf = capi.ExpertTable(capi.FMT_BF16, 64, 2048, 1280, 16 << 20, None, None)
    assert call(t=bf) == capi.ERR_UNSUPPORTED and "matrix cores" in capi.last_error()  # FP8 activations: block-FP8 (W8A8) or NVFP4 (W4A8) experts
    assert call(t=capi.ExpertTable(capi.FMT_NVFP4, 64, 2048, 1280, 16 << 20, None, None)) == capi.ERR_NULL  # W4A8 needs the global scales
    bf_shared = capi.SharedExpert(capi.FMT_BF16, 1280)
    assert call(t=nv, shared=ctypes.pointer(bf_shared), shared_out=512 << 20) == capi.ERR_UNSUPPORTED  # no BF16 shared expert next to FP8 activations
    nv_bare = capi.ExpertTable(capi.FMT_NVFP4, 64, 2048, 1280, 16 << 20, None, None)
    assert call(t=nv_bare, act_mode=capi.ACT_BF16) == capi.ERR_NULL   # W4A16 prefill: the table must bring its global scales
    odd16 = capi.ExpertTable(capi.FMT_BF16, 64, 2048 + 32, 1280, 16 << 20, None, None)
    assert call(t=odd16, act_mode=capi.ACT_BF16) == capi.ERR_SHAPE  # multiples of 64 on the BF16 matrix cores
    assert call(top_k=40) == capi.ERR_SHAPE
    assert call(swiglu=2, swiglu_limit=0.0) == capi.ERR_SHAPE
    assert call(swiglu=capi.SWIGLU_GELU_TWICE) == capi.ERR_UNSUPPORTED and "FFMOE_ACT_BF16" in capi.last_error()  # SiLU forms only on FP8 activations
    assert call(swiglu=5, act_mode=capi.ACT_BF16) == capi.ERR_UNSUPPORTED
    assert call(routed_weight=capi.WEIGHT_BEFORE_DOWN_F32) == capi.ERR_UNSUPPORTED
    assert call(scratch_bytes=4096) == capi.ERR_SCRATCH
    assert call(scratch=(256 << 20) + 16) == capi.ERR_ALIGN
    assert call(contributions=1 << 20) == capi.ERR_OVERLAP
    odd = capi.ExpertTable(capi.FMT_FP8_BLOCK128, 64, 2048, 1408, 16 << 20, None, None)  # 1408 = 11 * 128 is fine, 1400 is not
    assert call(t=odd, scratch_bytes=16) == capi.ERR_SCRATCH
    bad = capi.ExpertTable(capi.FMT_FP8_BLOCK128, 64, 2048, 1400, 16 << 20, None, None)
    assert call(t=bad) == capi.ERR_SHAPE
    mx = capi.ExpertTable(capi.FMT_E2M1_E8M0, 64, 2048, 1280, 16 << 20, None, None)
    mx_ok = dict(act_mode=capi.ACT_E4M3_E8M0_32, routed_weight=capi.WEIGHT_BEFORE_DOWN_F32, swiglu=capi.SWIGLU_CLAMPED_ONCE, swiglu_limit=7.0)
    assert call(t=mx) == capi.ERR_UNSUPPORTED and "E4M3_E8M0_32" in capi.last_error()        # FP8 block activations
    assert call(t=mx, **{**mx_ok, "routed_weight": capi.WEIGHT_AFTER_DOWN_BF16}) == capi.ERR_UNSUPPORTED
    assert call(t=mx, **{**mx_ok, "swiglu_limit": 0.0}) == capi.ERR_SHAPE
    assert call(t=mx, **{**mx_ok, "rows": 16384, "top_k": 8}) == capi.ERR_SHAPE and "65535" in capi.last_error()
    assert call(t=mx, scratch_bytes=64, **mx_ok) == capi.ERR_SCRATCH
    assert L.ffmoe_prefill_contribute_stage(ctypes.byref(table), ctypes.byref(_prefill_args()), 7, None) == capi.ERR_SHAPE
    assert L.ffmoe_prefill_scratch_bytes(0, 8, 256, 7168, 2048, 0) == 0
    need = L.ffmoe_prefill_scratch_bytes(4096, 8, 256, 7168, 2048, 0)
    assert need >= 4096 * 8 * 2048 * 3 + 4096 * 7168  # BF16 + E4M3 activations of every assignment, quantized x


def test_token_and_form_entry_contract_violations():
    L = capi.lib()
    fp8 = capi.ExpertTable(capi.FMT_FP8_BLOCK128, 256, 7168, 2048, 16 << 20, None, None)
    f = ctypes.c_float
    logits, y = 5 << 20, 6 << 20

    def from_logits(t=fp8, score=capi.NOAUX_SIGMOID, scaling=2.5, n_group=8, topk_group=4, lg=logits, **kw):
        a = _decode_args(**{**dict(top_k=8, weights_f32=1), **kw})
        return L.ffmoe_decode_contribute_from_logits(ctypes.byref(t), None, ctypes.byref(a), lg, None, score, f(scaling), n_group, topk_group, None)
    assert from_logits(rows=2) == capi.ERR_UNSUPPORTED and "one token row" in capi.last_error()
    assert from_logits(act_mode=capi.ACT_FP8_BLOCK128) == capi.ERR_UNSUPPORTED
    assert from_logits(weights_f32=0) == capi.ERR_UNSUPPORTED
    assert from_logits(t=capi.ExpertTable(capi.FMT_FP8_BLOCK128, 96, 7168, 2048, 16 << 20, None, None)) == capi.ERR_UNSUPPORTED
    assert from_logits(score=5) == capi.ERR_UNSUPPORTED
    assert from_logits(scaling=-1.0) == capi.ERR_SHAPE
    assert from_logits(n_group=8, topk_group=9) == capi.ERR_SHAPE
    assert from_logits(lg=logits + 2) == capi.ERR_ALIGN

    def token_layer(combine=capi.COMBINE_ROUTED, yy=y, **kw):
        a = _decode_args(**{**dict(top_k=8, weights_f32=1), **kw})
        return L.ffmoe_decode_token_layer(ctypes.byref(fp8), None, ctypes.byref(a), logits, None, capi.NOAUX_SIGMOID, f(2.5), 8, 4, None, yy, None,
                                          combine, None)
    assert token_layer(rows=4) == capi.ERR_UNSUPPORTED
    assert token_layer(combine=17) == capi.ERR_UNSUPPORTED
    assert token_layer(combine=capi.COMBINE_UNGATED) == capi.ERR_SHAPE and "shared expert" in capi.last_error()
    assert token_layer(yy=y + 2) == capi.ERR_ALIGN

    def form(t, form_id=capi.FORM_LANE16, **kw):
        a = _decode_args(**kw)
        return L.ffmoe_decode_contribute_form(ctypes.byref(t), None, ctypes.byref(a), form_id, None)
    bf16 = capi.ExpertTable(capi.FMT_BF16, 64, 2048, 1408, 16 << 20, None, None)
    assert form(fp8) == capi.ERR_UNSUPPORTED          # block-scaled experts have no Lane16 / Lane8 reference order
    assert form(bf16, form_id=3) == capi.ERR_UNSUPPORTED
    assert form(bf16, act_mode=capi.ACT_FP8_BLOCK128) == capi.ERR_UNSUPPORTED
    assert form(bf16, x=None) == capi.ERR_NULL


def test_e8m0_entry_contract_violations():
    L = capi.lib()
    t = capi.ExpertTable(capi.FMT_E2M1_E8M0, 16, 7168, 2048, 16 << 20, None, None)

    def call(tt=t, **kw):
        d = dict(top_k=8, act_mode=capi.ACT_E4M3_E8M0_32, swiglu=capi.SWIGLU_CLAMPED_ONCE, swiglu_limit=10.0,
                 routed_weight=capi.WEIGHT_BEFORE_DOWN_F32, weights_f32=1, scratch_bytes=1 << 30)
        d.update(kw)
        a = _decode_args(**d)
        return L.ffmoe_decode_contribute_e8m0(ctypes.byref(tt), None, ctypes.byref(a), None)
    assert L.ffmoe_decode_contribute_e8m0(None, None, None, None) == capi.ERR_NULL
    assert call(tt=capi.ExpertTable(capi.FMT_FP8_BLOCK128, 16, 7168, 2048, 16 << 20, None, None)) == capi.ERR_UNSUPPORTED
    assert call(act_mode=capi.ACT_BF16) == capi.ERR_UNSUPPORTED
    assert call(swiglu_limit=0.0) == capi.ERR_SHAPE
    assert call(routed_weight=capi.WEIGHT_AFTER_DOWN_BF16) == capi.ERR_UNSUPPORTED
    assert call(weights_f32=0) == capi.ERR_UNSUPPORTED
    assert call(tt=capi.ExpertTable(capi.FMT_E2M1_E8M0, 16, 7168 + 16, 2048, 16 << 20, None, None)) == capi.ERR_SHAPE
    assert call(scratch_bytes=64) == capi.ERR_SCRATCH and "ffmoe_e8m0_scratch_bytes" in capi.last_error()
    assert L.ffmoe_act_quant_e8m0(None, 1 << 20, 2 << 20, 1, 64, None) == capi.ERR_NULL
    assert L.ffmoe_act_quant_e8m0(1 << 20, 2 << 20, 3 << 20, 1, 48, None) == capi.ERR_SHAPE
    assert L.ffmoe_e8m0_scratch_bytes(1, 8, 7168, 2048, 2048) > 0


def test_slot_layout_matches_the_reference_catalogue():
    # src/experts/catalogue.rs:180-222: codes gate|up|down, then gate, up, down scales; BASELINE byte counts
    offs, size = ExpertTable.slot_layout(capi.FMT_FP8_BLOCK128, 7168, 2048)
    w = 7168 * 2048
    assert offs == [0, 3 * w, w, 3 * w + 16 * 56 * 4, 2 * w, 3 * w + 2 * 16 * 56 * 4]
    assert 3 * w + 3 * 16 * 56 * 4 == 44050944 and size >= 44050944 and size % 256 == 0
    offs, size = ExpertTable.slot_layout(capi.FMT_FP8_BLOCK128, 2048, 1408)
    assert 3 * 2048 * 1408 == 8650752 and offs[1] == 8650752 and (size - 8650752) // 1 >= 2112
    offs, size = ExpertTable.slot_layout(capi.FMT_NVFP4, 7168, 2048)
    assert 3 * w // 2 == 22020096 and 3 * w // 16 == 2752512 and offs[1] == 22020096
    # the published DeepSeek-V4.1 grid (tests/deepseek_contract.rs:587-644): hidden 5120, intermediate 2304, E2M1 codes with
    # [rows, cols / 32] E8M0 scales: 3 x 5,898,240 code bytes + 3 x 368,640 scale bytes, codes first, then the scales
    offs, size = ExpertTable.slot_layout(capi.FMT_E2M1_E8M0, 5120, 2304)
    assert offs == [0, 17_694_720, 5_898_240, 18_063_360, 11_796_480, 18_432_000] and size == 18_800_640


def test_synthetic_quantizers_equal_the_oracle():
    w = synth.normal((256, 384), 0.02, 1)
    c, s = synth.quant_fp8_block(w)
    oc, os_ = orc.quant_weight_fp8_block(w.numpy())
    assert np.array_equal(c.numpy(), oc) and np.array_equal(s.numpy().view(np.uint32), os_.view(np.uint32))
    c4, s4, g = synth.quant_nvfp4(w)
    o4, os4, og = orc.quant_weight_nvfp4(w.numpy())
    assert np.array_equal(c4.numpy(), o4) and np.array_equal(s4.numpy(), os4) and g == og
    x = torch.linspace(-448, 448, 200001)
    tc = synth.e4m3_encode(x).numpy()
    L = orc.lib()
    for i in range(0, x.numel(), 389):
        assert L.orc_encode_e4m3(float(x[i])) == tc[i]
    ragged = synth.normal((130, 200), 0.02, 2)
    c, s = synth.quant_fp8_block(ragged)
    oc, os_ = orc.quant_weight_fp8_block(ragged.numpy())
    assert np.array_equal(c.numpy(), oc) and np.array_equal(s.numpy().view(np.uint32), os_.view(np.uint32))


@pytest.mark.parametrize("threads", [1, 3, 8])
def test_cpu_baseline_equals_the_scalar_oracle(threads):
    rng = np.random.default_rng(0)
    H, I, n = 1024, 512, 3
    x = orc.f32_to_bf16(rng.normal(size=(2, H)).astype(np.float32))
    exs = []
    for a in range(n):
        mats = []
        for shape in [(I, H), (I, H), (H, I)]:
            c, s = orc.quant_weight_fp8_block(rng.normal(scale=0.02, size=shape).astype(np.float32))
            mats += [c, s]
        exs.append(tuple(mats))
    rows, w, ap = [0, 1, 1], [0.5, 0.25, 1.0], [1, 1, 0]
    for boundary in (orc.AFTER_DOWN_BF16, orc.BEFORE_CONTRIBUTION_BF16):
        out = orc.CpuDecodeJob(x, rows, exs, w, ap, boundary).run(threads)
        for a in range(n):
            g, u, d = (orc.dequant_fp8_block(exs[a][i], exs[a][i + 1]) for i in (0, 2, 4))
            ref = orc.expert_ffn(x[rows[a]], g, u, d, w[a], orc.TWICE, 0.0, boundary, orc.LANE16, orc.SILU_RCP, apply_weight=bool(ap[a]))
            assert np.array_equal(ref, out[a])


def test_struct_layouts_match_the_c_header(tmp_path):
    """The ctypes mirrors in flyingfish_amd/capi.py (and with them the #[repr(C)] structs a Rust binding declares) must
    have the size and field offsets a C compiler gives the structs of include/ffmoe.h (reference: MoeDecode,
    src/backend/cuda/moe/decode.rs:26-44; MoePrefillContribute, src/backend/cuda/moe/prefill.rs:57-91)."""
    import ctypes
    import subprocess
    structs = {"ffmoe_expert_table": capi.ExpertTable, "ffmoe_shared_expert": capi.SharedExpert, "ffmoe_decode": capi.Decode,
               "ffmoe_prefill": capi.Prefill}
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "ffmoe.h"', 'int main(void) {']
    for cname, cls in structs.items():
        lines.append('  printf("%s size %%zu\\n", sizeof(%s));' % (cname, cname))
        for field, _ in cls._fields_:
            lines.append('  printf("%s %s %%zu\\n", offsetof(%s, %s));' % (cname, field, cname, field))
    lines += ['  return 0;', '}']
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    include = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", include, str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    seen = 0
    for line in out.splitlines():
        cname, what, value = line.split()
        cls = structs[cname]
        if what == "size":
            assert ctypes.sizeof(cls) == int(value), "%s: ctypes size %d, C size %s" % (cname, ctypes.sizeof(cls), value)
        else:
            assert getattr(cls, what).offset == int(value), "%s.%s: ctypes offset %d, C offset %s" % (cname, what, getattr(cls, what).offset, value)
        seen += 1
    assert seen == sum(len(c._fields_) + 1 for c in structs.values())
