"""Host-side operator objects over libffmoe, mirroring the reference's operator structs.

  RouteOps      <- src/backend/cuda/moe/route.rs   (RouteOps::route / logits_f32 / topk_noaux)
  ExpertTable   <- NativeMoe's slots[E,6] table    (src/backend/cuda/moe/decode.rs:683-698)
  DecodeOps     <- src/backend/cuda/moe/decode.rs  (DecodeOps::contribute*, decode_scratch_bytes_mixed)
  CombineOps    <- src/backend/cuda/moe/combine.rs (shared_scale, combine, combine_bf16, combine_accum, combine_routed)
  Fp8Ops / NvFp4Ops / skinny <- src/backend/cuda/linear.rs
  NativeMoe     <- decode.rs:771-777, :1187-1297   (route -> contribute -> combine for one layer)

Tensors are torch CUDA tensors used as plain device buffers; the ops own nothing except scratch.
Errors from the library are raised as capi.FfmoeError with the library's message.
"""
import ctypes

import torch

from . import capi

_BF16 = torch.bfloat16


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dense(t, name):
    if not t.is_contiguous():
        raise ValueError("%s must be dense row-major" % name)
    return t


class ExpertTable:
    """All experts of one layer, resident in device memory.

    FP8 block slot layout (src/experts/catalogue.rs:180-222): gate codes [I,H], up codes [I,H],
    down codes [H,I], then gate/up scales [ceil(I/128), ceil(H/128)] f32 and down scales
    [ceil(H/128), ceil(I/128)] f32. NVFP4 slot: packed codes then E4M3 group-16 scales, same order.
    FP8 per-channel slot (catalogue.rs:31-39, :54-61): the three code matrices, then BF16 scales [I], [I], [H].
    """

    def __init__(self, fmt, experts, hidden, inter, storage, slots, global_scales=None, valid=None):
        self.format, self.experts, self.hidden, self.inter = fmt, experts, hidden, inter
        self.storage, self.slots, self.global_scales, self.valid = storage, slots, global_scales, valid

    @staticmethod
    def slot_layout(fmt, hidden, inter):
        """byte offsets of {gate codes, gate scales, up codes, up scales, down codes, down scales} and slot size."""
        if fmt == capi.FMT_FP8_BLOCK128:
            w = hidden * inter
            sgu = -(-inter // 128) * -(-hidden // 128) * 4
            sd = -(-hidden // 128) * -(-inter // 128) * 4
            offs = [0, 3 * w, w, 3 * w + sgu, 2 * w, 3 * w + 2 * sgu]
            size = 3 * w + 2 * sgu + sd
        elif fmt == capi.FMT_NVFP4:
            w = hidden * inter // 2
            s = hidden * inter // 16
            offs = [0, 3 * w, w, 3 * w + s, 2 * w, 3 * w + 2 * s]
            size = 3 * w + 3 * s
        elif fmt == capi.FMT_FP8_CHANNEL:
            w = hidden * inter
            offs = [0, 3 * w, w, 3 * w + 2 * inter, 2 * w, 3 * w + 4 * inter]
            size = 3 * w + 4 * inter + 2 * hidden
        elif fmt == capi.FMT_E2M1_E8M0:
            w = hidden * inter // 2
            s = hidden * inter // 32
            offs = [0, 3 * w, w, 3 * w + s, 2 * w, 3 * w + 2 * s]
            size = 3 * w + 3 * s
        elif fmt == capi.FMT_E4M3_E8M0_32:
            w = hidden * inter
            sgu = -(-inter // 32) * (hidden // 32)
            sd = -(-hidden // 32) * (inter // 32)
            offs = [0, 3 * w, w, 3 * w + sgu, 2 * w, 3 * w + 2 * sgu]
            size = 3 * w + 2 * sgu + sd
        elif fmt == capi.FMT_BF16:
            w = hidden * inter * 2
            offs = [0, 0, w, 0, 2 * w, 0]
            size = 3 * w
        else:
            raise ValueError("unknown format")
        size = (size + 255) // 256 * 256
        return offs, size

    @classmethod
    def allocate(cls, fmt, experts, hidden, inter, device="cuda"):
        offs, size = cls.slot_layout(fmt, hidden, inter)
        storage = torch.empty((experts, size), dtype=torch.uint8, device=device)
        base = storage.data_ptr()
        table = torch.tensor([[base + e * size + o for o in offs] for e in range(experts)], dtype=torch.int64)
        slots = table.to(device)
        gs = torch.ones((experts, 3), dtype=torch.float32, device=device) if fmt == capi.FMT_NVFP4 else None
        t = cls(fmt, experts, hidden, inter, storage, slots, gs)
        t.offsets, t.slot_bytes = offs, size
        return t

    def expert_views(self, e):
        """(gate codes, gate scales, up codes, up scales, down codes, down scales) views of expert e."""
        H, I = self.hidden, self.inter
        row = self.storage[e]
        o = self.offsets
        if self.format == capi.FMT_FP8_BLOCK128:
            sgu = (-(-I // 128), -(-H // 128))
            sd = (-(-H // 128), -(-I // 128))
            f32 = lambda off, shape: row[off:off + shape[0] * shape[1] * 4].view(torch.float32).view(shape)
            return (row[o[0]:o[0] + I * H].view(I, H), f32(o[1], sgu), row[o[2]:o[2] + I * H].view(I, H), f32(o[3], sgu),
                    row[o[4]:o[4] + H * I].view(H, I), f32(o[5], sd))
        if self.format == capi.FMT_NVFP4:
            return (row[o[0]:o[0] + I * H // 2].view(I, H // 2), row[o[1]:o[1] + I * H // 16].view(I, H // 16),
                    row[o[2]:o[2] + I * H // 2].view(I, H // 2), row[o[3]:o[3] + I * H // 16].view(I, H // 16),
                    row[o[4]:o[4] + H * I // 2].view(H, I // 2), row[o[5]:o[5] + H * I // 16].view(H, I // 16))
        if self.format == capi.FMT_E2M1_E8M0:
            return (row[o[0]:o[0] + I * H // 2].view(I, H // 2), row[o[1]:o[1] + I * H // 32].view(I, H // 32),
                    row[o[2]:o[2] + I * H // 2].view(I, H // 2), row[o[3]:o[3] + I * H // 32].view(I, H // 32),
                    row[o[4]:o[4] + H * I // 2].view(H, I // 2), row[o[5]:o[5] + H * I // 32].view(H, I // 32))
        if self.format == capi.FMT_E4M3_E8M0_32:
            gi, gh = -(-I // 32), -(-H // 32)
            return (row[o[0]:o[0] + I * H].view(I, H), row[o[1]:o[1] + gi * (H // 32)].view(gi, H // 32),
                    row[o[2]:o[2] + I * H].view(I, H), row[o[3]:o[3] + gi * (H // 32)].view(gi, H // 32),
                    row[o[4]:o[4] + H * I].view(H, I), row[o[5]:o[5] + gh * (I // 32)].view(gh, I // 32))
        if self.format == capi.FMT_FP8_CHANNEL:
            sc = lambda off, n: row[off:off + n * 2].view(_BF16)
            return (row[o[0]:o[0] + I * H].view(I, H), sc(o[1], I), row[o[2]:o[2] + I * H].view(I, H), sc(o[3], I),
                    row[o[4]:o[4] + H * I].view(H, I), sc(o[5], H))
        bf = lambda off, shape: row[off:off + shape[0] * shape[1] * 2].view(_BF16).view(shape)
        return (bf(o[0], (I, H)), None, bf(o[2], (I, H)), None, bf(o[4], (H, I)), None)

    def weight_bytes_per_expert(self):
        H, I = self.hidden, self.inter
        if self.format == capi.FMT_FP8_BLOCK128:
            return 3 * H * I + 4 * (2 * -(-I // 128) * -(-H // 128) + -(-H // 128) * -(-I // 128))
        if self.format == capi.FMT_NVFP4:
            return 3 * H * I // 2 + 3 * H * I // 16 + 12
        if self.format == capi.FMT_FP8_CHANNEL:
            return 3 * H * I + 2 * (2 * I + H)
        if self.format == capi.FMT_E2M1_E8M0:
            return 3 * H * I // 2 + 3 * H * I // 32
        if self.format == capi.FMT_E4M3_E8M0_32:
            return 3 * H * I + 2 * -(-I // 32) * (H // 32) + -(-H // 32) * (I // 32)
        return 3 * H * I * 2

    def c_struct(self):
        gen = getattr(self, "generation", None)
        return capi.ExpertTable(self.format, self.experts, self.hidden, self.inter, self.slots.data_ptr(),
                                self.valid.data_ptr() if self.valid is not None else None,
                                self.global_scales.data_ptr() if self.global_scales is not None else None,
                                gen.data_ptr() if gen is not None else None)

    def shared_struct(self, e=0):
        """Describe expert e of this table as an always-on shared expert."""
        s = capi.SharedExpert()
        s.format, s.inter = self.format, self.inter
        row = self.slots[e].tolist()
        for i in range(6):
            s.slot[i] = row[i]
        gl = self.global_scales[e].tolist() if self.global_scales is not None else [1.0, 1.0, 1.0]
        for i in range(3):
            s.global_scales[i] = gl[i]
        return s


class RouteOps:
    @staticmethod
    def logits_bf16(x, router):
        rows, hidden = x.shape
        experts = router.shape[0]
        out = torch.empty((rows, experts), dtype=_BF16, device=x.device)
        capi.check(capi.lib().ffmoe_route_logits_bf16(_ptr(_dense(x, "x")), _ptr(_dense(router, "router")), _ptr(out), rows, experts, hidden, _stream()))
        return out

    @staticmethod
    def logits_f32(x, router, out=None):
        rows, hidden = x.shape
        experts = router.shape[0]
        if out is None:
            out = torch.empty((rows, experts), dtype=torch.float32, device=x.device)
        capi.check(capi.lib().ffmoe_route_logits_f32(_ptr(_dense(x, "x")), _ptr(_dense(router, "router")), _ptr(out), rows, experts, hidden, _stream()))
        return out

    @staticmethod
    def topk(logits, top_k, score=capi.SCORE_SOFTMAX):
        rows, experts = logits.shape
        ids = torch.empty((rows, top_k), dtype=torch.int32, device=logits.device)
        w = torch.empty((rows, top_k), dtype=_BF16, device=logits.device)
        capi.check(capi.lib().ffmoe_route_topk(_ptr(_dense(logits, "logits")), _ptr(ids), _ptr(w), rows, experts, top_k, score, _stream()))
        return ids, w

    @staticmethod
    def topk_noaux(logits, bias, top_k, score_mode=capi.NOAUX_SIGMOID, routed_scaling=1.0, n_group=1, topk_group=1,
                   weights_f32=True, out=None):
        rows, experts = logits.shape
        if out is None:
            ids = torch.empty((rows, top_k), dtype=torch.int32, device=logits.device)
            w = torch.empty((rows, top_k), dtype=torch.float32 if weights_f32 else _BF16, device=logits.device)
        else:
            ids, w = out
        stride = 0 if bias is None or bias.dim() == 1 else experts
        capi.check(capi.lib().ffmoe_route_topk_noaux(_ptr(_dense(logits, "logits")), _ptr(bias), stride, _ptr(ids), _ptr(w),
                                                     int(weights_f32), rows, experts, top_k, score_mode, routed_scaling,
                                                     n_group, topk_group, _stream()))
        return ids, w

    @staticmethod
    def route_noaux(x, router, bias, top_k, logits, ids, weights, done=None, score_mode=capi.NOAUX_SIGMOID,
                    routed_scaling=1.0, n_group=1, topk_group=1):
        """FP32 logits + noaux selection; clears `done` for the routed rows."""
        rows, hidden = x.shape
        experts = router.shape[0]
        stride = 0 if bias is None or bias.dim() == 1 else experts
        capi.check(capi.lib().ffmoe_route_noaux_decode(_ptr(x), _ptr(router), _ptr(bias), stride, _ptr(logits), _ptr(ids), _ptr(weights),
                                                       int(weights.dtype == torch.float32), _ptr(done), rows, experts,
                                                       hidden, top_k, score_mode, routed_scaling, n_group, topk_group, _stream()))
        return ids, weights

    @staticmethod
    def route(x, router, top_k, score=capi.SCORE_SOFTMAX, logits=None, ids=None, weights=None):
        rows, hidden = x.shape
        experts = router.shape[0]
        logits = logits if logits is not None else torch.empty((rows, experts), dtype=_BF16, device=x.device)
        ids = ids if ids is not None else torch.empty((rows, top_k), dtype=torch.int32, device=x.device)
        w = weights if weights is not None else torch.empty((rows, top_k), dtype=_BF16, device=x.device)
        capi.check(capi.lib().ffmoe_route_decode(_ptr(_dense(x, "x")), _ptr(_dense(router, "router")), _ptr(logits), _ptr(ids), _ptr(w),
                                                 rows, experts, hidden, top_k, score, _stream()))
        return ids, w, logits


class Residency:
    """Expert residency protocol over an ExpertTable (src/experts/arena.rs:220-483): publish / retire slots on the
    stream, mask a routing result against the table."""

    @staticmethod
    def publish(table, incoming, slot_addresses, epoch, victim=-1, status=None):
        arr = (capi.U64 * 6)(*[int(a) for a in slot_addresses])
        capi.check(capi.lib().ffmoe_slot_publish(table.slots.data_ptr(), table.valid.data_ptr(), table.generation.data_ptr(), table.experts,
                                                 incoming, victim, ctypes.byref(arr), epoch, _ptr(status), _stream()))

    @staticmethod
    def mask(table, ids, status=None):
        active = torch.empty(ids.shape, dtype=torch.int32, device=ids.device)
        gen = torch.empty(ids.shape, dtype=torch.int64, device=ids.device)
        capi.check(capi.lib().ffmoe_route_mask(_ptr(ids), table.valid.data_ptr(), table.generation.data_ptr(), _ptr(active), _ptr(gen),
                                               _ptr(status), ids.numel(), table.experts, _stream()))
        return active, gen


class DecodeOps:
    """Expert contributions for a decode batch; owns its scratch arena and output buffers."""

    def __init__(self, table, shared=None, rows=1, top_k=8, act_mode=capi.ACT_BF16, swiglu=capi.SWIGLU_TWICE, swiglu_limit=0.0,
                 routed_weight=capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=False):
        self.table, self.shared = table, shared
        self.rows, self.top_k = rows, top_k
        self.cfg = (act_mode, swiglu, swiglu_limit, routed_weight, int(weights_f32))
        dev = table.slots.device
        si = shared.inter if shared is not None else 0
        nbytes = capi.lib().ffmoe_decode_scratch_bytes(rows, max(top_k, 1), table.experts, table.hidden, table.inter, si)
        # zero-filled once: the one-launch token layer accepts an activation word of the arena only with its launch's
        # (non-zero) tag, which a cleared arena cannot hold
        self.scratch = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        self.contributions = torch.empty((rows, max(top_k, 1), table.hidden), dtype=_BF16, device=dev)
        self.shared_out = torch.empty((rows, table.hidden), dtype=_BF16, device=dev) if shared is not None else None
        self.done = torch.zeros((rows, top_k), dtype=torch.int32, device=dev)
        self._table_c = table.c_struct()
        self._shared_c = shared

    def contribute(self, x, ids, weights, active=None, stage=None, assignment_gen=None, form=None):
        """stage None = both launches; 0 / 1 = only the gate-up / only the down launch. form = capi.FORM_LANE16 /
        FORM_LANE8: the reference's own summation orders, bit-equal to its CPU path (DecodeOps::new_invariant_*)."""
        act_mode, swiglu, limit, rw, wf32 = self.cfg
        d = capi.Decode(self.rows, self.top_k, act_mode, swiglu, limit, rw, wf32,
                        x.data_ptr(), ids.data_ptr(), active.data_ptr() if active is not None else None, weights.data_ptr(),
                        self.contributions.data_ptr(), self.shared_out.data_ptr() if self.shared_out is not None else None,
                        self.done.data_ptr(), self.scratch.data_ptr(), self.scratch.numel(), _ptr(assignment_gen))
        sh = ctypes.byref(self._shared_c) if self._shared_c is not None else None
        if form is not None:
            capi.check(capi.lib().ffmoe_decode_contribute_form(ctypes.byref(self._table_c), sh, ctypes.byref(d), form, _stream()))
        elif stage is None:
            capi.check(capi.lib().ffmoe_decode_contribute(ctypes.byref(self._table_c), sh, ctypes.byref(d), _stream()))
        else:
            capi.check(capi.lib().ffmoe_decode_contribute_stage(ctypes.byref(self._table_c), sh, ctypes.byref(d), stage, _stream()))
        return self.contributions, self.shared_out

    def contribute_static(self, x, ids, weights, active=None):
        """contribute() through ffmoe_decode_contribute_static: the library's built-in per-GPU arena replaces
        self.scratch (for callers that cannot allocate); results are bit-identical to contribute()."""
        act_mode, swiglu, limit, rw, wf32 = self.cfg
        d = capi.Decode(self.rows, self.top_k, act_mode, swiglu, limit, rw, wf32,
                        x.data_ptr(), ids.data_ptr(), active.data_ptr() if active is not None else None, weights.data_ptr(),
                        self.contributions.data_ptr(), self.shared_out.data_ptr() if self.shared_out is not None else None,
                        self.done.data_ptr(), None, 0, None)
        sh = ctypes.byref(self._shared_c) if self._shared_c is not None else None
        capi.check(capi.lib().ffmoe_decode_contribute_static(ctypes.byref(self._table_c), sh, ctypes.byref(d), _stream()))
        return self.contributions, self.shared_out

    def contribute_from_logits(self, x, logits, bias, ids, weights, score_mode=capi.NOAUX_SIGMOID, routed_scaling=1.0, n_group=1, topk_group=1):
        """One token: top-k selection inside the gate/up launch; ids / weights (f32) are written. Returns None when the
        shape is outside the fast path (nothing launched)."""
        act_mode, swiglu, limit, rw, wf32 = self.cfg
        d = capi.Decode(self.rows, self.top_k, act_mode, swiglu, limit, rw, wf32,
                        x.data_ptr(), ids.data_ptr(), None, weights.data_ptr(),
                        self.contributions.data_ptr(), self.shared_out.data_ptr() if self.shared_out is not None else None,
                        self.done.data_ptr(), self.scratch.data_ptr(), self.scratch.numel(), None)
        sh = ctypes.byref(self._shared_c) if self._shared_c is not None else None
        rc = capi.lib().ffmoe_decode_contribute_from_logits(ctypes.byref(self._table_c), sh, ctypes.byref(d), _ptr(logits), _ptr(bias),
                                                            score_mode, routed_scaling, n_group, topk_group, _stream())
        if rc == capi.ERR_UNSUPPORTED:
            return None
        capi.check(rc)
        return self.contributions, self.shared_out

    def finish(self, x, ids, weights, mode, y, status=None, scale=None, active=None):
        """rows == 1: down + routing weight + ordered combine in one launch, after contribute(stage=0) on the same
        arguments. Returns False (nothing launched) when the shape is outside the fast path."""
        act_mode, swiglu, limit, rw, wf32 = self.cfg
        d = capi.Decode(self.rows, self.top_k, act_mode, swiglu, limit, rw, wf32,
                        x.data_ptr(), ids.data_ptr(), active.data_ptr() if active is not None else None, weights.data_ptr(),
                        self.contributions.data_ptr(), self.shared_out.data_ptr() if self.shared_out is not None else None,
                        self.done.data_ptr(), self.scratch.data_ptr(), self.scratch.numel(), None)
        sh = ctypes.byref(self._shared_c) if self._shared_c is not None else None
        rc = capi.lib().ffmoe_decode_finish(ctypes.byref(self._table_c), sh, ctypes.byref(d), _ptr(scale), _ptr(y), _ptr(status), mode, _stream())
        if rc == capi.ERR_UNSUPPORTED:
            return False
        capi.check(rc)
        return True

    def token_forward(self, x, ids, weights, mode, y, logits, bias=None, status=None, scale=None, score_mode=capi.NOAUX_SIGMOID,
                      routed_scaling=1.0, n_group=1, topk_group=1, stage=None):
        """rows == 1, two launches: selection in the prologue of the gate/up launch (ids / weights are outputs), then
        down + routing weight + ordered combine into y. stage 0 / 1 = one of the launches alone. Returns False (nothing
        launched) when the shape is outside the fast path."""
        act_mode, swiglu, limit, rw, wf32 = self.cfg
        d = capi.Decode(self.rows, self.top_k, act_mode, swiglu, limit, rw, wf32,
                        x.data_ptr(), ids.data_ptr(), None, weights.data_ptr(),
                        self.contributions.data_ptr(), self.shared_out.data_ptr() if self.shared_out is not None else None,
                        self.done.data_ptr(), self.scratch.data_ptr(), self.scratch.numel(), None)
        sh = ctypes.byref(self._shared_c) if self._shared_c is not None else None
        L = capi.lib()
        if stage is None:
            rc = L.ffmoe_decode_token_forward(ctypes.byref(self._table_c), sh, ctypes.byref(d), _ptr(logits), _ptr(bias), score_mode,
                                              routed_scaling, n_group, topk_group, _ptr(scale), _ptr(y), _ptr(status), mode, _stream())
        else:
            rc = L.ffmoe_decode_token_forward_stage(ctypes.byref(self._table_c), sh, ctypes.byref(d), _ptr(logits), _ptr(bias), score_mode,
                                                    routed_scaling, n_group, topk_group, _ptr(scale), _ptr(y), _ptr(status), mode, stage, _stream())
        if rc == capi.ERR_UNSUPPORTED:
            return False
        capi.check(rc)
        return True

    def token_layer(self, x, ids, weights, mode, y, status=None, scale=None, logits=None, bias=None, score_mode=capi.NOAUX_SIGMOID,
                    routed_scaling=1.0, n_group=1, topk_group=1, active=None):
        """rows == 1: selection (when logits are given; ids / weights are then outputs), gate/up, down, routing weight and
        the ordered combine in ONE launch. Returns False (nothing launched) when the shape is outside the fast path."""
        act_mode, swiglu, limit, rw, wf32 = self.cfg
        # an arena of its own: the launch recognises its activations by a 16-bit tag in the upper half of each word, and
        # the untagged BF16 activations the other entry points leave in self.scratch could pass for a tagged word
        if getattr(self, "token_scratch", None) is None:
            self.token_scratch = torch.zeros_like(self.scratch)
        d = capi.Decode(self.rows, self.top_k, act_mode, swiglu, limit, rw, wf32,
                        x.data_ptr(), ids.data_ptr(), active.data_ptr() if active is not None else None, weights.data_ptr(),
                        self.contributions.data_ptr(), self.shared_out.data_ptr() if self.shared_out is not None else None,
                        self.done.data_ptr(), self.token_scratch.data_ptr(), self.token_scratch.numel(), None)
        sh = ctypes.byref(self._shared_c) if self._shared_c is not None else None
        rc = capi.lib().ffmoe_decode_token_layer(ctypes.byref(self._table_c), sh, ctypes.byref(d), _ptr(logits), _ptr(bias), score_mode,
                                                 routed_scaling, n_group, topk_group, _ptr(scale), _ptr(y), _ptr(status), mode, _stream())
        if rc == capi.ERR_UNSUPPORTED:
            return False
        capi.check(rc)
        return True


class E8m0DecodeOps:
    """Expert contributions in the E8M0 block-32 contract (W4A8 routed experts, W8A8 32x32-block shared expert, exact
    integer dots). Host mirror of MoeExpertW4A8 / the W8A8 shared expert ops (src/backend/cuda/moe/w4a8.rs:248-420),
    for rows x top_k choices per call; owns its scratch arena and output buffers."""

    def __init__(self, table, shared=None, rows=1, top_k=8, swiglu_limit=10.0, exact=True):
        self.table, self.shared, self.rows, self.top_k, self.limit = table, shared, rows, top_k, swiglu_limit
        self.act_mode = capi.ACT_E4M3_E8M0_32 if exact else capi.ACT_E4M3_E8M0_32_F32
        dev = table.slots.device
        si = shared.inter if shared is not None else 0
        nbytes = capi.lib().ffmoe_e8m0_scratch_bytes(rows, top_k, table.hidden, table.inter, si)
        self.scratch = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        self.contributions = torch.empty((rows, max(top_k, 1), table.hidden), dtype=_BF16, device=dev)
        self.shared_out = torch.empty((rows, table.hidden), dtype=_BF16, device=dev) if shared is not None else None
        self.done = torch.zeros((rows, max(top_k, 1)), dtype=torch.int32, device=dev)
        self._table_c = table.c_struct()
        self._shared_c = shared

    def contribute(self, x, ids, weights, active=None):
        d = capi.Decode(self.rows, self.top_k, self.act_mode, capi.SWIGLU_CLAMPED_ONCE, self.limit, capi.WEIGHT_BEFORE_DOWN_F32, 1,
                        x.data_ptr(), ids.data_ptr(), active.data_ptr() if active is not None else None, weights.data_ptr(),
                        self.contributions.data_ptr(), self.shared_out.data_ptr() if self.shared_out is not None else None,
                        self.done.data_ptr(), self.scratch.data_ptr(), self.scratch.numel(), None)
        sh = ctypes.byref(self._shared_c) if self._shared_c is not None else None
        capi.check(capi.lib().ffmoe_decode_contribute_e8m0(ctypes.byref(self._table_c), sh, ctypes.byref(d), _stream()))
        return self.contributions, self.shared_out

    @staticmethod
    def act_quant(x):
        rows, k = x.shape
        codes = torch.empty((rows, k), dtype=torch.uint8, device=x.device)
        scales = torch.empty((rows, k // 32), dtype=torch.uint8, device=x.device)
        capi.check(capi.lib().ffmoe_act_quant_e8m0(_ptr(_dense(x, "x")), _ptr(codes), _ptr(scales), rows, k, _stream()))
        return codes, scales


class PrefillOps:
    """Expert contributions for a prefill cohort (many rows): device-side grouping by expert and two grouped W8A8
    GEMMs. Host mirror of PrefillOps::prefill_contribute (src/backend/cuda/moe/prefill.rs:1033-1408); owns its scratch
    arena and the contributions / done buffers."""

    def __init__(self, table, rows, top_k, swiglu=capi.SWIGLU_TWICE, swiglu_limit=0.0,
                 routed_weight=capi.WEIGHT_AFTER_DOWN_BF16, weights_f32=True, shared=None, act_mode=capi.ACT_FP8_BLOCK128):
        """act_mode ACT_FP8_BLOCK128: W8A8 on the FP8 matrix cores (block-FP8 experts); ACT_BF16: the decode path's
        W*A16 arithmetic on the BF16 matrix cores, experts of any format."""
        self.table = table
        self.rows, self.top_k = rows, top_k
        self.act_mode = act_mode
        self.cfg = (swiglu, swiglu_limit, routed_weight, int(weights_f32))
        dev = table.slots.device
        si = shared.inter if shared is not None else 0
        nbytes = capi.lib().ffmoe_prefill_scratch_bytes(rows, top_k, table.experts, table.hidden, table.inter, si)
        self.scratch = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        self.contributions = torch.empty((rows, top_k, table.hidden), dtype=_BF16, device=dev)
        self.shared_out = torch.empty((rows, table.hidden), dtype=_BF16, device=dev) if shared is not None else None
        self.done = torch.zeros((rows, top_k), dtype=torch.int32, device=dev)
        self._table_c = table.c_struct()
        self._shared_c = shared

    def scratch_views(self):
        """The arena regions a caller may inspect after contribute(): same offsets as prefill_layout() in
        csrc/prefill.hip (every region rounded up to 256 bytes). act[pos] is the BF16 SwiGLU output of the assignment
        perm[pos]; offsets[e]..offsets[e+1] is expert e's segment; totals[3] is the number of live assignments."""
        return PrefillOps.arena_views(self.scratch, self.table, self.rows, self.top_k, self._shared_c)

    @staticmethod
    def arena_views(scratch, table, rows, top_k, shared):
        """scratch_views() of any arena a cohort call laid out, e.g. the scratch of a DecodeOps whose batch
        ffmoe_decode_contribute handed to the cohort kernels."""
        t = table
        R, K, E, H, I = rows, top_k, t.experts, t.hidden, t.inter
        A = R * K
        off = 0
        out = {}

        def take(name, nbytes, dtype, shape):
            nonlocal off
            out[name] = scratch[off:off + nbytes].view(dtype).view(shape)
            off += (nbytes + 255) // 256 * 256
        take("xq", R * H, torch.uint8, (R, H))
        take("sx", R * (H // 128) * 4, torch.float32, (R, H // 128))
        take("act", A * I * 2, _BF16, (A, I))
        take("aq", A * I, torch.uint8, (A, I))
        take("sa", A * (I // 128) * 4, torch.float32, (A, I // 128))
        take("counts", E * 4, torch.int32, (E,))
        take("offsets", (E + 1) * 4, torch.int32, (E + 1,))
        take("gbase", (E + 1) * 4, torch.int32, (E + 1,))
        take("totals", 16, torch.int32, (4,))
        take("perm", A * 4, torch.int32, (A,))
        if shared is not None:
            SI = shared.inter
            max_groups = E + (A + 15) // 16 + (R + 15) // 16
            take("groups", max_groups * 16, torch.uint8, (max_groups * 16,))
            take("units0", max_groups * (-(-I // 128)) * 8, torch.uint8, (-1,))
            take("units1", max_groups * (-(-H // 256)) * 8, torch.uint8, (-1,))
            take("sh_act", R * SI * 2, _BF16, (R, SI))
            take("sh_aq", R * SI, torch.uint8, (R, SI))
            take("sh_sa", R * (SI // 128) * 4, torch.float32, (R, SI // 128))
        return out

    def contribute(self, x, ids, weights, active=None, stage=None, assignment_gen=None):
        """stage None = the whole call; 0..3 = one step (plan, gate/up, re-quantize, down)."""
        swiglu, limit, rw, wf32 = self.cfg
        a = capi.Prefill(self.rows, self.top_k, self.act_mode, swiglu, limit, rw, wf32,
                         x.data_ptr(), ids.data_ptr(), active.data_ptr() if active is not None else None, weights.data_ptr(),
                         self.contributions.data_ptr(), self.done.data_ptr(), self.scratch.data_ptr(), self.scratch.numel(),
                         ctypes.pointer(self._shared_c) if self._shared_c is not None else None,
                         self.shared_out.data_ptr() if self.shared_out is not None else None, _ptr(assignment_gen))
        if stage is None:
            capi.check(capi.lib().ffmoe_prefill_contribute(ctypes.byref(self._table_c), ctypes.byref(a), _stream()))
        else:
            capi.check(capi.lib().ffmoe_prefill_contribute_stage(ctypes.byref(self._table_c), ctypes.byref(a), stage, _stream()))
        return self.contributions


class CombineOps:
    @staticmethod
    def shared_scale(x, seg):
        rows, hidden = x.shape
        out = torch.empty((rows,), dtype=_BF16, device=x.device)
        capi.check(capi.lib().ffmoe_shared_scale(_ptr(x), _ptr(seg), _ptr(out), rows, hidden, _stream()))
        return out

    @staticmethod
    def combine(contributions, shared_out, ids, mode, scale=None, done=None, final_active=None, status=None, out=None):
        rows, top_k, hidden = contributions.shape
        y = out if out is not None else torch.empty((rows, hidden), dtype=_BF16, device=contributions.device)
        capi.check(capi.lib().ffmoe_combine(_ptr(contributions), _ptr(shared_out), _ptr(scale), _ptr(ids), _ptr(done),
                                            _ptr(final_active), _ptr(y), _ptr(status), rows, top_k, hidden, mode, _stream()))
        return y


    @staticmethod
    def combine_residual(shared_out, residual=None, y_out=None, contributions=None, routed_in=None, ids=None, seg=None, x=None,
                         done=None, final_active=None, status=None):
        """ff = bf16(bf16(routed) + gated); y_out = ff, or residual += ff in place (combine_residual / join_routed_residual)."""
        rows, hidden = shared_out.shape
        top_k = contributions.shape[1] if contributions is not None else 1
        x_stride = x.stride(0) if x is not None else hidden
        capi.check(capi.lib().ffmoe_combine_residual(_ptr(contributions), _ptr(routed_in), _ptr(shared_out), _ptr(seg), _ptr(x), x_stride,
                                                     _ptr(ids), _ptr(done), _ptr(final_active), _ptr(residual), _ptr(y_out), _ptr(status),
                                                     rows, top_k, hidden, _stream()))
        return y_out if y_out is not None else residual


class Fp8Ops:
    @staticmethod
    def quantize(x):
        m, k = x.shape
        codes = torch.empty((m, k), dtype=torch.uint8, device=x.device)
        scales = torch.empty((m, -(-k // 128)), dtype=torch.float32, device=x.device)
        capi.check(capi.lib().ffmoe_quant_fp8_f32_128(_ptr(x), _ptr(codes), _ptr(scales), m, k, _stream()))
        return codes, scales

    @staticmethod
    def linear(w_codes, w_scales, x, act_mode=capi.ACT_BF16, out=None):
        n, k = w_codes.shape
        m = x.shape[0]
        y = out if out is not None else torch.empty((m, n), dtype=_BF16, device=x.device)
        scratch = None
        nbytes = 0
        if act_mode == capi.ACT_FP8_BLOCK128:
            nbytes = (m * k + 255) // 256 * 256 + m * -(-k // 128) * 4
            scratch = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        capi.check(capi.lib().ffmoe_linear_fp8_block(_ptr(w_codes), _ptr(w_scales), _ptr(x), _ptr(y), m, n, k, act_mode,
                                                     _ptr(scratch), nbytes, _stream()))
        return y

    @staticmethod
    def linear_batch_items(weights, xs, ys):
        """Device descriptor array for linear_batch: weights = [(codes, scales), ...], xs / ys = matching BF16 tensors."""
        rows = [[c.data_ptr(), s.data_ptr(), x.data_ptr(), y.data_ptr()] for (c, s), x, y in zip(weights, xs, ys)]
        return torch.tensor(rows, dtype=torch.int64).to(xs[0].device)

    @staticmethod
    def linear_batch(items, m, n, k):
        """All items (descriptor array from linear_batch_items) in one launch; m <= 4 activation rows each."""
        capi.check(capi.lib().ffmoe_linear_fp8_block_batch(_ptr(items), items.shape[0], m, n, k, _stream()))

    @staticmethod
    def linear_w8a8(w_codes, w_scales, x_codes, x_scales, out=None):
        n, k = w_codes.shape
        m = x_codes.shape[0]
        y = out if out is not None else torch.empty((m, n), dtype=_BF16, device=x_codes.device)
        capi.check(capi.lib().ffmoe_linear_fp8_block_w8a8(_ptr(w_codes), _ptr(w_scales), _ptr(x_codes), _ptr(x_scales), _ptr(y), m, n, k, _stream()))
        return y


class NvFp4Ops:
    @staticmethod
    def gemm(codes, scales, global_scale, x, out=None):
        n, kh = codes.shape
        k = kh * 2
        m = x.shape[0]
        y = out if out is not None else torch.empty((m, n), dtype=_BF16, device=x.device)
        capi.check(capi.lib().ffmoe_linear_nvfp4(_ptr(codes), _ptr(scales), _ptr(global_scale), _ptr(x), _ptr(y), m, n, k, _stream()))
        return y


def gemm_skinny_bf16(w, x, out=None):
    n, k = w.shape
    m = x.shape[0]
    y = out if out is not None else torch.empty((m, n), dtype=_BF16, device=x.device)
    capi.check(capi.lib().ffmoe_gemm_skinny_bf16(_ptr(w), _ptr(x), _ptr(y), m, n, k, _stream()))
    return y


def swiglu(gate, up, mode=capi.SWIGLU_TWICE, limit=0.0):
    rows, width = gate.shape
    y = torch.empty_like(gate)
    capi.check(capi.lib().ffmoe_swiglu(_ptr(gate), _ptr(up), _ptr(y), rows, width, mode, limit, _stream()))
    return y


class NativeMoe:
    """One MoE layer, decode: FP32 router logits -> noaux top-k -> expert contributions -> combine.

    Mirrors NativeMoe::new / run (decode.rs:683-698, :771-777, :1187-1297): geometry {hidden, intermediate, experts,
    top_k, scaling, limit}, weights {router, bias, slots, shared}, fixed row count, run(x) -> y.
    """

    def __init__(self, table, shared, router, bias, rows, top_k, routed_scaling=1.0, n_group=1, topk_group=1,
                 swiglu=capi.SWIGLU_TWICE, swiglu_limit=0.0, routed_weight=capi.WEIGHT_BEFORE_CONTRIBUTION_BF16,
                 combine_mode=capi.COMBINE_BF16):
        self.table, self.router, self.bias = table, router, bias
        self.rows, self.top_k = rows, top_k
        self.routing = (routed_scaling, n_group, topk_group)
        self.combine_mode = combine_mode
        dev = router.device
        self.decode = DecodeOps(table, shared, rows, top_k, capi.ACT_BF16, swiglu, swiglu_limit, routed_weight, weights_f32=True)
        self.logits = torch.empty((rows, table.experts), dtype=torch.float32, device=dev)
        self.ids = torch.empty((rows, top_k), dtype=torch.int32, device=dev)
        self.weights = torch.empty((rows, top_k), dtype=torch.float32, device=dev)
        self.y = torch.empty((rows, table.hidden), dtype=_BF16, device=dev)
        self.status = torch.zeros(1, dtype=torch.int32, device=dev)
        # one-token finish in a single launch (ffmoe_decode_finish). Off by default: on MI355X it measured 33 us
        # against 26 + 4.6 us for the separate down and combine launches at the DeepSeek-V3 shape.
        self.fused_finish = False
        # one token: run the top-k selection in the prologue of the gate/up launch (one launch less)
        self.inline_select = True
        # one token: selection + gate/up, then down + combine (ffmoe_decode_token_forward): three launches per layer with
        # the logits. contributions / shared_out / done are not written on this path; set False to get them.
        self.two_launch = True
        # one token: everything after the logits in one resident launch (ffmoe_decode_token_layer). Off by default: on
        # MI355X at the DeepSeek-V3 shape it measured 91 us against 79 us for the three launches it replaces.
        self.one_launch = False

    def run(self, x):
        scaling, ng, kg = self.routing
        if self.rows == 1 and self.one_launch:
            # one token: logits launch, then selection, gate/up, down and combine in one resident launch
            RouteOps.logits_f32(x, self.router, out=self.logits)
            mode = self.combine_mode if self.decode.shared_out is not None else capi.COMBINE_ROUTED
            if self.decode.token_layer(x, self.ids, self.weights, mode, self.y, status=self.status, logits=self.logits,
                                       bias=self.bias if self.bias.dim() == 1 else self.bias[0],
                                       routed_scaling=scaling, n_group=ng, topk_group=kg):
                return self.y
            self.one_launch = False
        if self.rows == 1 and self.two_launch:
            RouteOps.logits_f32(x, self.router, out=self.logits)
            mode = self.combine_mode if self.decode.shared_out is not None else capi.COMBINE_ROUTED
            if self.decode.token_forward(x, self.ids, self.weights, mode, self.y, self.logits, bias=self.bias if self.bias.dim() == 1 else self.bias[0],
                                         status=self.status, routed_scaling=scaling, n_group=ng, topk_group=kg):
                return self.y
            self.two_launch = False
        if self.rows == 1 and self.inline_select:
            # one token: logits launch, then gate/up with the selection in its prologue, down, combine (4 launches)
            RouteOps.logits_f32(x, self.router, out=self.logits)
            got = self.decode.contribute_from_logits(x, self.logits, self.bias if self.bias.dim() == 1 else self.bias[0], self.ids, self.weights,
                                                     routed_scaling=scaling, n_group=ng, topk_group=kg)
            if got is not None:
                contrib, shared_out = got
                mode = self.combine_mode if shared_out is not None else capi.COMBINE_ROUTED
                return CombineOps.combine(contrib, shared_out, self.ids, mode, done=self.decode.done, status=self.status, out=self.y)
            self.inline_select = False
        RouteOps.route_noaux(x, self.router, self.bias, self.top_k, self.logits, self.ids, self.weights,
                             done=self.decode.done, routed_scaling=scaling, n_group=ng, topk_group=kg)
        if self.rows == 1 and self.fused_finish:
            # one token: gate/up launch, then down + weighting + combine in a single launch
            self.decode.contribute(x, self.ids, self.weights, stage=0)
            mode = self.combine_mode if self.decode.shared_out is not None else capi.COMBINE_ROUTED
            if self.decode.finish(x, self.ids, self.weights, mode, self.y, status=self.status):
                return self.y
            self.fused_finish = False
            contrib, shared_out = self.decode.contribute(x, self.ids, self.weights, stage=1)
        else:
            contrib, shared_out = self.decode.contribute(x, self.ids, self.weights)
        mode = self.combine_mode if shared_out is not None else capi.COMBINE_ROUTED
        return CombineOps.combine(contrib, shared_out, self.ids, mode, done=self.decode.done, status=self.status, out=self.y)
