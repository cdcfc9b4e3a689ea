"""The model's step as one native call (csrc/step_plan.hip, interface in csrc/step_plan_api.h).

When a model is bound, every block lays its parts down in a `NativePlan` (`Block.emit`): norms and bodies
(mixers, feed-forwards) with their weights, sizes and constants, as raw pointers that the parts keep
alive, and a program of operations that says how the block arranges them.  A step is then one call
into the library, which queues every kernel, whatever their number; every choice of a kernel for a
shape is made there and nowhere else.

Parts that the package brings are native.  A part from elsewhere (a class registered by a test or
another architecture, written with tensor operations) needs nothing but its `forward`: the base
classes lay it down as a callback that the native step calls with the rows it is to read and the
buffer it is to fill.  A part alone (`Mixer.forward`, `Norm.forward`, `Block.forward` of the built-in
parts) runs through a small plan of its own, so it takes the code that a whole step takes.
"""
from __future__ import annotations

import ctypes
from ctypes import CFUNCTYPE, POINTER, c_int, c_long, c_void_p
from typing import Callable, List, Optional

import torch

from ..ops import lib as L
from ..ops.lib import KernelError


class StepArgs(ctypes.Structure):
    """GibbsStepArgs of csrc/step_plan_api.h."""
    _fields_ = [("ids", c_void_p), ("pos", c_void_p), ("row_req", c_void_p), ("cu", c_void_p), ("ctx", c_void_p),
                ("slot", c_void_p), ("logit_rows", c_void_p), ("tables", POINTER(c_void_p)), ("widths", POINTER(c_int)),
                ("n_groups", c_int), ("n_rows", c_int), ("n_req", c_int), ("n_logits", c_int), ("max_q", c_int),
                ("max_seq", c_int), ("lead_single", c_int), ("workspace", c_void_p), ("workspace_bytes", c_long),
                ("logits", c_void_p), ("stream", c_void_p), ("x_in", c_void_p), ("mirror_in", c_void_p),
                ("first_op", c_int), ("n_ops", c_int), ("settle", c_int)]


class DeltaSpec(ctypes.Structure):
    """GibbsDeltaSpec of csrc/step_plan_api.h."""
    _fields_ = [("w_in", c_void_p), ("w_out", c_void_p), ("w_a2", c_void_p), ("w_g2", c_void_p),
                ("taps", c_void_p), ("dt_bias", c_void_p), ("a_log", c_void_p), ("gain", c_void_p),
                ("conv_state", c_void_p), ("rule_state", c_void_p), ("slot_stride", c_long),
                ("in_rows", c_int), ("heads", c_int), ("kv_heads", c_int), ("dim", c_int), ("vdim", c_int),
                ("taps_per_channel", c_int), ("off_b", c_int), ("off_a", c_int), ("off_g", c_int), ("a_rank", c_int),
                ("g_rank", c_int), ("eps", ctypes.c_float), ("unit_eps", ctypes.c_float), ("q_scale", ctypes.c_float)]


class TimeMixSpec(ctypes.Structure):
    """GibbsTimeMixSpec of csrc/step_plan_api.h."""
    _fields_ = [("w_r", c_void_p), ("w_k", c_void_p), ("w_v", c_void_p), ("w_g", c_void_p), ("w_1", c_void_p), ("w_2", c_void_p),
                ("w_out", c_void_p), ("mu", c_void_p), ("w0", c_void_p), ("bonus", c_void_p), ("gain", c_void_p),
                ("shift_state", c_void_p), ("rule_state", c_void_p), ("slot_stride", c_long),
                ("heads", c_int), ("dim", c_int), ("rank", c_int), ("eps", ctypes.c_float)]


class LatentSpec(ctypes.Structure):
    """GibbsLatentSpec of csrc/step_plan_api.h."""
    _fields_ = [("w_in", c_void_p), ("w_uq", c_void_p), ("w_uk_t", c_void_p), ("w_uv", c_void_p), ("w_out", c_void_p),
                ("q_gain", c_void_p), ("kv_gain", c_void_p), ("sink", c_void_p), ("inv_freq", c_void_p), ("pages", c_void_p),
                ("in_rows", c_int), ("heads", c_int), ("dim", c_int), ("rot", c_int), ("vdim", c_int), ("rank", c_int),
                ("q_rank", c_int), ("rot_dims", c_int), ("variant", c_int), ("window", c_int), ("off_kv", c_int), ("off_g", c_int),
                ("num_pages", c_int), ("page_size", c_int), ("group", c_int), ("scale", ctypes.c_float), ("eps", ctypes.c_float)]


class SsdSpec(ctypes.Structure):
    """GibbsSsdSpec of csrc/step_plan_api.h."""
    _fields_ = [("w_in", c_void_p), ("w_out", c_void_p), ("taps", c_void_p), ("conv_bias", c_void_p), ("dt_bias", c_void_p),
                ("a_log", c_void_p), ("skip", c_void_p), ("gain", c_void_p), ("conv_state", c_void_p), ("rule_state", c_void_p),
                ("slot_stride", c_long), ("heads", c_int), ("vdim", c_int), ("state", c_int), ("groups", c_int),
                ("taps_per_channel", c_int), ("norm_groups", c_int), ("eps", ctypes.c_float)]


class MoeSpec(ctypes.Structure):
    """GibbsMoeSpec of csrc/step_plan_api.h."""
    _fields_ = [("router", c_void_p), ("router_bias", c_void_p), ("gate", c_void_p), ("up", c_void_p), ("down", c_void_p),
                ("shared_gate_up", c_void_p), ("shared_down", c_void_p), ("shared_gate", c_void_p),
                ("experts", c_int), ("top", c_int), ("F", c_int), ("act", c_int), ("shared_F", c_int), ("shared_act", c_int)]


HOST_BODY = CFUNCTYPE(c_int, c_void_p, POINTER(StepArgs), c_void_p, c_void_p)
HOST_NORM = CFUNCTYPE(c_int, c_void_p, POINTER(StepArgs), c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p)
HOST_ROWS = CFUNCTYPE(c_int, c_void_p, POINTER(StepArgs), c_void_p, c_long)


def _ptr(t) -> Optional[int]:
    """Device address of a tensor (or of a packed matrix's tiles), None for None."""
    return None if t is None else t.data_ptr()


def declare(lib) -> None:
    """Argument and result types of the plan's entry points."""
    P, I, F, LG = c_void_p, c_int, ctypes.c_float, c_long
    sigs = {
        "gibbs_plan_create": ([I, I, I, P, I, P, P, I, I], P),
        "gibbs_plan_destroy": ([P], None),
        "gibbs_plan_norm_rms": ([P, P, F], I),
        "gibbs_plan_norm_host": ([P, HOST_NORM, P], I),
        "gibbs_plan_body_conv": ([P, P, P, P, P, P, P, I, I, P, LG], I),
        "gibbs_plan_body_attention": ([P, P, P, P, P, I, I, I, F, I, P, P, F, P, I, I, P, I, P, P, I, I, I, I, P, HOST_ROWS, P], I),
        "gibbs_plan_body_glu": ([P, P, P, P, P, I, I], I),
        "gibbs_plan_body_host": ([P, HOST_BODY, P, I], I),
        "gibbs_plan_embedding": ([P, F, P], I),
        "gibbs_plan_attention_extras": ([P, I, I, I, I, F, I, P, P, I], I),
        "gibbs_plan_glu_clamped": ([P, I, F, F], I),
        "gibbs_plan_attention_projection": ([P, I, I, P, P, I, I, I, P], I),
        "gibbs_plan_body_moe": ([P, POINTER(MoeSpec)], I),
        "gibbs_plan_body_delta": ([P, POINTER(DeltaSpec)], I),
        "gibbs_plan_body_time_mix": ([P, POINTER(TimeMixSpec)], I),
        "gibbs_plan_norm_layer": ([P, P, P, F], I),
        "gibbs_plan_norm_group_rms": ([P, P, F, I], I),
        "gibbs_plan_attention_gated": ([P, I, P, P, F, I, I, P, I, I, F, I], I),
        "gibbs_plan_body_conv_input": ([P, P, I, P, LG], I),
        "gibbs_plan_body_ssd": ([P, POINTER(SsdSpec)], I),
        "gibbs_plan_logit_softcap": ([P, F], I),
        "gibbs_plan_moe_scores": ([P, I, I, I], I),
        "gibbs_plan_op_rows": ([P, I, I], I),
        "gibbs_plan_body_latent": ([P, POINTER(LatentSpec)], I),
        "gibbs_plan_body_mlp": ([P, P, P, I, P, F], I),
        "gibbs_plan_streams": ([P, I], I),
        "gibbs_plan_hyper": ([P, P, P, P], I),
        "gibbs_plan_embedding_tables": ([P, P, I, I, I, P, I, P, LG], I),
        "gibbs_plan_op_streams_norm": ([P, I, I], I),
        "gibbs_plan_op_streams_add": ([P, I, I], I),
        "gibbs_plan_op_norm_delta": ([P, I, I], I),
        "gibbs_plan_op_add_normed": ([P, I, I], I),
        "gibbs_plan_op_reinject": ([P], I),
        "gibbs_plan_op_half": ([P, I, I], I),
        "gibbs_plan_op_norm": ([P, I], I),
        "gibbs_plan_op_body": ([P, I, I], I),
        "gibbs_plan_op_add": ([P, I], I),
        "gibbs_plan_op_drop": ([P, I], I),
        "gibbs_plan_tail": ([P, I], I),
        "gibbs_plan_op_count": ([P], I),
        "gibbs_plan_workspace": ([P, P], LG),
        "gibbs_plan_step": ([P, P], I),
        "gibbs_plan_last_fused": ([P], I),
        "gibbs_plan_body_forward": ([P, I, P, P, POINTER(LG), POINTER(I)], LG),
        "gibbs_plan_norm_forward": ([P, I, P, P, P, I, P, I, POINTER(LG)], LG),
    }
    for name, (argtypes, restype) in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes, fn.restype = argtypes, restype


class _MinimalBatch:
    """The operands of a part that is run alone without a batch (a feed-forward reads none of them)."""
    def __init__(self, n_rows: int):
        self.n_rows, self.n_req, self.n_logits, self.max_q, self.max_seq, self.lead_single = n_rows, 0, 0, 0, 0, 0
        self.ids = self.pos = self.row_req = self.cu = self.ctx = self.slot = self.logit_rows = None
        self.tables = []


class NativePlan:
    """A plan under construction and, once built, the thing that steps."""

    def __init__(self, rt, hidden: int, vocab: int = 0, table: Optional[torch.Tensor] = None,
                 head: Optional[torch.Tensor] = None, head_packed=None):
        from ..ops import linear as lin
        self.rt, self.hidden, self.vocab, self.device = rt, hidden, vocab, rt.device
        lib = L.library()
        self.handle = lib.gibbs_plan_create(L.dtype_code(rt.act_dtype), int(hidden), int(vocab), _ptr(table),
                                            L.dtype_code(table.dtype) if table is not None else 0, _ptr(head),
                                            _ptr(head_packed), int(rt.fused_decode_rows), int(not lin.USE_LIBRARY_GEMM))
        if not self.handle:
            raise KernelError(lib.gibbs_last_error().decode(errors="replace"))
        self.keep: List = [table, head, head_packed]      # what the plan holds addresses of
        self._callbacks: List = []                         # ctypes thunks must outlive the plan
        self._arena: Optional[torch.Tensor] = None
        self._args = StepArgs()
        self._tables = self._widths = None
        # what a callback finds while a step is being queued
        self.batch = None
        self._workspace: Optional[torch.Tensor] = None
        self._x_in: Optional[torch.Tensor] = None
        self._error: Optional[BaseException] = None
        # the rows of a step are the table's rows and nothing else (a caller may then bring them itself, `x_in`)
        self.plain_embedding = True

    def __del__(self):
        if getattr(self, "handle", None):
            try:
                L.library().gibbs_plan_destroy(self.handle)
            except TypeError:              # (the interpreter is shutting down: the module is gone already)
                pass
            self.handle = None

    # ------------------------------------------------------------------ building: parts
    def _made(self, index: int) -> int:
        if index < 0:
            raise KernelError(L.library().gibbs_last_error().decode(errors="replace"))
        return index

    def _held(self, *tensors):
        self.keep += [t for t in tensors if t is not None]
        return [_ptr(t) for t in tensors]

    def rms_norm(self, gain: Optional[torch.Tensor], eps: float) -> int:
        (g,) = self._held(gain)
        return self._made(L.library().gibbs_plan_norm_rms(self.handle, g, float(eps)))

    def group_rms_norm(self, gain: torch.Tensor, eps: float, groups: int) -> int:
        """RMS norm in `groups` equal consecutive parts of the row, the gain over the whole row."""
        (g,) = self._held(gain)
        return self._made(L.library().gibbs_plan_norm_group_rms(self.handle, g, float(eps), int(groups)))

    def layer_norm(self, gain: Optional[torch.Tensor], bias: Optional[torch.Tensor], eps: float) -> int:
        g, b = self._held(gain, bias)
        return self._made(L.library().gibbs_plan_norm_layer(self.handle, g, b, float(eps)))

    def host_norm(self, forward: Callable) -> int:
        """A norm written with tensor operations: `forward(x, delta, rows, n_rows) -> normed rows` (the
        interface of `Norm.forward`)."""
        def thunk(_user, step, x_ptr, delta_ptr, delta_parts, rows_ptr, n_out, out_ptr):
            try:
                a = step.contents
                x = self._tensor(x_ptr, (a.n_rows, self.hidden), torch.float32)
                delta = None
                if delta_ptr:
                    delta = (self._tensor(delta_ptr, (delta_parts, a.n_rows, self.hidden), torch.float32) if delta_parts >= 2
                             else self._tensor(delta_ptr, (a.n_rows, self.hidden), self.rt.act_dtype))
                rows = self.batch.logit_rows if rows_ptr else None
                out = self._tensor(out_ptr, (n_out, self.hidden), self.rt.act_dtype)
                out.copy_(forward(x, delta, rows, n_out if rows_ptr else None))
                return 0
            except BaseException as exc:            # an exception cannot cross the native frames: it is raised after the call
                self._error = exc
                return 1
        cb = HOST_NORM(thunk)
        self._callbacks.append(cb)
        return self._made(L.library().gibbs_plan_norm_host(self.handle, cb, None))

    def short_conv(self, *, w_in, p_in, w_out, p_out, taps, bias, width: int, kernel: int, state) -> int:
        assert state.dtype == torch.float32 and state.stride(2) == 1 and state.stride(1) == width
        ptrs = self._held(w_in, p_in, w_out, p_out, taps, bias)
        self.keep.append(state)
        return self._made(L.library().gibbs_plan_body_conv(self.handle, *ptrs, int(width), int(kernel), state.data_ptr(),
                                                           int(state.stride(0))))

    def attention(self, *, w_qkv, p_qkv, w_out, p_out, heads: int, kv_heads: int, head_dim: int, scale: float, window,
                  q_gain, k_gain, qk_eps: float, rotation, kpages, vpages, group: int, owns: bool, slopes=None,
                  rows_hook: Optional[Callable] = None) -> int:
        """`rows_hook(q, k, batch)`: changes the step's q [N, heads, head_dim] and k [N, kv_heads, head_dim]
        (None for a mixer that reads another's cache) in place, after the q/k norm and before k is cached."""
        from ..ops import ROPE_VARIANTS
        inv_freq = cos_sin = None
        rot = variant = table_len = 0
        if rotation is not None:
            inv_freq, cos_sin, rot = rotation.inv_freq, rotation.cos_sin, int(rotation.rotary_dim)
            variant = ROPE_VARIANTS[rotation.variant]
            table_len = 0 if cos_sin is None else int(cos_sin.shape[0])
        assert kpages.is_contiguous() and vpages.is_contiguous() and kpages.shape[:-1] == vpages.shape[:-1]
        ptrs = self._held(w_qkv, p_qkv, w_out, p_out)
        gains = self._held(q_gain, k_gain)
        tables = self._held(inv_freq, cos_sin)
        (sl,) = self._held(slopes)
        self.keep += [kpages, vpages]
        hook = ctypes.cast(None, HOST_ROWS)
        if rows_hook is not None:
            kv = kv_heads if owns else 0

            def thunk(_user, step, qkv_ptr, ld):
                try:
                    n = step.contents.n_rows
                    rows = self._tensor(qkv_ptr, (n, ld), self.rt.act_dtype)
                    q = rows[:, :heads * head_dim].unflatten(1, (heads, head_dim))
                    k = rows[:, heads * head_dim:(heads + kv) * head_dim].unflatten(1, (kv, head_dim)) if owns else None
                    rows_hook(q, k, self.batch)
                    return 0
                except BaseException as exc:
                    self._error = exc
                    return 1
            hook = HOST_ROWS(thunk)
            self._callbacks.append(hook)
        return self._made(L.library().gibbs_plan_body_attention(
            self.handle, *ptrs, int(heads), int(kv_heads), int(head_dim), float(scale), int(window or 0), gains[0], gains[1],
            float(qk_eps), tables[0], rot, variant, tables[1], table_len, kpages.data_ptr(), vpages.data_ptr(),
            int(kpages.shape[0]), int(kpages.shape[2]), int(group), int(owns), sl, hook, None))

    def glu(self, *, w_gate_up, p_gate_up, w_down, p_down, inter: int, activation: int) -> int:
        ptrs = self._held(w_gate_up, p_gate_up, w_down, p_down)
        return self._made(L.library().gibbs_plan_body_glu(self.handle, *ptrs, int(inter), int(activation)))

    def attention_extras(self, body: int, *, v_head_dim: int, unit_qk: bool, temp_coef: float, temp_every: int, bias,
                         bias_over_scale=None, norm_dim: int = 0) -> None:
        """Options of an attention body without rotation: values of a head size of their own, q and k divided by
        their root mean square, a temperature on q, a table [distances, heads] of score biases (and the same as
        [heads, distances] divided by the score's scale, for the kernels that add it to unscaled scores)."""
        b, bt = self._held(bias, bias_over_scale)
        self._made(L.library().gibbs_plan_attention_extras(self.handle, int(body), int(v_head_dim), int(unit_qk), int(norm_dim),
                                                           float(temp_coef), int(temp_every), b, bt,
                                                           0 if bias is None else int(bias.shape[0])))

    def attention_projection(self, body: int, *, v_head_dim: int, bias, sink, keep_mode: int, keep_key: int, value_dim: int,
                             weight) -> None:
        """Options of an attention body with a rotation (or no encoding): values of a head size of their own, a float32
        bias on the projected rows, a sink per head in the softmax, and value mixing (`keep_mode` 1: the step's values
        are published under `keep_key`; 2: what was published is mixed in with `weight`, one float32 on the device)."""
        b, s, w = self._held(bias, sink, weight)
        self._made(L.library().gibbs_plan_attention_projection(self.handle, int(body), int(v_head_dim), b, s, int(keep_mode),
                                                               int(keep_key), int(value_dim), w))

    def attention_gated(self, body: int, *, q_gain, k_gain, qk_eps: float, norm_dim: int, values_from_keys: bool, v_inv_freq,
                        v_rot: int, chunk: int, softcap: float, gate: bool) -> None:
        """Further options of an attention body that takes the projection options: a q/k norm with gains before the
        rotation, values that are the keys as projected, values turned by their position (and the outputs turned back),
        chunks instead of a window, capped scores, a sigmoid gate from nh * vd further projected columns."""
        qg, kg, vf = self._held(q_gain, k_gain, v_inv_freq)
        self._made(L.library().gibbs_plan_attention_gated(self.handle, int(body), qg, kg, float(qk_eps), int(norm_dim), int(values_from_keys),
                                                          vf, int(v_rot), int(chunk or 0), float(softcap or 0.0), int(gate)))

    def conv_input(self, *, taps: torch.Tensor, kernel: int, state: torch.Tensor) -> int:
        """rows -> rows + conv(rows): taps float32 [hidden, kernel], state float32 [slots, kernel - 1, hidden] in the arena."""
        assert taps.dtype == torch.float32 and taps.is_contiguous() and state.dtype == torch.float32
        (t,) = self._held(taps)
        self.keep.append(state)
        return self._made(L.library().gibbs_plan_body_conv_input(self.handle, t, int(kernel), state.data_ptr(), int(state.stride(0))))

    def ssd(self, m, *, conv_state: torch.Tensor, rule_state: torch.Tensor) -> int:
        """The state-space mixer `m` (parts/ssd.py) over its states [slots, ...] in the arena."""
        assert rule_state.dtype == torch.float32 and conv_state.dtype == torch.float32 and rule_state.stride(0) == conv_state.stride(0)
        d = SsdSpec()
        d.w_in, d.w_out = self._held(m.w_in, m.w_out)
        d.taps, d.conv_bias, d.dt_bias, d.a_log, d.skip, d.gain = self._held(m.conv_taps, m.conv_bias, m.dt_bias, m.a_log, m.skip, m.gain)
        d.conv_state, d.rule_state, d.slot_stride = conv_state.data_ptr(), rule_state.data_ptr(), int(rule_state.stride(0))
        self.keep += [conv_state, rule_state]
        d.heads, d.vdim, d.state, d.groups, d.taps_per_channel, d.norm_groups = m.heads, m.vdim, m.state, m.groups, m.taps, m.norm_groups
        d.eps = m.norm_eps
        return self._made(L.library().gibbs_plan_body_ssd(self.handle, ctypes.byref(d)))

    def logit_softcap(self, cap: float) -> None:
        self._made(L.library().gibbs_plan_logit_softcap(self.handle, float(cap)))

    def filtered(self, body: int, value: int) -> int:
        """-> value: body(normed rows), which a later body reads as its rows (nothing is added to the stream)."""
        return self._made(L.library().gibbs_plan_op_rows(self.handle, body, value))

    def moe(self, m) -> int:
        """The mixture-of-experts feed-forward `m` (parts/moe.py)."""
        from ..ops import ACTIVATIONS
        d = MoeSpec()
        d.router, d.router_bias, d.gate, d.up, d.down = self._held(m.router, m.router_bias, m.w_gate, m.w_up, m.w_down)
        d.shared_gate_up, d.shared_down, d.shared_gate = self._held(m.shared_gate_up, m.shared_down, m.shared_gate)
        d.experts, d.top, d.F, d.act = m.experts, m.top, m.inter, ACTIVATIONS[m.activation]
        d.shared_F, d.shared_act = m.shared_inter, ACTIVATIONS[m.shared_activation]
        body = self._made(L.library().gibbs_plan_body_moe(self.handle, ctypes.byref(d)))
        if m.scores == "softmax_all" or m.identity:
            self._made(L.library().gibbs_plan_moe_scores(self.handle, body, int(m.scores == "softmax_all"), int(m.identity)))
        return body

    def glu_clamped(self, body: int, *, alpha: float, limit: float) -> None:
        self._made(L.library().gibbs_plan_glu_clamped(self.handle, int(body), float(alpha), float(limit)))

    def embedding(self, scale: float, inv_freq: Optional[torch.Tensor]) -> None:
        """The table's rows times `scale`, plus the sinusoidal position vector of `inv_freq` (float32 [hidden / 2])."""
        (f,) = self._held(inv_freq)
        self._made(L.library().gibbs_plan_embedding(self.handle, float(scale), f))
        self.plain_embedding = self.plain_embedding and scale == 1.0 and inv_freq is None

    def gated_delta(self, m, *, conv_state: torch.Tensor, rule_state: torch.Tensor) -> int:
        """The delta-rule mixer `m` (parts/delta.py) over its states [slots, ...] in the arena."""
        assert rule_state.dtype == torch.float32 and conv_state.dtype == torch.float32 and rule_state.stride(0) == conv_state.stride(0)
        d = DeltaSpec()
        d.w_in, d.w_out, d.w_a2, d.w_g2 = self._held(m.w_in, m.w_out, m.w_a2, m.w_g2)
        d.taps, d.dt_bias, d.a_log, d.gain = self._held(m.conv_taps, m.dt_bias, m.a_log, m.gain)
        d.conv_state, d.rule_state, d.slot_stride = conv_state.data_ptr(), rule_state.data_ptr(), int(rule_state.stride(0))
        self.keep += [conv_state, rule_state]
        d.in_rows, d.heads, d.kv_heads, d.dim, d.vdim = m.w_in.shape[0], m.heads, m.kv_heads, m.dim, m.vdim
        d.taps_per_channel, d.off_b, d.off_a, d.off_g = m.taps, m.off_b, m.off_a, m.off_g
        d.a_rank, d.g_rank = m.decay_rank, m.gate_rank
        d.eps, d.unit_eps, d.q_scale = m.norm_eps, m.unit_eps, m.q_scale
        return self._made(L.library().gibbs_plan_body_delta(self.handle, ctypes.byref(d)))

    def time_mix(self, m, *, shift_state: torch.Tensor, rule_state: torch.Tensor) -> int:
        """The time-mixing mixer `m` (parts/timemix.py) over its states [slots, ...] in the arena."""
        assert rule_state.dtype == torch.float32 and shift_state.dtype == torch.float32 and rule_state.stride(0) == shift_state.stride(0)
        d = TimeMixSpec()
        d.w_r, d.w_k, d.w_v, d.w_g, d.w_1, d.w_2, d.w_out = self._held(m.w_r, m.w_k, m.w_v, m.w_g, m.w_1, m.w_2, m.w_out)
        d.mu, d.w0, d.bonus, d.gain = self._held(m.mu, m.w0, m.bonus, m.gain)
        d.shift_state, d.rule_state, d.slot_stride = shift_state.data_ptr(), rule_state.data_ptr(), int(rule_state.stride(0))
        self.keep += [shift_state, rule_state]
        d.heads, d.dim, d.rank, d.eps = m.heads, m.dim, m.rank, m.norm_eps
        return self._made(L.library().gibbs_plan_body_time_mix(self.handle, ctypes.byref(d)))

    def latent_attention(self, m, *, pages: torch.Tensor, group: int) -> int:
        """The latent-attention mixer `m` (parts/latent.py) over its pages [num_pages, 1, page_size, kv_rank + rot_dim]."""
        from ..ops import ROPE_VARIANTS
        assert pages.is_contiguous() and pages.dtype == self.rt.act_dtype
        d = LatentSpec()
        d.w_in, d.w_uq, d.w_uk_t, d.w_uv, d.w_out = self._held(m.w_in, m.w_uq, m.w_uk_t, m.w_uv, m.w_out)
        d.q_gain, d.kv_gain, d.sink = self._held(m.q_gain, m.kv_gain, m.sinks)
        d.rot_dims = d.variant = 0
        if m.rot is not None:
            (d.inv_freq,) = self._held(m.rot.inv_freq)
            d.rot_dims, d.variant = int(m.rot.rotary_dim), ROPE_VARIANTS[m.rot.variant]
        d.pages = pages.data_ptr()
        self.keep.append(pages)
        d.in_rows, d.heads, d.dim, d.rot, d.vdim, d.rank, d.q_rank = m.w_in.shape[0], m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.q_rank
        d.window, d.off_kv, d.off_g = int(m.window or 0), m.off_kv, m.off_g
        d.num_pages, d.page_size, d.group = int(pages.shape[0]), int(pages.shape[2]), int(group)
        d.scale, d.eps = m.scale, m.norm_eps
        return self._made(L.library().gibbs_plan_body_latent(self.handle, ctypes.byref(d)))

    def mlp(self, *, w_up, w_down, inter: int, coef: torch.Tensor, eps: float) -> int:
        """down(act(up h)) with the polynomial-norm activation; coef: float32 [4] on the device."""
        assert coef.dtype == torch.float32 and coef.numel() == 4
        u, dn, c = self._held(w_up, w_down, coef)
        return self._made(L.library().gibbs_plan_body_mlp(self.handle, u, dn, int(inter), c, float(eps)))

    def streams(self, n: int) -> None:
        """The model keeps `n` residual streams, each starting as the embedding's output; its output is their sum."""
        self._made(L.library().gibbs_plan_streams(self.handle, int(n)))
        if n > 1:
            self.plain_embedding = False

    def hyper(self, w_in: torch.Tensor, w_mix: torch.Tensor, w_out: torch.Tensor) -> int:
        """A hyper-connection: in [streams], mix [streams, streams] indexed [from, to], out [streams], float32."""
        assert all(t.dtype == torch.float32 and t.is_contiguous() for t in (w_in, w_mix, w_out))
        return self._made(L.library().gibbs_plan_hyper(self.handle, *self._held(w_in, w_mix, w_out)))

    def embedding_tables(self, *, pair, buckets: int, mul_prev: int, mul_cur: int, position, prev_state) -> None:
        """Rows of a table over hashed token pairs and of a table over positions, added to the token table's row.
        `prev_state`: int32 [slots] (a column of the state arena): every request's last token."""
        pt, ps = self._held(pair, position)
        stride = 0
        if pair is not None:
            assert prev_state is not None and prev_state.dtype == torch.int32 and prev_state.dim() == 1
            stride = int(prev_state.stride(0))
            self.keep.append(prev_state)
        self._made(L.library().gibbs_plan_embedding_tables(
            self.handle, pt, int(buckets), int(mul_prev), int(mul_cur), ps, 0 if position is None else int(position.shape[0]),
            None if pair is None else prev_state.data_ptr(), stride))
        self.plain_embedding = False

    def streams_normed(self, norm: int, hyper: int) -> int:
        """-> value: norm(sum_s in[s] x_s)."""
        return self._made(L.library().gibbs_plan_op_streams_norm(self.handle, norm, hyper))

    def streams_add(self, hyper: int, value: int) -> None:
        """x_t <- sum_s mix[s, t] x_s + out[t] delta for all streams at once; the delta is used up."""
        self._made(L.library().gibbs_plan_op_streams_add(self.handle, hyper, value))

    def host_body(self, forward: Callable, group: Optional[int] = None) -> int:
        """A mixer or feed-forward written with tensor operations: `forward(h, batch) -> delta [N, hidden]`
        (or float32 partial sums [S, N, hidden]).  `group`: the cache group whose block table it reads."""
        def thunk(_user, step, h_ptr, out_ptr):
            try:
                n = step.contents.n_rows
                h = self._tensor(h_ptr, (n, self.hidden), self.rt.act_dtype)
                out = self._tensor(out_ptr, (n, self.hidden), self.rt.act_dtype)
                delta = forward(h, self.batch)
                out.copy_(delta.sum(0) if delta.dim() == 3 else delta)
                return 0
            except BaseException as exc:
                self._error = exc
                return 1
        cb = HOST_BODY(thunk)
        self._callbacks.append(cb)
        return self._made(L.library().gibbs_plan_body_host(self.handle, cb, None, -1 if group is None else int(group)))

    # ------------------------------------------------------------------ building: the program
    def half(self, norm: int, body: int) -> None:
        """x += body(norm(x)); in fused decode kernels where the step, the norm and the body allow them."""
        self._made(L.library().gibbs_plan_op_half(self.handle, norm, body))

    def normed(self, norm: int) -> int:
        """-> value: norm(x + what is pending)."""
        return self._made(L.library().gibbs_plan_op_norm(self.handle, norm))

    def apply(self, body: int, value: int) -> int:
        """-> value: body(normed rows)."""
        return self._made(L.library().gibbs_plan_op_body(self.handle, body, value))

    def add(self, value: int) -> None:
        """x += delta (it stays pending until the next norm reads x, which adds it on the way)."""
        self._made(L.library().gibbs_plan_op_add(self.handle, value))

    def normed_delta(self, norm: int, value: int) -> int:
        """-> value: norm(a body's delta), before it is added; the stream is not touched."""
        return self._made(L.library().gibbs_plan_op_norm_delta(self.handle, norm, value))

    def add_normed(self, norm: int, value: int) -> None:
        """x += norm(a body's delta): normed and added in one pass (float32), the delta is used up."""
        self._made(L.library().gibbs_plan_op_add_normed(self.handle, norm, value))

    def reinject(self) -> None:
        """x += the embedding's output (the rows as the step's first operation saw them)."""
        self._made(L.library().gibbs_plan_op_reinject(self.handle))
        self.plain_embedding = False

    def drop(self, value: int) -> None:
        self._made(L.library().gibbs_plan_op_drop(self.handle, value))

    def tail(self, norm: int) -> None:
        self._made(L.library().gibbs_plan_tail(self.handle, norm))

    def op_count(self) -> int:
        return int(L.library().gibbs_plan_op_count(self.handle))

    @classmethod
    def build(cls, model, views, rt, model_view=None) -> "NativePlan":
        """The plan of a bound `DecoderModel` (`views[run]`: the cache views of the run's mixers by role; `model_view`:
        the view of the state that the model itself keeps per request)."""
        plan = cls(rt, model.spec.hidden, model.spec.vocab, model.table, model.head, model.head_packed)
        if model.spec.embedding_scale != 1.0 or model.embedding_inv_freq is not None:
            plan.embedding(model.spec.embedding_scale, model.embedding_inv_freq)
        if model.spec.streams != 1:
            plan.streams(model.spec.streams)
        tables = model.spec.embedding_tables
        if tables is not None and (tables.pair is not None or tables.position is not None):
            prev = None
            if tables.pair is not None:
                if model_view is None or model.PREV_TOKEN not in model_view.states:
                    raise ValueError("a table over token pairs needs the requests' last tokens: no state view was given")
                prev = model_view.states[model.PREV_TOKEN]
            plan.embedding_tables(pair=model.pair_table, buckets=tables.buckets, mul_prev=tables.mul_prev, mul_cur=tables.mul_cur,
                                  position=model.position_table, prev_state=prev)
        for run, i in enumerate(model.spec.order):
            if run in model.spec.reinject_before:
                plan.reinject()
            model.blocks[i].emit(plan, views[run])
        plan.tail(model.final_norm.emit(plan))
        if model.spec.logit_softcap:
            plan.logit_softcap(model.spec.logit_softcap)
        return plan

    # ------------------------------------------------------------------ running
    def _tensor(self, ptr: int, shape, dtype: torch.dtype) -> torch.Tensor:
        """The tensor behind a pointer that the native step hands to a callback: a piece of the step's
        workspace, or the caller's own residual rows."""
        n = 1
        for s in shape:
            n *= s
        nbytes = n * torch.empty((), dtype=dtype).element_size()
        for base in (self._workspace, self._x_in):
            if base is None:
                continue
            off = ptr - base.data_ptr()
            if 0 <= off and off + nbytes <= base.numel() * base.element_size():
                return base.view(-1).view(torch.uint8)[off:off + nbytes].view(dtype).view(*shape)
        raise KernelError("a callback of the native step was handed memory that is neither the workspace nor the caller's rows")

    def _fill(self, batch, x_in=None, mirror_in=None, first_op: int = 0, n_ops: int = 0, settle: bool = False) -> StepArgs:
        a = self._args
        a.x_in, a.mirror_in = _ptr(x_in), _ptr(mirror_in)
        a.ids, a.pos, a.row_req = _ptr(batch.ids), _ptr(batch.pos), _ptr(batch.row_req)
        a.cu, a.ctx, a.slot = _ptr(batch.cu), _ptr(batch.ctx), _ptr(batch.slot)
        a.logit_rows = _ptr(batch.logit_rows) if batch.n_logits else None
        g = len(batch.tables)
        if self._tables is None or len(self._tables) != max(g, 1):
            self._tables, self._widths = (c_void_p * max(g, 1))(), (c_int * max(g, 1))()
        for i, t in enumerate(batch.tables):
            self._tables[i], self._widths[i] = t.data_ptr(), int(t.shape[1])
        a.tables, a.widths, a.n_groups = self._tables, self._widths, g
        a.n_rows, a.n_req, a.n_logits = batch.n_rows, batch.n_req, batch.n_logits
        a.max_q, a.max_seq, a.lead_single = batch.max_q, batch.max_seq, batch.lead_single
        a.first_op, a.n_ops, a.settle = first_op, n_ops, int(settle)
        a.workspace, a.workspace_bytes, a.logits = None, 0, None
        a.stream = L.stream()
        return a

    def _raise(self):
        exc, self._error = self._error, None
        if exc is not None:
            raise exc
        raise KernelError(L.library().gibbs_last_error().decode(errors="replace"))

    def _own_workspace(self, need: int) -> torch.Tensor:
        if self._arena is None or self._arena.numel() < need:
            self._arena = None                       # (give the old one back first)
            self._arena = torch.empty(max(int(need * 1.25), 1 << 20), dtype=torch.uint8, device=self.device)
        return self._arena

    def workspace_bytes(self, batch, x_in=None, mirror_in=None) -> int:
        need = L.library().gibbs_plan_workspace(self.handle, ctypes.byref(self._fill(batch, x_in, mirror_in)))
        if need < 0:
            self._raise()
        return int(need)

    def step(self, batch, workspace: Optional[torch.Tensor] = None, x_in: Optional[torch.Tensor] = None,
             mirror_in: Optional[torch.Tensor] = None, first_op: int = 0, n_ops: int = 0,
             settle: bool = False) -> Optional[torch.Tensor]:
        """Queues the whole step; returns float32 logits [wanted rows, vocab] (None if none are wanted).
        `workspace`: a byte buffer of the caller's that outlives the step's kernels (a captured graph
        replays over it); default: the plan's own, which grows when a step needs more.  `x_in` (float32
        [rows, hidden]) and `mirror_in` (its bfloat16 copy): the rows' embeddings, when the end of the
        previous step has written them already (the step then starts at its first layer and updates
        them in place).  `first_op`, `n_ops`: only these operations of the program run (no logits then);
        `settle`: whatever delta is still pending at the end is added into x."""
        lib = L.library()
        if x_in is not None:
            assert x_in.dtype == torch.float32 and x_in.is_contiguous() and x_in.shape[0] == batch.n_rows
            assert mirror_in is None or (mirror_in.dtype == torch.bfloat16 and mirror_in.shape == x_in.shape and mirror_in.is_contiguous())
        a = self._fill(batch, x_in, mirror_in, first_op, n_ops, settle)
        need = lib.gibbs_plan_workspace(self.handle, ctypes.byref(a))
        if need < 0:
            self._raise()
        if workspace is None:
            workspace = self._own_workspace(need)
        elif workspace.numel() < need:
            raise KernelError(f"the step needs {need} bytes of workspace, the caller's buffer has {workspace.numel()}")
        logits = None
        if batch.n_logits and n_ops == 0:
            logits = torch.empty((batch.n_logits, self.vocab), dtype=torch.float32, device=self.device)
        a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel()
        a.logits = None if logits is None else logits.data_ptr()
        self.batch, self._workspace, self._x_in = batch, workspace, x_in
        try:
            if lib.gibbs_plan_step(self.handle, ctypes.byref(a)) != 0:
                self._raise()
        finally:
            self.batch = self._workspace = self._x_in = None
        return logits

    def last_fused(self) -> int:
        """Halves of the last step that ran as fused decode kernels."""
        return int(L.library().gibbs_plan_last_fused(self.handle))

    # ------------------------------------------------------------------ one part alone
    def body_forward(self, body: int, h: torch.Tensor, batch) -> torch.Tensor:
        """delta of the normed rows `h` by body number `body`: [N, hidden], or float32 partial sums [S, N, hidden]."""
        lib = L.library()
        assert h.is_contiguous() and h.dtype == self.rt.act_dtype and h.shape[1] == self.hidden
        batch = _MinimalBatch(h.shape[0]) if batch is None else batch
        a = self._fill(batch)
        a.n_rows = h.shape[0]
        off, parts = c_long(0), c_int(0)
        need = lib.gibbs_plan_body_forward(self.handle, body, ctypes.byref(a), h.data_ptr(), ctypes.byref(off), ctypes.byref(parts))
        if need < 0:
            self._raise()
        workspace = torch.empty(max(int(need), 256), dtype=torch.uint8, device=self.device)   # (the result lives in it)
        a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel()
        self.batch, self._workspace = batch, workspace
        try:
            if lib.gibbs_plan_body_forward(self.handle, body, ctypes.byref(a), h.data_ptr(), ctypes.byref(off), ctypes.byref(parts)) != 0:
                self._raise()
        finally:
            self.batch = self._workspace = None
        n = h.shape[0]
        if parts.value >= 2:
            return workspace[off.value:off.value + parts.value * n * self.hidden * 4].view(torch.float32).view(parts.value, n, self.hidden)
        size = torch.empty((), dtype=self.rt.act_dtype).element_size()
        return workspace[off.value:off.value + n * self.hidden * size].view(self.rt.act_dtype).view(n, self.hidden)

    def norm_forward(self, norm: int, x: torch.Tensor, delta: Optional[torch.Tensor], rows: Optional[torch.Tensor],
                     n_rows: Optional[int]) -> torch.Tensor:
        lib = L.library()
        assert x.dtype == torch.float32 and x.is_contiguous() and x.shape[1] == self.hidden
        parts = 0
        if delta is not None:
            assert delta.is_contiguous()
            if delta.dim() == 3:
                assert delta.dtype == torch.float32 and delta.shape[1:] == x.shape
                parts = delta.shape[0]
            else:
                assert delta.shape == x.shape and delta.dtype == self.rt.act_dtype
                parts = 1
        n_out = x.shape[0] if rows is None else (rows.numel() if n_rows is None else n_rows)
        a = self._fill(_MinimalBatch(x.shape[0]))
        off = c_long(0)
        call = lambda: lib.gibbs_plan_norm_forward(self.handle, norm, ctypes.byref(a), x.data_ptr(), _ptr(delta), parts,
                                                   _ptr(rows), int(n_out), ctypes.byref(off))
        need = call()
        if need < 0:
            self._raise()
        workspace = torch.empty(max(int(need), 256), dtype=torch.uint8, device=self.device)
        a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel()
        if call() != 0:
            self._raise()
        size = torch.empty((), dtype=self.rt.act_dtype).element_size()
        return workspace[off.value:off.value + n_out * self.hidden * size].view(self.rt.act_dtype).view(n_out, self.hidden)
