"""Pre-bound launch plan: one filled `segpt_attn_params` plus every output / workspace buffer, so that a
tight loop (benchmark, serving) makes C-ABI calls without building structs or allocating per call."""

from __future__ import annotations

import math

import torch

from . import _lib
from .function import _fill_common, _rope_arg


class AttnPlan:
    """Binds canonical-layout tensors (q [B,H,S,D], k/v [B,Hkv,S,D], ...) once; `forward()`,
    `backward()` and `backward_stage(i)` then only enqueue kernels on the current stream.  Nothing is
    allocated, copied or cleared per call, so a forward + backward pair can be captured into a HIP graph
    (`torch.cuda.graph`) and replayed."""

    def __init__(self, x: dict, *, eps=1e-6, sm_scale=None, gate_scale=2.0, causal=True, q_start=0, backward=True,
                 rope_cos=None, rope_sin=None, rope_q_pos0=None, rope_k_pos0=0, qk_norm=True):
        self.lib = _lib.load()
        self.base_flags = 0 if qk_norm else _lib.SEGPT_FLAG_NO_NORM  # part of every call's flags
        q, k, v = x["q"], x["k"], x["v"]
        dev = q.device
        self.x = x
        f32 = lambda t: None if t is None else t.detach().to(device=dev, dtype=torch.float32).reshape(-1).contiguous()
        self.g_q, self.g_k, self.coef = f32(x["g_q"]), f32(x.get("g_k")), f32(x.get("vr_coef"))
        self.v_first, self.gate = x.get("v_first"), x.get("gate_logits")
        B, H, Sq, D = q.shape
        if sm_scale is None:
            sm_scale = 1.0 / math.sqrt(D)
        self.y = torch.empty_like(q)
        self.lse = torch.empty((B, H, Sq), dtype=torch.float32, device=dev)
        self.rope = _rope_arg(rope_cos, rope_sin, rope_q_pos0, rope_k_pos0, q_start, dev, D)  # keeps the tables alive
        p = _lib.new_params()
        _fill_common(p, q, k, v, self.y, self.lse, self.g_q, self.g_k, self.v_first, self.coef, self.gate, gate_scale,
                     eps, sm_scale, causal, q_start, self.rope)
        self.kv_ws = _lib.alloc_workspace(self.lib, p, _lib.SEGPT_WS_KV, dev)
        p.kv_workspace, p.kv_workspace_bytes = self.kv_ws.data_ptr(), self.kv_ws.numel()
        self.p = p
        self.has_bwd = backward
        if backward:
            self.d_o = x["d_o"]
            self.dq, self.dk, self.dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
            self.dv_first = None if self.v_first is None else torch.empty_like(self.v_first)
            self.dgate = None if self.gate is None else torch.empty_like(self.gate)
            self.dg_q = torch.empty_like(self.g_q)
            self.dg_k = None if self.g_k is None else torch.empty_like(self.g_k)
            self.dcoef = None if self.coef is None else torch.empty(2, dtype=torch.float32, device=dev)
            p.d_o, p.dq, p.dk, p.dv = _lib.t4(self.d_o), _lib.t4(self.dq), _lib.t4(self.dk), _lib.t4(self.dv)
            p.dv_first, p.dgate = _lib.t4(self.dv_first), _lib.t3(self.dgate)
            p.dg_q, p.dg_k, p.dvr_coef = _lib.ptr(self.dg_q), _lib.ptr(self.dg_k), _lib.ptr(self.dcoef)
            self.ws = _lib.alloc_workspace(self.lib, p, _lib.SEGPT_WS_BWD, dev)
            p.workspace, p.workspace_bytes = self.ws.data_ptr(), self.ws.numel()
        self.dev = dev

    @property
    def stream(self):
        """The device's current stream at call time (so that the calls can be captured into a graph)."""
        return torch.cuda.current_stream(self.dev).cuda_stream

    def _chk(self, rc, what):
        if rc != 0:
            raise _lib.SegptError(rc, what)

    def forward(self, flags: int = 0):
        """Key/value pre-pass + attention kernel; leaves the normalised keys in the plan's kv workspace."""
        self.p.flags = flags | self.base_flags
        self._chk(self.lib.segpt_attn_fwd(self.p, self.stream), "segpt_attn_fwd")

    def forward_stage(self, stage: int):
        self.p.flags = self.base_flags
        self._chk(self.lib.segpt_attn_fwd_stage(self.p, stage, self.stream), "segpt_attn_fwd_stage")

    def backward(self, kv_prepared: bool = False):
        """`kv_prepared`: forward() ran on this plan since k / v last changed, so the backward reuses its
        normalised keys instead of running the pre-pass again."""
        self.p.flags = (_lib.SEGPT_FLAG_KV_PREPARED if kv_prepared else 0) | self.base_flags
        self._chk(self.lib.segpt_attn_bwd(self.p, self.stream), "segpt_attn_bwd")

    def backward_stage(self, stage: int, kv_prepared: bool = False):
        self.p.flags = (_lib.SEGPT_FLAG_KV_PREPARED if kv_prepared else 0) | self.base_flags
        self._chk(self.lib.segpt_attn_bwd_stage(self.p, stage, self.stream), "segpt_attn_bwd_stage")
