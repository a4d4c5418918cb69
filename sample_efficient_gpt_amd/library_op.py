"""`torch.library` registration of the fused QK-norm attention, so that the op survives `torch.compile`
(the reference compiles the whole model, sample_efficient_gpt/training/trainer.py:227-228) and
non-reentrant activation checkpointing (transformer/transformer.py:123-132) as ONE opaque node with a fake
(shape-only) implementation instead of being traced into.

    y = torch.ops.segpt.qknorm_attention(q, k, v, g_q, g_k, v_first, vr_coef, gate_logits,
                                         gate_scale, eps, sm_scale, causal, q_start,
                                         rope_cos, rope_sin, rope_q_pos0, rope_k_pos0, qk_norm, out_bshd,
                                         inference)[0]

or the keyword wrapper ``qknorm_attention_op(...)`` below.  Canonical layout: q ``[B,H,Sq,D]``, k / v /
v_first ``[B,Hkv,Sk,D]`` (any strides, last dim contiguous), gate_logits ``[B,Sq,H]``; the optional tensors
are ``None`` when unused (rope_q_pos0 = -1 means "q_start"); ``inference=True`` promises that no backward
follows (decode-shaped calls may then take the split-key kernels, whose key/value workspace holds no keys).  Returns ``(y, lse, kv_ws)``: the output, the fp32 log-sum-exp ``[B,H,Sq]`` and the
key/value workspace the backward reuses.  Same kernels and C ABI as ``function.py``; no fallback.
"""

from __future__ import annotations

import math
from typing import List, Optional

import torch
from torch import Tensor

from . import _lib
from .function import (_backward, _check_inputs, _forward, _lastdim_contig, _no_backward_will_follow, _rope_arg,
                       _scale_arg)

__all__ = ["qknorm_attention_op"]


def _empty_out(q, out_bshd):
    """Output buffer [B,H,Sq,D]: contiguous, or (out_bshd) a view of a [B,Sq,H,D] buffer, the layout the
    output projection consumes (attention.py:243)."""
    B, H, Sq, D = q.shape
    if out_bshd:
        return q.new_empty((B, Sq, H, D)).permute(0, 2, 1, 3)
    return q.new_empty((B, H, Sq, D))


def _coef32(vr_coef, device):
    return None if vr_coef is None else vr_coef.detach().to(device=device, dtype=torch.float32).reshape(-1).contiguous()


@torch.library.custom_op("segpt::qknorm_attention", mutates_args=())
def _fwd_op(q: Tensor, k: Tensor, v: Tensor, g_q: Tensor, g_k: Optional[Tensor], v_first: Optional[Tensor],
            vr_coef: Optional[Tensor], gate_logits: Optional[Tensor], gate_scale: float, eps: float, sm_scale: float,
            causal: bool, q_start: int, rope_cos: Optional[Tensor], rope_sin: Optional[Tensor],
            rope_q_pos0: int, rope_k_pos0: int, qk_norm: bool, out_bshd: bool, inference: bool) -> List[Tensor]:
    rope = _rope_arg(rope_cos, rope_sin, None if rope_q_pos0 < 0 else rope_q_pos0, rope_k_pos0, q_start, q.device, q.shape[-1])
    gq32, gk32, c32 = _scale_arg(g_q, q.device), _scale_arg(g_k, q.device), _coef32(vr_coef, q.device)
    _check_inputs(q, k, v, gq32, gk32, v_first, c32, gate_logits)
    q, k, v = _lastdim_contig(q), _lastdim_contig(k), _lastdim_contig(v)
    v_first = None if v_first is None else _lastdim_contig(v_first)
    y = _empty_out(q, out_bshd)
    lse, kv_ws = _forward(q, k, v, gq32, gk32, v_first, c32, gate_logits, gate_scale, eps, sm_scale, causal, q_start, y, rope,
                          inference=inference, flags=0 if qk_norm else _lib.SEGPT_FLAG_NO_NORM)
    if inference:  # no backward will read it (and after the decode kernels it holds no keys)
        kv_ws = q.new_empty((0,), dtype=torch.uint8)
    return [y, lse, kv_ws]


@_fwd_op.register_fake
def _(q, k, v, g_q, g_k, v_first, vr_coef, gate_logits, gate_scale, eps, sm_scale, causal, q_start,
      rope_cos, rope_sin, rope_q_pos0, rope_k_pos0, qk_norm, out_bshd, inference):
    B, H, Sq, D = q.shape
    y = _empty_out(q, out_bshd)
    lse = q.new_empty((B, H, Sq), dtype=torch.float32)
    # normalised keys (+ mixed values) of the bf16 path, rounded up to 256 bytes each; 256 bytes otherwise
    nbytes = 256
    if q.numel() == 0 or inference:
        nbytes = 0
    elif q.dtype == torch.bfloat16:
        piece = (k.shape[0] * k.shape[1] * k.shape[2] * D * 2 + 255) // 256 * 256
        nbytes = piece * (2 if v_first is not None else 1)
    return [y, lse, q.new_empty((nbytes,), dtype=torch.uint8)]


@torch.library.custom_op("segpt::qknorm_attention_backward", mutates_args=())
def _bwd_op(dy: Tensor, q: Tensor, k: Tensor, v: Tensor, g_q: Tensor, g_k: Optional[Tensor], v_first: Optional[Tensor],
            vr_coef: Optional[Tensor], gate_logits: Optional[Tensor], y: Tensor, lse: Tensor, kv_ws: Tensor,
            gate_scale: float, eps: float, sm_scale: float, causal: bool, q_start: int,
            rope_cos: Optional[Tensor], rope_sin: Optional[Tensor], rope_q_pos0: int, rope_k_pos0: int,
            qk_norm: bool) -> List[Tensor]:
    """Returns [dq, dk, dv, dg_q, dg_k, dv_first, dvr_coef, dgate]; absent ones are empty tensors."""
    dev = q.device
    rope = _rope_arg(rope_cos, rope_sin, None if rope_q_pos0 < 0 else rope_q_pos0, rope_k_pos0, q_start, dev, q.shape[-1])
    gq32, gk32, c32 = _scale_arg(g_q, dev), _scale_arg(g_k, dev), _coef32(vr_coef, dev)
    q, k, v = _lastdim_contig(q), _lastdim_contig(k), _lastdim_contig(v)
    v_first = None if v_first is None else _lastdim_contig(v_first)
    dy = _lastdim_contig(dy)
    if dy.dtype != q.dtype:
        dy = dy.to(q.dtype)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dvf = None if v_first is None else torch.empty_like(v_first)
    dgate = None if gate_logits is None else torch.empty_like(gate_logits)
    dg_q, dg_k, dcoef = _backward(q, k, v, gq32, gk32, v_first, c32, gate_logits, gate_scale, eps, sm_scale, causal, q_start,
                                  y, lse, dy, dq, dk, dv, dvf, dgate, kv_ws, rope,
                                  0 if qk_norm else _lib.SEGPT_FLAG_NO_NORM)
    none = lambda: q.new_empty((0,))  # a fresh tensor each: returns of a custom op must not alias one another
    return [dq, dk, dv, dg_q.reshape(g_q.shape).to(g_q.dtype),
            none() if g_k is None else dg_k.reshape(g_k.shape).to(g_k.dtype),
            none() if dvf is None else dvf,
            none() if vr_coef is None else dcoef.reshape(vr_coef.shape).to(vr_coef.dtype),
            none() if dgate is None else dgate]


@_bwd_op.register_fake
def _(dy, q, k, v, g_q, g_k, v_first, vr_coef, gate_logits, y, lse, kv_ws, gate_scale, eps, sm_scale, causal, q_start,
      rope_cos, rope_sin, rope_q_pos0, rope_k_pos0, qk_norm):
    none = lambda: q.new_empty((0,))
    return [torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(g_q),
            none() if g_k is None else torch.empty_like(g_k),
            none() if v_first is None else torch.empty_like(v_first),
            none() if vr_coef is None else torch.empty_like(vr_coef),
            none() if gate_logits is None else torch.empty_like(gate_logits)]


def _setup_context(ctx, inputs, output):
    (q, k, v, g_q, g_k, v_first, vr_coef, gate_logits, gate_scale, eps, sm_scale, causal, q_start,
     rope_cos, rope_sin, rope_q_pos0, rope_k_pos0, qk_norm, out_bshd, _inference) = inputs
    y, lse, kv_ws = output
    ctx.save_for_backward(q, k, v, g_q, g_k, v_first, vr_coef, gate_logits, y, lse, kv_ws, rope_cos, rope_sin)
    ctx.cfg = (gate_scale, eps, sm_scale, causal, q_start, rope_q_pos0, rope_k_pos0, qk_norm)


def _autograd_backward(ctx, grads):
    dy = grads[0]
    q, k, v, g_q, g_k, v_first, vr_coef, gate_logits, y, lse, kv_ws, rope_cos, rope_sin = ctx.saved_tensors
    gate_scale, eps, sm_scale, causal, q_start, rope_q_pos0, rope_k_pos0, qk_norm = ctx.cfg
    dq, dk, dv, dg_q, dg_k, dvf, dcoef, dgate = torch.ops.segpt.qknorm_attention_backward(
        dy, q, k, v, g_q, g_k, v_first, vr_coef, gate_logits, y, lse, kv_ws, gate_scale, eps, sm_scale, causal, q_start,
        rope_cos, rope_sin, rope_q_pos0, rope_k_pos0, qk_norm)
    return (dq, dk, dv, dg_q, None if g_k is None else dg_k, None if v_first is None else dvf,
            None if vr_coef is None else dcoef, None if gate_logits is None else dgate, None, None, None, None, None,
            None, None, None, None, None, None, None)


_fwd_op.register_autograd(_autograd_backward, setup_context=_setup_context)


def qknorm_attention_op(q, k, v, g_q, g_k=None, *, v_first=None, vr_coef=None, gate_logits=None, gate_scale=2.0,
                        eps=1e-6, sm_scale=None, causal=True, q_start=0, return_lse=False,
                        rope_cos=None, rope_sin=None, rope_q_pos0=None, rope_k_pos0=0, qk_norm=True, out_bshd=False):
    """Keyword front end of ``torch.ops.segpt.qknorm_attention`` (same arguments as ``qknorm_attention``)."""
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(q.shape[-1])
    # decided here, in the caller's grad mode: a forward-only call (the reference's generate loop runs under
    # inference_mode, transformer.py:160) with few query rows takes the split-key decode kernels
    inference = _no_backward_will_follow(q, k, v, g_q, g_k, v_first, vr_coef, gate_logits)
    y, lse, _ = torch.ops.segpt.qknorm_attention(q, k, v, g_q, g_k, v_first, vr_coef, gate_logits, float(gate_scale),
                                                 float(eps), float(sm_scale), bool(causal), int(q_start),
                                                 rope_cos, rope_sin, -1 if rope_q_pos0 is None else int(rope_q_pos0),
                                                 int(rope_k_pos0), bool(qk_norm), bool(out_bshd), bool(inference))
    return (y, lse) if return_lse else y
