"""Autograd front end of the fused QK-norm flash attention (HIP kernels behind a C ABI).

Two entry points share one implementation:

* ``QKNormFlashAttnFunc.apply(Q, K, V, gain, is_causal=True, q_start=0, ...)`` -- positional drop-in
  for the reference's ``TritonFlashAttnQKNormFunc``
  (sample_efficient_gpt/transformer/ops/triton_flash_attn_qknorm.py:262-343): flattened
  ``[(h b), S, d]`` tensors, gradients for ``Q, K, V, gain`` and ``None`` for the flags.  Optional
  trailing positionals switch on what the reference's caller does around the op
  (sample_efficient_gpt/transformer/attention.py:207-255): un-expanded GQA K/V, the value-residual
  mix, the per-head sigmoid gate, a k-side scale vector.
* ``qknorm_attention(q, k, v, g_q, ...)`` -- the same op on canonical ``[B, H, S, D]`` /
  ``[B, Hkv, S, D]`` views with keyword arguments.

Defaults follow the live module (attention.py:51-80): RMS normaliser, eps 1e-6 on the mean,
logits scaled by 1/sqrt(d).  ``eps=1e-8/d, sm_scale=1/d`` reproduces the fused Triton kernel's
own formula (triton_flash_attn_qknorm.py:67-91).
"""

from __future__ import annotations

import math
import threading

import torch

from . import _lib

_DTYPES = {torch.bfloat16: _lib.SEGPT_DTYPE_BF16, torch.float32: _lib.SEGPT_DTYPE_FP32}


def _scale_arg(g, device):
    """Scale parameter -> contiguous fp32 device vector (or None)."""
    if g is None:
        return None
    return g.detach().to(device=device, dtype=torch.float32).reshape(-1).contiguous()


def _rope_arg(rope_cos, rope_sin, rope_q_pos0, rope_k_pos0, q_start, device, head_dim):
    """Normalise the rotary-embedding arguments to `(cos, sin, q_pos0, k_pos0)` (fp32 contiguous device tables
    of shape [len, head_dim // 2]) or None.  Query row i sits at position q_pos0 + i (default: q_start, as in
    the reference's caller, attention.py:191-204), key row j at k_pos0 + j."""
    if rope_cos is None and rope_sin is None:
        return None
    assert rope_cos is not None and rope_sin is not None, "rope_cos and rope_sin go together"
    cos = rope_cos.detach().to(device=device, dtype=torch.float32).contiguous()
    sin = rope_sin.detach().to(device=device, dtype=torch.float32).contiguous()
    assert cos.dim() == 2 and cos.shape == sin.shape and cos.shape[1] == head_dim // 2, "rope tables must be [len, head_dim // 2]"
    return cos, sin, int(q_start if rope_q_pos0 is None else rope_q_pos0), int(rope_k_pos0)


def _fill_common(p, q, k, v, y, lse, g_q, g_k, v_first, vr_coef, gate, gate_scale, eps, sm_scale, causal, q_start,
                 rope=None):
    B, H, Sq, D = q.shape
    p.dtype = _DTYPES[q.dtype]
    p.B, p.H, p.Hkv, p.Sq, p.Sk, p.D = B, H, k.shape[1], Sq, k.shape[2], D
    p.causal = int(bool(causal))
    p.q_start = int(q_start)
    p.gq_numel = g_q.numel()
    p.gk_numel = 0 if g_k is None else g_k.numel()
    p.eps, p.sm_scale, p.gate_scale = float(eps), float(sm_scale), float(gate_scale)
    p.q, p.k, p.v, p.o = _lib.t4(q), _lib.t4(k), _lib.t4(v), _lib.t4(y)
    p.v_first = _lib.t4(v_first)
    p.gate = _lib.t3(gate)
    p.lse = _lib.ptr(lse)
    p.g_q, p.g_k, p.vr_coef = _lib.ptr(g_q), _lib.ptr(g_k), _lib.ptr(vr_coef)
    if rope is not None:
        cos, sin, q_pos0, k_pos0 = rope
        p.rope_cos, p.rope_sin, p.rope_len = cos.data_ptr(), sin.data_ptr(), cos.shape[0]
        p.rope_q_pos0, p.rope_k_pos0 = q_pos0, k_pos0


def _check_inputs(q, k, v, g_q, g_k, v_first, vr_coef, gate):
    if q.dtype not in _DTYPES:
        raise TypeError(f"qknorm attention supports bfloat16 and float32 tensors, got {q.dtype}")
    for name, t in (("k", k), ("v", v), ("v_first", v_first), ("gate_logits", gate)):
        if t is not None and t.dtype != q.dtype:
            raise TypeError(f"{name} has dtype {t.dtype}, expected {q.dtype}")
    assert q.is_cuda and k.is_cuda and v.is_cuda, "q, k, v must be device tensors"
    B, H, Sq, D = q.shape
    assert k.dim() == 4 and v.shape == k.shape and k.shape[0] == B and k.shape[3] == D, "k/v shape mismatch"
    assert H % k.shape[1] == 0, "number of query heads must be a multiple of the kv heads"
    assert g_q.numel() in (1, D), "gain must have 1 or head_dim elements"
    assert g_k is None or g_k.numel() in (1, D), "k_gain must have 1 or head_dim elements"
    assert (v_first is None) == (vr_coef is None), "v_first and vr_coef go together"
    if v_first is not None:
        assert v_first.shape == v.shape and vr_coef.numel() == 2
    if gate is not None:
        assert gate.shape == (B, Sq, H), "gate_logits must be [B, Sq, H]"


def _forward(q, k, v, g_q, g_k, v_first, vr_coef, gate, gate_scale, eps, sm_scale, causal, q_start, y, rope=None,
             inference=False, flags=0):
    """Launch the forward on canonical 4-D views; returns (lse [B,H,Sq] fp32, kv workspace).  `y` is written.
    The kv workspace holds the normalised keys (and mixed values) the backward can reuse.  `inference`: no
    backward will follow, so a decode-shaped call (few query rows, long cache) may take the split-key kernels.
    `flags`: SEGPT_FLAG_* bits of the call itself (SEGPT_FLAG_NO_NORM for attention without QK-norm)."""
    lib = _lib.load()
    B, H, Sq, _ = q.shape
    lse = torch.empty((B, H, Sq), dtype=torch.float32, device=q.device)
    if q.numel() == 0:  # empty batch / no query rows: nothing to launch (the C ABI rejects zero sizes)
        return lse, torch.empty(0, dtype=torch.uint8, device=q.device)
    p = _lib.new_params()
    _fill_common(p, q, k, v, y, lse, g_q, g_k, v_first, vr_coef, gate, gate_scale, eps, sm_scale, causal, q_start, rope)
    p.flags = flags | (_lib.SEGPT_FLAG_DECODE if inference else 0)  # before sizing: a decode-shaped call needs less
    kv_ws = _lib.alloc_workspace(lib, p, _lib.SEGPT_WS_KV, q.device)
    p.kv_workspace, p.kv_workspace_bytes = kv_ws.data_ptr(), kv_ws.numel()
    with torch.cuda.device(q.device):  # the launch goes to the tensors' device, whatever the current one is
        rc = lib.segpt_attn_fwd(p, torch.cuda.current_stream(q.device).cuda_stream)
    if rc != 0:
        raise _lib.SegptError(rc, "segpt_attn_fwd")
    return lse, kv_ws


def _backward(q, k, v, g_q, g_k, v_first, vr_coef, gate, gate_scale, eps, sm_scale, causal, q_start, y, lse, dy,
              dq, dk, dv, dv_first, dgate, kv_ws=None, rope=None, flags=0):
    """Launch the backward; dq/dk/dv(/dv_first/dgate) are written; returns (dg_q, dg_k, dvr_coef) fp32.
    `kv_ws`: the forward's kv workspace (skips the key/value pre-pass); None allocates a fresh one."""
    lib = _lib.load()
    dev = q.device
    dg_q = torch.empty_like(g_q)
    dg_k = None if g_k is None else torch.empty_like(g_k)
    dcoef = None if vr_coef is None else torch.empty(2, dtype=torch.float32, device=dev)
    if q.numel() == 0:  # no query rows: every gradient is zero
        for t in (dq, dk, dv, dv_first, dgate, dg_q, dg_k, dcoef):
            if t is not None:
                t.zero_()
        return dg_q, dg_k, dcoef
    p = _lib.new_params()
    _fill_common(p, q, k, v, y, lse, g_q, g_k, v_first, vr_coef, gate, gate_scale, eps, sm_scale, causal, q_start, rope)
    p.d_o, p.dq, p.dk, p.dv = _lib.t4(dy), _lib.t4(dq), _lib.t4(dk), _lib.t4(dv)
    p.dv_first = _lib.t4(dv_first)
    p.dgate = _lib.t3(dgate)
    p.dg_q, p.dg_k, p.dvr_coef = _lib.ptr(dg_q), _lib.ptr(dg_k), _lib.ptr(dcoef)
    ws = _lib.alloc_workspace(lib, p, _lib.SEGPT_WS_BWD, dev)
    p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
    p.flags = flags
    if kv_ws is None:
        kv_ws = _lib.alloc_workspace(lib, p, _lib.SEGPT_WS_KV, dev)
    else:
        p.flags |= _lib.SEGPT_FLAG_KV_PREPARED
    p.kv_workspace, p.kv_workspace_bytes = kv_ws.data_ptr(), kv_ws.numel()
    with torch.cuda.device(dev):
        rc = lib.segpt_attn_bwd(p, torch.cuda.current_stream(dev).cuda_stream)
    if rc != 0:
        raise _lib.SegptError(rc, "segpt_attn_bwd")
    return dg_q, dg_k, dcoef


def _lastdim_contig(x):
    return x if x.stride(-1) == 1 else x.contiguous()


def _no_backward_will_follow(*tensors):
    """True when nothing can ask for a gradient of this call: grad mode is off (torch.no_grad / inference_mode,
    as in the reference's generate loop, transformer.py:160) or no tensor input requires one.  Must be evaluated
    by the CALLER of an autograd Function: inside ``forward`` grad mode is always off, and
    ``ctx.needs_input_grad`` mirrors ``requires_grad`` even under no_grad (a Parameter gain keeps it True)."""
    return (not torch.is_grad_enabled()) or not any(t is not None and t.requires_grad for t in tensors)


class _GradModeAtApply:
    """Mix-in for the positional drop-in Functions: records, in ``apply`` (the caller's context), whether a
    backward can follow, for ``forward`` to read."""

    _tls = threading.local()

    @classmethod
    @torch.compiler.disable  # Python-side bookkeeping the compiler cannot trace: a compiled caller breaks the graph here
    def apply(cls, *args, **kwargs):
        outer = getattr(cls._tls, "inference", False)  # a nested apply must leave the outer call's decision in place
        cls._tls.inference = _no_backward_will_follow(*(a for a in args if isinstance(a, torch.Tensor)))
        try:
            return super().apply(*args, **kwargs)
        finally:
            cls._tls.inference = outer

    @classmethod
    def _inference(cls):
        return bool(getattr(cls._tls, "inference", False))


class _CoreFunc(torch.autograd.Function):
    """Canonical-layout op: q [B,H,Sq,D], k/v/v_first [B,Hkv,Sk,D], gate [B,Sq,H]."""

    @staticmethod
    def forward(ctx, q, k, v, g_q, g_k, v_first, vr_coef, gate, gate_scale, eps, sm_scale, causal, q_start, rope=None,
                flags=0, out_bshd=False, inference=False):
        gq32, gk32 = _scale_arg(g_q, q.device), _scale_arg(g_k, q.device)
        coef32 = None if vr_coef is None else vr_coef.detach().to(device=q.device, dtype=torch.float32).reshape(-1).contiguous()
        _check_inputs(q, k, v, gq32, gk32, v_first, coef32, gate)
        q, k, v = _lastdim_contig(q), _lastdim_contig(k), _lastdim_contig(v)
        v_first = None if v_first is None else _lastdim_contig(v_first)
        if sm_scale is None:
            sm_scale = 1.0 / math.sqrt(q.shape[-1])
        if out_bshd:  # [B,H,Sq,D] view of a [B,Sq,H,D] buffer: the layout the output projection consumes
            B, H, Sq, D = q.shape
            y = torch.empty((B, Sq, H, D), dtype=q.dtype, device=q.device).permute(0, 2, 1, 3)
        else:
            y = torch.empty_like(q)
            if y.stride(-1) != 1:
                y = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        lse, kv_ws = _forward(q, k, v, gq32, gk32, v_first, coef32, gate, gate_scale, eps, sm_scale, causal, q_start, y, rope,
                              inference=inference, flags=flags)
        # the normalised keys (bf16 path) are kept for the backward: 1/rep of q's size
        ctx.save_for_backward(q, k, v, g_q, g_k, v_first, vr_coef, gate, y, lse, kv_ws)
        ctx.cfg = (gate_scale, eps, sm_scale, causal, q_start, rope, flags)
        ctx.mark_non_differentiable(lse)
        return y, lse

    @staticmethod
    def backward(ctx, dy, _dlse):
        q, k, v, g_q, g_k, v_first, vr_coef, gate, y, lse, kv_ws = ctx.saved_tensors
        gate_scale, eps, sm_scale, causal, q_start, rope, flags = ctx.cfg
        gq32, gk32 = _scale_arg(g_q, q.device), _scale_arg(g_k, q.device)
        coef32 = None if vr_coef is None else vr_coef.detach().to(device=q.device, dtype=torch.float32).reshape(-1).contiguous()
        dy = _lastdim_contig(dy)
        if dy.dtype != q.dtype:
            dy = dy.to(q.dtype)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        dv_first = None if v_first is None else torch.empty_like(v_first)
        dgate = None if gate is None else torch.empty_like(gate)
        dg_q, dg_k, dcoef = _backward(q, k, v, gq32, gk32, v_first, coef32, gate, gate_scale, eps, sm_scale, causal,
                                      q_start, y, lse, dy, dq, dk, dv, dv_first, dgate, kv_ws, rope, flags)
        dg_q = dg_q.reshape(g_q.shape).to(g_q.dtype)
        if g_k is not None:
            dg_k = dg_k.reshape(g_k.shape).to(g_k.dtype)
        if vr_coef is not None:
            dcoef = dcoef.reshape(vr_coef.shape).to(vr_coef.dtype)
        return dq, dk, dv, dg_q, dg_k, dv_first, dcoef, dgate, None, None, None, None, None, None, None, None, None


def qknorm_attention(q, k, v, g_q, g_k=None, *, v_first=None, vr_coef=None, gate_logits=None, gate_scale=2.0,
                     eps=1e-6, sm_scale=None, causal=True, q_start=0, return_lse=False,
                     rope_cos=None, rope_sin=None, rope_q_pos0=None, rope_k_pos0=0, qk_norm=True, out_bshd=False):
    """Fused QK-norm attention on canonical views.

    q ``[B,H,Sq,D]``; k, v, v_first ``[B,Hkv,Sk,D]`` (any strides, last dim contiguous, rows 16 B
    aligned); g_q, g_k scale parameters of 1 or D elements; vr_coef device tensor ``[2]`` = (c1, c2)
    with ``v' = c1 v + c2 v_first``; gate_logits ``[B,Sq,H]`` with ``y = gate_scale*sigmoid(z)*o``.
    rope_cos / rope_sin ``[len, D/2]``: q and k are the UNROTATED projections and the split-half rotary
    embedding (rope.py:36-56) is applied inside the kernels' loads; query row i sits at position
    ``rope_q_pos0 + i`` (default ``q_start``), key row j at ``rope_k_pos0 + j``.
    ``qk_norm=False``: no RMS normalisation of q and k (eps unused) -- the reference's attention without QK-norm
    (attention.py:233-240); the scale vectors still apply, pass ``g_q = ones(1)`` for the plain op.
    ``out_bshd=True``: the returned ``[B,H,Sq,D]`` tensor is a view of a ``[B,Sq,H,D]`` buffer, so that
    ``y.permute(0, 2, 1, 3).reshape(B, Sq, H*D)`` is the ``b seq (h head_d)`` tensor of attention.py:243 without a copy.
    """
    rope = _rope_arg(rope_cos, rope_sin, rope_q_pos0, rope_k_pos0, q_start, q.device, q.shape[-1])
    inference = _no_backward_will_follow(q, k, v, g_q, g_k, v_first, vr_coef, gate_logits)
    y, lse = _CoreFunc.apply(q, k, v, g_q, g_k, v_first, vr_coef, gate_logits, gate_scale, eps, sm_scale, causal, q_start,
                             rope, 0 if qk_norm else _lib.SEGPT_FLAG_NO_NORM, out_bshd, inference)
    return (y, lse) if return_lse else y


def _canon(x, n_heads):
    """[(h b), S, d] -> [B, H, S, d] view (no copy): head-major flatten of attention.py:199."""
    n, S, d = x.shape
    return x.view(n_heads, n // n_heads, S, d).permute(1, 0, 2, 3)


class QKNormFlashAttnFunc(_GradModeAtApply, torch.autograd.Function):
    """Drop-in for ``TritonFlashAttnQKNormFunc`` (triton_flash_attn_qknorm.py:262-343).

    ``apply(Q, K, V, gain, is_causal=True, q_start=0, k_gain=None, v_first=None, vr_coef=None,
    gate_logits=None, gate_scale=2.0, n_kv_heads=None, eps=1e-6, sm_scale=None, rope_cos=None,
    rope_sin=None)`` -- positional only, as autograd Functions are.  With the rope tables Q and K are the
    unrotated projections (positions ``q_start + i`` for queries, ``j`` for keys, attention.py:191-204).  ``Q [(h b), Nq, d]``, ``K, V [(h b) or (hkv b), Nk, d]`` contiguous
    device tensors (2-D inputs are promoted to 3-D, the output stays 3-D, :278-281).  When K/V carry
    fewer rows than Q they are un-expanded GQA tensors and ``n_kv_heads`` is required; query row
    ``n = h*B + b`` then reads kv row ``(h // rep)*B + b`` exactly as the reference's
    ``repeat_interleave`` expansion does (attention.py:207-218).  Returns ``O`` with Q's shape and dtype.
    """

    @staticmethod
    def forward(ctx, Q, K, V, gain, is_causal=True, q_start=0, k_gain=None, v_first=None, vr_coef=None,
                gate_logits=None, gate_scale=2.0, n_kv_heads=None, eps=1e-6, sm_scale=None, rope_cos=None,
                rope_sin=None):
        assert Q.is_cuda and Q.is_contiguous()
        assert K.is_cuda and K.is_contiguous()
        assert V.is_cuda and V.is_contiguous()
        assert gain.is_cuda
        if Q.ndim == 2:
            Q, K, V = Q.unsqueeze(0), K.unsqueeze(0), V.unsqueeze(0)
            if v_first is not None and v_first.ndim == 2:
                v_first = v_first.unsqueeze(0)
        nq, nk = Q.shape[0], K.shape[0]
        if nk != nq or n_kv_heads is not None or gate_logits is not None:
            if n_kv_heads is None:
                assert gate_logits is not None and nk == nq, "n_kv_heads is required for un-expanded GQA K/V"
                H = Hkv = gate_logits.shape[-1]
            else:
                Hkv = int(n_kv_heads)
                assert nq % nk == 0 and nk % Hkv == 0, "K/V rows must be n_kv_heads * batch"
                H = Hkv * (nq // nk)
        else:
            H = Hkv = 1  # every flattened row is its own (batch, head): plain MHA layout of the reference
        if v_first is not None:
            assert v_first.is_cuda and v_first.is_contiguous()
        q4, k4, v4 = _canon(Q, H), _canon(K, Hkv), _canon(V, Hkv)
        vf4 = None if v_first is None else _canon(v_first, Hkv)
        gq32, gk32 = _scale_arg(gain, Q.device), _scale_arg(k_gain, Q.device)
        coef32 = None if vr_coef is None else vr_coef.detach().to(device=Q.device, dtype=torch.float32).reshape(-1).contiguous()
        _check_inputs(q4, k4, v4, gq32, gk32, vf4, coef32, gate_logits)
        if sm_scale is None:
            sm_scale = 1.0 / math.sqrt(Q.shape[-1])
        O = torch.empty_like(Q)
        rope = _rope_arg(rope_cos, rope_sin, None, 0, q_start, Q.device, Q.shape[-1])
        lse, kv_ws = _forward(q4, k4, v4, gq32, gk32, vf4, coef32, gate_logits, gate_scale, eps, sm_scale, is_causal,
                              q_start, _canon(O, H), rope, inference=QKNormFlashAttnFunc._inference())
        ctx.save_for_backward(lse, Q, K, V, gain, O, k_gain, v_first, vr_coef, gate_logits, kv_ws)
        ctx.cfg = (H, Hkv, gate_scale, eps, sm_scale, bool(is_causal), int(q_start), rope)
        return O

    @staticmethod
    def backward(ctx, grad_output):
        lse, Q, K, V, gain, O, k_gain, v_first, vr_coef, gate, kv_ws = ctx.saved_tensors
        H, Hkv, gate_scale, eps, sm_scale, causal, q_start, rope = ctx.cfg
        grad_output = grad_output.contiguous()
        if grad_output.dtype != Q.dtype:
            grad_output = grad_output.to(Q.dtype)
        if grad_output.ndim == 2:
            grad_output = grad_output.unsqueeze(0)
        dQ, dK, dV = torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V)
        dVf = None if v_first is None else torch.empty_like(v_first)
        dgate = None if gate is None else torch.empty_like(gate)
        gq32, gk32 = _scale_arg(gain, Q.device), _scale_arg(k_gain, Q.device)
        coef32 = None if vr_coef is None else vr_coef.detach().to(device=Q.device, dtype=torch.float32).reshape(-1).contiguous()
        dg_q, dg_k, dcoef = _backward(
            _canon(Q, H), _canon(K, Hkv), _canon(V, Hkv), gq32, gk32,
            None if v_first is None else _canon(v_first, Hkv), coef32, gate, gate_scale, eps, sm_scale, causal, q_start,
            _canon(O, H), lse, _canon(grad_output, H), _canon(dQ, H), _canon(dK, Hkv), _canon(dV, Hkv),
            None if dVf is None else _canon(dVf, Hkv), dgate, kv_ws, rope)
        dgain = dg_q.reshape(gain.shape).to(gain.dtype)
        dk_gain = None if k_gain is None else dg_k.reshape(k_gain.shape).to(k_gain.dtype)
        dcoef = None if vr_coef is None else dcoef.reshape(vr_coef.shape).to(vr_coef.dtype)
        #      Q   K   V   gain   causal q_start k_gain  v_first vr_coef gate  gate_scale n_kv eps sm_scale rope tables
        return dQ, dK, dV, dgain, None, None, dk_gain, dVf, dcoef, dgate, None, None, None, None, None, None


class TritonFlashAttnQKNormFunc(QKNormFlashAttnFunc):
    """The reference's class name WITH the reference kernel's own formula as the default
    (triton_flash_attn_qknorm.py:67-91: L2 normaliser ``rsqrt(sum x^2 + 1e-8)``, logits ``gain * cos``), i.e. the
    family at ``eps = 1e-8 / d, sm_scale = 1 / d``.  ``QKNormFlashAttnFunc`` keeps the live module's defaults
    (RMS normaliser, eps 1e-6, 1/sqrt(d); attention.py:51-80).  Same positional signature; explicit ``eps`` /
    ``sm_scale`` override the defaults."""

    @staticmethod
    def forward(ctx, Q, K, V, gain, is_causal=True, q_start=0, k_gain=None, v_first=None, vr_coef=None,
                gate_logits=None, gate_scale=2.0, n_kv_heads=None, eps=None, sm_scale=None, rope_cos=None,
                rope_sin=None):
        d = Q.shape[-1]
        return QKNormFlashAttnFunc.forward(ctx, Q, K, V, gain, is_causal, q_start, k_gain, v_first, vr_coef, gate_logits,
                                           gate_scale, n_kv_heads, 1e-8 / d if eps is None else eps,
                                           1.0 / d if sm_scale is None else sm_scale, rope_cos, rope_sin)


class FlashAttnFunc(_GradModeAtApply, torch.autograd.Function):
    """Drop-in for the reference's attention WITHOUT QK-norm, ``TritonFlashAttnFunc``
    (triton_flash_attn.py:208-297; called at attention.py:240): ``apply(Q, K, V, q_start=0, is_causal=True,
    n_kv_heads=None)`` -- note the argument order, which differs from the QK-norm op's.  ``Q [(h b), Nq, d]``,
    ``K, V [(h b) or (hkv b), Nk, d]`` contiguous device tensors (2-D promoted to 3-D, :222-226); logits are
    ``Q K^T / sqrt(d)`` (:232).  Same kernels as the QK-norm op with both normalisers fixed at 1
    (SEGPT_FLAG_NO_NORM).  The reference backward's mis-masked diagonal tile (BQ=32 != BK=64,
    triton_flash_attn.py:176,292-293) is not reproduced: gradients are the exact ones."""

    @staticmethod
    def forward(ctx, Q, K, V, q_start=0, is_causal=True, n_kv_heads=None):
        assert Q.is_cuda and Q.is_contiguous()
        assert K.is_cuda and K.is_contiguous()
        assert V.is_cuda and V.is_contiguous()
        if Q.ndim == 2:
            Q, K, V = Q.unsqueeze(0), K.unsqueeze(0), V.unsqueeze(0)
        nq, nk = Q.shape[0], K.shape[0]
        if n_kv_heads is None:
            assert nk == nq, "n_kv_heads is required for un-expanded GQA K/V"
            H = Hkv = 1
        else:
            Hkv = int(n_kv_heads)
            assert nq % nk == 0 and nk % Hkv == 0, "K/V rows must be n_kv_heads * batch"
            H = Hkv * (nq // nk)
        q4, k4, v4 = _canon(Q, H), _canon(K, Hkv), _canon(V, Hkv)
        one = torch.ones(1, dtype=torch.float32, device=Q.device)
        _check_inputs(q4, k4, v4, one, None, None, None, None)
        sm_scale = 1.0 / math.sqrt(Q.shape[-1])
        O = torch.empty_like(Q)
        lse, kv_ws = _forward(q4, k4, v4, one, None, None, None, None, 1.0, 0.0, sm_scale, is_causal, q_start, _canon(O, H),
                              None, inference=FlashAttnFunc._inference(), flags=_lib.SEGPT_FLAG_NO_NORM)
        ctx.save_for_backward(lse, Q, K, V, O, one, kv_ws)
        ctx.cfg = (H, Hkv, sm_scale, bool(is_causal), int(q_start))
        return O

    @staticmethod
    def backward(ctx, grad_output):
        lse, Q, K, V, O, one, kv_ws = ctx.saved_tensors
        H, Hkv, sm_scale, causal, q_start = ctx.cfg
        grad_output = grad_output.contiguous()
        if grad_output.dtype != Q.dtype:
            grad_output = grad_output.to(Q.dtype)
        if grad_output.ndim == 2:
            grad_output = grad_output.unsqueeze(0)
        dQ, dK, dV = torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V)
        _backward(_canon(Q, H), _canon(K, Hkv), _canon(V, Hkv), one, None, None, None, None, 1.0, 0.0, sm_scale, causal,
                  q_start, _canon(O, H), lse, _canon(grad_output, H), _canon(dQ, H), _canon(dK, Hkv), _canon(dV, Hkv),
                  None, None, kv_ws, None, _lib.SEGPT_FLAG_NO_NORM)
        return dQ, dK, dV, None, None, None
