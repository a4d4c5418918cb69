"""nn.Module with the interface and state-dict layout of the reference's QK-norm attention module."""

from __future__ import annotations

import torch
import torch.nn as nn

from .function import QKNormFlashAttnFunc


class SelfDotProductAttnQKNorm(nn.Module):
    """Same constructor, parameter (``gain`` of shape ``[1]``, fp32, init 1) and forward signature as
    sample_efficient_gpt/transformer/attention.py:30-80; the normalise + SDPA sequence of its forward
    is replaced by one fused kernel call.  Inputs are the flattened ``[(h b), S, d]`` tensors the
    reference's MultiHeadSelfAttention passes (attention.py:231-232); K/V may be left un-expanded when
    ``n_kv_heads`` is given.
    """

    def __init__(self, head_dim: int, n_kv_heads: int | None = None):
        super().__init__()
        self.head_dim = head_dim
        self.n_kv_heads = n_kv_heads
        self.gain = nn.Parameter(torch.tensor([1.0], dtype=torch.float32))

    def forward(self, Q, K, V, is_causal: bool = True, q_start: int = 0):
        lead = Q.shape[:-2]
        if Q.dim() > 3:  # "... seq_len d_k" inputs: fold the leading dims like the reference's kernels expect
            Q, K, V = (t.reshape(-1, *t.shape[-2:]) for t in (Q, K, V))
        n_kv = self.n_kv_heads if K.shape[0] != Q.shape[0] else None
        out = QKNormFlashAttnFunc.apply(Q.contiguous(), K.contiguous(), V.contiguous(), self.gain, is_causal, q_start,
                                        None, None, None, None, 2.0, n_kv)
        return out.reshape(*lead, *out.shape[-2:]) if len(lead) > 1 else out


class KVCache:
    """Key/value cache with the interface of the reference's (attention.py:15-27: no-argument constructor,
    ``append(k, v) -> (keys, values)``, ``keys`` / ``values`` None until the first append), held the way the fused
    kernels read it: canonical ``[B, Hkv, len, D]`` views of one pre-allocated buffer per tensor that grows by
    doubling (the reference concatenates on every step), un-expanded GQA heads, and RAW projections -- the
    rotary embedding and the RMS normalisation of the keys are applied by the kernel as it reads them."""

    def __init__(self, capacity: int = 0):
        self.keys = None
        self.values = None
        self.length = 0
        self._cap = int(capacity)
        self._kbuf = self._vbuf = None
        self._mbuf = None  # mixed values c1 v + c2 v_first of the layer that hands them on as v1 (filled on demand)
        self._mlen = 0

    def append(self, k, v):
        B, Hkv, S, D = k.shape
        need = self.length + S
        if self._kbuf is None or need > self._kbuf.shape[2]:
            cap = max(need, 2 * (0 if self._kbuf is None else self._kbuf.shape[2]), self._cap, 128)
            kb = torch.empty((B, Hkv, cap, D), dtype=k.dtype, device=k.device)
            vb = torch.empty((B, Hkv, cap, D), dtype=v.dtype, device=v.device)
            if self._kbuf is not None:
                kb[:, :, : self.length].copy_(self._kbuf[:, :, : self.length])
                vb[:, :, : self.length].copy_(self._vbuf[:, :, : self.length])
            self._kbuf, self._vbuf = kb, vb
        self._kbuf[:, :, self.length : need].copy_(k)
        self._vbuf[:, :, self.length : need].copy_(v)
        self.length = need
        self.keys, self.values = self._kbuf[:, :, :need], self._vbuf[:, :, :need]
        return self.keys, self.values

    @property
    def mixed_length(self):
        """Rows of the mixed value tensor kept so far (see ``append_mixed``)."""
        return self._mlen

    def append_mixed(self, vm_new):
        """Rows [mixed_length, length) of the mixed value tensor (the ``V`` a value-residual layer returns for later
        layers, attention.py:228,267), kept beside the raw values so that a generation step mixes only its new
        rows instead of the whole cache.  Call after ``append`` of the same step with exactly the rows that are
        missing (``length - mixed_length`` of them: more than the step's own when earlier steps did not keep
        theirs, e.g. a prefill that ran with gradients enabled); returns the ``[B, Hkv, length, D]`` view."""
        S = vm_new.shape[2]
        if self._mlen + S != self.length:
            raise ValueError(f"append_mixed got {S} rows, the cache is missing rows [{self._mlen}, {self.length})")
        if self._mbuf is None or self._mbuf.shape[2] < self._vbuf.shape[2]:
            mb = torch.empty_like(self._vbuf)
            if self._mbuf is not None:
                mb[:, :, : self._mlen].copy_(self._mbuf[:, :, : self._mlen])
            self._mbuf = mb
        self._mbuf[:, :, self._mlen : self.length].copy_(vm_new)
        self._mlen = self.length
        return self._mbuf[:, :, : self.length]


class _Linear(nn.Module):
    """Bias-free linear layer with the reference's parameter name (`<name>.linear.weight`) and
    initialisation (core.py:11-23)."""

    def __init__(self, in_features, out_features, device=None, dtype=None):
        super().__init__()
        self.linear = nn.Linear(in_features, out_features, bias=False, device=device, dtype=dtype)
        sigma = 1.0 / (in_features**0.5)
        nn.init.trunc_normal_(self.linear.weight, std=sigma, a=-3 * sigma, b=3 * sigma)

    def forward(self, x):
        return self.linear(x)


class MultiHeadSelfAttention(nn.Module):
    """The reference's attention module (attention.py:84-267) around ONE fused kernel call: same constructor,
    state-dict names (``qkv.linear.weight``, ``out.linear.weight``, ``sdpa_qknorm.gain``, ``alpha1`` / ``alpha2`` /
    ``scale``, ``attn_gate.linear.weight``) and ``forward(x, token_positions=None, v1=None, kv_cache=None)
    -> (attn_out, V)``.

    What the reference does in separate passes happens inside the kernels here: q / k / v are strided views of
    the projection output (no ``rearrange(...).contiguous()``), the rotary embedding and the RMS normalisation
    are applied as the rows are loaded, GQA heads are indexed instead of expanded, the value-residual mix is
    folded into the V loads, the per-head gate into the output write, and the output lands in ``b seq (h d)``
    layout for the output projection.  ``kv_cache`` is this package's ``KVCache`` (raw, un-expanded keys).

    Differences a caller can see: a layer that is handed ``v1`` returns ``None`` as its second output unless
    ``always_return_values`` is set (the reference's model only ever uses the first layer's, transformer.py:135-136);
    the returned ``V`` (the tensor later layers take as ``v1``, attention.py:267) is
    the mixed value tensor as an un-expanded ``[b, hkv, Sk, d]`` view (the reference returns the flattened,
    ``repeat_interleave``-expanded ``[(h b), Sk, d]`` one, whose rows are equal within a GQA group); ``v1`` is
    accepted in that layout, in the reference's, and as ``[(hkv b), Sk, d]``.  As in the reference, ``token_positions`` is not used (positions follow from the cache length,
    attention.py:185-195).  ``gating="elementwise"`` is applied after the kernel (it is not per head).
    """

    def __init__(self, d_model: int, n_heads: int, n_kv_heads: int | None = None, theta: float = 10_000,
                 max_seq_len: int = 4096, qknorm: bool = False, value_residual: bool = False, gating=False,
                 device=None, dtype=None):
        super().__init__()
        assert d_model % n_heads == 0, "Hidden dim must be divisible by n_heads"
        self.n_heads = n_heads
        self.n_kv_heads = int(n_kv_heads) if n_kv_heads is not None else n_heads
        if self.n_heads % self.n_kv_heads != 0:
            raise ValueError(f"Invalid GQA: n_heads={self.n_heads} not divisible by n_kv_heads={self.n_kv_heads}")
        head_dim = d_model // n_heads
        # rope.py:12-34: angle(pos, j) = pos * theta^(-2j/d); non-persistent buffers named as in the reference
        j = torch.arange(0, head_dim // 2, device=device)
        ang = torch.outer(torch.arange(max_seq_len, device=device), theta ** (-2 * j / head_dim))
        self.rope = nn.Module()
        self.rope.register_buffer("cos", ang.cos().float(), persistent=False)
        self.rope.register_buffer("sin", ang.sin().float(), persistent=False)
        self.qkv = _Linear(d_model, (n_heads + 2 * self.n_kv_heads) * head_dim, device=device, dtype=dtype)
        self.out = _Linear(d_model, d_model, device=device, dtype=dtype)
        self.qknorm = qknorm
        if qknorm:
            self.sdpa_qknorm = SelfDotProductAttnQKNorm(head_dim, self.n_kv_heads)
            if device is not None:
                self.sdpa_qknorm.to(device)
        else:
            self.register_buffer("_unit_gain", torch.ones(1, device=device), persistent=False)
        self.value_residual = bool(value_residual)
        if value_residual:
            self.alpha1 = nn.Parameter(torch.tensor([1.0], device=device))
            self.alpha2 = nn.Parameter(torch.tensor([0.0], device=device))
            self.scale = nn.Parameter(torch.tensor([1.0], device=device))
        else:
            self.register_buffer("alpha1", torch.tensor([1.0], device=device), persistent=False)
            self.register_buffer("alpha2", torch.tensor([0.0], device=device), persistent=False)
            self.register_buffer("scale", torch.tensor([1.0], device=device), persistent=False)
        # attention.py:267 returns the mixed V from every layer, but only the first layer's is ever used
        # (transformer.py:135-136: `if v1 is None: v1 = v`).  False: layers that are GIVEN v1 return None instead
        # of spending an elementwise pass (over the whole cache at generation time) on a tensor nobody reads.
        self.always_return_values = False
        self.gating = gating
        if gating:
            gate_in, gate_out = {"elementwise": (d_model, d_model), "per-head": (d_model, n_heads),
                                 "per-head-hd": (head_dim, n_heads)}.get(gating, (None, None))
            if gate_in is None:
                raise ValueError(f"{self.gating=} is undefined")
            self.attn_gate = _Linear(gate_in, gate_out, device=device, dtype=dtype)

    def forward(self, x, token_positions=None, v1=None, kv_cache: KVCache | None = None):
        from .function import _canon
        from .library_op import qknorm_attention_op

        b, S, d_model = x.shape
        H, Hkv = self.n_heads, self.n_kv_heads
        d = d_model // H
        q_out, kv_out = H * d, Hkv * d
        proj = self.qkv(x)
        # strided [B, heads, S, d] views of the projection output: nothing is copied or re-laid out
        q = proj[..., :q_out].unflatten(-1, (H, d)).permute(0, 2, 1, 3)
        k = proj[..., q_out : q_out + kv_out].unflatten(-1, (Hkv, d)).permute(0, 2, 1, 3)
        v = proj[..., q_out + kv_out :].unflatten(-1, (Hkv, d)).permute(0, 2, 1, 3)
        q_start = 0
        if kv_cache is not None:
            q_start = kv_cache.length
            k, v = kv_cache.append(k, v)
        Sk = k.shape[2]
        v_first = vr_coef = None
        v_mixed = v if v1 is None or self.always_return_values else None
        if self.value_residual:  # attention.py:222-228; with the buffers (1, 0, 1) the line is the identity in fp32
            if v1 is None:
                v_first = v
            elif v1.dim() == 4:
                v_first = v1
            elif v1.shape[0] == Hkv * b:
                v_first = _canon(v1.reshape(Hkv * b, Sk, d), Hkv)
            else:  # the reference's expanded layout: rows of a GQA group are copies, take the first of each
                v_first = _canon(v1.reshape(H * b, Sk, d), H)[:, :: H // Hkv]
            n = torch.rsqrt(self.alpha1**2 + self.alpha2**2 + 1e-8)
            vr_coef = torch.cat([self.scale * self.alpha1 * n, self.scale * self.alpha2 * n]).float()
            # The returned tensor only (the kernel mixes on its own, in fp32): built when a later layer can take it
            # as v1, with fp32 coefficients like the reference's promotion (attention.py:228), and, during cached
            # generation, for the new rows only.
            if v_mixed is not None:
                mix = lambda a, f: (vr_coef[0] * a.float() + vr_coef[1] * f.float()).to(v.dtype)
                if kv_cache is not None and v1 is None and not torch.is_grad_enabled():
                    # every row the cache does not hold yet: the step's own, and any that earlier steps mixed
                    # outside the cache (a prefill with gradients enabled takes the full mix below)
                    m0 = kv_cache.mixed_length
                    v_mixed = kv_cache.append_mixed(mix(v[:, :, m0:], v_first[:, :, m0:]))
                else:
                    v_mixed = mix(v, v_first)
        gate_logits = None
        if self.gating == "per-head":
            gate_logits = self.attn_gate(x)
        elif self.gating == "per-head-hd":
            gate_logits = self.attn_gate(x[..., :d])
        gain = self.sdpa_qknorm.gain if self.qknorm else self._unit_gain
        # the registered op: one opaque node under torch.compile and non-reentrant checkpointing
        y = qknorm_attention_op(q, k, v, gain, None, v_first=v_first, vr_coef=vr_coef, gate_logits=gate_logits, gate_scale=2.0,
                             causal=True, q_start=q_start, rope_cos=self.rope.cos, rope_sin=self.rope.sin,
                             rope_q_pos0=q_start, rope_k_pos0=0, qk_norm=self.qknorm, out_bshd=True)
        attn_cat = y.permute(0, 2, 1, 3).reshape(b, S, H * d)  # a view: the kernel wrote this layout
        if self.gating == "elementwise":
            attn_cat = (2.0 * self.attn_gate(x).sigmoid()) * attn_cat
        return self.out(attn_cat), v_mixed  # later layers take the second one as v1
