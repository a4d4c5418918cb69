"""CPU oracle: QK-norm causal GQA attention, forward and backward.

TEST INFRASTRUCTURE ONLY -- the product path (sample_efficient_gpt_amd) never
imports this file.  It restates, in plain CPU PyTorch (fp32/fp64), what the
reference computes on its attention path:

* the live QK-norm module, `sample_efficient_gpt/transformer/attention.py:43-80`
  (RMS normaliser, eps 1e-6 on the mean, scalar gain on q, SDPA's 1/sqrt(d),
  `k_idx <= q_start + q_idx` mask)                        -> ``live_module_variant_a``
* the fused Triton op's dense mathematics,
  `sample_efficient_gpt/transformer/ops/triton_flash_attn_qknorm.py:57-115`
  (L2 normaliser, eps 1e-8 on the sum, logit = gain*cos)  -> ``fused_kernel_variant_b``
* the CPU monkey patch `sample_efficient_gpt/scripts/hf/convert_imu1_checkpoint.py:73-89`
  (RMS, eps 1e-8, logit = gain*d*cos)                     -> ``cpu_patch_variant_c``
* the attention without QK-norm, `attention.py:233-240` (SDPA) and `TritonFlashAttnFunc`,
  `sample_efficient_gpt/transformer/ops/triton_flash_attn.py:208-297`   -> ``plain_flash_variant``
  (the family with ``qk_norm=False``)
* the whole module `MultiHeadSelfAttention.forward`, `attention.py:175-267` (projection, RoPE, GQA
  expansion, KV cache, value residual, attention, gate, output projection)   -> ``mhsa_forward``
* the caller glue of `attention.py:199-255`: `(h b)` head-major flatten, GQA
  `repeat_interleave`, value-residual mix, per-head `2*sigmoid` gate
                                                          -> ``flatten_heads`` ... ``caller_glue``

and the one generalised family all three are members of (``attention_forward``):

    s_ij = sm_scale * (a_i q_i * g_q) . (b_j k_j * g_k),   a_i = rsqrt(mean(q_i^2) + eps)

What pins each function (the reference holds no tests or golden vectors for
this path, so every pin is mathematical -- see tests/test_oracle.py):

* ``attention_forward``   brute-force masked softmax; pinned against
  ``torch.nn.functional.scaled_dot_product_attention`` (library routine),
  ``torch.logsumexp``, scale invariance of q/k rows, causality perturbation,
  V=1 => O=1, row 0 == v'[0], GQA native == expanded.
* ``attention_backward_explicit``  hand-derived chain rule; pinned against
  ``torch.autograd`` through ``attention_forward`` in fp64 and ``gradcheck``.
* variants A/B/C           each written from its own reference lines with its own
  normaliser; pinned by the family remap (eps, sm_scale) equality in fp64.
* ``plain_flash_variant``   pinned against ``F.scaled_dot_product_attention`` and the family with
  ``qk_norm=False``; the ``qk_norm=False`` explicit backward against autograd in fp64.
* layout helpers           pinned by brute-force python indexing on tiny tensors.
* ``mhsa_forward``          the whole module forward (attention.py:175-267) in the reference's flattened
  layouts; pinned against the separately written ``caller_glue`` + ``apply_rope`` composition, a per-(batch,
  head) python loop over plain softmax attention, and prefill + cached single-token steps == one full pass.

The exact bf16 rounding order of variant A (normalise -> round -> times
bf16(gain) -> round, attention.py:59-62) is restated in ``live_module_variant_a``
but no reference-held vector exists for it: that rounding order is
"parity unpinned"; its effect (<= 1 bf16 ulp on the normalised q) is far inside
the 2e-2 tolerance the GPU parity tests use.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------- helpers


def rms_inv(x: torch.Tensor, eps: float) -> torch.Tensor:
    """rsqrt(mean(x^2, last dim) + eps), keepdim.  attention.py:56-57."""
    return torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def visibility_mask(sq: int, sk: int, causal: bool, q_start: int, device=None) -> torch.Tensor:
    """[sq, sk] bool, True where key j is visible to query i.  attention.py:72-77."""
    if not causal:
        return torch.ones(sq, sk, dtype=torch.bool, device=device)
    qi = q_start + torch.arange(sq, device=device)
    kj = torch.arange(sk, device=device)
    return kj[None, :] <= qi[:, None]


def _vec(g, d, like):
    """Scale parameter as a [d] vector: None -> ones, numel 1 -> broadcast."""
    if g is None:
        return torch.ones(d, dtype=like.dtype, device=like.device)
    g = g.to(like.dtype).reshape(-1)
    if g.numel() == 1:
        return g.expand(d)
    assert g.numel() == d, f"scale vector must have 1 or {d} elements"
    return g


# --------------------------------------------------------------------------- rotary embedding (the step before)


def rope_tables(max_seq_len: int, theta_base: float, d_k: int, dtype=torch.float64):
    """cos, sin [max_seq_len, d_k // 2] with angle(pos, j) = pos * theta_base ** (-2 j / d_k).  rope.py:12-24."""
    j = torch.arange(0, d_k // 2, dtype=dtype)
    inv_freqs = torch.as_tensor(theta_base, dtype=dtype) ** (-2 * j / d_k)
    ang = torch.outer(torch.arange(max_seq_len, dtype=dtype), inv_freqs)
    return ang.cos(), ang.sin()


def apply_rope(x, cos, sin, pos0: int = 0):
    """Split-half rotation of x [..., S, D]: pairs (j, j + D/2); row s uses table row pos0 + s.  rope.py:36-56
    (the reference computes in fp32 and casts back to the input dtype; here the caller's dtype is kept)."""
    S, D = x.shape[-2], x.shape[-1]
    half = D // 2
    c = cos[pos0 : pos0 + S].to(x.dtype)
    sn = sin[pos0 : pos0 + S].to(x.dtype)
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * c - x2 * sn, x1 * sn + x2 * c], dim=-1)


# --------------------------------------------------------------------------- family forward


def attention_forward(
    q,
    k,
    v,
    g_q=None,
    g_k=None,
    *,
    eps: float = 1e-6,
    sm_scale: float | None = None,
    causal: bool = True,
    q_start: int = 0,
    v_first=None,
    vr_coef=None,
    gate_logits=None,
    gate_scale: float = 2.0,
    rope=None,
    rope_q_pos0: int | None = None,
    rope_k_pos0: int = 0,
    qk_norm: bool = True,
):
    """Generalised QK-norm attention in canonical layout.

    q [B,H,Sq,D]; k, v, v_first [B,Hkv,Sk,D]; g_q, g_k numel 1 or D;
    vr_coef (c1, c2) tensor/sequence; gate_logits [B,Sq,H].
    Query head h reads kv head h // (H // Hkv)  (attention.py:207-218).
    rope = (cos, sin) tables: q and k are rotated before the normalisation, as the reference's caller does
    (attention.py:202-204); query row i sits at position rope_q_pos0 + i (default q_start, attention.py:191-195),
    key row j at rope_k_pos0 + j.
    qk_norm=False: both normalisers are 1 (eps unused) -- the reference's attention without QK-norm
    (attention.py:233-240, triton_flash_attn.py:208-297) when g_q = 1 and g_k is None.
    Computes in the dtype of ``q`` (callers pass fp32 or fp64).
    Returns (y, lse, o_ungated, v_mixed); lse is in natural-log units.
    """
    B, H, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    assert H % Hkv == 0
    rep = H // Hkv
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    gq = _vec(g_q, D, q)
    gk = _vec(g_k, D, q)
    if rope is not None:
        q = apply_rope(q, rope[0], rope[1], q_start if rope_q_pos0 is None else rope_q_pos0)
        k = apply_rope(k, rope[0], rope[1], rope_k_pos0)

    qn = q * (rms_inv(q, eps) if qk_norm else 1.0) * gq
    kn = k * (rms_inv(k, eps) if qk_norm else 1.0) * gk
    if vr_coef is not None:
        assert v_first is not None
        c = vr_coef if torch.is_tensor(vr_coef) else torch.tensor(vr_coef, dtype=q.dtype)
        c = c.to(q.dtype)
        vm = c[0] * v + c[1] * v_first
    else:
        vm = v
    kx = kn.repeat_interleave(rep, dim=1)
    vx = vm.repeat_interleave(rep, dim=1)

    s = torch.einsum("bhid,bhjd->bhij", qn, kx) * sm_scale
    vis = visibility_mask(Sq, Sk, causal, q_start, device=q.device)
    s = s.masked_fill(~vis, float("-inf"))
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse[..., None])
    o = torch.einsum("bhij,bhjd->bhid", p, vx)
    if gate_logits is not None:
        gate = gate_scale * torch.sigmoid(gate_logits.to(q.dtype))  # [B,Sq,H]
        y = o * gate.permute(0, 2, 1)[..., None]
    else:
        y = o
    return y, lse, o, vm


def attention_forward_sdpa(q, k, v, g_q=None, g_k=None, *, eps=1e-6, sm_scale=None, causal=True):
    """Same family through the library routine SDPA (q_start == 0, no extras).

    This is also the shape of the reference's live path (normalise, then
    `F.scaled_dot_product_attention(is_causal=True)`, attention.py:80) and is
    what bench.py times as the CPU baseline.
    """
    B, H, Sq, D = q.shape
    rep = H // k.shape[1]
    gq = _vec(g_q, D, q)
    gk = _vec(g_k, D, q)
    qn = q * rms_inv(q, eps) * gq
    kn = (k * rms_inv(k, eps) * gk).repeat_interleave(rep, dim=1)
    vx = v.repeat_interleave(rep, dim=1)
    return F.scaled_dot_product_attention(qn, kn, vx, is_causal=causal, scale=sm_scale)


# --------------------------------------------------------------------------- explicit backward


def attention_backward_explicit(
    q,
    k,
    v,
    g_q,
    g_k,
    dy,
    *,
    eps=1e-6,
    sm_scale=None,
    causal=True,
    q_start=0,
    v_first=None,
    vr_coef=None,
    gate_logits=None,
    gate_scale=2.0,
    qk_norm=True,
):
    """Hand-written chain rule (no autograd).  Returns a dict of gradients.

    Follows the structure of the reference backward kernel
    (triton_flash_attn_qknorm.py:177-255: P from LSE, dV = P^T dO, dP = dO V^T,
    dS = P*(dP - D), then through both normalisers), written for the mean
    normaliser and vector scales.
    """
    B, H, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    rep = H // Hkv
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    gq = _vec(g_q, D, q)
    gk = _vec(g_k, D, q)
    y, lse, o, vm = attention_forward(
        q, k, v, g_q, g_k, eps=eps, sm_scale=sm_scale, causal=causal, q_start=q_start,
        v_first=v_first, vr_coef=vr_coef, gate_logits=gate_logits, gate_scale=gate_scale, qk_norm=qk_norm,
    )
    out = {}
    # gate
    if gate_logits is not None:
        sig = torch.sigmoid(gate_logits.to(q.dtype)).permute(0, 2, 1)  # [B,H,Sq]
        r = (dy * o).sum(-1)
        do = gate_scale * sig[..., None] * dy
        out["dgate_logits"] = (gate_scale * sig * (1 - sig) * r).permute(0, 2, 1)
    else:
        do = dy
    delta = (do * o).sum(-1)  # [B,H,Sq]

    a = rms_inv(q, eps) if qk_norm else torch.ones_like(q[..., :1])  # [B,H,Sq,1]
    b = rms_inv(k, eps) if qk_norm else torch.ones_like(k[..., :1])
    proj = 1.0 if qk_norm else 0.0  # without a normaliser its own gradient term vanishes
    qn = q * a * gq
    kn = k * b * gk
    kx = kn.repeat_interleave(rep, dim=1)
    vx = vm.repeat_interleave(rep, dim=1)
    s = torch.einsum("bhid,bhjd->bhij", qn, kx) * sm_scale
    vis = visibility_mask(Sq, Sk, causal, q_start, device=q.device)
    p = torch.exp(s - lse[..., None]).masked_fill(~vis, 0.0)

    dvx = torch.einsum("bhij,bhid->bhjd", p, do)
    dp = torch.einsum("bhid,bhjd->bhij", do, vx)
    ds = p * (dp - delta[..., None])
    dqn = sm_scale * torch.einsum("bhij,bhjd->bhid", ds, kx)
    dknx = sm_scale * torch.einsum("bhij,bhid->bhjd", ds, qn)
    # sum the rep query heads of each kv group
    dkn = dknx.reshape(B, Hkv, rep, Sk, D).sum(2)
    dvm = dvx.reshape(B, Hkv, rep, Sk, D).sum(2)

    # through the normalisers:  x~ = a x * g,  a = rsqrt(mean x^2 + eps)
    u = dqn * gq
    out["dq"] = a * u - proj * (a**3 / D) * (u * q).sum(-1, keepdim=True) * q
    out["dg_q"] = (dqn * (a * q)).sum(dim=(0, 1, 2))
    w = dkn * gk
    out["dk"] = b * w - proj * (b**3 / D) * (w * k).sum(-1, keepdim=True) * k
    out["dg_k"] = (dkn * (b * k)).sum(dim=(0, 1, 2))

    if vr_coef is not None:
        c = vr_coef if torch.is_tensor(vr_coef) else torch.tensor(vr_coef, dtype=q.dtype)
        c = c.to(q.dtype)
        out["dv"] = c[0] * dvm
        out["dv_first"] = c[1] * dvm
        out["dvr_coef"] = torch.stack([(dvm * v).sum(), (dvm * v_first).sum()])
    else:
        out["dv"] = dvm
    out["y"], out["lse"] = y, lse
    return out


def attention_backward_autograd(q, k, v, g_q, g_k, dy, **kw):
    """Gradients by torch.autograd through ``attention_forward``."""
    v_first = kw.get("v_first")
    vr_coef = kw.get("vr_coef")
    gate_logits = kw.get("gate_logits")
    leaves = {"dq": q, "dk": k, "dv": v, "dg_q": g_q}
    if g_k is not None:
        leaves["dg_k"] = g_k
    if v_first is not None:
        leaves["dv_first"] = v_first
    if vr_coef is not None:
        leaves["dvr_coef"] = vr_coef
    if gate_logits is not None:
        leaves["dgate_logits"] = gate_logits
    req = {n: t.detach().clone().requires_grad_(True) for n, t in leaves.items()}
    kw = dict(kw)
    if v_first is not None:
        kw["v_first"] = req["dv_first"]
    if vr_coef is not None:
        kw["vr_coef"] = req["dvr_coef"]
    if gate_logits is not None:
        kw["gate_logits"] = req["dgate_logits"]
    y, lse, _, _ = attention_forward(req["dq"], req["dk"], req["dv"], req["dg_q"], req.get("dg_k"), **kw)
    names = list(req)
    grads = torch.autograd.grad(y, [req[n] for n in names], grad_outputs=dy)
    out = dict(zip(names, grads))
    out["y"], out["lse"] = y.detach(), lse.detach()
    return out


# --------------------------------------------------------------------------- the three reference variants


def family_params(variant: str, d: int) -> tuple[float, float]:
    """(eps, sm_scale) that place reference variant A/B/C in the family."""
    if variant == "A":
        return 1e-6, 1.0 / math.sqrt(d)
    if variant == "B":
        return 1e-8 / d, 1.0 / d
    if variant == "C":
        return 1e-8, 1.0
    raise ValueError(variant)


def live_module_variant_a(Q, K, V, gain, is_causal: bool = True, q_start: int = 0):
    """The live module, attention.py:43-80, on flattened `[n, S, d]` inputs.

    Normalises in fp32, rounds back to the input dtype, multiplies q by the gain
    cast to the input dtype (a second rounding), then softmax(QK^T/sqrt(d))V with
    the `k_idx <= q_start + q_idx` mask.  The core is written as brute force in
    fp32 so that it also runs for bf16 inputs on CPU without a fused backend.
    """
    eps = 1e-6
    ct = torch.float64 if Q.dtype == torch.float64 else torch.float32  # fp64 callers keep their precision
    qf, kf = Q.to(ct), K.to(ct)
    qn = (qf * rms_inv(qf, eps)).to(Q.dtype)
    kn = (kf * rms_inv(kf, eps)).to(K.dtype)
    qn = qn * gain.to(qn.dtype)
    d = Q.shape[-1]
    s = torch.einsum("nid,njd->nij", qn.to(ct), kn.to(ct)) / math.sqrt(d)
    vis = visibility_mask(Q.shape[-2], K.shape[-2], is_causal, q_start)
    s = s.masked_fill(~vis, float("-inf"))
    return (torch.softmax(s, dim=-1) @ V.to(ct)).to(Q.dtype)


def fused_kernel_variant_b(Q, K, V, gain, is_causal: bool = True, q_start: int = 0):
    """Dense mathematics of the fused Triton op, triton_flash_attn_qknorm.py:57-115.

    alpha = rsqrt(sum q^2 + 1e-8) (:67), beta likewise (:86), logits
    = (q.k) * alpha * beta * gain (:91), no further scaling; LSE = m + log l (:112).
    Returns (O, L).  Computed in the dtype of Q without the kernel's bf16 casts.
    """
    alpha = torch.rsqrt((Q * Q).sum(-1, keepdim=True) + 1e-8)
    beta = torch.rsqrt((K * K).sum(-1, keepdim=True) + 1e-8)
    s = torch.einsum("nid,njd->nij", Q, K) * alpha * beta.transpose(-1, -2) * gain.to(Q.dtype)
    vis = visibility_mask(Q.shape[-2], K.shape[-2], is_causal, q_start)
    s = s.masked_fill(~vis, float("-inf"))
    L = torch.logsumexp(s, dim=-1)
    return torch.exp(s - L[..., None]) @ V, L


def cpu_patch_variant_c(Q, K, V, gain, is_causal: bool = True, q_start: int = 0):
    """The CPU monkey patch, convert_imu1_checkpoint.py:73-89 (RMS, eps 1e-8, no 1/sqrt(d))."""
    qn = Q * rms_inv(Q, 1e-8)
    kn = K * rms_inv(K, 1e-8)
    s = torch.bmm(qn, kn.transpose(1, 2)) * gain.to(Q.dtype)
    vis = visibility_mask(Q.shape[-2], K.shape[-2], is_causal, q_start)
    s = s.masked_fill(~vis, float("-inf"))
    return torch.bmm(torch.softmax(s, dim=-1), V)


# --------------------------------------------------------------------------- caller glue (attention.py:199-255)


def plain_flash_variant(Q, K, V, q_start: int = 0, is_causal: bool = True):
    """The reference's attention WITHOUT QK-norm on flattened [(h b), S, d] tensors: softmax(Q K^T / sqrt(d)) V
    with the `k_idx <= q_start + q_idx` mask -- TritonFlashAttnFunc (triton_flash_attn.py:208-297, scale at
    :232; note the argument order q_start, is_causal) and the SDPA call attention.py:233-236.  Written as
    the brute-force softmax; the family reaches it with qk_norm=False, g_q = 1.  The reference kernel's
    backward mis-masks one diagonal tile when BQ != BK (triton_flash_attn.py:176,292-293); this restatement
    is the exact mathematics instead."""
    d = Q.shape[-1]
    s = torch.einsum("nid,njd->nij", Q, K) / math.sqrt(d)
    vis = visibility_mask(Q.shape[1], K.shape[1], is_causal, q_start, device=Q.device)
    s = s.masked_fill(~vis, float("-inf"))
    return torch.einsum("nij,njd->nid", torch.softmax(s, dim=-1), V)


def flatten_heads(x):
    """[B,H,S,D] -> [(h b),S,D], head-major: n = h*B + b  (attention.py:199-200)."""
    B, H, S, D = x.shape
    return x.permute(1, 0, 2, 3).reshape(H * B, S, D)


def unflatten_heads(x, n_heads: int):
    """[(h b),S,D] -> [B,H,S,D]."""
    n, S, D = x.shape
    B = n // n_heads
    return x.reshape(n_heads, B, S, D).permute(1, 0, 2, 3)


def expand_kv_flat(x, n_kv_heads: int, n_heads: int):
    """GQA expansion on the flattened layout, attention.py:207-218.

    `(h b)` -> `h b`, repeat_interleave(rep) over heads, back to `(h b)`:
    flat query index n = h*B + b reads flat kv index (h // rep)*B + b.
    """
    n, S, D = x.shape
    B = n // n_kv_heads
    rep = n_heads // n_kv_heads
    x = x.reshape(n_kv_heads, B, S, D).repeat_interleave(rep, dim=0)
    return x.reshape(n_heads * B, S, D)


def value_residual_coefs(alpha1, alpha2, scale):
    """(c1, c2) with V' = c1 V + c2 V1 for attention.py:228:
    V <- scale*(alpha1 V + alpha2 V1)*rsqrt(alpha1^2 + alpha2^2 + 1e-8)."""
    n = torch.rsqrt(alpha1**2 + alpha2**2 + 1e-8)
    return scale * alpha1 * n, scale * alpha2 * n


def caller_glue(q, k, v, gain, *, v1=None, alpha1=None, alpha2=None, scale=None, gate_logits=None):
    """attention.py:199-255 from post-RoPE q [B,H,S,D], k/v [B,Hkv,S,D] to the gated
    `b seq (h head_d)` tensor, going through the reference's flattened layout,
    `repeat_interleave` expansion, value-residual line and per-head `2*sigmoid` gate,
    with the live QK-norm module (variant A) in the middle.  Returns (attn_cat, V_mixed_flat).
    """
    B, H, S, D = q.shape
    Hkv = k.shape[1]
    Q = flatten_heads(q)
    K = expand_kv_flat(flatten_heads(k), Hkv, H)
    V = expand_kv_flat(flatten_heads(v), Hkv, H)
    V1 = V if v1 is None else v1.view_as(V)
    one = torch.ones(1, dtype=q.dtype)
    a1 = one if alpha1 is None else alpha1
    a2 = torch.zeros(1, dtype=q.dtype) if alpha2 is None else alpha2
    sc = one if scale is None else scale
    V = sc * (a1 * V + a2 * V1) * torch.rsqrt(a1**2 + a2**2 + 1e-8)
    attn = live_module_variant_a(Q, K, V, gain, True, 0)
    attn = attn.reshape(H, B, S, D).permute(1, 2, 0, 3)  # b seq h head_d
    if gate_logits is not None:
        attn = (2.0 * torch.sigmoid(gate_logits)).unsqueeze(-1) * attn
    return attn.reshape(B, S, H * D), V


# --------------------------------------------------------------------------- the whole attention module


def mhsa_forward(x, w, *, n_heads, n_kv_heads=None, theta=10000.0, max_seq_len=4096, qknorm=True, gating=False,
                 v1=None, cache=None, rope=None):
    """`MultiHeadSelfAttention.forward`, attention.py:175-267, step by step in the reference's own layouts.

    x [b, S, d_model]; `w` holds the weights under the reference's state-dict names: ``qkv.linear.weight``
    [(H+2Hkv)d, d_model], ``out.linear.weight`` [d_model, d_model] (bias-free Linear, core.py:18),
    ``sdpa_qknorm.gain`` [1] when qknorm, ``alpha1`` / ``alpha2`` / ``scale`` [1] (absent: the buffers 1, 0, 1 of
    attention.py:154-159), ``attn_gate.linear.weight`` when gating ("elementwise" / "per-head" / "per-head-hd",
    attention.py:162-171).  `cache`: None or a dict with "keys" / "values" (None or the flattened, head-expanded,
    ROTATED keys and raw values KVCache holds, attention.py:15-27); it is updated like `KVCache.append`.
    `rope`: (cos, sin) tables to use instead of building them from theta (e.g. the fp32 tables of the module under
    test, rope.py:12-24 computes them in fp32).
    Returns (attn_out [b, S, d_model], V [(h b), Sk, d]) -- V is the mixed, expanded value tensor the
    reference hands to later layers (attention.py:267).
    """
    b, S, d_model = x.shape
    H = n_heads
    Hkv = H if n_kv_heads is None else n_kv_heads
    d = d_model // H
    q_out, kv_out = H * d, Hkv * d
    proj = x @ w["qkv.linear.weight"].T                                           # :180
    Q, K, V = proj[..., :q_out], proj[..., q_out:q_out + kv_out], proj[..., q_out + kv_out:]
    past = 0
    if cache is not None and cache.get("keys") is not None:
        past = cache["keys"].shape[1]                                             # :186
    q_start = past if cache is not None else 0
    Q = flatten_heads(Q.reshape(b, S, H, d).permute(0, 2, 1, 3))                  # :199 "b seq (h head_d) -> (h b) seq head_d"
    K = flatten_heads(K.reshape(b, S, Hkv, d).permute(0, 2, 1, 3))
    cos, sin = rope if rope is not None else rope_tables(
        max_seq_len, theta, d, dtype=torch.float64 if x.dtype == torch.float64 else torch.float32)
    Q = apply_rope(Q, cos, sin, q_start)                                          # :202-204, positions past .. past+S-1
    K = apply_rope(K, cos, sin, q_start)
    if Hkv != H:
        K = expand_kv_flat(K, Hkv, H)                                             # :207-211
    V = flatten_heads(V.reshape(b, S, Hkv, d).permute(0, 2, 1, 3))                # :213
    if Hkv != H:
        V = expand_kv_flat(V, Hkv, H)
    if cache is not None:                                                         # :220-221 / KVCache.append
        if cache.get("keys") is not None:
            K, V = torch.cat((cache["keys"], K), dim=1), torch.cat((cache["values"], V), dim=1)
        cache["keys"], cache["values"] = K, V
    V1 = V if v1 is None else v1.reshape(V.shape)                                 # :222-225
    one, zero = torch.ones(1, dtype=x.dtype), torch.zeros(1, dtype=x.dtype)
    a1, a2, sc = w.get("alpha1", one), w.get("alpha2", zero), w.get("scale", one)
    V = sc * (a1 * V + a2 * V1) * torch.rsqrt(a1**2 + a2**2 + 1e-8)               # :228
    if qknorm:
        attn = live_module_variant_a(Q, K, V, w["sdpa_qknorm.gain"], True, q_start)   # :232
    else:
        attn = plain_flash_variant(Q, K, V, q_start, True)                        # :236 / :240
    attn = attn.reshape(H, b, S, d).permute(1, 2, 0, 3)                           # b seq h head_d
    if not gating:
        attn_cat = attn.reshape(b, S, H * d)                                      # :243
    elif gating == "elementwise":
        attn_cat = (2.0 * torch.sigmoid(x @ w["attn_gate.linear.weight"].T)) * attn.reshape(b, S, H * d)   # :246-248
    elif gating == "per-head":
        gate = (2.0 * torch.sigmoid(x @ w["attn_gate.linear.weight"].T)).unsqueeze(-1)                   # :251
        attn_cat = (gate * attn).reshape(b, S, H * d)
    elif gating == "per-head-hd":
        gate = (2.0 * torch.sigmoid(x[..., :d] @ w["attn_gate.linear.weight"].T)).unsqueeze(-1)          # :259
        attn_cat = (gate * attn).reshape(b, S, H * d)
    else:
        raise ValueError(f"gating={gating!r} is undefined")
    return attn_cat @ w["out.linear.weight"].T, V                                 # :265-267
