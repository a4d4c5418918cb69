"""Pins the CPU oracle (oracle/qknorm_attn_oracle.py) by mathematics.

The reference holds no tests, golden vectors or fixtures for its attention path,
so each oracle function is pinned against a library routine, a closed form, an
invariant or brute force chosen so that a dropped term, wrong sign/index or
transposed operand fails at least one check.
"""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import qknorm_attn_oracle as orc

torch.manual_seed(0)
F64 = torch.float64


def _rand(B=2, H=4, Hkv=2, Sq=24, Sk=None, D=8, dtype=F64, seed=0):
    g = torch.Generator().manual_seed(seed)
    Sk = Sq if Sk is None else Sk
    q = torch.randn(B, H, Sq, D, generator=g, dtype=dtype)
    k = torch.randn(B, Hkv, Sk, D, generator=g, dtype=dtype)
    v = torch.randn(B, Hkv, Sk, D, generator=g, dtype=dtype)
    gq = 1 + 0.2 * torch.randn(D, generator=g, dtype=dtype)
    gk = 1 + 0.2 * torch.randn(D, generator=g, dtype=dtype)
    return q, k, v, gq, gk


# ------------------------------------------------------------------ forward core


def test_forward_matches_sdpa_library_routine():
    q, k, v, gq, gk = _rand()
    y, lse, o, _ = orc.attention_forward(q, k, v, gq, gk)
    ref = orc.attention_forward_sdpa(q, k, v, gq, gk)
    assert torch.allclose(y, ref, atol=1e-12)
    assert torch.equal(y, o)


def test_forward_python_loop_bruteforce():
    # element-by-element python loops on a tiny case: catches transposed operands / wrong GQA map
    B, H, Hkv, S, D = 1, 4, 2, 5, 4
    q, k, v, gq, gk = _rand(B, H, Hkv, S, None, D)
    eps, sc = 1e-6, 1 / math.sqrt(D)
    y, lse, _, _ = orc.attention_forward(q, k, v, gq, gk, eps=eps, sm_scale=sc)
    for h in range(H):
        g = h // (H // Hkv)
        for i in range(S):
            qi = q[0, h, i]
            qi = qi / math.sqrt(float((qi * qi).sum()) / D + eps) * gq
            logits = []
            for j in range(i + 1):
                kj = k[0, g, j]
                kj = kj / math.sqrt(float((kj * kj).sum()) / D + eps) * gk
                logits.append(float((qi * kj).sum()) * sc)
            m = max(logits)
            w = [math.exp(x - m) for x in logits]
            z = sum(w)
            out = sum(wj / z * v[0, g, j] for j, wj in enumerate(w))
            assert torch.allclose(y[0, h, i], out, atol=1e-12)
            assert abs(float(lse[0, h, i]) - (m + math.log(z))) < 1e-12


def test_lse_is_logsumexp_of_masked_scores():
    q, k, v, gq, gk = _rand(Sq=16)
    _, lse, _, _ = orc.attention_forward(q, k, v, None, None, eps=0.0, sm_scale=0.5)
    qn = q / q.pow(2).mean(-1, keepdim=True).sqrt()
    kn = (k / k.pow(2).mean(-1, keepdim=True).sqrt()).repeat_interleave(2, 1)
    s = 0.5 * qn @ kn.transpose(-1, -2)
    s = s.masked_fill(torch.triu(torch.ones(16, 16, dtype=torch.bool), 1), -math.inf)
    assert torch.allclose(lse, torch.logsumexp(s, -1), atol=1e-12)


def test_row_scale_invariance():
    q, k, v, gq, gk = _rand()
    y0, l0, _, _ = orc.attention_forward(q, k, v, gq, gk, eps=0.0)
    cq = torch.rand(q.shape[:-1], dtype=F64)[..., None] * 3 + 0.1
    ck = torch.rand(k.shape[:-1], dtype=F64)[..., None] * 3 + 0.1
    y1, l1, _, _ = orc.attention_forward(q * cq, k * ck, v, gq, gk, eps=0.0)
    assert torch.allclose(y0, y1, atol=1e-11) and torch.allclose(l0, l1, atol=1e-11)


def test_prenormalised_unit_scales_reduce_to_plain_sdpa():
    q, k, v, _, _ = _rand(H=2, Hkv=2)
    q = q / q.pow(2).mean(-1, keepdim=True).sqrt()
    k = k / k.pow(2).mean(-1, keepdim=True).sqrt()
    y, _, _, _ = orc.attention_forward(q, k, v, None, None, eps=0.0)
    assert torch.allclose(y, F.scaled_dot_product_attention(q, k, v, is_causal=True), atol=1e-12)


def test_causality_and_simple_closed_forms():
    q, k, v, gq, gk = _rand(Sq=12)
    y, _, _, _ = orc.attention_forward(q, k, v, gq, gk)
    # row 0 sees only key 0
    assert torch.allclose(y[:, :, 0], v.repeat_interleave(2, 1)[:, :, 0], atol=1e-12)
    # perturbing token t leaves rows < t unchanged
    t = 7
    k2, v2, q2 = k.clone(), v.clone(), q.clone()
    k2[:, :, t] += 1.0
    v2[:, :, t] -= 2.0
    q2[:, :, t] *= -1.0
    y2, _, _, _ = orc.attention_forward(q2, k2, v2, gq, gk)
    assert torch.equal(y[:, :, :t], y2[:, :, :t])
    assert not torch.allclose(y[:, :, t:], y2[:, :, t:])
    # V == 1  =>  O == 1
    y1, _, _, _ = orc.attention_forward(q, k, torch.ones_like(v), gq, gk)
    assert torch.allclose(y1, torch.ones_like(y1), atol=1e-12)


def test_noncausal_is_full_softmax():
    q, k, v, gq, gk = _rand(H=2, Hkv=2, Sq=6, Sk=9)
    y, _, _, _ = orc.attention_forward(q, k, v, gq, gk, causal=False)
    ref = orc.attention_forward_sdpa(q, k, v, gq, gk, causal=False)
    assert torch.allclose(y, ref, atol=1e-12)


def test_q_start_mask_is_suffix_of_full_problem():
    # decode: the last 3 queries of a length-10 problem, against all 10 keys
    q, k, v, gq, gk = _rand(Sq=10)
    y, lse, _, _ = orc.attention_forward(q, k, v, gq, gk)
    y2, lse2, _, _ = orc.attention_forward(q[:, :, 7:], k, v, gq, gk, q_start=7)
    assert torch.allclose(y[:, :, 7:], y2, atol=1e-12) and torch.allclose(lse[:, :, 7:], lse2, atol=1e-12)
    m = orc.visibility_mask(3, 10, True, 7)
    assert m.tolist() == [[j <= 7 + i for j in range(10)] for i in range(3)]


def test_gqa_native_equals_expanded():
    q, k, v, gq, gk = _rand(H=6, Hkv=2)
    y, l, _, _ = orc.attention_forward(q, k, v, gq, gk)
    ye, le, _, _ = orc.attention_forward(q, k.repeat_interleave(3, 1), v.repeat_interleave(3, 1), gq, gk)
    assert torch.equal(y, ye) and torch.equal(l, le)


def test_scalar_gain_is_vector_of_equal_entries():
    q, k, v, _, _ = _rand()
    gain = torch.tensor([1.7], dtype=F64)
    y, _, _, _ = orc.attention_forward(q, k, v, gain, None)
    y2, _, _, _ = orc.attention_forward(q, k, v, gain.expand(8).clone(), torch.ones(8, dtype=F64))
    assert torch.equal(y, y2)


# ------------------------------------------------------------------ extras


def test_gate_identities():
    q, k, v, gq, gk = _rand()
    z = torch.randn(2, 24, 4, dtype=F64)
    y0, _, o, _ = orc.attention_forward(q, k, v, gq, gk)
    yg, _, og, _ = orc.attention_forward(q, k, v, gq, gk, gate_logits=z, gate_scale=2.0)
    assert torch.equal(o, og)
    assert torch.allclose(yg, 2 * torch.sigmoid(z).permute(0, 2, 1)[..., None] * y0, atol=1e-14)
    # zero logits and scale 2 => identity (why the reference uses 2*sigmoid)
    yi, _, _, _ = orc.attention_forward(q, k, v, gq, gk, gate_logits=torch.zeros_like(z), gate_scale=2.0)
    assert torch.allclose(yi, y0, atol=1e-14)


def test_value_residual_identities_and_linearity():
    q, k, v, gq, gk = _rand()
    vf = torch.randn_like(v)
    y0, _, _, _ = orc.attention_forward(q, k, v, gq, gk)
    y1, _, _, vm = orc.attention_forward(q, k, v, gq, gk, v_first=vf, vr_coef=(1.0, 0.0))
    assert torch.equal(y0, y1) and torch.equal(vm, v)
    yf, _, _, _ = orc.attention_forward(q, k, vf, gq, gk)
    ym, _, _, _ = orc.attention_forward(q, k, v, gq, gk, v_first=vf, vr_coef=(0.3, 0.7))
    assert torch.allclose(ym, 0.3 * y0 + 0.7 * yf, atol=1e-12)
    c1, c2 = orc.value_residual_coefs(torch.tensor([1.0], dtype=F64), torch.tensor([0.0], dtype=F64), torch.tensor([1.0], dtype=F64))
    assert abs(float(c1) - 1 / math.sqrt(1 + 1e-8)) < 1e-15 and float(c2) == 0.0
    a1, a2, sc = torch.tensor([0.6], dtype=F64), torch.tensor([-0.8], dtype=F64), torch.tensor([1.5], dtype=F64)
    c1, c2 = orc.value_residual_coefs(a1, a2, sc)
    direct = sc * (a1 * v + a2 * vf) * torch.rsqrt(a1**2 + a2**2 + 1e-8)
    assert torch.allclose(c1 * v + c2 * vf, direct, atol=1e-14)


# ------------------------------------------------------------------ reference variants and the family remap


def _flat(Bn=3, S=20, D=16, seed=3):
    g = torch.Generator().manual_seed(seed)
    Q, K, V = (torch.randn(Bn, S, D, generator=g, dtype=F64) for _ in range(3))
    gain = torch.tensor([1.3], dtype=F64)
    return Q, K, V, gain


@pytest.mark.parametrize("variant", ["A", "B", "C"])
def test_variants_are_family_members(variant):
    Q, K, V, gain = _flat()
    D = Q.shape[-1]
    fn = {"A": orc.live_module_variant_a, "B": orc.fused_kernel_variant_b, "C": orc.cpu_patch_variant_c}[variant]
    out = fn(Q, K, V, gain, True, 0)
    L = None
    if variant == "B":
        out, L = out
    eps, sc = orc.family_params(variant, D)
    y, lse, _, _ = orc.attention_forward(Q[None].transpose(0, 1), K[None].transpose(0, 1), V[None].transpose(0, 1), gain, None, eps=eps, sm_scale=sc)
    tol = 1e-6 if variant == "A" else 1e-12  # variant A normalises in fp32 by construction
    assert torch.allclose(y[:, 0], out, atol=tol)
    if L is not None:
        assert torch.allclose(lse[:, 0], L, atol=1e-12)


def test_variants_differ_from_each_other():
    # guards against the remap test passing vacuously (e.g. all three collapsing to one formula)
    Q, K, V, gain = _flat()
    a = orc.live_module_variant_a(Q, K, V, gain)
    b, _ = orc.fused_kernel_variant_b(Q, K, V, gain)
    c = orc.cpu_patch_variant_c(Q, K, V, gain)
    assert (a - b).abs().max() > 1e-3 and (a - c).abs().max() > 1e-3 and (b - c).abs().max() > 1e-3


def test_variant_a_q_start_and_bf16_rounding_points():
    Q, K, V, gain = _flat(S=12)
    full = orc.live_module_variant_a(Q, K, V, gain)
    tail = orc.live_module_variant_a(Q[:, 9:], K, V, gain, True, 9)
    assert torch.allclose(full[:, 9:], tail, atol=1e-12)
    # bf16: output dtype follows input; result close to the fp64 one
    ob = orc.live_module_variant_a(Q.bfloat16(), K.bfloat16(), V.bfloat16(), gain.float())
    assert ob.dtype == torch.bfloat16
    ref = orc.live_module_variant_a(Q.bfloat16().double(), K.bfloat16().double(), V.bfloat16().double(), gain)
    assert (ob.double() - ref).abs().max() < 2e-2


# ------------------------------------------------------------------ layout glue


def test_flatten_and_gqa_expansion_by_indexing():
    B, H, Hkv, S, D = 3, 6, 2, 2, 2
    q = torch.arange(B * H * S * D, dtype=F64).reshape(B, H, S, D)
    k = torch.arange(B * Hkv * S * D, dtype=F64).reshape(B, Hkv, S, D) + 1000
    Q = orc.flatten_heads(q)
    Kx = orc.expand_kv_flat(orc.flatten_heads(k), Hkv, H)
    rep = H // Hkv
    for h in range(H):
        for b in range(B):
            assert torch.equal(Q[h * B + b], q[b, h])
            assert torch.equal(Kx[h * B + b], k[b, h // rep])
    assert torch.equal(orc.unflatten_heads(Q, H), q)


def test_caller_glue_equals_native_family_call():
    B, H, Hkv, S, D = 2, 6, 2, 10, 8
    q, k, v, _, _ = _rand(B, H, Hkv, S, None, D)
    gain = torch.tensor([0.9], dtype=F64)
    z = torch.randn(B, S, H, dtype=F64)
    v1 = torch.randn(B, Hkv, S, D, dtype=F64)
    a1, a2, sc = (torch.tensor([x], dtype=F64) for x in (0.8, 0.5, 1.1))
    v1_flat = orc.expand_kv_flat(orc.flatten_heads(v1), Hkv, H)
    cat, vmix = orc.caller_glue(q, k, v, gain, v1=v1_flat, alpha1=a1, alpha2=a2, scale=sc, gate_logits=z)
    c1, c2 = orc.value_residual_coefs(a1, a2, sc)
    y, _, _, vm = orc.attention_forward(q, k, v, gain, None, v_first=v1, vr_coef=torch.cat([c1, c2]), gate_logits=z, gate_scale=2.0)
    assert torch.allclose(cat, y.permute(0, 2, 1, 3).reshape(B, S, H * D), atol=1e-6)
    assert torch.allclose(vmix, orc.expand_kv_flat(orc.flatten_heads(vm), Hkv, H), atol=1e-12)


# ------------------------------------------------------------------ backward


def _bwd_case(extras):
    q, k, v, gq, gk = _rand(B=2, H=4, Hkv=2, Sq=10, D=8, seed=5)
    kw = {}
    if extras:
        g = torch.Generator().manual_seed(9)
        kw = dict(
            v_first=torch.randn(v.shape, generator=g, dtype=F64),
            vr_coef=torch.tensor([0.4, 0.6], dtype=F64),
            gate_logits=torch.randn(2, 10, 4, generator=g, dtype=F64),
            gate_scale=1.0,
        )
    dy = torch.randn(q.shape, generator=torch.Generator().manual_seed(11), dtype=F64)
    return q, k, v, gq, gk, dy, kw


@pytest.mark.parametrize("extras", [False, True])
def test_explicit_backward_matches_autograd(extras):
    q, k, v, gq, gk, dy, kw = _bwd_case(extras)
    ex = orc.attention_backward_explicit(q, k, v, gq, gk, dy, **kw)
    ag = orc.attention_backward_autograd(q, k, v, gq, gk, dy, **kw)
    for name in ag:
        assert torch.allclose(ex[name], ag[name], atol=1e-10), name
    assert set(ag) <= set(ex)


def test_gradcheck_tiny():
    g = torch.Generator().manual_seed(2)
    q = torch.randn(1, 2, 8, 4, generator=g, dtype=F64, requires_grad=True)
    k = torch.randn(1, 1, 8, 4, generator=g, dtype=F64, requires_grad=True)
    v = torch.randn(1, 1, 8, 4, generator=g, dtype=F64, requires_grad=True)
    vf = torch.randn(1, 1, 8, 4, generator=g, dtype=F64, requires_grad=True)
    gq = (1 + 0.1 * torch.randn(4, generator=g, dtype=F64)).requires_grad_(True)
    gk = (1 + 0.1 * torch.randn(4, generator=g, dtype=F64)).requires_grad_(True)
    c = torch.tensor([0.4, 0.6], dtype=F64, requires_grad=True)
    z = torch.randn(1, 8, 2, generator=g, dtype=F64, requires_grad=True)

    def f(q, k, v, vf, gq, gk, c, z):
        return orc.attention_forward(q, k, v, gq, gk, v_first=vf, vr_coef=c, gate_logits=z, gate_scale=2.0)[0]

    assert torch.autograd.gradcheck(f, (q, k, v, vf, gq, gk, c, z), atol=1e-6)


def test_scalar_gain_grad_is_sum_of_vector_grad_and_gqa_grad_sums_group():
    q, k, v, _, _, dy, _ = _bwd_case(False)
    gain = torch.tensor([1.2], dtype=F64)
    ag = orc.attention_backward_autograd(q, k, v, gain, None, dy)
    ex = orc.attention_backward_explicit(q, k, v, gain.expand(8).clone(), None, dy)
    assert torch.allclose(ag["dg_q"], ex["dg_q"].sum().reshape(1), atol=1e-11)
    # native dK == sum over the group's expanded dK
    rep = 2
    exx = orc.attention_backward_explicit(q, k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1), gain, None, dy)
    assert torch.allclose(ex["dk"], exx["dk"].reshape(2, 2, rep, 10, 8).sum(2), atol=1e-11)
    assert torch.allclose(ex["dv"], exx["dv"].reshape(2, 2, rep, 10, 8).sum(2), atol=1e-11)


def test_variant_b_reference_backward_form_matches_family():
    # the reference kernel's t1/t2 form (triton_flash_attn_qknorm.py:219-246) for the sum normaliser
    Q, K, V, gain = _flat(Bn=2, S=9, D=8)
    D = Q.shape[-1]
    dO = torch.randn_like(Q)
    O, L = orc.fused_kernel_variant_b(Q, K, V, gain)
    alpha = torch.rsqrt((Q * Q).sum(-1, keepdim=True) + 1e-8)
    beta = torch.rsqrt((K * K).sum(-1, keepdim=True) + 1e-8)
    s = (Q @ K.transpose(1, 2)) * alpha * beta.transpose(1, 2) * gain
    vis = orc.visibility_mask(9, 9, True, 0)
    p = torch.exp(s - L[..., None]).masked_fill(~vis, 0.0)
    ds = p * (dO @ V.transpose(1, 2) - (dO * O).sum(-1, keepdim=True))
    t1q = (ds * beta.transpose(1, 2)) @ K
    dq = gain * (alpha * t1q - alpha**3 * (t1q * Q).sum(-1, keepdim=True) * Q)
    t1k = (ds * alpha).transpose(1, 2) @ Q
    dk = gain * (beta * t1k - beta**3 * (t1k * K).sum(-1, keepdim=True) * K)
    dg = (alpha[..., 0] * (Q * t1q).sum(-1)).sum()
    eps, sc = orc.family_params("B", D)
    ex = orc.attention_backward_explicit(Q[None].transpose(0, 1), K[None].transpose(0, 1), V[None].transpose(0, 1), gain.expand(D).clone(), None, dO[None].transpose(0, 1), eps=eps, sm_scale=sc)
    assert torch.allclose(ex["dq"][:, 0], dq, atol=1e-10)
    assert torch.allclose(ex["dk"][:, 0], dk, atol=1e-10)
    assert torch.allclose(ex["dv"][:, 0], p.transpose(1, 2) @ dO, atol=1e-10)
    assert abs(float(ex["dg_q"].sum() - dg)) < 1e-10


# ------------------------------------------------------------------ rotary embedding (rope.py:12-56)


def test_rope_tables_closed_form():
    cos, sin = orc.rope_tables(37, 10000.0, 16)
    assert cos.shape == sin.shape == (37, 8)
    assert torch.allclose(cos[0], torch.ones(8, dtype=F64)) and torch.allclose(sin[0], torch.zeros(8, dtype=F64))
    for pos, j in ((1, 0), (5, 3), (36, 7)):
        ang = pos * 10000.0 ** (-2 * j / 16)
        assert abs(float(cos[pos, j]) - math.cos(ang)) < 1e-12 and abs(float(sin[pos, j]) - math.sin(ang)) < 1e-12
    assert abs(float(cos[9, 0]) - math.cos(9.0)) < 1e-12  # pair 0 turns by one radian per position


def test_rope_is_the_complex_rotation_of_split_half_pairs():
    # independent formulation: z_j = x_j + i x_{j+D/2},  z_j -> z_j * exp(i * angle(pos, j))
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 3, 11, 8, generator=g, dtype=F64)
    cos, sin = orc.rope_tables(32, 100.0, 8)
    pos0 = 5
    got = orc.apply_rope(x, cos, sin, pos0)
    z = torch.complex(x[..., :4], x[..., 4:])
    ang = torch.outer(torch.arange(pos0, pos0 + 11, dtype=F64), 100.0 ** (-2 * torch.arange(4, dtype=F64) / 8))
    zr = z * torch.polar(torch.ones_like(ang), ang)
    assert torch.allclose(got, torch.cat([zr.real, zr.imag], -1), atol=1e-12)
    # a rotation: pair norms and hence the row RMS are unchanged; position 0 is the identity
    assert torch.allclose(got.pow(2).sum(-1), x.pow(2).sum(-1), atol=1e-12)
    assert torch.allclose(orc.apply_rope(x[..., :1, :], cos, sin, 0), x[..., :1, :], atol=1e-15)
    # rotating by pos then by -pos (sin -> -sin) restores x
    assert torch.allclose(orc.apply_rope(got, cos, -sin, pos0), x, atol=1e-12)


def test_rope_in_attention_depends_on_relative_positions_only():
    q, k, v, _, _ = _rand(Sq=20, D=8, seed=5)
    cos, sin = orc.rope_tables(64, 50.0, 8)
    y0, l0, _, _ = orc.attention_forward(q, k, v, None, None, rope=(cos, sin))
    # same relative offsets, every absolute position shifted by 13: logits q_i.k_j are unchanged
    y1, l1, _, _ = orc.attention_forward(q, k, v, None, None, rope=(cos, sin), rope_q_pos0=13, rope_k_pos0=13)
    assert torch.allclose(y0, y1, atol=1e-10) and torch.allclose(l0, l1, atol=1e-10)
    # it is not a no-op, and it equals rotating the inputs by hand
    y_plain, _, _, _ = orc.attention_forward(q, k, v, None, None)
    assert (y0 - y_plain).abs().max() > 1e-3
    y2, _, _, _ = orc.attention_forward(orc.apply_rope(q, cos, sin), orc.apply_rope(k, cos, sin), v, None, None)
    assert torch.allclose(y0, y2, atol=1e-12)
    # decode-style suffix: queries 7.. with q_start=7 sit at positions 7.. by default (attention.py:191-195)
    y3, _, _, _ = orc.attention_forward(q[:, :, 7:], k, v, None, None, q_start=7, rope=(cos, sin))
    assert torch.allclose(y3, y0[:, :, 7:], atol=1e-10)


def test_rope_gradients_by_gradcheck():
    g = torch.Generator().manual_seed(9)
    q = torch.randn(1, 2, 5, 4, generator=g, dtype=F64, requires_grad=True)
    k = torch.randn(1, 1, 5, 4, generator=g, dtype=F64, requires_grad=True)
    v = torch.randn(1, 1, 5, 4, generator=g, dtype=F64, requires_grad=True)
    gq = (1 + 0.2 * torch.randn(4, generator=g, dtype=F64)).requires_grad_(True)
    cos, sin = orc.rope_tables(8, 10.0, 4)
    fn = lambda q, k, v, gq: orc.attention_forward(q, k, v, gq, None, rope=(cos, sin))[0]
    assert torch.autograd.gradcheck(fn, (q, k, v, gq), eps=1e-6, atol=1e-6)


# ------------------------------------------------------------------ attention without QK-norm (plain flash path)


def test_plain_variant_is_sdpa_and_the_family_without_normalisers():
    g = torch.Generator().manual_seed(21)
    n, S, D = 6, 19, 8
    Q = 1.7 * torch.randn(n, S, D, generator=g, dtype=F64)  # NOT unit-RMS rows: a stray normaliser would show
    K = 0.6 * torch.randn(n, S, D, generator=g, dtype=F64)
    V = torch.randn(n, S, D, generator=g, dtype=F64)
    out = orc.plain_flash_variant(Q, K, V)
    assert torch.allclose(out, F.scaled_dot_product_attention(Q, K, V, is_causal=True), atol=1e-12)
    y = orc.attention_forward(Q[None], K[None], V[None], torch.ones(1, dtype=F64), None, qk_norm=False)[0][0]
    assert torch.allclose(out, y, atol=1e-12)
    # with normalisers the result differs (the switch is not a no-op) ...
    y_n = orc.attention_forward(Q[None], K[None], V[None], torch.ones(1, dtype=F64), None)[0][0]
    assert (y_n - out).abs().max() > 1e-2
    # ... and scaling a query row now changes the logits (no scale invariance left)
    Q2 = Q.clone()
    Q2[:, 5] *= 3.0
    assert (orc.plain_flash_variant(Q2, K, V)[:, 5] - out[:, 5]).abs().max() > 1e-3
    # q_start / non-causal arguments (note the order: q_start, is_causal -- triton_flash_attn.py:215-216)
    full = orc.plain_flash_variant(Q, K, V, 0, True)
    tail = orc.plain_flash_variant(Q[:, 12:], K, V, 12, True)
    assert torch.allclose(tail, full[:, 12:], atol=1e-12)
    assert torch.allclose(orc.plain_flash_variant(Q, K, V, 0, False), F.scaled_dot_product_attention(Q, K, V), atol=1e-12)


@pytest.mark.parametrize("extras", [False, True])
def test_plain_explicit_backward_matches_autograd(extras):
    q, k, v, gq, gk, dy, kw = _bwd_case(extras)
    q = 1.5 * q
    ex = orc.attention_backward_explicit(q, k, v, gq, gk, dy, qk_norm=False, **kw)
    ag = orc.attention_backward_autograd(q, k, v, gq, gk, dy, qk_norm=False, **kw)
    for name in ag:
        assert torch.allclose(ex[name], ag[name], atol=1e-10), name
    # against the normalised family the gradients differ
    ex_n = orc.attention_backward_explicit(q, k, v, gq, gk, dy, **kw)
    assert (ex_n["dq"] - ex["dq"]).abs().max() > 1e-3


# ------------------------------------------------------------------ the whole module (attention.py:175-267)


def _mhsa_weights(d_model, H, Hkv, gating, value_residual, qknorm, seed=5):
    g = torch.Generator().manual_seed(seed)
    d = d_model // H
    r = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    w = {"qkv.linear.weight": r((H + 2 * Hkv) * d, d_model) / math.sqrt(d_model), "out.linear.weight": r(d_model, d_model) / math.sqrt(d_model)}
    if qknorm:
        w["sdpa_qknorm.gain"] = torch.tensor([1.3], dtype=F64)
    if value_residual:
        w.update(alpha1=torch.tensor([0.8], dtype=F64), alpha2=torch.tensor([0.5], dtype=F64), scale=torch.tensor([1.1], dtype=F64))
    if gating:
        shape = {"elementwise": (d_model, d_model), "per-head": (H, d_model), "per-head-hd": (H, d)}[gating]
        w["attn_gate.linear.weight"] = r(*shape) / math.sqrt(shape[1])
    return w


@pytest.mark.parametrize("gating", [False, "per-head", "per-head-hd", "elementwise"])
def test_mhsa_equals_separately_written_glue(gating):
    """mhsa_forward against the composition projection -> apply_rope -> caller_glue -> output projection
    (caller_glue covers the gate only in its per-head form: the other two are applied here by hand)."""
    b, S, H, Hkv, d = 2, 11, 4, 2, 8
    d_model = H * d
    w = _mhsa_weights(d_model, H, Hkv, gating, True, True)
    g = torch.Generator().manual_seed(6)
    x = torch.randn(b, S, d_model, generator=g, dtype=F64)
    v1 = torch.randn(H * b, S, d, generator=g, dtype=F64)
    out, V = orc.mhsa_forward(x, w, n_heads=H, n_kv_heads=Hkv, max_seq_len=32, qknorm=True, gating=gating, v1=v1)
    proj = x @ w["qkv.linear.weight"].T
    q = proj[..., : H * d].reshape(b, S, H, d).permute(0, 2, 1, 3)
    k = proj[..., H * d : (H + Hkv) * d].reshape(b, S, Hkv, d).permute(0, 2, 1, 3)
    v = proj[..., (H + Hkv) * d :].reshape(b, S, Hkv, d).permute(0, 2, 1, 3)
    cos, sin = orc.rope_tables(32, 10000.0, d)
    gl = None
    if gating == "per-head":
        gl = x @ w["attn_gate.linear.weight"].T
    elif gating == "per-head-hd":
        gl = x[..., :d] @ w["attn_gate.linear.weight"].T
    cat, V2 = orc.caller_glue(orc.apply_rope(q, cos, sin), orc.apply_rope(k, cos, sin), v, w["sdpa_qknorm.gain"], v1=v1,
                              alpha1=w["alpha1"], alpha2=w["alpha2"], scale=w["scale"], gate_logits=gl)
    if gating == "elementwise":
        cat = 2.0 * torch.sigmoid(x @ w["attn_gate.linear.weight"].T) * cat
    assert torch.allclose(out, cat @ w["out.linear.weight"].T, atol=1e-11)
    assert torch.allclose(V, V2, atol=1e-12)


def test_mhsa_python_loop_without_qknorm():
    """Per (batch, head) loops over plain softmax attention on a tiny case: catches a wrong head split of the
    projection, a wrong GQA map or a wrong concat order."""
    b, S, H, Hkv, d = 2, 5, 4, 2, 4
    d_model = H * d
    w = _mhsa_weights(d_model, H, Hkv, False, False, False)
    x = torch.randn(b, S, d_model, generator=torch.Generator().manual_seed(8), dtype=F64)
    out, V = orc.mhsa_forward(x, w, n_heads=H, n_kv_heads=Hkv, max_seq_len=16, qknorm=False)
    cos, sin = orc.rope_tables(16, 10000.0, d)
    proj = x @ w["qkv.linear.weight"].T
    cat = torch.zeros(b, S, d_model, dtype=F64)
    for bi in range(b):
        for h in range(H):
            gkv = h // (H // Hkv)
            qh = orc.apply_rope(proj[bi, :, h * d : (h + 1) * d], cos, sin)
            kh = orc.apply_rope(proj[bi, :, (H + gkv) * d : (H + gkv + 1) * d], cos, sin)
            vh = proj[bi, :, (H + Hkv + gkv) * d : (H + Hkv + gkv + 1) * d]
            for i in range(S):
                sc = torch.stack([(qh[i] * kh[j]).sum() / math.sqrt(d) for j in range(i + 1)])
                pr = torch.softmax(sc, 0)
                cat[bi, i, h * d : (h + 1) * d] = sum(pr[j] * vh[j] for j in range(i + 1))
            # with the buffers (1, 0, 1) the value-residual line only multiplies by rsqrt(1 + 1e-8)
            assert torch.allclose(V[h * b + bi], vh * (1 + 1e-8) ** -0.5, atol=1e-12)
    assert torch.allclose(out, (cat * (1 + 1e-8) ** -0.5) @ w["out.linear.weight"].T, atol=1e-11)


@pytest.mark.parametrize("qknorm", [True, False])
def test_mhsa_cached_steps_equal_one_full_pass(qknorm):
    """Prefill + single-token steps through the KV cache reproduce the rows of one full causal pass
    (positions and the causal diagonal both shift by the cache length, attention.py:185-198)."""
    b, S, H, Hkv, d = 2, 9, 4, 2, 8
    d_model = H * d
    w = _mhsa_weights(d_model, H, Hkv, "per-head", True, qknorm)
    x = torch.randn(b, S, d_model, generator=torch.Generator().manual_seed(10), dtype=F64)
    kw = dict(n_heads=H, n_kv_heads=Hkv, max_seq_len=16, qknorm=qknorm, gating="per-head")
    full, V_full = orc.mhsa_forward(x, w, **kw)
    cache = {"keys": None, "values": None}
    outs = [orc.mhsa_forward(x[:, :6], w, cache=cache, **kw)[0]]
    for t in range(6, S):
        o, V_t = orc.mhsa_forward(x[:, t : t + 1], w, cache=cache, **kw)
        outs.append(o)
    assert cache["keys"].shape == (H * b, S, d)
    assert torch.allclose(torch.cat(outs, dim=1), full, atol=1e-11)
    assert torch.allclose(V_t, V_full, atol=1e-12)
