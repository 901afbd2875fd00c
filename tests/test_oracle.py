"""Pins the CPU oracle (oracle/llama_layer_ref.py) with facts that do not come from the oracle
itself: closed forms, invariants, library routines and brute-force loops.  A dropped term, a
wrong sign, a transposed operand or a wrong head map fails at least one of these."""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import llama_layer_ref as R

torch.manual_seed(0)
D = torch.float64


# ------------------------------------------------------------------ rmsnorm
def test_rmsnorm_matches_library_and_closed_form():
    x = torch.randn(7, 48, dtype=D)
    g = torch.randn(48, dtype=D)
    assert torch.allclose(R.rmsnorm(x, g, 1e-5), F.rms_norm(x, (48,), g, 1e-5), atol=1e-12)
    # constant row x_i = c  ->  y = gamma * c / sqrt(c^2 + eps)
    c, eps = 3.0, 1e-5
    y = R.rmsnorm(torch.full((1, 16), c, dtype=D), g[:16], eps)
    assert torch.allclose(y[0], g[:16] * c / math.sqrt(c * c + eps), atol=1e-12)


def test_rmsnorm_scale_invariance_and_orthogonal_gradient():
    x = torch.randn(5, 32, dtype=D, requires_grad=True)
    g = torch.randn(32, dtype=D)
    assert torch.allclose(R.rmsnorm(x, g, 0.0), R.rmsnorm(3.7 * x, g, 0.0), atol=1e-12)
    dy = torch.randn(5, 32, dtype=D)
    R.rmsnorm(x, g, 0.0).backward(dy)
    # y is invariant to scaling x, so the input gradient has no component along x
    assert (x.grad * x.detach()).sum(dim=-1).abs().max() < 1e-10


def test_rmsnorm_backward_formula_equals_autograd():
    x = torch.randn(9, 40, dtype=D, requires_grad=True)
    g = torch.randn(40, dtype=D, requires_grad=True)
    dy = torch.randn(9, 40, dtype=D)
    R.rmsnorm(x, g, 1e-5).backward(dy)
    dx, dg = R.rmsnorm_bwd_formula(dy, x.detach(), g.detach(), 1e-5)
    assert torch.allclose(dx, x.grad, atol=1e-11) and torch.allclose(dg, g.grad, atol=1e-11)


# ------------------------------------------------------------------ linear / split
def test_linear_against_triple_loop():
    x = torch.randn(3, 5, dtype=D)
    w = torch.randn(4, 5, dtype=D)
    y = R.linear(x, w)
    for i in range(3):
        for j in range(4):
            assert abs(y[i, j] - sum(x[i, k] * w[j, k] for k in range(5))) < 1e-12
    # one-hot row picks a weight column; identity weight is the identity map
    assert torch.equal(R.linear(torch.eye(5, dtype=D)[2:3], w)[0], w[:, 2])
    assert torch.equal(R.linear(x, torch.eye(5, dtype=D)), x)


@pytest.mark.parametrize("nq,nkv", [(8, 8), (3, 1), (24, 8), (8, 2), (32, 8)])
def test_split_qkv_index_map(nq, nkv):
    hd, per = 4, nq // nkv
    width = (nq + 2 * nkv) * hd
    mixed = torch.arange(2 * width, dtype=torch.float32).reshape(1, 2, width)
    q, k, v = R.split_qkv(mixed, nq, nkv, hd)
    assert q.shape == (1, 2, nq, hd) and k.shape == (1, 2, nkv, hd) == v.shape
    for b in range(2):
        for g in range(nkv):
            base = b * width + g * (per + 2) * hd
            for j in range(per):
                assert q[0, b, g * per + j].tolist() == list(range(base + j * hd, base + (j + 1) * hd))
            assert k[0, b, g].tolist() == list(range(base + per * hd, base + (per + 1) * hd))
            assert v[0, b, g].tolist() == list(range(base + (per + 1) * hd, base + (per + 2) * hd))


# ------------------------------------------------------------------ rope
def test_rope_table_values():
    f = R.rope_table(5, 8, 10000.0, dtype=D)
    assert f.shape == (5, 1, 1, 8)
    for pos in range(5):
        for i in range(4):
            want = pos * 10000.0 ** (-2 * i / 8)
            assert abs(f[pos, 0, 0, i] - want) < 1e-12 and abs(f[pos, 0, 0, i + 4] - want) < 1e-12


def test_rope_identity_norm_inverse_and_relative_position():
    s, hd = 12, 16
    f = R.rope_table(s, hd, 500000.0, dtype=D)
    t = torch.randn(s, 2, 3, hd, dtype=D)
    y = R.rope(t, f)
    assert torch.allclose(y[0], t[0], atol=1e-14)  # position 0 is the identity
    pair = lambda z: z[..., : hd // 2] ** 2 + z[..., hd // 2:] ** 2
    assert torch.allclose(pair(y), pair(t), atol=1e-12)  # each (i, i+hd/2) pair is rotated
    assert torch.allclose(R.rope(y, -f), t, atol=1e-12)  # rotation by -f undoes it
    # the adjoint of a rotation is the inverse rotation: <R t, g> == <t, R^-1 g>
    g = torch.randn_like(t)
    assert abs((y * g).sum() - (t * R.rope(g, -f)).sum()) < 1e-10
    # <R_m q, R_n k> depends on m - n only
    q, k = torch.randn(hd, dtype=D), torch.randn(hd, dtype=D)
    rot = lambda vec, p: R.rope(vec.expand(s, 1, 1, hd), f)[p, 0, 0]
    assert abs(rot(q, 7) @ rot(k, 3) - rot(q, 9) @ rot(k, 5)) < 1e-10
    assert abs(rot(q, 4) @ rot(k, 0) - rot(q, 4) @ k) < 1e-10
    # sign convention: rotate_half([a, b]) = [-b, a]  =>  one pair at angle th
    th = f[3, 0, 0, 0]
    e = torch.zeros(s, 1, 1, hd, dtype=D)
    e[..., 0] = 1.0
    r = R.rope(e, f)[3, 0, 0]
    assert abs(r[0] - torch.cos(th)) < 1e-12 and abs(r[hd // 2] - torch.sin(th)) < 1e-12


# ------------------------------------------------------------------ swiglu
def test_swiglu_value_and_gradient():
    x = torch.randn(6, 20, dtype=D, requires_grad=True)
    y = R.swiglu(x)
    assert torch.allclose(y, F.silu(x[:, :10]) * x[:, 10:], atol=1e-14)  # first half gates
    dy = torch.randn(6, 10, dtype=D)
    y.backward(dy)
    assert torch.allclose(R.swiglu_bwd_formula(dy, x.detach()), x.grad, atol=1e-12)
    # central finite differences on a few coordinates
    xd = x.detach()
    for (i, j) in [(0, 0), (2, 7), (5, 13), (3, 19)]:
        h = 1e-6
        xp, xm = xd.clone(), xd.clone()
        xp[i, j] += h
        xm[i, j] -= h
        fd = ((R.swiglu(xp) - R.swiglu(xm)) * dy).sum() / (2 * h)
        assert abs(fd - x.grad[i, j]) < 1e-7


# ------------------------------------------------------------------ attention
def _brute_attention(q, k, v):
    s, b, nq, hd = q.shape
    rep = nq // k.shape[2]
    out = torch.zeros_like(q)
    lse = torch.zeros(b, nq, s, dtype=q.dtype)
    for bi in range(b):
        for h in range(nq):
            kv = h // rep
            for i in range(s):
                sc = torch.stack([(q[i, bi, h] @ k[j, bi, kv]) / math.sqrt(hd) for j in range(i + 1)])
                p = torch.exp(sc - sc.max())
                lse[bi, h, i] = sc.max() + torch.log(p.sum())
                p = p / p.sum()
                out[i, bi, h] = sum(p[j] * v[j, bi, kv] for j in range(i + 1))
    return out, lse


@pytest.mark.parametrize("nq,nkv", [(4, 2), (3, 1), (2, 2)])
def test_attention_against_brute_force_and_sdpa(nq, nkv):
    s, b, hd = 9, 2, 8
    q = torch.randn(s, b, nq, hd, dtype=D)
    k = torch.randn(s, b, nkv, hd, dtype=D)
    v = torch.randn(s, b, nkv, hd, dtype=D)
    out, lse = R.causal_gqa_attention(q, k, v, return_lse=True)
    bo, bl = _brute_attention(q, k, v)
    assert torch.allclose(out, bo, atol=1e-12) and torch.allclose(lse, bl, atol=1e-12)
    sd = F.scaled_dot_product_attention(q.permute(1, 2, 0, 3), k.permute(1, 2, 0, 3), v.permute(1, 2, 0, 3),
                                        is_causal=True, enable_gqa=True).permute(2, 0, 1, 3)
    assert torch.allclose(out, sd, atol=1e-10)


def test_attention_special_cases():
    hd = 8
    q = torch.randn(1, 1, 2, hd, dtype=D)
    k, v = torch.randn(1, 1, 1, hd, dtype=D), torch.randn(1, 1, 1, hd, dtype=D)
    assert torch.allclose(R.causal_gqa_attention(q, k, v)[0, 0, 1], v[0, 0, 0], atol=1e-14)  # s = 1: o = v
    # all keys equal -> uniform weights over the visible prefix -> running mean of v
    s = 6
    q = torch.randn(s, 1, 1, hd, dtype=D)
    k = torch.randn(1, 1, 1, hd, dtype=D).expand(s, 1, 1, hd)
    v = torch.randn(s, 1, 1, hd, dtype=D)
    out = R.causal_gqa_attention(q, k, v)
    for i in range(s):
        assert torch.allclose(out[i, 0, 0], v[: i + 1, 0, 0].mean(dim=0), atol=1e-12)
    # the first row never sees later values (causality): change v[3:] and row 2 is unchanged
    v2 = v.clone()
    v2[3:] += 5.0
    assert torch.equal(R.causal_gqa_attention(q, k, v2)[:3], out[:3])


# ------------------------------------------------------------------ whole layer
def test_layer_is_per_sample_and_param_order():
    dims = R.LayerDims(hidden=32, nq=4, nkv=2, hd=8, ffn=24)
    gen = torch.Generator().manual_seed(1)
    p = [R.init_layer_params(dims, gen, dtype=D)]
    assert tuple(p[0]) == R.PARAM_ORDER
    assert p[0]["w_qkv"].shape == (dims.qkv_width, 32) and p[0]["w_fc1"].shape == (48, 32)
    x = torch.randn(10, 4, 32, dtype=D)
    go = torch.randn(10, 4, 32, dtype=D)
    y, dx, grads = R.stack_forward_backward(x, p, dims, go)
    # batch entries never interact: halves of the batch give the halves of the result, and the
    # weight gradients of the halves add up to the full one (what nanobatching relies on)
    ya, dxa, ga = R.stack_forward_backward(x[:, :2], p, dims, go[:, :2])
    yb, dxb, gb = R.stack_forward_backward(x[:, 2:], p, dims, go[:, 2:])
    assert torch.allclose(torch.cat((ya, yb), 1), y, atol=1e-12)
    assert torch.allclose(torch.cat((dxa, dxb), 1), dx, atol=1e-12)
    for name in R.PARAM_ORDER:
        assert torch.allclose(ga[0][name] + gb[0][name], grads[0][name], atol=1e-10)
    # residual structure: with zero projection weights each block is the identity
    z = {k: (torch.zeros_like(t) if k in ("w_proj", "w_fc2") else t) for k, t in p[0].items()}
    f = R.rope_table(10, dims.hd, dims.rope_base, dtype=D)
    assert torch.equal(R.layer_forward(x, z, dims, f), x)


def _library_layer(x, p, dims, skip_rope=False):
    """The layer built from PyTorch library routines only, in the operator order of
    kareus/megatron/core/transformer/transformer_layer.py:148-174: rms_norm -> linear -> per-group
    (q.., k, v) split -> rotary position embedding as a complex multiplication -> causal
    grouped-query scaled_dot_product_attention -> linear -> residual add -> rms_norm -> linear ->
    silu(gate) * up -> linear -> residual add.  Shares no code with the oracle."""
    F = torch.nn.functional
    s, b, h = x.shape
    per, hd = dims.nq // dims.nkv, dims.hd
    h1 = F.rms_norm(x, (h,), p["ln1"], dims.eps)
    mixed = F.linear(h1, p["w_qkv"]).view(s, b, dims.nkv, per + 2, hd)
    q, k, v = mixed[:, :, :, :per].reshape(s, b, dims.nq, hd), mixed[:, :, :, per], mixed[:, :, :, per + 1]
    if "q_norm" in p:
        q, k = F.rms_norm(q, (hd,), p["q_norm"], dims.eps), F.rms_norm(k, (hd,), p["k_norm"], dims.eps)
    if not skip_rope:
        # halves layout: channel i pairs with i + hd/2; rotating the pair by angle a_i is the
        # complex product (t_i + j t_{i+hd/2}) * exp(j a_i)
        inv = dims.rope_base ** (-torch.arange(0, hd, 2, dtype=x.dtype) / hd)
        rot = torch.polar(torch.ones(s, hd // 2, dtype=x.dtype), torch.arange(s, dtype=x.dtype)[:, None] * inv)

        def rotate(t):
            z = torch.complex(t[..., : hd // 2], t[..., hd // 2:]) * rot[:, None, None, :]
            return torch.cat((z.real, z.imag), dim=-1)

        q, k = rotate(q), rotate(k)
    o = F.scaled_dot_product_attention(q.permute(1, 2, 0, 3), k.permute(1, 2, 0, 3), v.permute(1, 2, 0, 3),
                                       is_causal=True, enable_gqa=True)
    x = x + F.linear(o.permute(2, 0, 1, 3).reshape(s, b, dims.nq * hd), p["w_proj"])
    gate, up = F.linear(F.rms_norm(x, (h,), p["ln2"], dims.eps), p["w_fc1"]).chunk(2, dim=-1)
    return x + F.linear(F.silu(gate) * up, p["w_fc2"])


def test_layer_composition_equals_a_layer_of_library_routines():
    """Pins the composition (operator order, the q/k/v split feeding rope and attention, both residual adds):
    the oracle's layer equals one assembled from library routines in fp64, for values and for every gradient,
    and the comparison notices a missing rotary embedding."""
    dims = R.LayerDims(hidden=48, nq=6, nkv=2, hd=16, ffn=40)
    gen = torch.Generator().manual_seed(7)
    p = R.init_layer_params(dims, gen, std=0.3, dtype=D)
    p["ln1"] = 1 + 0.2 * torch.randn(48, generator=gen, dtype=D)
    p["ln2"] = 1 + 0.2 * torch.randn(48, generator=gen, dtype=D)
    x = torch.randn(12, 3, 48, generator=gen, dtype=D)
    go = torch.randn(12, 3, 48, generator=gen, dtype=D)
    y, dx, grads = R.stack_forward_backward(x, [p], dims, go)
    xl = x.clone().requires_grad_(True)
    pl = {k: t.clone().requires_grad_(True) for k, t in p.items()}
    yl = _library_layer(xl, pl, dims)
    yl.backward(go)
    assert torch.allclose(yl, y, atol=1e-11) and torch.allclose(xl.grad, dx, atol=1e-10)
    for name in R.PARAM_ORDER:
        assert torch.allclose(pl[name].grad, grads[0][name], atol=1e-9), name
    # two layers: the stack is the composition of the layers
    p2 = R.init_layer_params(dims, gen, std=0.3, dtype=D)
    f = R.rope_table(12, dims.hd, dims.rope_base, dtype=D)
    assert torch.allclose(R.stack_forward(x, [p, p2], dims, f),
                          _library_layer(_library_layer(x, p, dims), p2, dims), atol=1e-11)
    # the check has teeth: without the rotary embedding the library layer is somewhere else
    assert (_library_layer(x, p, dims, skip_rope=True) - y).abs().max() > 1e-3


def test_layer_with_query_and_key_norms():
    """The q / k layernorm of the QKV split (qkv_postprocess.py:115-118): an RMSNorm per head over the head
    dimension, on queries and keys, in front of the rotary embedding, not on values.  Pinned by the library
    routine in the library layer and by what the norm makes invariant: scaling the QKV weight rows of ONE query
    head, or of one key head, leaves the layer's output alone (a norm over all heads together, or none, would
    not), scaling a value head's rows does not."""
    dims = R.LayerDims(hidden=48, nq=6, nkv=2, hd=16, ffn=40, eps=1e-12)
    gen = torch.Generator().manual_seed(11)
    p = R.init_layer_params(dims, gen, std=0.3, dtype=D)
    p["q_norm"] = 1 + 0.3 * torch.randn(16, generator=gen, dtype=D)
    p["k_norm"] = 1 + 0.3 * torch.randn(16, generator=gen, dtype=D)
    x = torch.randn(12, 3, 48, generator=gen, dtype=D)
    go = torch.randn(12, 3, 48, generator=gen, dtype=D)
    y, dx, grads = R.stack_forward_backward(x, [p], dims, go)
    xl = x.clone().requires_grad_(True)
    pl = {k: t.clone().requires_grad_(True) for k, t in p.items()}
    yl = _library_layer(xl, pl, dims)
    yl.backward(go)
    assert torch.allclose(yl, y, atol=1e-11) and torch.allclose(xl.grad, dx, atol=1e-10)
    for name in p:
        assert torch.allclose(pl[name].grad, grads[0][name], atol=1e-9), name
    plain = {k: t for k, t in p.items() if k not in ("q_norm", "k_norm")}
    f = R.rope_table(12, dims.hd, dims.rope_base, dtype=D)
    assert (R.layer_forward(x, plain, dims, f) - y).abs().max() > 1e-3     # the norms do something
    per, hd = dims.nq // dims.nkv, dims.hd

    def scaled(slot, group=1, factor=3.0):
        w = p["w_qkv"].clone().view(dims.nkv, per + 2, hd, dims.hidden)
        w[group, slot] *= factor
        return {**p, "w_qkv": w.view(-1, dims.hidden)}

    for slot in (0, per - 1, per):                     # a query head, another, the group's key head
        assert torch.allclose(R.layer_forward(x, scaled(slot), dims, f), y, atol=1e-9), slot
        assert (R.layer_forward(x, {**plain, "w_qkv": scaled(slot)["w_qkv"]}, dims, f)
                - R.layer_forward(x, plain, dims, f)).abs().max() > 1e-3
    assert (R.layer_forward(x, scaled(per + 1), dims, f) - y).abs().max() > 1e-3   # values are not normalised


def test_dropout_with_mask_is_native_dropout_given_its_mask():
    """The oracle's hidden dropout takes the mask as an input; for the mask the library routine drew, it is that
    routine's output, and its gradient is native_dropout_backward (bias_dropout_add.py:24-32, 40-43)."""
    torch.manual_seed(0)
    x = torch.randn(64, 96, dtype=torch.float64, requires_grad=True)
    out, mask = torch.ops.aten.native_dropout(x, 0.3, True)
    mine = R.dropout_with_mask(x, mask, 0.3)
    assert torch.allclose(mine, out, rtol=1e-15, atol=0) and 0.6 < mask.double().mean() < 0.8
    g = torch.randn(64, 96, dtype=torch.float64)
    (dx,) = torch.autograd.grad(mine, x, g)
    assert torch.allclose(dx, torch.ops.aten.native_dropout_backward(g, mask, 1 / 0.7), rtol=1e-15, atol=0)
    assert torch.equal(R.dropout_with_mask(x, torch.ones_like(mask), 0.0), x)

