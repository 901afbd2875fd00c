"""Parity of every HIP kernel with the CPU oracle, called through the C ABI (ctypes) on the same
seeded inputs.  Integer-exact where the arithmetic is exact (residual add, index maps), otherwise
bf16 tolerance: max |err| / max |ref| <= 2e-2 against the fp32 oracle evaluated on the bf16-rounded
inputs (the stated bf16 tolerance of the benchmark); observed errors are ~3e-3, one bf16 ulp."""

import math

import pytest
import torch

from oracle import llama_layer_ref as R

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a HIP device")]
TOL = 2e-2
DEV = "cuda"


@pytest.fixture(scope="module")
def be():
    from kareus_amd.backend import get_backend

    return get_backend("hip")


def rel(got, want):
    got, want = got.float().cpu(), want.float().cpu()
    return ((got - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


def rnd(*shape, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(DEV, torch.bfloat16)


# ------------------------------------------------------------------ elementwise
@pytest.mark.parametrize("shape,p", [((64, 2, 512), 0.1), ((257, 3, 1024), 0.5), ((16, 8), 0.0), ((1000, 4096), 0.25)])
def test_dropout_add_and_its_backward(be, shape, p):
    """out = residual + dropout(x) (bias_dropout_add.py:15-45): with the mask the kernel wrote, the reference's
    arithmetic gives the same bits (dropout output rounded to bf16, then the add); about 1 - p of the elements
    are kept; the mask follows from PyTorch's CPU generator alone; the backward is dy * mask / (1 - p)."""
    x, r = rnd(*shape, seed=3), rnd(*shape, seed=4)
    torch.manual_seed(11)
    out, mask = be.dropout_add(x, r, p)
    assert mask.dtype == torch.uint8 and mask.shape == x.shape and int(mask.max()) <= 1
    keep = mask.float().mean().item()
    n = mask.numel()
    assert abs(keep - (1 - p)) <= 5 * (p * (1 - p) / n) ** 0.5 + 1e-9
    want = (r.float() + (x.float() * mask / (1 - p)).to(torch.bfloat16).float()).to(torch.bfloat16)
    assert torch.equal(out, want)
    torch.manual_seed(11)
    out2, mask2 = be.dropout_add(x, r, p)
    assert torch.equal(mask, mask2) and torch.equal(out, out2)
    if p > 0:
        torch.manual_seed(12)
        assert not torch.equal(be.dropout_add(x, r, p)[1], mask)
        # no structure along rows or between neighbours: the kept fraction of every column and of the
        # products of neighbouring mask bits is what independent draws give
        m2 = mask.view(-1, mask.shape[-1]).float()
        if m2.shape[0] >= 64:
            col = m2.mean(0)
            assert (col - (1 - p)).abs().max() <= 6 * (p * (1 - p) / m2.shape[0]) ** 0.5
        pair = (m2[:, 1:] * m2[:, :-1]).mean().item()
        assert abs(pair - (1 - p) ** 2) <= 0.02
    dy = rnd(*shape, seed=5)
    dx = be.dropout_bwd(dy, mask, 1 / (1 - p))
    assert torch.equal(dx, (dy.float() * mask / (1 - p)).to(torch.bfloat16))
    # a strided nanobatch slice as operand and as output
    if len(shape) == 3 and shape[1] >= 2:
        big_x, big_r, big_o = rnd(shape[0], 2 * shape[1], shape[2], seed=6), rnd(shape[0], 2 * shape[1], shape[2], seed=7), \
            torch.zeros(shape[0], 2 * shape[1], shape[2], device=DEV, dtype=torch.bfloat16)
        xs, rs, os_ = big_x[:, :shape[1]], big_r[:, shape[1]:], big_o[:, shape[1]:]
        torch.manual_seed(13)
        o3, m3 = be.dropout_add(xs, rs, p, out=os_)
        torch.manual_seed(13)
        o4, m4 = be.dropout_add(xs.contiguous(), rs.contiguous(), p)
        assert o3.data_ptr() == os_.data_ptr() and torch.equal(os_, o4) and torch.equal(m3, m4)
        assert not big_o[:, :shape[1]].any()


@pytest.mark.parametrize("s,b,ng,per,hd", [(64, 2, 2, 4, 128), (333, 1, 1, 1, 64), (50, 3, 3, 2, 256),
                                           (4096, 2, 2, 4, 128)])
def test_query_key_norm_and_its_backward(be, s, b, ng, per, hd):
    """The q / k layernorm of the QKV split on the fused buffer (qkv_postprocess.py:115-118, 150-157): query and
    key heads against the oracle's RMSNorm over the head dimension and its backward formula, value heads carried
    along bit for bit, weight gradients summed over all heads of the kind.  (The last case has more rows than
    the launch has row slots, so every workgroup walks several.)"""
    eps = 1e-5
    mixed = rnd(s, b, ng, per + 2, hd, seed=1)
    gq = (1 + 0.3 * torch.randn(hd, generator=torch.Generator().manual_seed(2))).to(DEV, torch.bfloat16)
    gk = (1 + 0.3 * torch.randn(hd, generator=torch.Generator().manual_seed(3))).to(DEV, torch.bfloat16)
    before = mixed.clone()
    out, rstd = be.qk_norm_fwd(mixed, gq, gk, eps)
    assert torch.equal(mixed, before) and out.shape == mixed.shape and rstd.shape == (s, b, ng, per + 1)
    xq, xk = mixed[..., :per, :].float(), mixed[..., per, :].float()
    assert rel(out[..., :per, :], R.rmsnorm(xq, gq.float(), eps)) <= TOL
    assert rel(out[..., per, :], R.rmsnorm(xk, gk.float(), eps)) <= TOL
    assert torch.equal(out[..., per + 1, :], mixed[..., per + 1, :])
    assert rel(rstd, torch.rsqrt(mixed[..., :per + 1, :].float().pow(2).mean(-1) + eps)) <= 1e-5
    dy = rnd(s, b, ng, per + 2, hd, seed=4)
    rdq, rdgq = R.rmsnorm_bwd_formula(dy[..., :per, :].float(), xq, gq.float(), eps)
    rdk, rdgk = R.rmsnorm_bwd_formula(dy[..., per, :].float(), xk, gk.float(), eps)
    dvalue = dy[..., per + 1, :].clone()
    dx, dgq, dgk = be.qk_norm_bwd(dy, mixed, rstd, gq, gk)
    assert dx.data_ptr() == dy.data_ptr()                                   # in place
    assert rel(dx[..., :per, :], rdq) <= TOL and rel(dx[..., per, :], rdk) <= TOL
    assert torch.equal(dx[..., per + 1, :], dvalue)
    assert rel(dgq, rdgq) <= TOL and rel(dgk, rdgk) <= TOL
    # the same call again gives the same bits (fixed summation order, no atomics)
    dy2 = rnd(s, b, ng, per + 2, hd, seed=4)
    dx2, dgq2, dgk2 = be.qk_norm_bwd(dy2, mixed, rstd, gq, gk)
    assert torch.equal(dx2, dx) and torch.equal(dgq2, dgq) and torch.equal(dgk2, dgk)
    with pytest.raises(RuntimeError, match="dense fused buffer"):
        be.qk_norm_fwd(mixed[:, :, :, :per + 1], gq, gk, eps)
    with pytest.raises(RuntimeError, match="head dimension"):
        be.qk_norm_fwd(mixed, gq[: hd // 2], gk, eps)


@pytest.mark.parametrize("n", [8, 1000 * 512, 4096 * 4096, 13 * 8 + 5])
def test_add_is_exact(be, n):
    a, b = rnd(n, seed=1), rnd(n, seed=2)
    assert torch.equal(be.add(a, b), a + b)
    assert torch.equal(be.add(a, a), a + a)  # aliasing inputs (ResidualFork with identical grads)


@pytest.mark.parametrize("rows,f", [(512, 1376), (64, 8), (1000, 1024), (2048, 3584)])
def test_swiglu(be, rows, f):
    x, dy = rnd(rows, 2 * f, seed=3), rnd(rows, f, seed=4)
    assert rel(be.swiglu_fwd(x), R.swiglu(x.float())) <= TOL
    assert rel(be.swiglu_bwd(dy, x), R.swiglu_bwd_formula(dy.float(), x.float())) <= TOL
    big = torch.full((8, 16), 30.0, device=DEV, dtype=torch.bfloat16)  # saturated gate: y = x1*x2, finite
    big[:, :8] *= -1
    assert torch.isfinite(be.swiglu_fwd(big)).all() and be.swiglu_fwd(big).abs().max() < 1e-8


@pytest.mark.parametrize("s,b,heads,hd", [(256, 2, 8, 128), (64, 1, 3, 64), (4096, 1, 2, 128)])
def test_rope(be, s, b, heads, hd):
    t = rnd(s, b, heads, hd, seed=5)
    f = R.rope_table(s, hd, 500000.0).to(DEV)
    y = be.rope_fwd(t, f)
    assert rel(y, R.rope(t.float().cpu(), f.cpu())) <= TOL
    assert rel(be.rope_bwd(t, f), R.rope(t.float().cpu(), -f.cpu())) <= TOL
    assert torch.equal(y[0], t[0])  # position 0 is the identity, exactly
    # strided input (a view into a wider buffer) gives the same result as its contiguous copy
    wide = rnd(s, b, heads + 2, hd, seed=6)
    assert torch.equal(be.rope_fwd(wide[:, :, 1:-1], f), be.rope_fwd(wide[:, :, 1:-1].contiguous(), f))


def test_rope_fused_in_place_leaves_value_heads(be):
    s, b, ng, per, hd = 128, 2, 2, 3, 128
    fused = rnd(s, b, ng, per + 2, hd, seed=7)
    before = fused.clone()
    f = R.rope_table(s, hd, 500000.0).to(DEV)
    be.rope_fused_inplace(fused, per, f, False)
    ref = R.rope(before[:, :, :, : per + 1].flatten(2, 3).float().cpu(), f.cpu()).view(s, b, ng, per + 1, hd)
    assert rel(fused[:, :, :, : per + 1], ref) <= TOL
    assert torch.equal(fused[:, :, :, per + 1], before[:, :, :, per + 1])
    be.rope_fused_inplace(fused, per, f, True)  # backward rotation undoes it up to rounding
    assert rel(fused, before) <= TOL


# ------------------------------------------------------------------ rmsnorm
@pytest.mark.parametrize("rows,cols", [(1024, 512), (130, 1024), (67, 1536), (129, 2048), (4096, 3072), (1000, 4096),
                                       (3, 8), (70, 8192), (257, 1376), (33, 2560), (40, 3584), (45, 5120), (31, 6144), (9, 4104)])
def test_rmsnorm(be, rows, cols):
    x, dy = rnd(rows, cols, seed=8), rnd(rows, cols, seed=9)
    g = (1 + 0.1 * torch.randn(cols, generator=torch.Generator().manual_seed(10))).to(DEV, torch.bfloat16)
    y, rstd = be.rmsnorm_fwd(x, g, 1e-5)
    assert rel(y, R.rmsnorm(x.float(), g.float(), 1e-5)) <= TOL
    assert rel(rstd, torch.rsqrt(x.float().pow(2).mean(-1) + 1e-5)) <= 1e-5
    dx, dg = be.rmsnorm_bwd(dy, x, rstd, g)
    rdx, rdg = R.rmsnorm_bwd_formula(dy.float(), x.float(), g.float(), 1e-5)
    assert rel(dx, rdx) <= TOL and rel(dg, rdg) <= TOL
    const = torch.full((4, cols), 3.0, device=DEV, dtype=torch.bfloat16)  # closed form for a constant row
    yc, _ = be.rmsnorm_fwd(const, torch.ones(cols, device=DEV, dtype=torch.bfloat16), 1e-5)
    assert (yc.float() - 3.0 / math.sqrt(9.0 + 1e-5)).abs().max() < 1e-2


@pytest.mark.parametrize("cols", [512, 1376, 2560, 3072, 4096, 5000, 6144, 8192])
def test_rmsnorm_backward_fused_with_residual_add_is_bit_identical(be, cols):
    """RMSNorm backward + the residual fork's gradient sum in one kernel: same bits as the two
    kernels one after the other, also when the residual gradient is a row-strided slice and the
    result goes into a slice of a larger tensor; the weight gradient is untouched."""
    rows, batch = 300, 3
    x, dy = rnd(rows, cols, seed=40), rnd(rows, cols, seed=41)
    res_full = rnd(rows, batch, cols, seed=42)
    g = (1 + 0.1 * torch.randn(cols, generator=torch.Generator().manual_seed(43))).to(DEV, torch.bfloat16)
    _, rstd = be.rmsnorm_fwd(x, g, 1e-5)
    dx_plain, dg_plain = be.rmsnorm_bwd(dy, x, rstd, g)
    res = res_full[:, 1, :]
    want = be.add(dx_plain, res)
    got, dg = be.rmsnorm_bwd(dy, x, rstd, g, residual_grad=res)
    assert torch.equal(got, want) and torch.equal(dg, dg_plain)
    whole = torch.zeros(rows, batch, cols, device=DEV, dtype=torch.bfloat16)
    sink = whole[:, 2, :]
    back, _ = be.rmsnorm_bwd(dy, x, rstd, g, residual_grad=res.contiguous(), out=sink)
    assert back.data_ptr() == sink.data_ptr() and torch.equal(whole[:, 2, :], want)
    assert not whole[:, :2, :].any()
    oracle = R.rmsnorm_bwd_formula(dy.float(), x.float(), g.float(), 1e-5)[0] + res.float()
    assert rel(got, oracle) <= TOL


def test_add_writes_into_a_batch_slice(be):
    """The residual add can put its sum into a [seq, nb, hidden] slice of a [seq, batch, hidden]
    tensor (one row stride addresses seq rows of nb*hidden elements)."""
    seq, batch, hidden = 96, 4, 512
    for nb in (1, 2):
        a, b = rnd(seq, nb, hidden, seed=50 + nb), rnd(seq, nb, hidden, seed=60 + nb)
        whole = torch.zeros(seq, batch, hidden, device=DEV, dtype=torch.bfloat16)
        out = be.add(a, b, out=whole[:, nb:2 * nb])
        assert out.data_ptr() == whole[:, nb:2 * nb].data_ptr()
        assert torch.equal(whole[:, nb:2 * nb], a + b) and not whole[:, :nb].any() and not whole[:, 2 * nb:].any()
    with pytest.raises(RuntimeError):
        be.add(a, b, out=torch.zeros(seq, hidden, 2 * nb, device=DEV, dtype=torch.bfloat16).transpose(1, 2)[:, :nb])


def test_row_strided_nanobatch_slices_need_no_copy(be):
    """One sequence out of a [seq, batch, hidden] tensor is a matrix with row stride batch*hidden:
    RMSNorm (forward and backward) and the residual add must read it in place and give exactly
    what they give on a dense copy."""
    seq, batch, hidden = 384, 4, 1024
    full, gfull = rnd(seq, batch, hidden, seed=30), rnd(seq, batch, hidden, seed=31)
    g = (1 + 0.1 * torch.randn(hidden, generator=torch.Generator().manual_seed(32))).to(DEV, torch.bfloat16)
    xs, dys = full[:, 2, :], gfull[:, 1, :]
    assert not xs.is_contiguous() and xs.stride(0) == batch * hidden
    y, rstd = be.rmsnorm_fwd(xs, g, 1e-5)
    yd, rstdd = be.rmsnorm_fwd(xs.contiguous(), g, 1e-5)
    assert torch.equal(y, yd) and torch.equal(rstd, rstdd) and y.is_contiguous()
    dx, dg = be.rmsnorm_bwd(dys, xs, rstd, g)
    dxd, dgd = be.rmsnorm_bwd(dys.contiguous(), xs.contiguous(), rstd, g)
    assert torch.equal(dx, dxd) and torch.equal(dg, dgd)
    dense = rnd(seq, 1, hidden, seed=33)
    out = be.add(full[:, 2:3, :], dense)                      # strided + dense, 3-D as the engine passes them
    assert out.shape == dense.shape and out.is_contiguous()
    assert torch.equal(out, full[:, 2:3, :] + dense)
    assert torch.equal(be.add(dense, gfull[:, 0:1, :]), dense + gfull[:, 0:1, :])
    assert torch.equal(be.add(full[:, 0:1, :], gfull[:, 3:4, :]), full[:, 0:1, :] + gfull[:, 3:4, :])
    wide = be.add(full[:, 0:2, :], gfull[:, 2:4, :])           # two sequences: no single row stride, copied
    assert torch.equal(wide, full[:, 0:2, :] + gfull[:, 2:4, :])


# ------------------------------------------------------------------ GEMM
SHAPES = [(256, 256, 64), (512, 768, 512), (264, 520, 200), (1024, 2752, 512), (2048, 512, 1376),
          (8, 8, 8), (4096, 640, 384), (40, 1536, 4096),
          # outputs of 192 tiles or more, where the library picks narrower tiles than 256 columns:
          (4096, 3584, 128),    # 224 columns (16 x 16 tiles fill one round of workgroups)
          (16384, 768, 64),     # 192 columns
          (16384, 640, 72),     # 160 columns, and a contraction tail
          # outputs of fewer than 192 full tiles, where narrower tiles and cuts of the contraction compete:
          (4096, 1536, 4096),   # forward: 128-column tiles uncut; the other two layouts take other plans
          (4088, 1000, 2056),   # the same with ragged edges in all three dimensions
          (1536, 4096, 1024)]


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_gemm_three_layouts(be, m, n, k):
    x, w, dy = rnd(m, k, seed=11), rnd(n, k, scale=0.05, seed=12), rnd(m, n, seed=13)
    assert rel(be.linear_fwd(x, w), x.float() @ w.float().t()) <= TOL
    assert rel(be.linear_dgrad(dy, w), dy.float() @ w.float()) <= TOL
    assert rel(be.linear_wgrad(dy, x), dy.float().t() @ x.float()) <= TOL


def test_gemm_plan_does_not_change_the_sums_much(be):
    """The library picks tile width and cuts of the contraction by a cost model that depends on the
    workspace it is given (alone on the GPU: cuts allowed; beside other streams: fewer or none; never:
    no workspace).  All plans compute the same sums, up to the rounding of a cut's fp32 partial tiles."""
    for (m, n, k) in [(4096, 1536, 4096), (4096, 1024, 4096), (1536, 4096, 4096), (520, 264, 8192)]:
        x, w, dy, xx = rnd(m, k, seed=31), rnd(n, k, scale=0.05, seed=32), rnd(k, m, scale=0.1, seed=33), rnd(k, n, seed=34)
        for layout, a, b, ref in ((0, x, w, x.float() @ w.float().t()), (1, x, w.t().contiguous(), x.float() @ w.float().t()),
                                  (2, dy, xx, dy.float().t() @ xx.float())):
            outs = [be.gemm(layout, a, b, m, n, k, split_k=mode) for mode in (True, False, None)]
            for o in outs:
                assert rel(o, ref) <= TOL
            assert rel(outs[0], outs[2]) <= 1e-2 and rel(outs[1], outs[2]) <= 1e-2
            c0 = rnd(m, n, seed=35)
            acc = be.gemm(layout, a, b, m, n, k, out=c0.clone(), accumulate=True, split_k=None)
            assert rel(acc, ref + c0.float()) <= TOL


def test_gemm_is_reproducible(be):
    """No atomics and a fixed order of accumulation: repeated launches give the same bits (a
    race on an LDS tile between the waves of a workgroup would show up here)."""
    m, n, k = 4096, 3584, 1088
    x, w, dy = rnd(m, k, seed=14), rnd(n, k, scale=0.05, seed=15), rnd(m, n, seed=16)
    first = (be.linear_fwd(x, w).clone(), be.linear_dgrad(dy, w).clone(), be.linear_wgrad(dy, x).clone())
    for _ in range(5):
        again = (be.linear_fwd(x, w), be.linear_dgrad(dy, w), be.linear_wgrad(dy, x))
        assert all(torch.equal(a, b) for a, b in zip(again, first))


def test_gemm_closed_forms(be):
    eye = torch.eye(512, device=DEV, dtype=torch.bfloat16)
    x = rnd(264, 512, seed=14)
    assert torch.equal(be.linear_fwd(x, eye), x) and torch.equal(be.linear_dgrad(x, eye), x)  # identity weight
    ones = torch.ones(128, 512, device=DEV, dtype=torch.bfloat16)
    small = (torch.arange(264 * 512) % 7 - 3).reshape(264, 512).to(DEV, torch.bfloat16)  # exact small ints
    assert torch.equal(be.linear_fwd(small, ones).float(), small.float().sum(1, keepdim=True).expand(264, 128))
    onehot = torch.zeros(264, 8, device=DEV, dtype=torch.bfloat16)  # dW = dy^T x with one-hot dy picks rows of x
    onehot[5, 3] = 1
    dw = be.linear_wgrad(onehot, x)
    assert torch.equal(dw[3], x[5]) and dw.abs().sum() == x[5].abs().sum()


def test_gemm_split_k_accumulate_and_strides(be):
    for (m, n, k) in [(512, 768, 4096), (264, 520, 2440)]:
        dy, x = rnd(k, m, scale=0.1, seed=15), rnd(k, n, seed=16)
        assert be.lib.kr_gemm_workspace_bytes(2, m, n, k) > 0  # this shape is computed split-K
        ref = dy.float().t() @ x.float()
        assert rel(be.linear_wgrad(dy, x), ref) <= TOL
        c0 = rnd(m, n, seed=17)
        assert rel(be.gemm(2, dy, x, m, n, k, out=c0.clone(), accumulate=True), ref + c0.float()) <= TOL
    a, w, c0 = rnd(296, 512, seed=18), rnd(264, 512, seed=19), rnd(296, 264, seed=20)
    assert rel(be.gemm(0, a, w, 296, 264, 512, out=c0.clone(), accumulate=True), a.float() @ w.float().t() + c0.float()) <= TOL
    wide = rnd(296, 1024, seed=21)  # lda > K: operand is a column slice of a wider matrix
    assert torch.equal(be.gemm(0, wide[:, 256:768], w, 296, 264, 512), be.gemm(0, wide[:, 256:768].contiguous(), w, 296, 264, 512))
    with pytest.raises(RuntimeError, match="not supported"):
        be.gemm(0, a[:295], w, 295, 264, 512)


# ------------------------------------------------------------------ attention
def _grouped(s, b, nq, nkv, hd, seed):
    per = nq // nkv
    fused = rnd(s, b, nkv, per + 2, hd, seed=seed)
    return fused, fused[:, :, :, :per], fused[:, :, :, per], fused[:, :, :, per + 1]


@pytest.mark.parametrize("s,b,nq,nkv", [(128, 1, 1, 1), (256, 2, 4, 2), (512, 1, 3, 1), (384, 1, 8, 8), (1024, 1, 4, 1),
                                        (2048, 1, 2, 1),    # 32 query tiles per key tile: the steady state of the pipelines
                                        (512, 17, 8, 8),    # 544 workgroups, one query head per KV head: dK/dV written directly
                                        (640, 3, 6, 2),     # odd tile count, three query heads per KV head
                                        (256, 1, 24, 8),    # the head map of benchmark configuration 3 (Llama-3.2-3B)
                                        (256, 2, 32, 8),    # ... and of configuration 5 (Llama-3.1-8B), four query heads per KV head
                                        # enough 256-query tiles for every compute unit: the forward kernel whose halves share K / V tiles
                                        (1024, 8, 8, 2),    # 4 tiles x 64 (batch, head) pairs, eight pairs start together on an XCD
                                        (768, 11, 8, 8),    # 3 tiles per pair: plain longest-first order
                                        (512, 33, 8, 2),    # 2 tiles per pair, 264 pairs: the last group of 16 pairs is incomplete
                                        (2304, 4, 8, 2),    # 9 tiles per pair: an odd tile count, half 0 idles through two steps of 36
                                        (512, 6, 24, 8),    # three query heads per KV head in the shared-tile kernels
                                        # enough key tiles that a dK/dV workgroup serves several query heads of its KV group:
                                        (512, 32, 8, 4),    # both heads of a group: dK/dV stored directly, no partial results
                                        (512, 64, 8, 2),    # all four heads of a group
                                        (256, 128, 6, 2)])  # all three heads of a group
def test_attention_forward_backward(be, s, b, nq, nkv):
    hd = 128
    _, q, k, v = _grouped(s, b, nq, nkv, hd, seed=22)
    do = rnd(s, b, nq, hd, seed=23)
    o, lse = be.attn_fwd(q, k, v, hd ** -0.5)
    qf, kf, vf = (t.float().cpu().clone().requires_grad_(True) for t in (q.flatten(2, 3), k, v))
    ro, rlse = R.causal_gqa_attention(qf, kf, vf, return_lse=True)
    assert rel(o, ro) <= TOL and rel(lse, rlse) <= 1e-4
    ro.backward(do.float().cpu())
    dq, dk, dv = be.attn_bwd(do, q, k, v, o, lse, hd ** -0.5)
    assert rel(dq.flatten(2, 3), qf.grad) <= TOL and rel(dk, kf.grad) <= TOL and rel(dv, vf.grad) <= TOL
    assert dq._kr_mixed.shape == (s, b, (nq + 2 * nkv) * hd)  # gradients share one fused buffer
    again = be.attn_bwd(do, q, k, v, o, lse, hd ** -0.5)       # no atomics, fixed reduction order: same bits
    assert all(torch.equal(x, y) for x, y in zip(again, (dq, dk, dv)))
    # dense [s, b, nq, hd] tensors go through the same kernels
    qd = q.flatten(2, 3).contiguous()
    od, lsed = be.attn_fwd(qd, k.contiguous(), v.contiguous(), hd ** -0.5)
    assert torch.equal(od, o) and torch.equal(lsed, lse)
    dqd, dkd, dvd = be.attn_bwd(do, qd, k.contiguous(), v.contiguous(), od, lsed, hd ** -0.5)
    assert torch.equal(dqd, dq.flatten(2, 3)) and torch.equal(dkd, dk) and torch.equal(dvd, dv)


def test_attention_at_sequence_8192(be):
    """The sequence length of benchmark configuration 5, against the brute-force oracle (two query heads on
    one KV head keep the oracle's 8192 x 8192 score matrices within a few seconds of CPU time)."""
    s, b, nq, nkv, hd = 8192, 1, 2, 1, 128
    _, q, k, v = _grouped(s, b, nq, nkv, hd, seed=70)
    do = rnd(s, b, nq, hd, seed=71)
    o, lse = be.attn_fwd(q, k, v, hd ** -0.5)
    dq, dk, dv = be.attn_bwd(do, q, k, v, o, lse, hd ** -0.5)
    qf, kf, vf = (t.float().cpu().clone().requires_grad_(True) for t in (q.flatten(2, 3), k, v))
    ro, rlse = R.causal_gqa_attention(qf, kf, vf, return_lse=True)
    assert rel(o, ro) <= TOL and rel(lse, rlse) <= 1e-4
    ro.backward(do.float().cpu())
    assert rel(dq.flatten(2, 3), qf.grad) <= TOL and rel(dk, kf.grad) <= TOL and rel(dv, vf.grad) <= TOL
    # the whole forms (256-query workgroups: the query gradient with one wave per SIMD walks 128 key tiles here)
    o2, lse2 = be.attn_fwd(q, k, v, hd ** -0.5, beside_other_streams=True)
    assert rel(o2, ro) <= TOL and rel(lse2, rlse) <= 1e-4
    dq2, dk2, dv2 = be.attn_bwd(do, q, k, v, o2, lse2, hd ** -0.5, beside_other_streams=True)
    assert rel(dq2.flatten(2, 3), qf.grad) <= TOL and rel(dk2, kf.grad) <= TOL and rel(dv2, vf.grad) <= TOL


def test_attention_does_not_depend_on_the_launch_size(be):
    """Forward and query-gradient kernels come in two variants chosen by workgroup count (forward:
    halves of a workgroup share K / V tiles once there is a 256-query tile for every compute unit;
    query gradient: up to 1024 workgroups each row's keys are split between two halves of a
    workgroup).  Within a variant a sequence gives the same bits whatever the batch around it;
    across variants the results agree to rounding."""
    s, nq, nkv, hd, b = 1024, 8, 2, 128, 17                   # 4 x 8 x 17 = 544 tiles of 256 queries
    q, k, v = rnd(s, b, nq, hd, seed=40), rnd(s, b, nkv, hd, seed=41), rnd(s, b, nkv, hd, seed=42)
    o_all, lse_all = be.attn_fwd(q, k, v, hd ** -0.5)
    o_9, lse_9 = be.attn_fwd(q[:, 4:13].contiguous(), k[:, 4:13].contiguous(), v[:, 4:13].contiguous(), hd ** -0.5)  # 288 tiles
    assert torch.equal(o_all[:, 4:13], o_9) and torch.equal(lse_all[4:13], lse_9)
    for bi in (0, 9, 16):
        o1, lse1 = be.attn_fwd(q[:, bi:bi + 1].contiguous(), k[:, bi:bi + 1].contiguous(),
                               v[:, bi:bi + 1].contiguous(), hd ** -0.5)   # 64 workgroups of 128 queries
        assert rel(o_all[:, bi:bi + 1], o1) <= 1e-2 and rel(lse_all[bi], lse1[0]) <= 1e-5
        o2, lse2 = be.attn_fwd(q[:, bi:bi + 2].contiguous(), k[:, bi:bi + 2].contiguous(),
                               v[:, bi:bi + 2].contiguous(), hd ** -0.5)   # 128 workgroups, same variant
        assert torch.equal(o2[:, :1], o1) and torch.equal(lse2[0], lse1[0])
    ro, rlse = R.causal_gqa_attention(q[:, 3:4].float(), k[:, 3:4].float(), v[:, 3:4].float(), return_lse=True)
    assert rel(o_all[:, 3:4], ro) <= TOL and rel(lse_all[3:4], rlse) <= 1e-4
    # the query-gradient kernel: unsplit variant for the whole batch, split variant for one sequence
    do = rnd(s, b, nq, hd, seed=43)
    dq_all, dk_all, dv_all = be.attn_bwd(do, q, k, v, o_all, lse_all, hd ** -0.5)
    for bi in (0, 16):
        sl = slice(bi, bi + 1)
        one = [t[:, sl].contiguous() for t in (do, q, k, v, o_all)]
        dq1, dk1, dv1 = be.attn_bwd(one[0], one[1], one[2], one[3], one[4], lse_all[sl].contiguous(), hd ** -0.5)
        assert rel(dq_all[:, sl], dq1) <= 1e-2 and rel(dk_all[:, sl], dk1) <= 1e-2 and rel(dv_all[:, sl], dv1) <= 1e-2


@pytest.mark.parametrize("s,b,nq,nkv", [(512, 1, 8, 2), (768, 2, 4, 4), (256, 1, 6, 2), (384, 1, 2, 1), (1024, 1, 24, 8)])
def test_attention_beside_other_streams(be, s, b, nq, nkv):
    """The forms the engine launches on its nanobatch streams (KR_ATTN_BESIDE_OTHER_STREAMS: whole rows and whole
    key tiles per workgroup whatever their number; a length that is not a multiple of 256 keeps the 128-query
    forms): against the fp32 oracle like the default forms, the same bits on every call, and — unlike the default
    forms, which pick a variant by workgroup count — the same bits for a sequence whatever the batch around it."""
    hd = 128
    _, q, k, v = _grouped(s, b, nq, nkv, hd, seed=222)
    do = rnd(s, b, nq, hd, seed=223)
    o, lse = be.attn_fwd(q, k, v, hd ** -0.5, beside_other_streams=True)
    qf, kf, vf = (t.float().cpu().clone().requires_grad_(True) for t in (q.flatten(2, 3), k, v))
    ro, rlse = R.causal_gqa_attention(qf, kf, vf, return_lse=True)
    assert rel(o, ro) <= TOL and rel(lse, rlse) <= 1e-4
    ro.backward(do.float().cpu())
    dq, dk, dv = be.attn_bwd(do, q, k, v, o, lse, hd ** -0.5, beside_other_streams=True)
    assert rel(dq.flatten(2, 3), qf.grad) <= TOL and rel(dk, kf.grad) <= TOL and rel(dv, vf.grad) <= TOL
    again = be.attn_bwd(do, q, k, v, o, lse, hd ** -0.5, beside_other_streams=True)
    assert all(torch.equal(x, y) for x, y in zip(again, (dq, dk, dv)))
    # against the default forms: equal to rounding
    o0, lse0 = be.attn_fwd(q, k, v, hd ** -0.5)
    assert rel(o, o0) <= 1e-2 and rel(lse, lse0) <= 1e-5
    # a batch of 40 such sequences (enough tiles for every compute unit) gives each of them the same bits
    if s % 256 == 0 and nq == 8:
        big = 40
        qb, kb, vb = (t.repeat_interleave(big, dim=1) for t in (q, k, v))
        ob, lseb = be.attn_fwd(qb, kb, vb, hd ** -0.5, beside_other_streams=True)
        assert torch.equal(ob[:, 7:8], o) and torch.equal(lseb[7:8], lse)
        ob2, _ = be.attn_fwd(qb, kb, vb, hd ** -0.5)            # alone on the GPU it takes the same form
        assert torch.equal(ob2, ob)
        dob = do.repeat_interleave(big, dim=1)
        dqb, dkb, dvb = be.attn_bwd(dob, qb, kb, vb, ob, lseb, hd ** -0.5, beside_other_streams=True)
        assert torch.equal(dqb[:, 7:8], dq)


def test_attention_special_cases(be):
    hd, s = 128, 256
    # all keys equal -> output row i is the mean of v[0..i]
    q = rnd(s, 1, 1, hd, seed=24)
    k = rnd(1, 1, 1, hd, seed=25).expand(s, 1, 1, hd).contiguous()
    v = rnd(s, 1, 1, hd, seed=26)
    o, lse = be.attn_fwd(q, k, v, hd ** -0.5)
    want = torch.cumsum(v.float(), 0) / torch.arange(1, s + 1, device=DEV).view(s, 1, 1, 1)
    assert rel(o, want) <= TOL
    assert torch.equal(o[0], v[0])  # a single visible key: o = v exactly
    # causality: changing later keys/values leaves earlier rows bit-identical
    k2, v2 = k.clone(), v.clone()
    k2[200:] += 1
    v2[200:] -= 3
    o2, _ = be.attn_fwd(q, k2, v2, hd ** -0.5)
    assert torch.equal(o2[:200], o[:200])
    with pytest.raises(RuntimeError, match="not supported"):
        be.attn_fwd(rnd(128, 1, 1, 136), rnd(128, 1, 1, 136), rnd(128, 1, 1, 136), 1.0)  # head_dim above 128


@pytest.mark.parametrize("s,b,nq,nkv", [(512, 2, 4, 2),       # split-key forward (few 256-query tiles)
                                         (512, 64, 8, 2)])     # forward over shared tiles
@pytest.mark.parametrize("kind", ["wide", "rising", "falling"])
def test_attention_when_the_row_maximum_keeps_moving(be, s, b, nq, nkv, kind):
    """The forward kernels move the reference point of a row's exponents only when its maximum has grown
    by more than 2^8.  Scores N(0,1) never do that after the first tile, so: scores spread over +-40
    (jumps of every size), scores that rise along the keys (a new maximum in every tile, by a little or
    by a lot depending on the row) and scores that fall (the first reference stays for good, later
    probabilities underflow).  Checked against the fp32 oracle like every other shape, lse included."""
    hd = 128
    _, q, k, v = _grouped(s, b, nq, nkv, hd, seed=300)
    q, k = q.clone(), k.clone()
    if kind == "wide":
        k *= 12.0                                         # scores ~ N(0, 12^2): jumps of many powers of two
    else:
        # one shared direction u: score(i, j) = (q_i . u)(k_j . u) + noise, |k_j . u| growing with j
        u = torch.nn.functional.normalize(rnd(hd, seed=301).float(), dim=0).bfloat16()
        ramp = torch.linspace(0.0, 30.0, s, device=DEV).view(s, 1, 1, 1)
        if kind == "falling":
            ramp = -ramp
        k += (ramp * u.float()).bfloat16()
        q += (torch.linspace(0.2, 4.0, s, device=DEV).view(s, 1, 1, 1, 1) * u.float()).bfloat16()
    scale = hd ** -0.5
    o, lse = be.attn_fwd(q, k, v, scale)
    qf, kf, vf = (t.float().cpu() for t in (q.flatten(2, 3), k, v))
    ro, rlse = R.causal_gqa_attention(qf, kf, vf, return_lse=True)
    assert torch.isfinite(o.float()).all() and torch.isfinite(lse).all()
    assert rel(o, ro) <= TOL and rel(lse, rlse) <= 1e-4
    assert torch.equal(o[0], v[0].repeat_interleave(nq // nkv, dim=1))     # one visible key: o = v exactly


@pytest.mark.parametrize("s,b,nq,nkv,hd", [(100, 1, 1, 1, 128),    # ragged length at the fast kernels' head dimension
                                            (256, 2, 8, 8, 64),     # benchmark configuration 1: 8 heads of 64
                                            (77, 3, 6, 2, 64),      # ragged, grouped queries
                                            (200, 1, 4, 1, 96), (1, 1, 1, 1, 64), (130, 2, 4, 2, 128), (33, 1, 2, 2, 8),
                                            (1000, 2, 8, 2, 128),   # a ragged length at a training width
                                            (640, 2, 8, 8, 64)])    # whole tiles, half the head dimension
@pytest.mark.parametrize("general", [False, True])
def test_attention_general_shapes(be, s, b, nq, nkv, hd, general):
    """Head dimensions other than 128 and sequence lengths that are not whole 128-row tiles: padded into the MFMA
    kernels through the workspace (``general=False``, what the engine runs) or on the general fp32 kernels — same
    interface and layouts (fused QKV views, dense tensors), checked like the fast path."""
    _, q, k, v = _grouped(s, b, nq, nkv, hd, seed=100)
    do = rnd(s, b, nq, hd, seed=101)
    scale = hd ** -0.5
    attn_fwd = lambda *a: be.attn_fwd(*a, general_kernels=general)
    attn_bwd = lambda *a: be.attn_bwd(*a, general_kernels=general)
    o, lse = attn_fwd(q, k, v, scale)
    qf, kf, vf = (t.float().cpu().clone().requires_grad_(True) for t in (q.flatten(2, 3), k, v))
    ro, rlse = R.causal_gqa_attention(qf, kf, vf, return_lse=True)
    assert rel(o, ro) <= TOL and rel(lse, rlse) <= 1e-4
    assert torch.equal(o[0], v[0].repeat_interleave(nq // nkv, dim=1))     # one visible key: o = v exactly
    ro.backward(do.float().cpu())
    dq, dk, dv = attn_bwd(do, q, k, v, o, lse, scale)
    assert all(torch.isfinite(t.float()).all() for t in (o, dq, dk, dv))
    assert rel(dq.flatten(2, 3), qf.grad) <= TOL and rel(dk, kf.grad) <= TOL and rel(dv, vf.grad) <= TOL
    again = attn_bwd(do, q, k, v, o, lse, scale)                            # fixed order of every sum: same bits
    assert all(torch.equal(x, y) for x, y in zip(again, (dq, dk, dv)))
    qd = q.flatten(2, 3).contiguous()
    od, lsed = attn_fwd(qd, k.contiguous(), v.contiguous(), scale)
    assert torch.equal(od, o) and torch.equal(lsed, lse)


def test_attention_padded_into_the_mfma_kernels_equals_the_whole_tile_call(be):
    """A ragged length is the whole-tile problem with rows taken away: queries below s see the same keys, so the
    padded call must give the bits of the MFMA kernels on the next multiple of 128 restricted to the first s
    rows (forward), and gradients that ignore the rows beyond s."""
    s, sp, b, nq, nkv, hd = 300, 384, 2, 4, 2, 128
    _, q, k, v = _grouped(sp, b, nq, nkv, hd, seed=110)
    scale = hd ** -0.5
    o_full, lse_full = be.attn_fwd(q, k, v, scale)
    o, lse = be.attn_fwd(q[:s], k[:s], v[:s], scale)
    assert torch.equal(o, o_full[:s]) and torch.equal(lse, lse_full[..., :s])
    # backward: the whole-tile call with zero upstream gradient beyond s gives the same dq, dk, dv rows below s
    do_full = rnd(sp, b, nq, hd, seed=111)
    do_full[s:] = 0
    dq_f, dk_f, dv_f = be.attn_bwd(do_full, q, k, v, o_full, lse_full, scale)
    dq, dk, dv = be.attn_bwd(do_full[:s], q[:s], k[:s], v[:s], o, lse, scale)
    assert torch.equal(dq, dq_f[:s]) and torch.equal(dk, dk_f[:s]) and torch.equal(dv, dv_f[:s])


# ------------------------------------------------------------------ fused GEMM epilogues
@pytest.mark.parametrize("m,n,k", [(512, 768, 512), (264, 520, 200), (4096, 4096, 1024), (1000, 3072, 640),
                                   (16384, 640, 72)])
def test_gemm_with_fused_residual_equals_gemm_then_add(be, m, n, k):
    """C = bf16(bf16(A.B) + R) in the GEMM's epilogue: the same bits as the GEMM followed by the residual add,
    also with a row-strided residual and a row-strided output (a nanobatch slice of the block's output).
    (The unfused reference runs without split-K, as a fused launch always does: splitting the contraction
    changes the order of the sum.)"""
    x, w = rnd(m, k, seed=80), rnd(n, k, scale=0.05, seed=81)
    res_wide = rnd(m, 2 * n, seed=82)
    res = res_wide[:, n // 2: n // 2 + n] if (n // 2) % 8 == 0 else res_wide[:, :n]
    want = be.add(res.contiguous(), be.linear_fwd(x, w, split_k=None))
    got = be.linear_fwd(x, w, residual=res)
    assert torch.equal(got, want)
    whole = torch.zeros(m, 3 * n, device=DEV, dtype=torch.bfloat16)
    be.linear_fwd(x, w, residual=res, out=whole[:, n:2 * n])
    assert torch.equal(whole[:, n:2 * n], want) and not whole[:, :n].any() and not whole[:, 2 * n:].any()
    assert rel(got, x.float() @ w.float().t() + res.float()) <= TOL
    with pytest.raises(RuntimeError, match="not supported"):   # fused epilogues exist for the forward layout only
        be.gemm(1, rnd(m, n, seed=83), w, m, k, n, residual=rnd(m, k, seed=84))


@pytest.mark.parametrize("m,f,k", [(512, 128, 256), (264, 384, 200), (4096, 3584, 4096), (1000, 1024, 3072),
                                   (16384, 320, 72), (8192, 672, 136), (304, 14336, 64)])
def test_gemm_with_fused_swiglu_equals_gemm_then_swiglu(be, m, f, k):
    """fc1 with the activation in its epilogue: x = A.W^T [m, 2f] and y = silu(x[:, :f]) * x[:, f:] from one
    launch, the same bits as the GEMM followed by the SwiGLU kernel."""
    a, w = rnd(m, k, seed=85), rnd(2 * f, k, scale=0.05, seed=86)
    x_want = be.linear_fwd(a, w, split_k=None)
    y_want = be.swiglu_fwd(x_want)
    y = torch.empty(m, f, device=DEV, dtype=torch.bfloat16)
    x = be.linear_fwd(a, w, swiglu_out=y)
    assert torch.equal(x, x_want) and torch.equal(y, y_want)
    assert rel(y, R.swiglu(a.float() @ w.float().t())) <= TOL
    assert be.can_fuse_swiglu(2 * f)
    with pytest.raises(RuntimeError, match="not supported"):   # no tile width divides 2f = 144: the caller keeps the two launches
        be.linear_fwd(a[:, :k], rnd(2 * 72, k, seed=87), swiglu_out=torch.empty(m, 72, device=DEV, dtype=torch.bfloat16))


def test_gemm_compute_unit_budget_changes_nothing_but_the_launch(be):
    m, n, k = 4096, 3584, 1088
    x, w = rnd(m, k, seed=88), rnd(n, k, scale=0.05, seed=89)
    full = be.linear_fwd(x, w, split_k=None)
    for cus in (1, 64, 200, 256, 1000):
        assert torch.equal(be.linear_fwd(x, w, split_k=False, max_cus=cus), full)


@pytest.mark.parametrize("m,n,k", [(7168, 4096, 256), (7160, 4088, 200), (4096, 7168, 128), (3584, 8192, 72)])
def test_weight_gradient_with_transposed_store(be, m, n, k):
    """A weight gradient whose tile grid fits the device better the other way round (fc1 of workload c4:
    7168 x 4096) is computed as the transposed product with a transposing store; results are those of the
    direct form (which a call that accumulates still takes) and do not depend on the form bit for bit."""
    dy, x = rnd(k, m, scale=0.1, seed=90), rnd(k, n, seed=91)
    ref = dy.float().t() @ x.float()
    got = be.linear_wgrad(dy, x, split_k=None)
    assert rel(got, ref) <= TOL
    direct = be.gemm(2, dy, x, m, n, k, out=torch.zeros(m, n, device=DEV, dtype=torch.bfloat16), accumulate=True,
                     split_k=None)
    assert torch.equal(got, direct)
    wide = torch.zeros(m, n + 64, device=DEV, dtype=torch.bfloat16)        # row-strided output
    be.gemm(2, dy, x, m, n, k, out=wide[:, :n], split_k=None)
    assert torch.equal(wide[:, :n], got) and not wide[:, n:].any()
    assert torch.equal(be.linear_wgrad(dy, x, split_k=None), got)


@pytest.mark.parametrize("m,f,h", [(512, 128, 256), (264, 520, 200), (4096, 3584, 1024), (1000, 1024, 640), (16384, 72, 3072)])
def test_input_gradient_with_fused_swiglu_backward_equals_the_two_kernels(be, m, f, h):
    """fc2's input-gradient GEMM with the SwiGLU backward in its epilogue: dy . W is never written, the
    gradient of the activation's input comes out of the one launch with the bits of the GEMM followed by
    kr_swiglu_bwd."""
    dy, w = rnd(m, h, seed=110), rnd(h, f, scale=0.05, seed=111)        # W_fc2 [hidden, ffn]
    x = rnd(m, 2 * f, seed=112)                                         # the activation's input (fc1's output)
    want = be.swiglu_bwd(be.linear_dgrad(dy, w, split_k=None), x)
    got = be.linear_dgrad(dy, w, swiglu_bwd_x=x)
    assert got.shape == (m, 2 * f) and torch.equal(got, want)
    assert rel(got, R.swiglu_bwd_formula(dy.float() @ w.float(), x.float())) <= TOL
    wide = rnd(m, 2 * f + 16, seed=113)                                 # row-strided activation input
    assert torch.equal(be.linear_dgrad(dy, w, swiglu_bwd_x=wide[:, :2 * f]),
                       be.swiglu_bwd(be.linear_dgrad(dy, w, split_k=None), wide[:, :2 * f].contiguous()))
