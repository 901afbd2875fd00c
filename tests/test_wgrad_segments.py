"""The weight gradient of a linear layer over all nanobatches of a microbatch in one launch.

The reference computes dW = dy^T . x once per nanobatch and sums the products in main_grad
(kareus/transformer_engine/pytorch/ops/basic/basic_linear_bias.py:229-263, GEMM call basic_linear.py:898-909).
The sum over nanobatches is the same contraction continued over more tokens, so `kr_gemm_bf16_nt_segments`
takes the nanobatches' operand pairs where they lie and contracts them one after the other in one GEMM.
Only the operand base changes at a piece boundary, so the result must equal, bit for bit, the plain layout-NT
kernel fed the concatenation of the pieces (same tiling, same order of the fp32 sum); against the per-nanobatch
accumulation, which rounds to bf16 once per nanobatch, and against an fp32 product it must agree within the
bf16 tolerance of the layer tests.
"""

import ctypes

import pytest
import torch

DEV = "cuda"
TOL = 2e-2


def gpu(test):
    """Marks a test that needs the device."""
    return pytest.mark.gpu(pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a HIP device")(test))


# ---- host logic ---------------------------------------------------------------------------------------
def test_entry_point_rejects_bad_pieces_without_a_device():
    from kareus_amd.backend import hip

    lib = hip.load_library()
    ptrs = (ctypes.c_void_p * 2)(4096, 8192)

    def call(m=64, n=64, k_seg=64, nseg=2, a=ptrs, b=ptrs, flags=0, run_rows=1, run_ld=0):
        return lib.kr_gemm_bf16_nt_segments(m, n, k_seg, nseg, a, 64, run_rows, run_ld, b, 64, 4096, 64, 0, flags, 0,
                                            None, 0, None)

    assert call(nseg=0) == -1 and call(nseg=9) == -1 and call(k_seg=0) == -1
    assert call(a=None) == -1 and call(flags=2) == -1
    assert call(k_seg=96) == -2                                         # pieces are whole K-steps of 64 rows
    assert call(a=(ctypes.c_void_p * 2)(4096, 0)) == -1                  # a missing piece
    assert call(a=(ctypes.c_void_p * 2)(4096, 8200)) == -1               # not 16-byte aligned
    assert call(run_rows=3, run_ld=512) == -1 and call(run_rows=32, run_ld=4096) == -2 and call(run_rows=2, run_ld=0) == -1
    assert call(run_rows=2, run_ld=500) == -2                            # run starts a multiple of 8 elements apart


def test_operand_pairs_on_the_host_are_turned_down():
    from kareus_amd.backend.hip import HipBackend

    be = HipBackend.__new__(HipBackend)                                  # the check needs no library
    dys = [torch.empty(128, 64, dtype=torch.bfloat16) for _ in range(2)]
    xs = [torch.empty(128, 32, dtype=torch.bfloat16) for _ in range(2)]
    assert not be.wgrad_segments_ok(dys, xs)                             # host tensors: never
    assert not be.wgrad_segments_ok(dys, xs[:1]) and not be.wgrad_segments_ok([], [])


# ---- kernels ------------------------------------------------------------------------------------------
def _rnd(*shape, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(DEV, torch.bfloat16)


@pytest.fixture(scope="module")
def be():
    from kareus_amd.backend import get_backend

    return get_backend("hip")


CASES = [
    # M (out features), N (in features), rows per piece, pieces
    (7168, 4096, 4096, 4),     # fc1 of workload c4: the transposed-store form, 256 K-steps
    (4096, 3584, 4096, 4),     # fc2
    (1536, 4096, 4096, 4),     # qkv: few tiles, the contraction is cut (cuts cross piece boundaries or not)
    (4096, 1024, 4096, 4),     # out-projection
    (1024, 512, 256, 2),       # the plumbing layer's sizes
    (520, 200, 64, 3),         # ragged tiles, one K-step per piece, an odd number of pieces
    (768, 768, 192, 8),        # the most pieces, three K-steps each
    (256, 256, 64, 1),         # a single piece is the plain product
]


@gpu
@pytest.mark.parametrize("m,n,k_seg,nseg", CASES)
@pytest.mark.parametrize("split_k", [True, False])
def test_pieces_equal_the_concatenation_bit_for_bit(be, m, n, k_seg, nseg, split_k):
    dys = [_rnd(k_seg, m, seed=10 + i) for i in range(nseg)]
    xs = [_rnd(k_seg, n, seed=50 + i) for i in range(nseg)]
    assert be.wgrad_segments_ok(dys, xs)
    got = be.linear_wgrad_segments(dys, xs, split_k=split_k)
    want = be.linear_wgrad(torch.cat(dys), torch.cat(xs), split_k=split_k)
    assert torch.equal(got, want)
    ref = torch.cat(dys).float().t() @ torch.cat(xs).float()
    assert (got.float() - ref).abs().max() <= TOL * ref.abs().max()
    # accumulating into an existing gradient
    base = _rnd(m, n, seed=99)
    acc = be.linear_wgrad_segments(dys, xs, out=base.clone(), accumulate=True, split_k=split_k)
    acc0 = be.linear_wgrad(torch.cat(dys), torch.cat(xs), out=base.clone(), accumulate=True, split_k=split_k)
    assert torch.equal(acc, acc0)


@gpu
def test_pieces_that_are_strided_views_in_any_order(be):
    """One-sequence nanobatches of a [s, b, h] tensor are matrices with row stride b*h: pieces of one
    allocation, interleaved; the order of the pieces is the order of the sum."""
    s, b, m, n = 512, 4, 1024, 768
    dy_all, x_all = _rnd(s, b, m, seed=1), _rnd(s, b, n, seed=2)
    dys = [be.rows_view(dy_all[:, i:i + 1]) for i in range(b)]
    xs = [be.rows_view(x_all[:, i:i + 1]) for i in range(b)]
    assert all(d.stride(0) == b * m for d in dys) and be.wgrad_segments_ok(dys, xs)
    got = be.linear_wgrad_segments(dys, xs)
    want = be.linear_wgrad(torch.cat([d.contiguous() for d in dys]), torch.cat([x.contiguous() for x in xs]))
    assert torch.equal(got, want)
    back = be.linear_wgrad_segments(dys[::-1], xs[::-1])
    want_back = be.linear_wgrad(torch.cat([d.contiguous() for d in dys[::-1]]), torch.cat([x.contiguous() for x in xs[::-1]]))
    assert torch.equal(back, want_back)
    ref = dy_all.float().reshape(-1, m).t() @ x_all.float().reshape(-1, n)
    for r in (got, back):
        assert (r.float() - ref).abs().max() <= TOL * ref.abs().max()


@gpu
@pytest.mark.parametrize("s,b,r,m,n", [(256, 8, 4, 768, 512), (64, 16, 8, 4096, 1024), (1024, 4, 2, 3072, 1024),
                                       (128, 32, 16, 640, 384), (4096, 8, 4, 3072, 1024)])
@pytest.mark.parametrize("split_k", [True, False])
def test_pieces_in_row_runs_equal_dense_copies(be, s, b, r, m, n, split_k):
    """The incoming gradient of a layer stack cut into nanobatches of r sequences: every piece of dy is a
    [s, r, m] slice whose rows come in runs, read where it lies; bit-equal to the launch on dense copies."""
    dy_all = _rnd(s, b, m, seed=3)
    dys = [dy_all[:, lo:lo + r] for lo in range(0, b, r)][:8]
    xs = [_rnd(s * r, n, seed=20 + i) for i in range(len(dys))]
    assert be.rows_view(dys[0]).dim() == 3 and be.wgrad_segments_ok(dys, xs)
    got = be.linear_wgrad_segments(dys, xs, split_k=split_k)
    want = be.linear_wgrad_segments([d.reshape(-1, m).contiguous() for d in dys], xs, split_k=split_k)
    assert torch.equal(got, want)
    ref = torch.cat([d.reshape(-1, m) for d in dys]).float().t() @ torch.cat(xs).float()
    assert (got.float() - ref).abs().max() <= TOL * ref.abs().max()


@gpu
def test_pairs_the_backend_turns_down(be):
    dys = [_rnd(128, 256, seed=i) for i in range(2)]
    xs = [_rnd(128, 512, seed=5 + i) for i in range(2)]
    assert be.wgrad_segments_ok(dys, xs)
    assert not be.wgrad_segments_ok(dys, [xs[0], _rnd(128, 520, seed=7)[:, :512]])     # another row stride
    assert not be.wgrad_segments_ok([d[:96] for d in dys], [x[:96] for x in xs])        # not whole K-steps
    assert not be.wgrad_segments_ok(dys * 5, xs * 5)                                    # more than eight pairs
    whole = _rnd(64, 8, 256, seed=9)
    assert be.wgrad_segments_ok([whole[:, 0:2], whole[:, 2:4]], xs)                     # rows in runs, both alike
    assert not be.wgrad_segments_ok([whole[:, 0:2], dys[1]], xs)                        # ... one in runs, one dense
    assert not be.wgrad_segments_ok([whole[:, 0:2], whole[:, 2:4]], [xs[0], whole[:, 4:6]])   # only dy may be in runs
    with pytest.raises(RuntimeError):
        be.linear_wgrad_segments([d[:96] for d in dys], [x[:96] for x in xs])


def _layer_grads(whole, nnb, b, s=256, at_end=None, recompute=False):
    from kareus_amd import LayerConfig, LayerStack

    cfg = LayerConfig(hidden_size=1024, num_attention_heads=8, num_query_groups=2, kv_channels=128,
                      ffn_hidden_size=1792, num_layers=2, num_nanobatches=nnb, backend="hip",
                      wgrad_over_all_nanobatches=whole, wgrad_launches_at_end=at_end,
                      checkpoint_activations=recompute)
    model = LayerStack(cfg, device=DEV, seed=1234)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(s, b, 1024, generator=g).to(DEV, torch.bfloat16).requires_grad_(True)
    go = torch.randn(s, b, 1024, generator=g).to(DEV, torch.bfloat16)
    outs = []
    for _ in range(2):                                                  # twice: the second pass reuses freed blocks
        for p in model.parameters():
            p.grad = None
        x.grad = None
        y = model(x)
        y.backward(go)
        torch.cuda.synchronize()
        outs.append((y.detach().clone(), x.grad.clone(), [p.grad.clone() for p in model.parameters()]))
    (y1, dx1, g1), (y2, dx2, g2) = outs
    assert torch.equal(y1, y2) and torch.equal(dx1, dx2) and all(torch.equal(a, c) for a, c in zip(g1, g2))
    return outs[0]


@gpu
@pytest.mark.parametrize("nnb,b", [(4, 4), (2, 4), (2, 2)])
def test_layer_step_with_one_weight_gradient_per_layer(nnb, b):
    """Two layers, nanobatches on their own streams: outputs and input gradients do not depend on how the
    weight gradients are summed (bit-equal); the weight gradients agree with the per-nanobatch
    accumulation within bf16 rounding and are the same on every pass."""
    y_w, dx_w, g_w = _layer_grads(True, nnb, b, at_end=False)
    y_p, dx_p, g_p = _layer_grads(False, nnb, b)
    assert torch.equal(y_w, y_p) and torch.equal(dx_w, dx_p)
    for a, c in zip(g_w, g_p):
        assert (a.float() - c.float()).abs().max() <= TOL * c.float().abs().max()
    # issued at the end of the backward pass instead of where the last nanobatch delivers: the same launches
    y_e, dx_e, g_e = _layer_grads(True, nnb, b, at_end=True)
    assert torch.equal(y_e, y_w) and torch.equal(dx_e, dx_w) and all(torch.equal(a, c) for a, c in zip(g_e, g_w))


@gpu
def test_recomputed_activations_feed_the_same_weight_gradient():
    """Activation recompute rebuilds the saved inputs inside the backward pass; the one weight-gradient launch
    per layer, issued at the end of that pass, must read them as it reads the saved ones."""
    kept = _layer_grads(True, 4, 4)
    again = _layer_grads(True, 4, 4, recompute=True)
    assert torch.equal(kept[0], again[0]) and torch.equal(kept[1], again[1])
    assert all(torch.equal(a, c) for a, c in zip(kept[2], again[2]))
