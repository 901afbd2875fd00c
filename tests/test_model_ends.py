"""Embedding, final norm, output layer and loss around the layer stack: the oracle's new functions
pinned by library routines and closed forms, the host engine against the oracle, the kernels
against the oracle on the device."""

import math

import pytest
import torch
import torch.nn.functional as F

from kareus_amd import GPTModelShard, LayerConfig
from kareus_amd.backend import get_backend
from oracle import llama_layer_ref as R

DIMS = R.LayerDims(hidden=64, nq=4, nkv=2, hd=16, ffn=48)
PARAMS = [("input_layernorm", "ln1"), ("linear_qkv", "w_qkv"), ("linear_proj", "w_proj"),
          ("pre_mlp_layernorm", "ln2"), ("linear_fc1", "w_fc1"), ("linear_fc2", "w_fc2")]


# ---- the oracle's own pins -----------------------------------------------------------------------
def test_oracle_cross_entropy_against_library_and_closed_forms():
    g = torch.Generator().manual_seed(0)
    logits, labels = torch.randn(5, 3, 40, generator=g, dtype=torch.float64), torch.randint(0, 40, (3, 5), generator=g)
    want = F.cross_entropy(logits.reshape(-1, 40), labels.t().reshape(-1), reduction="none").view(5, 3).t()
    assert torch.allclose(R.cross_entropy(logits, labels), want, atol=1e-12)
    # uniform logits: loss = log(vocab) whatever the label; one dominant logit on the label: loss -> 0
    assert torch.allclose(R.cross_entropy(torch.full((2, 2, 40), 3.0), torch.zeros(2, 2, dtype=torch.long)),
                          torch.full((2, 2), math.log(40.0)))
    peaked = torch.zeros(1, 1, 40)
    peaked[0, 0, 7] = 50.0
    assert R.cross_entropy(peaked, torch.tensor([[7]])).item() < 1e-6
    assert R.cross_entropy(peaked, torch.tensor([[8]])).item() == pytest.approx(50.0, abs=1e-4)
    # gradient of the summed loss: softmax - onehot, rows sum to zero
    x = logits.clone().requires_grad_(True)
    R.cross_entropy(x, labels).sum().backward()
    assert torch.allclose(x.grad.sum(-1), torch.zeros(5, 3, dtype=torch.float64), atol=1e-12)
    assert torch.allclose(x.grad, torch.softmax(logits, -1) - F.one_hot(labels.t(), 40), atol=1e-12)


def test_oracle_embedding_index_map_and_shard_mask():
    w = torch.arange(6 * 4, dtype=torch.float64).view(6, 4)          # row r holds 4r .. 4r+3
    ids = torch.tensor([[0, 5, 2], [3, 3, 1]])                       # [b=2, s=3]
    out = R.embedding(ids, w)
    assert out.shape == (3, 2, 4)
    for bi in range(2):
        for si in range(3):
            assert torch.equal(out[si, bi], w[ids[bi, si]])
    assert torch.allclose(out, F.embedding(ids, w).transpose(0, 1))
    shard = R.embedding(ids + 10, w[2:5], vocab_start=12)            # shard holds ids 12..14
    for bi in range(2):
        for si in range(3):
            tok = int(ids[bi, si]) + 10
            assert torch.equal(shard[si, bi], w[tok - 10] if 12 <= tok <= 14 else torch.zeros(4, dtype=torch.float64))
    # gradient: row r receives the sum of the upstream rows of the tokens that picked it
    wl = w.clone().requires_grad_(True)
    up = torch.arange(3 * 2 * 4, dtype=torch.float64).view(3, 2, 4)
    R.embedding(ids, wl).backward(up)
    assert torch.equal(wl.grad[3], up[0, 1] + up[1, 1]) and torch.equal(wl.grad[4], torch.zeros(4, dtype=torch.float64))


# ---- host engine -----------------------------------------------------------------------------------
def _cfg(backend, dtype, nnb=2, layers=2):
    return LayerConfig(hidden_size=DIMS.hidden, num_attention_heads=DIMS.nq, num_query_groups=DIMS.nkv,
                       kv_channels=DIMS.hd, ffn_hidden_size=DIMS.ffn, num_layers=layers, num_nanobatches=nnb,
                       params_dtype=dtype, backend=backend)


def _reference(model, ids, labels, loss_grad, vocab_start=0):
    f = lambda t: t.detach().float().cpu()
    layers = [{n: f(getattr(layer, a).weight) for a, n in PARAMS} for layer in model.decoder.layers]
    return R.model_forward_backward(ids.cpu(), labels.cpu(), f(model.embedding.weight), layers,
                                    f(model.final_layernorm), f(model.output_layer), DIMS, loss_grad.cpu(),
                                    vocab_start)


def _check(model, ids, labels, loss_grad, tol, vocab_start=0):
    loss = model(ids, labels)
    loss.backward(loss_grad.to(loss.device))
    rloss, rg = _reference(model, ids, labels, loss_grad, vocab_start)
    rel = lambda a, b: ((a.detach().float().cpu() - b).abs().max() / b.abs().max()).item()
    assert loss.shape == labels.shape and loss.dtype == torch.float32
    assert rel(loss, rloss) <= tol
    assert rel(model.embedding.weight.grad, rg["emb"]) <= tol
    assert rel(model.final_layernorm.grad, rg["final_gamma"]) <= tol
    assert rel(model.output_layer.grad, rg["w_out"]) <= tol
    for li, layer in enumerate(model.decoder.layers):
        for a, n in PARAMS:
            assert rel(getattr(layer, a).weight.grad, rg["layers"][li][n]) <= tol, (li, n)


@pytest.mark.parametrize("nnb", [1, 2])
def test_host_model_matches_oracle(nnb):
    g = torch.Generator().manual_seed(3)
    ids, labels = torch.randint(0, 96, (4, 32), generator=g), torch.randint(0, 96, (4, 32), generator=g)
    model = GPTModelShard(_cfg("eager", torch.float32, nnb), vocab_rows=96, seed=1234)
    _check(model, ids, labels, torch.rand(4, 32, generator=g), 2e-4)
    logits = model(ids)
    assert logits.shape == (32, 4, 96)


def test_host_vocabulary_shard_semantics():
    """A shard embeds foreign ids to zero; labels outside the shard's columns are ignored rows."""
    be = get_backend("eager")
    w = torch.randn(8, 16)
    ids = torch.tensor([[3, 20, 9], [10, 4, 17]])
    out = be.embedding_fwd(ids, w, vocab_start=4)
    assert torch.equal(out, R.embedding(ids, w, 4).contiguous())
    assert torch.equal(out[1, 0], torch.zeros(16)) and torch.equal(out[0, 1], w[6])
    dw = be.embedding_bwd(ids, torch.ones(3, 2, 16), 8, vocab_start=4)
    assert torch.equal(dw[:, 0], torch.tensor([1., 0, 0, 0, 0, 1, 1, 0]))      # ids 4, 9, 10 are inside
    loss, lse = be.cross_entropy_fwd(torch.zeros(3, 8), torch.tensor([2, -1, 8]))
    assert torch.allclose(loss, torch.tensor([math.log(8.0), 0.0, 0.0]))
    d = be.cross_entropy_bwd(torch.zeros(3, 8), torch.tensor([2, -1, 8]), lse, torch.ones(3))
    assert torch.equal(d[1], torch.zeros(8)) and d[0, 2] == pytest.approx(1 / 8 - 1)


# ---- kernels -----------------------------------------------------------------------------------------
gpu = pytest.mark.gpu


@gpu
@pytest.mark.parametrize("b,s,hidden,rows,start", [(2, 128, 512, 1000, 0), (4, 96, 4096, 520, 256), (1, 64, 1032, 37, 5)])
def test_embedding_kernels(b, s, hidden, rows, start):
    be = get_backend("hip")
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, rows + 2 * start + 3, (b, s), generator=g).cuda()
    w = torch.randn(rows, hidden, generator=g).cuda().bfloat16()
    out = be.embedding_fwd(ids, w, start)
    assert torch.equal(out.float().cpu(), R.embedding(ids.cpu(), w.float().cpu(), start))     # a gather: exact
    dout = torch.randn(s, b, hidden, generator=g).cuda().bfloat16()
    dw = be.embedding_bwd(ids, dout, rows, start)
    wl = w.float().cpu().requires_grad_(True)
    R.embedding(ids.cpu(), wl, start).backward(dout.float().cpu())
    assert ((dw.float().cpu() - wl.grad).abs().max() / wl.grad.abs().max()).item() <= 2e-2    # bf16 store
    untouched = wl.grad.abs().sum(-1) == 0
    assert torch.equal(dw.float().cpu()[untouched], torch.zeros_like(wl.grad[untouched]))    # written as zeros
    assert torch.equal(dw, be.embedding_bwd(ids, dout, rows, start))                          # reproducible


@gpu
def test_embedding_backward_with_heavily_repeated_ids():
    """A block of 64 vocabulary rows that attracts more tokens than its LDS key list holds (4096) falls
    back to one in-order scan per row; a sparse block in the same launch takes the sorted-list path."""
    be = get_backend("hip")
    g = torch.Generator().manual_seed(8)
    b, s, hidden, rows = 4, 2048, 256, 200
    ids = torch.randint(0, 4, (b, s), generator=g)                  # four ids only: 8192 tokens in block 0
    ids[3, -3:] = torch.tensor([150, 199, 150])                     # block 2 sees three tokens
    ids[0, :5] = torch.tensor([63, 62, 40, 40, 9])
    dout = torch.randn(s, b, hidden, generator=g).cuda().bfloat16()
    dw = be.embedding_bwd(ids.cuda(), dout, rows)
    wl = torch.zeros(rows, hidden).requires_grad_(True)
    R.embedding(ids, wl).backward(dout.float().cpu())
    assert ((dw.float().cpu() - wl.grad).abs().max() / wl.grad.abs().max()).item() <= 2e-2
    assert torch.equal(dw[40].float().cpu(), (dout[2, 0].float() + dout[3, 0].float()).cpu().bfloat16().float())
    assert torch.equal(dw[9], dout[4, 0]) and torch.equal(dw[63], dout[0, 0]) and torch.equal(dw[199], dout[-2, 3])
    assert torch.equal(dw[100], torch.zeros_like(dw[100]))


@gpu
@pytest.mark.parametrize("rows,vocab", [(64, 32064), (200, 1000), (7, 8)])
def test_cross_entropy_kernels(rows, vocab):
    be = get_backend("hip")
    g = torch.Generator().manual_seed(6)
    logits = (4 * torch.randn(rows, vocab, generator=g)).cuda().bfloat16()
    labels = torch.randint(0, vocab, (rows,), generator=g)
    labels[1] = -1                                                                            # an ignored row
    labels = labels.cuda()
    loss, lse = be.cross_entropy_fwd(logits, labels)
    lf = logits.float().cpu()
    want_lse = torch.logsumexp(lf, -1)
    live = labels.cpu() >= 0
    want = torch.where(live, want_lse - lf.gather(1, labels.cpu().clamp(min=0)[:, None])[:, 0], torch.zeros(rows))
    assert (lse.cpu() - want_lse).abs().max() <= 1e-3 and (loss.cpu() - want).abs().max() <= 1e-3
    dloss = torch.rand(rows, generator=g).cuda()
    d = be.cross_entropy_bwd(logits, labels, lse, dloss)
    ref = torch.softmax(lf, -1)
    ref[live, labels.cpu()[live]] -= 1
    ref = ref * (dloss.cpu() * live)[:, None]
    assert ((d.float().cpu() - ref).abs().max() / ref.abs().max()).item() <= 2e-2
    assert torch.equal(d[1], torch.zeros_like(d[1]))
    same = be.cross_entropy_bwd(logits.clone(), labels, lse, dloss, in_place=True)            # may overwrite the logits
    assert torch.equal(same, d)
    # uniform logits: loss = log(vocab)
    u, _ = be.cross_entropy_fwd(torch.zeros(4, vocab, device="cuda", dtype=torch.bfloat16), torch.zeros(4, dtype=torch.long, device="cuda"))
    assert (u.cpu() - math.log(vocab)).abs().max() <= 1e-3


@gpu
def test_device_model_matches_oracle():
    global DIMS
    dims = R.LayerDims(hidden=512, nq=4, nkv=2, hd=128, ffn=640)
    cfg = LayerConfig(hidden_size=512, num_attention_heads=4, num_query_groups=2, kv_channels=128,
                      ffn_hidden_size=640, num_layers=2, num_nanobatches=2, backend="hip")
    g = torch.Generator().manual_seed(7)
    ids, labels = torch.randint(0, 2048, (4, 256), generator=g), torch.randint(0, 2048, (4, 256), generator=g)
    model = GPTModelShard(cfg, vocab_rows=2048, device="cuda", seed=1234)
    saved, DIMS = DIMS, dims
    try:
        _check(model, ids.cuda(), labels.cuda(), torch.rand(4, 256, generator=g), 2e-2)       # bf16 vs fp32: 2e-2
    finally:
        DIMS = saved
