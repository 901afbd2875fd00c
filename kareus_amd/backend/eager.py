"""Eager-PyTorch implementation of the operator primitives (host plumbing only).

Each primitive states the formula of the native call it stands in for; the HIP
backend implements the same contracts on the device.
"""

from __future__ import annotations

import math
from typing import Tuple

import torch
from torch import Tensor


class EagerBackend:
    name = "eager"

    # y = x . W^T, dx = dy . W, dW = dy^T . x   (reference call sites:
    # kareus/transformer_engine/pytorch/ops/basic/basic_linear.py:571-582, 847-859, 898-909)
    def linear_fwd(self, x: Tensor, w: Tensor, split_k: bool = True, out: Tensor = None,
                   residual: Tensor = None, swiglu_out: Tensor = None, max_cus: int = 0) -> Tensor:
        y = x @ w.t()
        if residual is not None:       # rounded product first, then the add: as the two separate ops
            y = residual + y
        if swiglu_out is not None:
            a, b = y.chunk(2, dim=-1)
            swiglu_out.copy_((torch.nn.functional.silu(a.float()) * b.float()).to(y.dtype))
        if out is not None:
            out.copy_(y)
            return out
        return y

    @staticmethod
    def can_fuse_swiglu(two_f: int) -> bool:
        return two_f % 2 == 0

    # the eager ops take [rows, cols] matrices; anything a view cannot express is copied
    supports_row_runs = False

    @staticmethod
    def rows_view(t: Tensor):
        try:
            return t.view(-1, t.shape[-1])
        except RuntimeError:
            return None

    @staticmethod
    def rows_in_place(t: Tensor) -> Tensor:
        return t.reshape(-1, t.shape[-1])

    def linear_dgrad(self, dy: Tensor, w: Tensor, split_k: bool = True, swiglu_bwd_x: Tensor = None) -> Tensor:
        g = dy @ w
        return g if swiglu_bwd_x is None else self.swiglu_bwd(g, swiglu_bwd_x)

    can_fuse_swiglu_bwd = True

    def linear_wgrad(self, dy: Tensor, x: Tensor, out: Tensor = None, accumulate: bool = False,
                     split_k: bool = True) -> Tensor:
        dw = dy.t() @ x
        if out is None:
            return dw
        if accumulate:
            out.add_(dw)
        else:
            out.copy_(dw)
        return out

    @staticmethod
    def wgrad_segments_ok(dys, xs) -> bool:
        return len(dys) == len(xs) >= 1

    def linear_wgrad_segments(self, dys, xs, out: Tensor = None, accumulate: bool = False,
                              split_k: bool = True) -> Tensor:
        """``sum_i dys[i]^T . xs[i]`` as one product over all rows."""
        return self.linear_wgrad(torch.cat(list(dys)), torch.cat(list(xs)), out=out, accumulate=accumulate)

    # rs = rsqrt(mean(x^2) + eps) in fp32, y = (x * rs) * gamma
    # (3rdparty/TransformerEngine/transformer_engine/common/normalization/rmsnorm/
    #  rmsnorm_fwd_kernels.cuh:90-121)
    def rmsnorm_fwd(self, x: Tensor, gamma: Tensor, eps: float) -> Tuple[Tensor, Tensor]:
        xf = x.float()
        rstd = torch.rsqrt(xf.pow(2).mean(dim=-1) + eps)
        y = (xf * rstd[:, None]) * gamma.float()
        return y.to(x.dtype), rstd

    # dx = rs * (g - xhat * mean(g * xhat)), g = gamma * dy ; dgamma = sum_rows dy * xhat
    # (rmsnorm_bwd_kernels.cuh:95-128)
    def rmsnorm_partial_rows(self, rows: int, cols: int) -> int:
        return 1

    def rmsnorm_dgamma(self, partials: Tensor, gamma: Tensor) -> Tensor:
        return partials.sum(dim=0).to(gamma.dtype)

    def rmsnorm_bwd(self, dy: Tensor, x: Tensor, rstd: Tensor, gamma: Tensor,
                    residual_grad: Tensor = None, out: Tensor = None,
                    partials_out: Tensor = None) -> Tuple[Tensor, Tensor]:
        xhat = x.float() * rstd[:, None]
        dyf = dy.float()
        g = dyf * gamma.float()
        dx = rstd[:, None] * (g - xhat * (g * xhat).mean(dim=-1, keepdim=True))
        dgamma = (dyf * xhat).sum(dim=0)
        dx = dx.to(x.dtype)
        if residual_grad is not None:
            dx = dx + residual_grad        # rounded first, then added: as the two separate ops do
        if out is not None:
            out.copy_(dx)
            dx = out
        if partials_out is not None:
            partials_out.copy_(dgamma.view(1, -1))
            return dx, None
        return dx, dgamma.to(gamma.dtype)

    # y = t cos f + rotate_half(t) sin f, rotate_half([a, b]) = [-b, a]; trig in fp32
    # (kareus/megatron/core/models/common/embedding/rope_utils.py:147-182)
    @staticmethod
    def _rope(t: Tensor, freqs: Tensor, sign: float) -> Tensor:
        rot = freqs.shape[-1]
        cos, sin = torch.cos(freqs.float()), torch.sin(freqs.float()) * sign
        tr = t[..., :rot].float()
        a, b = tr.chunk(2, dim=-1)
        out = tr * cos + torch.cat((-b, a), dim=-1) * sin
        if rot < t.shape[-1]:
            out = torch.cat((out, t[..., rot:].float()), dim=-1)
        return out.to(t.dtype)

    def rope_fwd(self, t: Tensor, freqs: Tensor) -> Tensor:
        if t.dim() == 5:  # grouped [s, b, ng, per, hd] query view
            t = t.flatten(2, 3)
        return self._rope(t, freqs, 1.0)

    # The gradient of a rotation is the rotation by the opposite angle (rope_utils.py:207-222).
    def rope_bwd(self, g: Tensor, freqs: Tensor) -> Tensor:
        if g.dim() == 5:
            g = g.flatten(2, 3)
        return self._rope(g, freqs, -1.0)

    # y = silu(x1) * x2 with x1, x2 = chunk(x, 2, -1)
    # (kareus/megatron/core/extensions/ops/bias_swiglu.py:14-20, 34-44)
    def swiglu_fwd(self, x: Tensor) -> Tensor:
        x1, x2 = x.float().chunk(2, dim=-1)
        return (torch.nn.functional.silu(x1) * x2).to(x.dtype)

    def swiglu_bwd(self, dy: Tensor, x: Tensor) -> Tensor:
        x1, x2 = x.float().chunk(2, dim=-1)
        g = dy.float()
        sig = torch.sigmoid(x1)
        d1 = g * sig * (1 + x1 * (1 - sig)) * x2
        d2 = g * x1 * sig
        return torch.cat((d1, d2), dim=-1).to(x.dtype)

    def add(self, a: Tensor, b: Tensor, out: Tensor = None) -> Tensor:
        if out is None:
            return a + b
        if out.shape != a.shape:
            raise RuntimeError(f"add: out has shape {tuple(out.shape)}, operands {tuple(a.shape)}")
        return torch.add(a, b, out=out)

    # residual + dropout(x) and the byte mask (kareus/megatron/core/extensions/ops/bias_dropout_add.py:15-45)
    def dropout_add(self, x: Tensor, residual: Tensor, p: float, out: Tensor = None):
        seed = int(torch.randint(0, 1 << 62, (1,), dtype=torch.int64).item())   # as the hip backend draws it
        gen = torch.Generator(device=x.device).manual_seed(seed)
        keep = torch.rand(x.shape, generator=gen, device=x.device) >= p
        dropped = (x.float() * keep / (1.0 - p)).to(x.dtype)
        total = (residual.float() + dropped.float()).to(x.dtype)
        if out is not None:
            if out.shape != x.shape:
                raise RuntimeError(f"dropout_add: out has shape {tuple(out.shape)}, operands {tuple(x.shape)}")
            out.copy_(total)
            total = out
        return total, keep.to(torch.uint8)

    def dropout_bwd(self, dy: Tensor, mask: Tensor, scale: float) -> Tensor:
        return (dy.float() * mask * scale).to(dy.dtype)

    # RMSNorm over the head dimension of the query and key heads of a fused QKV buffer
    # [s, b, groups, per + 2, hd]; value heads carried along (qkv_postprocess.py:115-118, 150-157).
    @staticmethod
    def _qk_weights(gamma_q: Tensor, gamma_k: Tensor, per: int) -> Tensor:
        return torch.cat([gamma_q.float().expand(per, -1), gamma_k.float()[None]], dim=0)  # [per + 1, hd]

    def qk_norm_fwd(self, mixed5: Tensor, gamma_q: Tensor, gamma_k: Tensor, eps: float) -> Tuple[Tensor, Tensor]:
        per = mixed5.shape[3] - 2
        x = mixed5[..., :per + 1, :].float()
        rstd = torch.rsqrt(x.pow(2).mean(-1) + eps)
        y = (x * rstd[..., None] * self._qk_weights(gamma_q, gamma_k, per)).to(mixed5.dtype)
        return torch.cat([y, mixed5[..., per + 1:, :]], dim=3), rstd

    def qk_norm_bwd(self, dmixed5: Tensor, mixed5: Tensor, rstd: Tensor, gamma_q: Tensor,
                    gamma_k: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
        per = mixed5.shape[3] - 2
        xhat = mixed5[..., :per + 1, :].float() * rstd[..., None]
        dy = dmixed5[..., :per + 1, :].float()
        dyg = dy * self._qk_weights(gamma_q, gamma_k, per)
        dx = rstd[..., None] * (dyg - xhat * (dyg * xhat).mean(-1, keepdim=True))
        dgam = (dy * xhat).sum(dim=(0, 1, 2))                      # [per + 1, hd]
        out = torch.cat([dx.to(dmixed5.dtype), dmixed5[..., per + 1:, :]], dim=3)
        return out, dgam[:per].sum(0).to(gamma_q.dtype), dgam[per].to(gamma_k.dtype)

    # Causal GQA attention on [s, b, heads, hd] tensors; query head i reads KV head
    # i // (nq / nkv); lse = logsumexp of the scaled, masked scores, [b, nq, s] fp32
    # (kareus/flash_attn/flash_attn_interface.py:473-493).
    def attn_fwd(self, q: Tensor, k: Tensor, v: Tensor, scale: float, causal: bool = True,
                 beside_other_streams: bool = False):
        if q.dim() == 5:
            q = q.flatten(2, 3)
        s, b, nq, hd = q.shape
        nkv = k.shape[2]
        rep = nq // nkv
        qf = q.float().permute(1, 2, 0, 3)
        kf = k.float().permute(1, 2, 0, 3).repeat_interleave(rep, dim=1)
        vf = v.float().permute(1, 2, 0, 3).repeat_interleave(rep, dim=1)
        scores = (qf @ kf.transpose(-1, -2)) * scale
        if causal:
            mask = torch.ones(s, s, dtype=torch.bool, device=q.device).tril()
            scores = scores.masked_fill(~mask, float("-inf"))
        lse = torch.logsumexp(scores, dim=-1)
        p = torch.exp(scores - lse[..., None])
        o = (p @ vf).permute(2, 0, 1, 3).contiguous()
        return o.to(q.dtype), lse.contiguous()

    def attn_bwd(self, do, q, k, v, o, lse, scale: float, causal: bool = True, beside_other_streams: bool = False):
        if q.dim() == 5:
            q = q.flatten(2, 3)
        s, b, nq, hd = q.shape
        nkv = k.shape[2]
        rep = nq // nkv
        qf = q.float().permute(1, 2, 0, 3)
        kf = k.float().permute(1, 2, 0, 3).repeat_interleave(rep, dim=1)
        vf = v.float().permute(1, 2, 0, 3).repeat_interleave(rep, dim=1)
        dof = do.float().reshape(s, b, nq, hd).permute(1, 2, 0, 3)
        of = o.float().reshape(s, b, nq, hd).permute(1, 2, 0, 3)
        scores = (qf @ kf.transpose(-1, -2)) * scale
        if causal:
            mask = torch.ones(s, s, dtype=torch.bool, device=q.device).tril()
            scores = scores.masked_fill(~mask, float("-inf"))
        p = torch.exp(scores - lse[..., None])
        dv = p.transpose(-1, -2) @ dof
        dp = dof @ vf.transpose(-1, -2)
        delta = (dof * of).sum(dim=-1, keepdim=True)
        ds = p * (dp - delta) * scale
        dq = ds @ kf
        dk = ds.transpose(-1, -2) @ qf
        dk = dk.reshape(b, nkv, rep, s, hd).sum(dim=2)
        dv = dv.reshape(b, nkv, rep, s, hd).sum(dim=2)
        back = lambda t: t.permute(2, 0, 1, 3).contiguous()
        return back(dq).to(q.dtype), back(dk).to(k.dtype), back(dv).to(v.dtype)

    # Vocabulary-shard embedding: rows of other shards give zeros
    # (3rdparty/Megatron-LM/megatron/core/tensor_parallel/layers.py:245-263); output [s, b, h]
    # (models/common/embeddings/language_model_embedding.py:114-116).
    def embedding_fwd(self, ids: Tensor, weight: Tensor, vocab_start: int = 0) -> Tensor:
        rel = ids - vocab_start
        other = (rel < 0) | (rel >= weight.shape[0])
        out = weight[rel.masked_fill(other, 0)]
        out = out.masked_fill(other[..., None], 0.0)
        return out.transpose(0, 1).contiguous()

    def embedding_bwd(self, ids: Tensor, dout: Tensor, vocab_rows: int, vocab_start: int = 0) -> Tensor:
        rel = (ids - vocab_start).transpose(0, 1).reshape(-1)          # [s, b] order like dout
        keep = (rel >= 0) & (rel < vocab_rows)
        dw = torch.zeros(vocab_rows, dout.shape[-1], dtype=torch.float32, device=dout.device)
        dw.index_add_(0, rel[keep], dout.reshape(-1, dout.shape[-1])[keep].float())
        return dw.to(dout.dtype)

    # loss = logsumexp(logits) - logits[label]; rows whose label is outside [0, vocab) are ignored
    def cross_entropy_fwd(self, logits: Tensor, labels: Tensor) -> Tuple[Tensor, Tensor]:
        lf = logits.float()
        lse = torch.logsumexp(lf, dim=-1)
        live = (labels >= 0) & (labels < logits.shape[-1])
        picked = lf.gather(1, labels.masked_fill(~live, 0)[:, None])[:, 0]
        return torch.where(live, lse - picked, torch.zeros_like(lse)), lse

    def cross_entropy_bwd(self, logits: Tensor, labels: Tensor, lse: Tensor, dloss: Tensor,
                          in_place: bool = False) -> Tensor:
        live = (labels >= 0) & (labels < logits.shape[-1])
        d = torch.exp(logits.float() - lse[:, None])
        d[live, labels[live]] -= 1.0
        d = d * torch.where(live, dloss.float(), torch.zeros_like(lse))[:, None]
        return d.to(logits.dtype)

    def default_scale(self, hd: int) -> float:
        return 1.0 / math.sqrt(hd)
