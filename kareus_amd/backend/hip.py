"""The product backend: gfx950 kernels of ``libkareus_hip.so`` called through its C ABI.

PyTorch supplies device memory and the current HIP stream; every arithmetic step is a
hand-written kernel.  There is no fallback: a missing library, a non-HIP tensor or a
dtype other than bf16 raises.
"""

from __future__ import annotations

import ctypes
import os
from typing import Tuple

import torch
from torch import Tensor

from . import reserved_compute_units

_LIB_NAME = "libkareus_hip.so"
_c_void_p, _c_int, _c_i64, _c_float, _c_size_t = (
    ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_size_t,
)

# name -> (restype, argtypes); mirrors include/kareus_hip.h
_SIGNATURES = {
    "kr_version": (_c_int, []),
    "kr_error_string": (ctypes.c_char_p, [_c_int]),
    "kr_device_clock_mhz": (_c_int, []),
    "kr_gemm_workspace_bytes": (_c_size_t, [_c_int, _c_int, _c_int, _c_int]),
    "kr_gemm_workspace_bytes_shared": (_c_size_t, [_c_int, _c_int, _c_int, _c_int, _c_float]),
    "kr_gemm_bf16": (_c_int, [_c_int, _c_int, _c_int, _c_int, _c_void_p, _c_i64, _c_void_p, _c_i64,
                              _c_void_p, _c_i64, _c_int, _c_void_p, _c_size_t, _c_void_p]),
    "kr_gemm_bf16_fused": (_c_int, [_c_int, _c_int, _c_int, _c_int, _c_void_p, _c_i64, _c_void_p, _c_i64,
                                    _c_void_p, _c_i64, _c_int, _c_int, _c_void_p, _c_i64, _c_void_p, _c_i64,
                                    _c_int, _c_void_p, _c_size_t, _c_void_p]),
    "kr_gemm_bf16_runs": (_c_int, [_c_int, _c_int, _c_int, _c_int, _c_void_p, _c_i64, _c_int, _c_i64, _c_void_p, _c_i64,
                                   _c_void_p, _c_i64, _c_int, _c_i64, _c_int, _c_int, _c_void_p, _c_i64, _c_int, _c_i64,
                                   _c_void_p, _c_i64, _c_int, _c_void_p, _c_size_t, _c_void_p]),
    "kr_gemm_bf16_nt_segments": (_c_int, [_c_int, _c_int, _c_int, _c_int, _c_void_p, _c_i64, _c_int, _c_i64, _c_void_p, _c_i64,
                                          _c_void_p, _c_i64, _c_int, _c_int, _c_int, _c_void_p, _c_size_t, _c_void_p]),
    "kr_rmsnorm_fwd": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_i64, _c_float, _c_void_p]),
    "kr_rmsnorm_fwd_runs": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_i64, _c_int, _c_i64,
                                     _c_float, _c_void_p]),
    "kr_rmsnorm_bwd_add_runs": (_c_int, [_c_void_p] * 8 + [_c_int, _c_int, _c_i64, _c_i64, _c_int, _c_i64, _c_i64, _c_int,
                                                           _c_i64, _c_i64, _c_int, _c_i64, _c_void_p]),
    "kr_rmsnorm_bwd_workspace_bytes": (_c_size_t, [_c_int, _c_int]),
    "kr_rmsnorm_bwd": (_c_int, [_c_void_p] * 7 + [_c_int, _c_int, _c_i64, _c_i64, _c_void_p]),
    "kr_rmsnorm_bwd_add": (_c_int, [_c_void_p] * 8 + [_c_int, _c_int] + [_c_i64] * 4 + [_c_void_p]),
    "kr_rmsnorm_bwd_partial_rows": (_c_int, [_c_int, _c_int]),
    "kr_rmsnorm_dgamma": (_c_int, [_c_void_p, _c_int, _c_int, _c_void_p, _c_void_p]),
    "kr_rmsnorm_bwd_add_noalloc": (_c_int, [_c_void_p] * 7 + [_c_int, _c_int] + [_c_i64] * 4 + [_c_void_p]),
    "kr_rope": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int] + [_c_i64] * 6
                + [_c_int, _c_int, _c_int, _c_void_p]),
    "kr_swiglu_fwd": (_c_int, [_c_void_p, _c_void_p, _c_i64, _c_int, _c_void_p]),
    "kr_swiglu_bwd": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_i64, _c_int, _c_void_p]),
    "kr_add": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_i64, _c_void_p]),
    "kr_add_rows": (_c_int, [_c_void_p, _c_i64, _c_void_p, _c_i64, _c_void_p, _c_i64, _c_i64, _c_int, _c_void_p]),
    "kr_dropout_add": (_c_int, [_c_void_p, _c_i64, _c_void_p, _c_i64, _c_void_p, _c_i64, _c_void_p, _c_i64, _c_int,
                                _c_float, ctypes.c_uint64, ctypes.c_uint64, _c_void_p]),
    "kr_dropout_bwd": (_c_int, [_c_void_p, _c_i64, _c_void_p, _c_void_p, _c_i64, _c_i64, _c_int, _c_float, _c_void_p]),
    "kr_qk_norm_bwd_workspace_bytes": (_c_size_t, [_c_i64, _c_int, _c_int, _c_int]),
    "kr_qk_norm_fwd": (_c_int, [_c_void_p] * 5 + [_c_i64, _c_int, _c_int, _c_int, _c_float, _c_void_p]),
    "kr_qk_norm_bwd": (_c_int, [_c_void_p] * 8 + [_c_i64, _c_int, _c_int, _c_int, _c_void_p]),
    "kr_embedding_fwd": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_i64, _c_i64, _c_void_p]),
    "kr_embedding_bwd": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_i64, _c_i64, _c_void_p]),
    "kr_cross_entropy_fwd": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_i64, _c_int, _c_i64, _c_void_p]),
    "kr_cross_entropy_bwd": (_c_int, [_c_void_p] * 5 + [_c_i64, _c_int, _c_i64, _c_i64, _c_void_p]),
    "kr_attn_fwd": (_c_int, [_c_void_p] * 5 + [_c_int] * 5 + [_c_float] + [_c_i64] * 14 + [_c_void_p]),
    "kr_attn_fwd_flags": (_c_int, [_c_void_p] * 5 + [_c_int] * 5 + [_c_float] + [_c_i64] * 14 + [_c_int, _c_void_p]),
    "kr_attn_fwd_workspace_bytes": (_c_size_t, [_c_int] * 5),
    "kr_attn_fwd_ws": (_c_int, [_c_void_p] * 5 + [_c_int] * 5 + [_c_float] + [_c_i64] * 14 +
                       [_c_int, _c_void_p, _c_size_t, _c_void_p]),
    "kr_attn_bwd_workspace_bytes": (_c_size_t, [_c_int] * 5),
    "kr_attn_bwd": (_c_int, [_c_void_p] * 10 + [_c_int] * 5 + [_c_float] + [_c_i64] * 28 + [_c_void_p]),
    "kr_attn_bwd_flags": (_c_int, [_c_void_p] * 10 + [_c_int] * 5 + [_c_float] + [_c_i64] * 28 + [_c_int, _c_void_p]),
}

KR_GEMM_TN, KR_GEMM_NN, KR_GEMM_NT = 0, 1, 2
KR_ATTN_BESIDE_OTHER_STREAMS = 0x100
KR_ATTN_GENERAL_KERNELS = 0x200


def library_path() -> str:
    return os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), _LIB_NAME)


def load_library() -> ctypes.CDLL:
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} is missing: build it with `make -C kareus_amd/csrc` "
            "(or __graft_entry__.build()). The hip backend has no fallback."
        )
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


class HipBackend:
    name = "hip"

    def __init__(self) -> None:
        self.lib = load_library()
        self._gemm_ws_bytes: dict = {}  # (layout, m, n, k, split_k) -> workspace bytes
        self._ws_cache: dict = {}       # (stream, device) -> reusable workspace buffer
        self._cu_count: dict = {}       # device index -> compute units
        self._attn_ws_bytes: dict = {}  # (s, b, nq, nkv, hd) -> forward workspace bytes of a padded shape

    # -- plumbing -------------------------------------------------------------------
    # the raw handle of the current stream without building a torch.cuda.Stream object: this is
    # asked once per kernel launch
    _raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    _raw_device = getattr(torch._C, "_cuda_getDevice", None)

    @classmethod
    def _stream(cls) -> int:
        if cls._raw_stream is not None and cls._raw_device is not None:
            return cls._raw_stream(cls._raw_device())
        return torch.cuda.current_stream().cuda_stream

    def _check(self, rc: int, what: str) -> None:
        if rc != 0:
            raise RuntimeError(f"{what} failed: {self.lib.kr_error_string(rc).decode()} (code {rc})")

    @staticmethod
    def _dev(*tensors: Tensor) -> None:
        for t in tensors:
            if not t.is_cuda:
                raise RuntimeError("the hip backend needs tensors on the HIP device")
            if t.dtype not in (torch.bfloat16, torch.float32):
                raise RuntimeError(f"unsupported dtype {t.dtype}")

    @staticmethod
    def _on_device(index: Tensor) -> None:
        if not index.is_cuda or index.dtype != torch.int64:
            raise RuntimeError("index tensors must be int64 on the HIP device")

    @staticmethod
    def _bf16(*tensors: Tensor) -> None:
        for t in tensors:
            if t.dtype != torch.bfloat16:
                raise RuntimeError(f"the hip backend computes in bf16, got {t.dtype}")

    # -- row runs ---------------------------------------------------------------------
    # A nanobatch of r sequences of a [s, b, h] tensor is a [s, r, h] view with strides (b*h, h, 1): its
    # rows come in runs of r (stride h) whose starts are b*h apart.  The *_runs entry points address it
    # in place; r has to be a power of two (at most MAX_RUN_ROWS for the GEMM).
    supports_row_runs = True
    MAX_RUN_ROWS = 16

    @staticmethod
    def _operand(t: Tensor):
        """``(rows, ld, run_rows, run_ld)`` of a [rows, cols] matrix or a [s, r, cols] run tensor that the
        kernels address in place, or None when ``t`` has to be copied."""
        if t.stride(-1) != 1:
            return None
        cols = t.shape[-1]
        if t.dim() == 2:
            ld = t.stride(0)
            return (t.shape[0], ld, 1, 0) if (ld % 8 == 0 and ld >= cols) or t.shape[0] == 1 else None
        if t.dim() != 3:
            return None
        s_, r, _ = t.shape
        outer, ld = t.stride(0), t.stride(1)
        if r == 1:
            return (s_, outer, 1, 0) if outer % 8 == 0 and outer >= cols else None
        if ld % 8 or ld < cols or outer % 8:
            return None
        if outer == r * ld or s_ == 1:
            return (s_ * r, ld, 1, 0)
        if r & (r - 1) or r > HipBackend.MAX_RUN_ROWS or outer < r * ld:
            return None
        return (s_ * r, ld, r, outer)

    def rows_view(self, t: Tensor):
        """``t`` ([..., cols]) as the kernels can address it in place: a [rows, cols] view when its rows have
        one stride, ``t`` itself when it is a [s, r, cols] tensor whose rows come in runs; None when only a
        copy would do."""
        cols = t.shape[-1]
        # (whether the leading dimensions merge into one is read off the strides: asking ``view`` and catching
        # its error costs 10 us per nanobatch slice that does not)
        lead = [(n, st) for n, st in zip(t.shape[:-1], t.stride()[:-1]) if n != 1]
        if all(a[1] == b[0] * b[1] for a, b in zip(lead, lead[1:])) and t.numel():
            m = t.view(-1, cols)
            if self._operand(m) is not None:
                return m
        if t.dim() == 3 and self._operand(t) is not None:
            return t
        return None

    def rows_in_place(self, t: Tensor) -> Tensor:
        """``rows_view(t)``, or a dense [rows, cols] copy when the kernels cannot address ``t`` as it lies."""
        v = self.rows_view(t)
        return v if v is not None else t.reshape(-1, t.shape[-1]).contiguous()

    # -- GEMM -------------------------------------------------------------------------
    def _num_cus(self, device) -> int:
        n = self._cu_count.get(device.index)
        if n is None:
            n = self._cu_count[device.index] = torch.cuda.get_device_properties(device).multi_processor_count
        return n

    # the weight the library's planner gives a launch's own latency (against its compute-unit time) when the
    # launch runs beside other streams' kernels (KR_GEMM_BESIDE_OTHER_STREAMS): the workspace is sized with
    # the same weight, so the cuts the dispatcher plans are the cuts the buffer holds
    SHARED_LATENCY_WEIGHT = 0.1

    def _workspace(self, nbytes: int, device) -> Tensor:
        """A workspace of at least ``nbytes`` for the current stream.  One buffer per (stream, size
        class) is kept and reused: kernels on one stream run in order, so consecutive launches may
        share it, and a fresh ``torch.empty`` per launch costs more host time than the launch."""
        key = (self._stream(), device.index)
        buf = self._ws_cache.get(key)
        if buf is None or buf.numel() < nbytes:
            buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
            self._ws_cache[key] = buf
        return buf

    def gemm(self, layout: int, a: Tensor, b: Tensor, m: int, n: int, k: int,
             out: Tensor = None, accumulate: bool = False, split_k: bool = True,
             residual: Tensor = None, swiglu_out: Tensor = None, max_cus: int = 0,
             swiglu_bwd_x: Tensor = None) -> Tensor:
        """``split_k=True``: the GEMM has the GPU to itself and splits the contraction of a small
        output for the shortest latency.  ``split_k=False``: kernels of other streams are there
        to use the CUs a small output leaves idle, so the split count is chosen mostly for the
        least CU-time (often no split at all).
        ``residual`` ([m, n], row-strided): added to the bf16-rounded product in the epilogue.
        ``swiglu_out`` ([m, n/2]): also receives silu(out[:, :n/2]) * out[:, n/2:] (layout TN).
        ``max_cus``: compute-unit budget of the launch (0 = the whole device).
        ``swiglu_bwd_x`` ([m, 2n], layout NN): the product is the gradient of a SwiGLU output and
        is not stored; ``out`` ([m, 2n]) receives the gradient of the activation's input instead."""
        self._dev(a, b)
        self._bf16(a, b)
        if a.stride(-1) != 1 or b.stride(-1) != 1:
            raise RuntimeError("GEMM operands must have a contiguous last dimension")
        a_op = self._operand(a)
        if a_op is None or b.dim() != 2:
            raise RuntimeError("GEMM operands must be matrices with one row stride (A may have row runs)")
        if out is None:
            out = torch.empty((m, 2 * n if swiglu_bwd_x is not None else n), dtype=torch.bfloat16, device=a.device)
        epi, aux_ptr, aux_ld, out2_ptr, out2_ld = 0, None, 0, None, 0
        if swiglu_bwd_x is not None:
            if residual is not None or swiglu_out is not None or accumulate:
                raise RuntimeError("one fused epilogue at a time")
            self._dev(swiglu_bwd_x)
            self._bf16(swiglu_bwd_x)
            if tuple(swiglu_bwd_x.shape) != (m, 2 * n) or swiglu_bwd_x.stride(1) != 1 or tuple(out.shape) != (m, 2 * n):
                raise RuntimeError("swiglu_bwd_x and out must be [M, 2N] with a contiguous last dimension")
            epi, aux_ptr, aux_ld = 4, swiglu_bwd_x.data_ptr(), swiglu_bwd_x.stride(0)
        aux_op = None
        if residual is not None:
            self._dev(residual)
            self._bf16(residual)
            aux_op = self._operand(residual)
            if aux_op is None or aux_op[0] != m or residual.shape[-1] != n:
                raise RuntimeError("GEMM residual must be [M, N] (or [s, r, N] in row runs) with a contiguous last dimension")
            epi, aux_ptr, aux_ld = 1, residual.data_ptr(), aux_op[1]
        if swiglu_out is not None:
            if residual is not None:
                raise RuntimeError("one fused epilogue at a time")
            self._dev(swiglu_out)
            self._bf16(swiglu_out)
            if tuple(swiglu_out.shape) != (m, n // 2) or swiglu_out.stride(1) != 1:
                raise RuntimeError("swiglu_out must be [M, N/2] with a contiguous last dimension")
            epi, out2_ptr, out2_ld = 2, swiglu_out.data_ptr(), swiglu_out.stride(0)
        ws_bytes, ws_ptr = 0, None
        fused = epi != 0
        if not fused and split_k is not None:   # split_k=None: never split (no workspace is handed over)
            key = (layout, m, n, k, split_k)
            ws_bytes = self._gemm_ws_bytes.get(key)
            if ws_bytes is None:
                ws_bytes = (self.lib.kr_gemm_workspace_bytes(layout, m, n, k) if split_k else
                            self.lib.kr_gemm_workspace_bytes_shared(layout, m, n, k, self.SHARED_LATENCY_WEIGHT))
                self._gemm_ws_bytes[key] = ws_bytes
            if ws_bytes:
                ws_ptr = self._workspace(ws_bytes, a.device).data_ptr()
        if max_cus == 0:
            reserved = reserved_compute_units()
            if reserved:
                max_cus = max(self._num_cus(a.device) - reserved, 8)
        if split_k is False:
            epi |= 0x100   # KR_GEMM_BESIDE_OTHER_STREAMS
        c_op = self._operand(out)
        if c_op is None or c_op[0] != m:
            raise RuntimeError("GEMM output must be [M, ...] with one row stride (or [s, r, ...] in row runs)")
        lda, ldc = a_op[1], c_op[1]
        if a_op[2] > 1 or c_op[2] > 1 or (aux_op is not None and aux_op[2] > 1):
            if c_op[2] > 1:
                ws_ptr, ws_bytes = None, 0      # an output in row runs is stored by the GEMM itself: no cuts
            rc = self.lib.kr_gemm_bf16_runs(layout, m, n, k, a.data_ptr(), lda, a_op[2], a_op[3], b.data_ptr(),
                                            b.stride(0), out.data_ptr(), ldc, c_op[2], c_op[3], int(accumulate),
                                            epi, aux_ptr, aux_ld, aux_op[2] if aux_op else 1, aux_op[3] if aux_op else 0,
                                            out2_ptr, out2_ld, int(max_cus), ws_ptr, ws_bytes, self._stream())
        elif epi == 0 and max_cus == 0:
            rc = self.lib.kr_gemm_bf16(layout, m, n, k, a.data_ptr(), lda, b.data_ptr(), b.stride(0),
                                       out.data_ptr(), ldc, int(accumulate), ws_ptr, ws_bytes,
                                       self._stream())
        else:
            rc = self.lib.kr_gemm_bf16_fused(layout, m, n, k, a.data_ptr(), lda, b.data_ptr(),
                                             b.stride(0), out.data_ptr(), ldc, int(accumulate),
                                             epi, aux_ptr, aux_ld, out2_ptr, out2_ld, int(max_cus),
                                             ws_ptr, ws_bytes, self._stream())
        self._check(rc, f"kr_gemm_bf16(layout={layout}, M={m}, N={n}, K={k}, epilogue={epi & 0xff})")
        return out

    def linear_fwd(self, x: Tensor, w: Tensor, split_k: bool = True, out: Tensor = None,
                   residual: Tensor = None, swiglu_out: Tensor = None, max_cus: int = 0) -> Tensor:
        return self.gemm(KR_GEMM_TN, x, w, self._nrows(x), w.shape[0], x.shape[-1], out=out, split_k=split_k,
                         residual=residual, swiglu_out=swiglu_out, max_cus=max_cus)

    @staticmethod
    def _nrows(t: Tensor) -> int:
        return t.shape[0] if t.dim() == 2 else t.shape[0] * t.shape[1]

    @staticmethod
    def can_fuse_swiglu(two_f: int) -> bool:
        """Whether a projection of this output width can produce the SwiGLU activation in its epilogue."""
        return two_f % 2 == 0 and any(two_f % (32 * wn) == 0 for wn in (5, 6, 7, 8))

    def linear_dgrad(self, dy: Tensor, w: Tensor, split_k: bool = True, swiglu_bwd_x: Tensor = None) -> Tensor:
        """``dy . W``; with ``swiglu_bwd_x`` (the input of the SwiGLU activation that fed this layer) the
        result is the gradient of that input, [rows, 2 * in_features], computed in the GEMM's epilogue."""
        return self.gemm(KR_GEMM_NN, dy, w, self._nrows(dy), w.shape[1], dy.shape[-1], split_k=split_k,
                         swiglu_bwd_x=swiglu_bwd_x)

    can_fuse_swiglu_bwd = True

    def linear_wgrad(self, dy: Tensor, x: Tensor, out: Tensor = None, accumulate: bool = False,
                     split_k: bool = True) -> Tensor:
        return self.gemm(KR_GEMM_NT, dy, x, dy.shape[-1], x.shape[1], self._nrows(dy), out=out,
                         accumulate=accumulate, split_k=split_k)

    MAX_WGRAD_SEGMENTS = 8   # KR_GEMM_MAX_SEGMENTS

    def wgrad_segments_ok(self, dys, xs) -> bool:
        """Whether ``linear_wgrad_segments`` takes these operand pairs: matrices of one shape and one row
        stride in every pair (the ``dys`` may be nanobatch slices in row runs, all alike), a multiple of 64 rows
        each, at most MAX_WGRAD_SEGMENTS pairs."""
        if not 1 <= len(dys) == len(xs) <= self.MAX_WGRAD_SEGMENTS:
            return False
        first = None
        for dy, x in zip(dys, xs):
            a, b = self._operand(dy), self._operand(x)
            if a is None or b is None or b[2] > 1 or a[0] != b[0] or a[0] % 64:
                return False
            if dy.dtype != torch.bfloat16 or x.dtype != torch.bfloat16 or not dy.is_cuda or x.device != dy.device:
                return False
            key = (a[0], a[1], a[2], a[3], b[1], dy.shape[-1], x.shape[-1])
            if first is None:
                first = key
            elif key != first:
                return False
        return True

    def linear_wgrad_segments(self, dys, xs, out: Tensor = None, accumulate: bool = False,
                              split_k: bool = True) -> Tensor:
        """``sum_i dys[i]^T . xs[i]`` in one launch: the weight gradient over all nanobatches of a
        microbatch, each pair read where it lies (``wgrad_segments_ok`` says whether the pairs qualify)."""
        if not self.wgrad_segments_ok(dys, xs):
            raise RuntimeError("linear_wgrad_segments: operand pairs must be matrices of one shape and row stride "
                               "with a multiple of 64 rows each")
        nseg = len(dys)
        a0, b0 = self._operand(dys[0]), self._operand(xs[0])
        k_seg, m, n = a0[0], dys[0].shape[-1], xs[0].shape[-1]
        if out is None:
            out = torch.empty((m, n), dtype=torch.bfloat16, device=dys[0].device)
        c_op = self._operand(out)
        if c_op is None or c_op[2] > 1 or tuple(out.shape) != (m, n):
            raise RuntimeError("linear_wgrad_segments: out must be a [M, N] matrix with one row stride")
        ws_bytes, ws_ptr = 0, None
        if split_k is not None:
            key = (KR_GEMM_NT, m, n, k_seg * nseg, split_k)
            ws_bytes = self._gemm_ws_bytes.get(key)
            if ws_bytes is None:
                ws_bytes = (self.lib.kr_gemm_workspace_bytes(KR_GEMM_NT, m, n, k_seg * nseg) if split_k else
                            self.lib.kr_gemm_workspace_bytes_shared(KR_GEMM_NT, m, n, k_seg * nseg, self.SHARED_LATENCY_WEIGHT))
                self._gemm_ws_bytes[key] = ws_bytes
            if ws_bytes:
                ws_ptr = self._workspace(ws_bytes, out.device).data_ptr()
        max_cus = 0
        reserved = reserved_compute_units()
        if reserved:
            max_cus = max(self._num_cus(out.device) - reserved, 8)
        ptrs = ctypes.c_void_p * nseg
        a_ptrs = ptrs(*[t.data_ptr() for t in dys])
        b_ptrs = ptrs(*[t.data_ptr() for t in xs])
        rc = self.lib.kr_gemm_bf16_nt_segments(m, n, k_seg, nseg, a_ptrs, a0[1], a0[2], a0[3], b_ptrs, b0[1], out.data_ptr(), c_op[1],
                                               int(accumulate), 0x100 if split_k is False else 0, int(max_cus),
                                               ws_ptr, ws_bytes, self._stream())
        self._check(rc, f"kr_gemm_bf16_nt_segments(M={m}, N={n}, k_seg={k_seg}, nseg={nseg})")
        return out

    # -- RMSNorm ----------------------------------------------------------------------
    @staticmethod
    def _rows(t: Tensor) -> Tensor:
        """A [rows, cols] matrix the kernels can address with one row stride: unit column
        stride, row stride a multiple of 8 elements; anything else is copied."""
        if t.dim() == 2 and t.stride(1) == 1 and t.stride(0) % 8 == 0 and t.stride(0) >= t.shape[1]:
            return t
        return t.contiguous()

    def rmsnorm_fwd(self, x: Tensor, gamma: Tensor, eps: float) -> Tuple[Tensor, Tensor]:
        """``x``: [rows, cols], or a [s, r, cols] nanobatch slice whose rows come in runs (read in place).
        Returns the dense [rows, cols] result and rstd [rows]."""
        self._dev(x, gamma)
        self._bf16(x, gamma)
        op = self._operand(x)
        if op is None:
            x = x.reshape(-1, x.shape[-1]).contiguous()
            op = self._operand(x)
        rows, ld, run_rows, run_ld = op
        cols = x.shape[-1]
        y = torch.empty((rows, cols), dtype=x.dtype, device=x.device)
        rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
        if run_rows > 1:
            rc = self.lib.kr_rmsnorm_fwd_runs(x.data_ptr(), gamma.data_ptr(), y.data_ptr(), rstd.data_ptr(),
                                              rows, cols, ld, run_rows, run_ld, eps, self._stream())
        else:
            rc = self.lib.kr_rmsnorm_fwd(x.data_ptr(), gamma.data_ptr(), y.data_ptr(), rstd.data_ptr(),
                                         rows, cols, ld, eps, self._stream())
        self._check(rc, "kr_rmsnorm_fwd")
        return y, rstd

    def rmsnorm_partial_rows(self, rows: int, cols: int) -> int:
        """fp32 partial rows of the weight gradient one backward call over [rows, cols] leaves."""
        return self.lib.kr_rmsnorm_bwd_partial_rows(rows, cols)

    def rmsnorm_dgamma(self, partials: Tensor, gamma: Tensor) -> Tensor:
        """Sum of the partial rows ([n, cols] fp32) of all nanobatches -> the weight gradient."""
        dgamma = torch.empty_like(gamma)
        self._check(self.lib.kr_rmsnorm_dgamma(partials.data_ptr(), partials.shape[0], partials.shape[1],
                                               dgamma.data_ptr(), self._stream()), "kr_rmsnorm_dgamma")
        return dgamma

    def rmsnorm_bwd(self, dy: Tensor, x: Tensor, rstd: Tensor, gamma: Tensor,
                    residual_grad: Tensor = None, out: Tensor = None,
                    partials_out: Tensor = None) -> Tuple[Tensor, Tensor]:
        """``residual_grad`` (same shape as ``x``): the gradient of the residual branch forked off
        in front of the norm is added to the norm's input gradient in the same pass.  ``out``: the
        [rows, cols] tensor (possibly a row-strided slice) the input gradient is written into.
        ``partials_out`` ([rmsnorm_partial_rows, cols] fp32, contiguous): the weight gradient is
        left there as partial rows for ``rmsnorm_dgamma`` and None is returned in its place."""
        self._dev(dy, x, rstd, gamma)
        self._bf16(dy, x, gamma)
        dy = self._rows(dy)
        x_op = self._operand(x)
        if x_op is None:
            x = x.reshape(-1, x.shape[-1]).contiguous()
            x_op = self._operand(x)
        rows, cols = x_op[0], x.shape[-1]
        if tuple(dy.shape) != (rows, cols):
            raise RuntimeError("rmsnorm_bwd: dy must be [rows, cols] like x")
        if out is None:
            dx = torch.empty((rows, cols), dtype=x.dtype, device=x.device)
            dx_op = (rows, cols, 1, 0)
        else:
            self._dev(out)
            self._bf16(out)
            dx = out
            dx_op = self._operand(dx)
            if dx_op is None or dx_op[0] != rows or dx.shape[-1] != cols:
                raise RuntimeError("rmsnorm_bwd: out must be [rows, cols] with a single row stride, or in row runs")
        res_ptr, res_op = None, (rows, 0, 1, 0)
        if residual_grad is not None:
            self._dev(residual_grad)
            self._bf16(residual_grad)
            res_op = self._operand(residual_grad)
            if res_op is None:
                residual_grad = residual_grad.reshape(-1, cols).contiguous()
                res_op = self._operand(residual_grad)
            if res_op[0] != rows or residual_grad.shape[-1] != cols:
                raise RuntimeError("rmsnorm_bwd: residual_grad must have the shape of x")
            res_ptr = residual_grad.data_ptr()
        if partials_out is not None:
            if (partials_out.dtype != torch.float32 or not partials_out.is_contiguous()
                    or tuple(partials_out.shape) != (self.rmsnorm_partial_rows(rows, cols), cols)):
                raise RuntimeError("rmsnorm_bwd: partials_out must be fp32 [partial rows, cols]")
            dgamma, dg_ptr, ws = None, None, partials_out
        else:
            dgamma = torch.empty_like(gamma)
            dg_ptr = dgamma.data_ptr()
            ws = self._workspace(self.lib.kr_rmsnorm_bwd_workspace_bytes(rows, cols), x.device)
        if x_op[2] > 1 or res_op[2] > 1 or dx_op[2] > 1:
            rc = self.lib.kr_rmsnorm_bwd_add_runs(dy.data_ptr(), x.data_ptr(), rstd.data_ptr(), gamma.data_ptr(),
                                                  res_ptr, dx.data_ptr(), dg_ptr, ws.data_ptr(), rows, cols,
                                                  dy.stride(0), x_op[1], x_op[2], x_op[3], res_op[1], res_op[2],
                                                  res_op[3], dx_op[1], dx_op[2], dx_op[3], self._stream())
        else:
            rc = self.lib.kr_rmsnorm_bwd_add(dy.data_ptr(), x.data_ptr(), rstd.data_ptr(), gamma.data_ptr(),
                                             res_ptr, dx.data_ptr(), dg_ptr, ws.data_ptr(), rows, cols,
                                             dy.stride(0), x_op[1], res_op[1], dx_op[1], self._stream())
        self._check(rc, "kr_rmsnorm_bwd_add")
        return dx, dgamma

    # -- RoPE -------------------------------------------------------------------------
    def _freqs2d(self, freqs: Tensor, hd: int) -> Tensor:
        if freqs.dtype != torch.float32:
            raise RuntimeError("the rotary table must be fp32")
        if freqs.shape[-1] != hd:
            raise RuntimeError("partial rotary (rot_dim < head_dim) is not supported")
        f2d = freqs.reshape(freqs.shape[0], hd)
        return f2d if f2d.is_contiguous() else f2d.contiguous()

    def _rope(self, t: Tensor, freqs: Tensor, backward: bool, out: Tensor = None,
              group_size: int = 1, group_rotate: int = 1) -> Tensor:
        self._dev(t, freqs)
        self._bf16(t)
        s, b, heads, hd = t.shape
        if t.stride(3) != 1:
            raise RuntimeError("rotary input needs a contiguous head dimension")
        f2d = self._freqs2d(freqs, hd)
        if out is None:
            out = torch.empty((s, b, heads, hd), dtype=t.dtype, device=t.device)
        rc = self.lib.kr_rope(t.data_ptr(), out.data_ptr(), f2d.data_ptr(), s, b, heads, hd,
                              t.stride(0), t.stride(1), t.stride(2),
                              out.stride(0), out.stride(1), out.stride(2), int(backward),
                              group_size, group_rotate, self._stream())
        self._check(rc, "kr_rope")
        return out

    def rope_fwd(self, t: Tensor, freqs: Tensor) -> Tensor:
        if t.dim() == 5:
            t = t.flatten(2, 3)
        return self._rope(t, freqs, False)

    def rope_bwd(self, g: Tensor, freqs: Tensor) -> Tensor:
        if g.dim() == 5:
            g = g.flatten(2, 3)
        return self._rope(g, freqs, True)

    def rope_fused_inplace(self, fused: Tensor, per: int, freqs: Tensor, backward: bool) -> None:
        """Rotate the query and key heads of a fused QKV buffer [s, b, ng, per+2, hd] in place
        (one launch); the value heads are left untouched."""
        s, b, ng, slots, hd = fused.shape
        if slots != per + 2 or not fused.is_contiguous():
            raise RuntimeError("fused QKV buffer must be contiguous [s, b, ng, per+2, hd]")
        flat = fused.view(s, b, ng * slots, hd)
        self._rope(flat, freqs, backward, out=flat, group_size=slots, group_rotate=per + 1)

    # -- SwiGLU / add -------------------------------------------------------------------
    def swiglu_fwd(self, x: Tensor) -> Tensor:
        self._dev(x)
        self._bf16(x)
        rows, two_f = x.shape
        y = torch.empty((rows, two_f // 2), dtype=x.dtype, device=x.device)
        self._check(self.lib.kr_swiglu_fwd(x.data_ptr(), y.data_ptr(), rows, two_f // 2, self._stream()),
                    "kr_swiglu_fwd")
        return y

    def swiglu_bwd(self, dy: Tensor, x: Tensor) -> Tensor:
        self._dev(dy, x)
        self._bf16(dy, x)
        rows, two_f = x.shape
        dx = torch.empty_like(x)
        self._check(self.lib.kr_swiglu_bwd(dy.data_ptr(), x.data_ptr(), dx.data_ptr(), rows, two_f // 2,
                                           self._stream()), "kr_swiglu_bwd")
        return dx

    def add(self, a: Tensor, b: Tensor, out: Tensor = None) -> Tensor:
        """``a + b``; with ``out`` the sum is written there (a slice of a larger tensor is fine as
        long as one row stride addresses it) instead of into a new tensor."""
        self._dev(a, b)
        self._bf16(a, b)
        if a.shape != b.shape:
            raise RuntimeError(f"add: shapes differ, {tuple(a.shape)} vs {tuple(b.shape)}")
        if out is None and a.is_contiguous() and b.is_contiguous():
            out = torch.empty_like(a)
            self._check(self.lib.kr_add(a.data_ptr(), b.data_ptr(), out.data_ptr(), a.numel(), self._stream()),
                        "kr_add")
            return out
        # a strided nanobatch slice (some sequences of a [seq, batch, hidden] tensor) is a matrix
        # [seq, batch_slice * hidden] with a long row stride: add it in place, do not copy it first
        a2, b2 = self._rows(self._leading_rows(a)), self._rows(self._leading_rows(b))
        if out is None:
            out = torch.empty(a.shape, dtype=a.dtype, device=a.device)
        else:
            self._dev(out)
            self._bf16(out)
            if out.shape != a.shape:
                raise RuntimeError(f"add: out has shape {tuple(out.shape)}, operands {tuple(a.shape)}")
        try:
            o2 = out.view(a2.shape)
        except RuntimeError:
            o2 = None
        if o2 is None or o2.stride(1) != 1 or o2.stride(0) % 8 or o2.stride(0) < o2.shape[1]:
            raise RuntimeError("add: out cannot be addressed with a single row stride")
        rows, cols = a2.shape
        self._check(self.lib.kr_add_rows(a2.data_ptr(), a2.stride(0), b2.data_ptr(), b2.stride(0),
                                         o2.data_ptr(), o2.stride(0), rows, cols, self._stream()), "kr_add_rows")
        return out

    def dropout_add(self, x: Tensor, residual: Tensor, p: float, out: Tensor = None) -> Tuple[Tensor, Tensor]:
        """``residual + dropout(x, p)`` and the byte mask of kept elements (same shape, dense).  The
        mask is keyed by a seed drawn from PyTorch's CPU generator, so ``torch.manual_seed`` fixes it
        and a restored CPU generator state (activation recomputation) reproduces it."""
        self._dev(x, residual)
        self._bf16(x, residual)
        if x.shape != residual.shape:
            raise RuntimeError(f"dropout_add: shapes differ, {tuple(x.shape)} vs {tuple(residual.shape)}")
        if not 0.0 <= p < 1.0:
            raise RuntimeError(f"dropout_add: probability {p} is outside [0, 1)")
        x2, r2 = self._rows(self._leading_rows(x)), self._rows(self._leading_rows(residual))
        if out is None:
            out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        else:
            self._dev(out)
            self._bf16(out)
            if out.shape != x.shape:
                raise RuntimeError(f"dropout_add: out has shape {tuple(out.shape)}, operands {tuple(x.shape)}")
        try:
            o2 = out.view(x2.shape)
        except RuntimeError:
            o2 = None
        if o2 is None or o2.stride(1) != 1 or o2.stride(0) % 8 or o2.stride(0) < o2.shape[1]:
            raise RuntimeError("dropout_add: out cannot be addressed with a single row stride")
        rows, cols = x2.shape
        mask = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
        seed = int(torch.randint(0, 1 << 62, (1,), dtype=torch.int64).item())
        self._check(self.lib.kr_dropout_add(x2.data_ptr(), x2.stride(0), r2.data_ptr(), r2.stride(0), o2.data_ptr(),
                                            o2.stride(0), mask.data_ptr(), rows, cols, float(p), seed, 0,
                                            self._stream()), "kr_dropout_add")
        return out, mask

    def dropout_bwd(self, dy: Tensor, mask: Tensor, scale: float) -> Tensor:
        """``dy * mask * scale``: native_dropout_backward."""
        self._dev(dy)
        self._bf16(dy)
        if (not mask.is_cuda or mask.dtype != torch.uint8 or mask.shape != dy.shape
                or not mask.is_contiguous()):
            raise RuntimeError("dropout_bwd: the mask must be the dense byte mask the forward wrote")
        d2 = self._rows(self._leading_rows(dy))
        dx = torch.empty(dy.shape, dtype=dy.dtype, device=dy.device)
        rows, cols = d2.shape
        self._check(self.lib.kr_dropout_bwd(d2.data_ptr(), d2.stride(0), mask.data_ptr(), dx.data_ptr(), cols, rows, cols,
                                            float(scale), self._stream()), "kr_dropout_bwd")
        return dx

    # -- query / key layernorm of the QKV split ----------------------------------------------
    def _fused5(self, name: str, t: Tensor) -> Tuple[int, int, int, int]:
        self._dev(t)
        self._bf16(t)
        if t.dim() != 5 or not t.is_contiguous() or t.shape[3] < 3:
            raise RuntimeError(f"{name}: needs a dense fused buffer [s, b, groups, per + 2, hd], got "
                               f"{tuple(t.shape)} with strides {t.stride()}")
        s, b, ng, slots, hd = t.shape
        return s * b, ng, slots - 2, hd

    def _qk_gammas(self, name: str, hd: int, gamma_q: Tensor, gamma_k: Tensor) -> None:
        self._dev(gamma_q, gamma_k)
        self._bf16(gamma_q, gamma_k)
        for g in (gamma_q, gamma_k):
            if g.shape != (hd,) or not g.is_contiguous():
                raise RuntimeError(f"{name}: a weight vector has shape {tuple(g.shape)}, the head dimension is {hd}")

    def qk_norm_fwd(self, mixed5: Tensor, gamma_q: Tensor, gamma_k: Tensor, eps: float) -> Tuple[Tensor, Tensor]:
        """RMSNorm over the head dimension of the query and key heads of a fused QKV buffer
        ``[s, b, groups, per + 2, hd]``; the value heads are copied.  Returns the new fused buffer and
        ``rstd [s, b, groups, per + 1]`` (qkv_postprocess.py:115-118)."""
        tokens, ng, per, hd = self._fused5("qk_norm_fwd", mixed5)
        self._qk_gammas("qk_norm_fwd", hd, gamma_q, gamma_k)
        out = torch.empty_like(mixed5)
        rstd = torch.empty(mixed5.shape[:3] + (per + 1,), dtype=torch.float32, device=mixed5.device)
        self._check(self.lib.kr_qk_norm_fwd(mixed5.data_ptr(), gamma_q.data_ptr(), gamma_k.data_ptr(), out.data_ptr(),
                                            rstd.data_ptr(), tokens, ng, per, hd, float(eps), self._stream()),
                    "kr_qk_norm_fwd")
        return out, rstd

    def qk_norm_bwd(self, dmixed5: Tensor, mixed5: Tensor, rstd: Tensor, gamma_q: Tensor,
                    gamma_k: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
        """The backward of :meth:`qk_norm_fwd`, in place on the query and key heads of ``dmixed5``
        (qkv_postprocess.py:150-157).  Returns ``(dmixed5, dgamma_q, dgamma_k)``."""
        tokens, ng, per, hd = self._fused5("qk_norm_bwd", dmixed5)
        if self._fused5("qk_norm_bwd", mixed5) != (tokens, ng, per, hd):
            raise RuntimeError(f"qk_norm_bwd: gradient {tuple(dmixed5.shape)} and input {tuple(mixed5.shape)} differ")
        self._qk_gammas("qk_norm_bwd", hd, gamma_q, gamma_k)
        self._dev(rstd)
        if rstd.dtype != torch.float32 or rstd.shape != mixed5.shape[:3] + (per + 1,) or not rstd.is_contiguous():
            raise RuntimeError("qk_norm_bwd: rstd is not the fp32 [s, b, groups, per + 1] tensor of the forward")
        dgq, dgk = torch.empty_like(gamma_q), torch.empty_like(gamma_k)
        nbytes = self.lib.kr_qk_norm_bwd_workspace_bytes(tokens, ng, per, hd)
        ws = self._workspace(max(nbytes, 16), mixed5.device)
        self._check(self.lib.kr_qk_norm_bwd(dmixed5.data_ptr(), mixed5.data_ptr(), rstd.data_ptr(), gamma_q.data_ptr(),
                                            gamma_k.data_ptr(), dgq.data_ptr(), dgk.data_ptr(), ws.data_ptr(),
                                            tokens, ng, per, hd, self._stream()), "kr_qk_norm_bwd")
        return dmixed5, dgq, dgk

    @staticmethod
    def _leading_rows(t: Tensor) -> Tensor:
        """``[d0, ...] -> [d0, rest]`` without a copy when the trailing dimensions are dense."""
        if t.dim() == 1:
            return t.view(1, -1)
        try:
            return t.view(t.shape[0], -1)
        except RuntimeError:
            return t.reshape(t.shape[0], -1)

    # -- embedding and loss ---------------------------------------------------------------
    def embedding_fwd(self, ids: Tensor, weight: Tensor, vocab_start: int = 0) -> Tensor:
        """ids [b, s] int64 -> [s, b, hidden]; ids outside this shard's rows give zeros."""
        self._dev(weight)
        self._on_device(ids)
        self._bf16(weight)
        if ids.dtype != torch.int64 or ids.dim() != 2:
            raise RuntimeError("token ids must be a [batch, seq] int64 tensor")
        ids = ids.contiguous()
        b, s = ids.shape
        out = torch.empty((s, b, weight.shape[1]), dtype=weight.dtype, device=weight.device)
        rc = self.lib.kr_embedding_fwd(ids.data_ptr(), weight.data_ptr(), out.data_ptr(), s, b,
                                       weight.shape[1], vocab_start, weight.shape[0], self._stream())
        self._check(rc, "kr_embedding_fwd")
        return out

    def embedding_bwd(self, ids: Tensor, dout: Tensor, vocab_rows: int, vocab_start: int = 0) -> Tensor:
        self._dev(dout)
        self._on_device(ids)
        self._bf16(dout)
        ids, dout = ids.contiguous(), dout.contiguous()
        b, s = ids.shape
        dw = torch.empty((vocab_rows, dout.shape[-1]), dtype=dout.dtype, device=dout.device)
        rc = self.lib.kr_embedding_bwd(ids.data_ptr(), dout.data_ptr(), dw.data_ptr(), s, b, dout.shape[-1],
                                       vocab_start, vocab_rows, self._stream())
        self._check(rc, "kr_embedding_bwd")
        return dw

    def cross_entropy_fwd(self, logits: Tensor, labels: Tensor) -> Tuple[Tensor, Tensor]:
        """logits [rows, vocab] bf16, labels [rows] int64 -> (loss [rows] fp32, lse [rows] fp32)."""
        self._dev(logits)
        self._on_device(labels)
        self._bf16(logits)
        logits, labels = self._rows(logits), labels.contiguous()
        rows, vocab = logits.shape
        loss = torch.empty(rows, dtype=torch.float32, device=logits.device)
        lse = torch.empty(rows, dtype=torch.float32, device=logits.device)
        rc = self.lib.kr_cross_entropy_fwd(logits.data_ptr(), labels.data_ptr(), loss.data_ptr(), lse.data_ptr(),
                                           rows, vocab, logits.stride(0), self._stream())
        self._check(rc, "kr_cross_entropy_fwd")
        return loss, lse

    def cross_entropy_bwd(self, logits: Tensor, labels: Tensor, lse: Tensor, dloss: Tensor,
                          in_place: bool = False) -> Tensor:
        self._dev(logits, lse, dloss)
        self._on_device(labels)
        self._bf16(logits)
        logits = self._rows(logits)
        rows, vocab = logits.shape
        out = logits if in_place else torch.empty((rows, vocab), dtype=logits.dtype, device=logits.device)
        dloss = dloss.to(torch.float32).contiguous()
        rc = self.lib.kr_cross_entropy_bwd(logits.data_ptr(), labels.contiguous().data_ptr(), lse.data_ptr(),
                                           dloss.data_ptr(), out.data_ptr(), rows, vocab, logits.stride(0),
                                           out.stride(0), self._stream())
        self._check(rc, "kr_cross_entropy_bwd")
        return out

    # -- attention ----------------------------------------------------------------------
    @staticmethod
    def _k_strides(t: Tensor):
        if t.stride(-1) != 1:
            raise RuntimeError("attention tensors need a contiguous head dimension")
        return t.stride(0), t.stride(1), t.stride(2)

    @staticmethod
    def _q_strides(t: Tensor, per: int):
        """(seq, batch, group, head-in-group) strides of a dense [s, b, nq, hd] or a grouped
        [s, b, ng, per, hd] query-like tensor."""
        if t.stride(-1) != 1:
            raise RuntimeError("attention tensors need a contiguous head dimension")
        if t.dim() == 5:
            return t.stride(0), t.stride(1), t.stride(2), t.stride(3)
        return t.stride(0), t.stride(1), per * t.stride(2), t.stride(2)

    @staticmethod
    def _q_dims(q: Tensor, k: Tensor):
        s, b = q.shape[0], q.shape[1]
        nkv, hd = k.shape[2], k.shape[3]
        nq = q.shape[2] * q.shape[3] if q.dim() == 5 else q.shape[2]
        if q.dim() == 5 and q.shape[2] != nkv:
            raise RuntimeError("grouped query tensor must have one group per KV head")
        return s, b, nq, nkv, hd

    def attn_fwd(self, q: Tensor, k: Tensor, v: Tensor, scale: float, causal: bool = True,
                 beside_other_streams: bool = False, general_kernels: bool = False):
        """``beside_other_streams``: kernels of other streams use the compute units this launch leaves idle,
        so it is shaped for the least compute-unit time, not for its own latency.
        ``general_kernels``: a shape outside the MFMA kernels (head dimension below 128, a ragged length)
        takes the general fp32 kernels instead of being padded into the MFMA ones."""
        if not causal:
            raise RuntimeError("only causal attention is implemented")
        self._dev(q, k, v)
        self._bf16(q, k, v)
        s, b, nq, nkv, hd = self._q_dims(q, k)
        per = nq // nkv
        o = torch.empty((s, b, nq, hd), dtype=q.dtype, device=q.device)
        lse = torch.empty((b, nq, s), dtype=torch.float32, device=q.device)
        flags = (KR_ATTN_BESIDE_OTHER_STREAMS if beside_other_streams else 0) | (KR_ATTN_GENERAL_KERNELS if general_kernels else 0)
        nbytes = 0 if general_kernels else self._attn_fwd_ws_bytes(s, b, nq, nkv, hd)
        ws_ptr = self._workspace(nbytes, q.device).data_ptr() if nbytes else None
        rc = self.lib.kr_attn_fwd_ws(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                                     s, b, nq, nkv, hd, scale, *self._q_strides(q, per), *self._k_strides(k),
                                     *self._k_strides(v), *self._q_strides(o, per), flags, ws_ptr, nbytes, self._stream())
        self._check(rc, f"kr_attn_fwd(s={s}, b={b}, nq={nq}, nkv={nkv}, hd={hd})")
        return o, lse

    def _attn_fwd_ws_bytes(self, s, b, nq, nkv, hd) -> int:
        if hd == 128 and s % 128 == 0:
            return 0
        key = (s, b, nq, nkv, hd)
        n = self._attn_ws_bytes.get(key)
        if n is None:
            n = self._attn_ws_bytes[key] = self.lib.kr_attn_fwd_workspace_bytes(s, b, nq, nkv, hd)
        return n

    def attn_bwd(self, do: Tensor, q: Tensor, k: Tensor, v: Tensor, o: Tensor, lse: Tensor,
                 scale: float, causal: bool = True, beside_other_streams: bool = False,
                 general_kernels: bool = False):
        """Returns (dq, dk, dv).  If ``q`` is a grouped [s, b, ng, per, hd] view, the three
        gradients are views of one buffer laid out like the fused QKV projection output and
        carry it as ``_kr_mixed`` so the QKV-split backward can hand it on without a copy."""
        if not causal:
            raise RuntimeError("only causal attention is implemented")
        self._dev(do, q, k, v, o, lse)
        self._bf16(do, q, k, v, o)
        s, b, nq, nkv, hd = self._q_dims(q, k)
        per = nq // nkv
        do4 = do.reshape(s, b, nq, hd)
        o4 = o.reshape(s, b, nq, hd)
        mixed = None
        if q.dim() == 5:
            fused = torch.empty((s, b, nkv, per + 2, hd), dtype=q.dtype, device=q.device)
            dq, dk, dv = fused[:, :, :, :per], fused[:, :, :, per], fused[:, :, :, per + 1]
            mixed = fused.view(s, b, nkv * (per + 2) * hd)
        else:
            dq = torch.empty((s, b, nq, hd), dtype=q.dtype, device=q.device)
            dk = torch.empty((s, b, nkv, hd), dtype=q.dtype, device=q.device)
            dv = torch.empty((s, b, nkv, hd), dtype=q.dtype, device=q.device)
        nbytes = self.lib.kr_attn_bwd_workspace_bytes(s, b, nq, nkv, hd)
        ws = self._workspace(max(nbytes, 16), q.device)
        flags = (KR_ATTN_BESIDE_OTHER_STREAMS if beside_other_streams else 0) | (KR_ATTN_GENERAL_KERNELS if general_kernels else 0)
        rc = self.lib.kr_attn_bwd_flags(do4.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), o4.data_ptr(),
                                        lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ws.data_ptr(),
                                        s, b, nq, nkv, hd, scale,
                                        *self._q_strides(q, per), *self._k_strides(k), *self._k_strides(v),
                                        *self._q_strides(o4, per), *self._q_strides(do4, per),
                                        *self._q_strides(dq, per), *self._k_strides(dk), *self._k_strides(dv),
                                        flags, self._stream())
        self._check(rc, f"kr_attn_bwd(s={s}, b={b}, nq={nq}, nkv={nkv}, hd={hd})")
        if mixed is not None:
            for t in (dq, dk, dv):
                t._kr_mixed = mixed
                t._kr_fused5 = fused
        return dq, dk, dv
