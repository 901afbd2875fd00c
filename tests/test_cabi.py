"""The C-ABI library loads on a machine without a GPU and exports exactly what include/*.h declares."""

import ctypes
import glob
import os
import re

from kareus_amd.backend import hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    names = set()
    for header in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = re.sub(r"/\*.*?\*/", "", open(header).read(), flags=re.S)
        names.update(re.findall(r"\b(kr_[a-z0-9_]+)\s*\(", text))
    return names


def test_library_exports_every_declared_symbol():
    declared = _declared()
    assert {"kr_gemm_bf16", "kr_attn_fwd", "kr_attn_bwd", "kr_rmsnorm_fwd", "kr_rmsnorm_bwd", "kr_rope",
            "kr_swiglu_fwd", "kr_swiglu_bwd", "kr_add", "kr_version", "kr_error_string"} <= declared
    lib = ctypes.CDLL(hip.library_path())
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/ but not exported"
    # and the Python binding table covers the same set
    assert set(hip._SIGNATURES) == declared


def test_argument_checks_run_without_a_device():
    lib = hip.load_library()
    assert lib.kr_version() >= 100
    assert lib.kr_error_string(0) == b"ok" and b"unknown" in lib.kr_error_string(-99)
    assert lib.kr_device_clock_mhz() >= 0                         # 0 where no device can be asked
    # invalid arguments are rejected before anything touches the GPU
    assert lib.kr_add(None, None, None, 8, None) == -1
    assert lib.kr_swiglu_fwd(16, 16, 4, 12, None) == -2          # F not a multiple of 8
    assert lib.kr_rmsnorm_fwd(16, 16, 16, 16, 4, 8200, 8200, 1e-5, None) == -2    # wider than 8192
    assert lib.kr_rmsnorm_fwd(16, 16, 16, 16, 4, 64, 32, 1e-5, None) == -1        # row stride < width
    assert lib.kr_rmsnorm_bwd(16, 16, 16, 16, 16, 16, 16, 4, 64, 64, 68, None) == -2  # stride not x8
    assert lib.kr_add_rows(16, 64, 16, 64, 16, 32, 4, 64, None) == -1             # output stride < width
    assert lib.kr_add_rows(16, 64, 16, 64, 16, 64, 4, 60, None) == -2             # width not x8
    assert lib.kr_dropout_add(16, 64, 16, 64, 16, 64, 8, 4, 64, 1.0, 1, 0, None) == -1   # p outside [0, 1)
    assert lib.kr_dropout_add(16, 64, 16, 64, 16, 64, 12, 4, 64, 0.1, 1, 0, None) == -1  # mask not 8-byte aligned
    assert lib.kr_dropout_add(16, 64, 16, 64, 16, 64, 8, 4, 60, 0.1, 1, 0, None) == -2   # width not x8
    assert lib.kr_dropout_bwd(16, 32, 8, 16, 64, 4, 64, 1.25, None) == -1                # gradient stride < width
    assert lib.kr_qk_norm_fwd(16, 32, 48, 64, 80, 4, 2, 4, 96, 1e-5, None) == -2         # head dimension not 64/128/256
    assert lib.kr_qk_norm_fwd(16, 32, 40, 64, 80, 4, 2, 4, 128, 1e-5, None) == -1        # misaligned weight
    assert lib.kr_qk_norm_fwd(16, 32, 48, 64, 80, 4, 2, 0, 128, 1e-5, None) == -1        # no query head in a group
    assert lib.kr_qk_norm_fwd(16, 32, 48, 16, 64, 4, 2, 4, 128, 1e-5, None) == -1        # output on top of the input
    assert lib.kr_qk_norm_bwd(16, 16, 16, 16, 16, 16, 16, None, 4, 2, 4, 128, None) == -1  # no workspace
    assert lib.kr_qk_norm_bwd_workspace_bytes(4, 2, 4, 96) == 0
    # 8192 tokens x 2 groups x 6 heads of 128 channels: 16 rows per workgroup, capped at 1024 workgroups, each
    # leaving 2 x 128 fp32 partial sums
    assert lib.kr_qk_norm_bwd_workspace_bytes(8192, 2, 4, 128) == 1024 * 2 * 128 * 4
    assert lib.kr_qk_norm_bwd_workspace_bytes(16, 1, 2, 64) == 2 * 2 * 64 * 4              # 64 rows, 32 a workgroup
    assert lib.kr_gemm_workspace_bytes_shared(2, 1536, 4096, 4096, 0.3) <= lib.kr_gemm_workspace_bytes(2, 1536, 4096, 4096)
    assert lib.kr_gemm_bf16(0, 8, 8, 7, 16, 8, 16, 8, 16, 8, 0, None, 0, None) == -2
    assert lib.kr_gemm_bf16(9, 8, 8, 8, 16, 8, 16, 8, 16, 8, 0, None, 0, None) == -1
    assert lib.kr_gemm_bf16(0, 8, 8, 8, 16, 8, 16, 8, 18, 8, 0, None, 0, None) == -1   # misaligned C
    assert lib.kr_attn_bwd_workspace_bytes(256, 1, 4, 2, 136) == 0  # head dimensions above 128 are unsupported
    # a shape padded into the MFMA kernels (256 rows, 128 channels): four query-sized and four key-sized bf16
    # copies, the padded log-sum-exp, and the MFMA backward's own workspace at the padded shape
    padded = 4 * 256 * 4 * 128 * 2 + 4 * 256 * 2 * 128 * 2 + 256 * 4 * 4
    assert lib.kr_attn_bwd_workspace_bytes(250, 1, 4, 2, 64) == padded + lib.kr_attn_bwd_workspace_bytes(256, 1, 4, 2, 128)
    assert lib.kr_attn_fwd_workspace_bytes(250, 1, 4, 2, 64) == 2 * 256 * 4 * 128 * 2 + 2 * 256 * 2 * 128 * 2 + 256 * 4 * 4
    assert lib.kr_attn_fwd_workspace_bytes(256, 1, 4, 2, 128) == 0 and lib.kr_attn_fwd_workspace_bytes(256, 1, 4, 2, 136) == 0
    assert lib.kr_attn_fwd_ws(16, 16, 16, 16, 16, 250, 1, 4, 2, 64, 0.125, *([64] * 14), 0x400, None, 0, None) == -1   # unknown flag
    assert lib.kr_attn_fwd_ws(16, 16, 16, 16, 16, 250, 1, 4, 2, 64, 0.125, *([64] * 14), 0, 24, 1 << 30, None) == -1   # misaligned workspace
    assert lib.kr_attn_fwd_ws(16, 16, 16, 16, 16, 250, 1, 4, 2, 64, 0.125, *([64] * 14), 0, 32, 1024, None) == -1      # workspace too small
    # delta and the rescaled lse, plus fp32 dK/dV partials per query head when heads share KV heads ...
    assert lib.kr_attn_bwd_workspace_bytes(4096, 4, 32, 32, 128) == 2 * 4 * 32 * 4096 * 4
    assert lib.kr_attn_bwd_workspace_bytes(4096, 4, 32, 8, 128) == 2 * 4 * 32 * 4096 * 4 + 2 * 4 * 32 * 4096 * 128 * 4
    # ... and per (query head, half of the query tiles) when the launch has few workgroups
    assert lib.kr_attn_bwd_workspace_bytes(256, 1, 4, 4, 128) == 2 * 256 * 4 * 4 + 2 * 256 * 4 * 2 * 128 * 4
    assert lib.kr_attn_bwd_workspace_bytes(256, 1, 4, 2, 128) == 2 * 256 * 4 * 4 + 2 * 256 * 4 * 2 * 128 * 4
    assert lib.kr_gemm_workspace_bytes(2, 1536, 4096, 16384) > 0 and lib.kr_gemm_workspace_bytes(0, 4096, 7168, 4096) == 0
    assert lib.kr_rmsnorm_bwd_workspace_bytes(8192, 4096) == 512 * 4096 * 4


def test_strides_the_kernels_cannot_index_are_refused():
    """Attention keeps sequence strides in 32 bits (per-lane byte offsets up to (48 * stride + 128) * 2) and no
    kernel walks backwards: a stride that is not positive or too long is an error, not a wild load."""
    lib = hip.load_library()
    good = [1024, 256, 128, 128] + [1024, 256, 128] * 2 + [1024, 256, 128, 128]
    args = lambda st: [16, 16, 16, 16, 16, 128, 1, 1, 1, 128, 1.0] + st + [None]
    too_long = (1 << 31) // 48 // 8 * 8
    for pos in (0, 4, 7, 10):                                  # the four sequence strides
        bad = list(good)
        bad[pos] = too_long
        assert lib.kr_attn_fwd(*args(bad)) == -2
        bad[pos] = -1024
        assert lib.kr_attn_fwd(*args(bad)) == -2
    bad = list(good)
    bad[1] = 0                                                 # a batch stride of zero
    assert lib.kr_attn_fwd(*args(bad)) == -2
    bwd_good = good + [1024, 256, 128, 128] * 2 + [1024, 256, 128] * 2
    bwd = lambda st: [16] * 10 + [128, 1, 1, 1, 128, 1.0] + st + [None]
    for pos in (0, 14, 18, 22, 25):
        bad = list(bwd_good)
        bad[pos] = too_long
        assert lib.kr_attn_bwd(*bwd(bad)) == -2
        bad[pos] = -8
        assert lib.kr_attn_bwd(*bwd(bad)) == -2
    rope = lambda st: [16, 16, 16, 4, 1, 2, 128] + st + [0, 1, 1, None]
    assert lib.kr_rope(*rope([-256, 256, 128, 256, 256, 128])) == -2
    assert lib.kr_rope(*rope([256, 256, 128, 256, 0, 128])) == -2


def test_fused_gemm_argument_checks():
    lib = hip.load_library()
    base = [0, 256, 256, 64, 16, 64, 16, 64, 16, 256, 0]
    call = lambda epi, aux, ld_aux, out2, ld_out2, cus=0, acc=0, layout=0, n=256: lib.kr_gemm_bf16_fused(
        layout, 256, n, 64, 16, 64, 16, 64, 16, n, acc, epi, aux, ld_aux, out2, ld_out2, cus, None, 0, None)
    assert call(1, None, 256, None, 0) == -1                 # residual epilogue without a residual
    assert call(1, 16, 128, None, 0) == -1                   # residual row stride below N
    assert call(1, 16, 256, None, 0, acc=1) == -1            # a fused epilogue cannot accumulate into C
    assert call(2, None, 0, None, 0) == -1                   # SwiGLU without its second output
    assert call(2, None, 0, 16, 128, layout=1) == -2         # fused epilogues are built for the forward layout
    assert call(1, 16, 256, None, 0, layout=2) == -2
    assert call(2, None, 0, 16, 136, n=272) == -2            # no tile width divides 2F = 272
    assert call(7, None, 0, None, 0) == -1                   # unknown epilogue
    assert call(4, 16, 512, None, 0, layout=0) == -2         # the SwiGLU backward epilogue belongs to the NN layout
    assert call(4, None, 512, None, 0, layout=1) == -1       # ... and needs the activation's input
    assert call(4, 16, 256, None, 0, layout=1) == -1         # ... of twice the product's width
    assert lib.kr_gemm_bf16_fused(1, 256, 256, 64, 16, 64, 16, 256, 16, 256, 0, 4, 16, 512, None, 0, 0, None, 0,
                                  None) == -1                # ... and an output of that width
    assert call(0, None, 0, None, 0, cus=-3) == -1


def test_swiglu_epilogue_index_model():
    """A CPU model of the store addresses of the GEMM's SwiGLU epilogue and of its gate / up interleave of
    the weight rows (kr_gemm.hip), for every tile width: every element of x [M, 2F] and of the activation
    [M, F] is written exactly once, no address leaves the tensors, and no offset that the kernel keeps in an
    unsigned register is negative (the mistake that once sent a store 8 GB past the output)."""
    import numpy as np

    def check(M, F, WN):
        N = 2 * F
        assert N % (32 * WN) == 0
        x_hits, y_hits = np.zeros((M, N), int), np.zeros((M, F), int)
        for tm in range((M + 255) // 256):
            for tn in range(N // (32 * WN)):
                out_m0, out_n0 = tm * 256, tn * 16 * WN
                for wave in range(4):
                    wm, wn = wave >> 1, wave & 1
                    m_wave = out_m0 + wm * 128
                    rows_in = m_wave + 128 <= M
                    n_store = out_n0 + (F if wn else 0)
                    for lane in range(64):
                        quad, rch = lane >> 4, lane & 15
                        if 8 * rch >= 16 * WN:
                            continue
                        for mt in range(8):
                            for q in range(4):                      # x: rows 4 q + quad of the block
                                rr = 4 * q + quad
                                row = m_wave + mt * 16 + rr
                                if rows_in or row < M:
                                    nlo = rr * N + 8 * rch          # kept unsigned in the kernel
                                    assert nlo >= 0
                                    r, c = divmod((m_wave + mt * 16) * N + n_store + nlo, N)
                                    assert 0 <= r < M and c + 8 <= N
                                    x_hits[r, c:c + 8] += 1
                            for qq in range(2):                     # activation: this wave's half of the rows
                                rr = 4 * (2 * wn + qq) + quad
                                row = m_wave + mt * 16 + rr
                                if rows_in or row < M:
                                    c = out_n0 + 8 * rch
                                    assert c + 8 <= F
                                    y_hits[row, c:c + 8] += 1
                for row in range(32 * WN):                          # B tile row -> weight row
                    r = out_n0 + row if row < 16 * WN else out_n0 + (row - 16 * WN) + F
                    assert 0 <= r < N and (row < 16 * WN) == (r < F)
        assert (x_hits == 1).all() and (y_hits == 1).all()

    for M, F, WN in [(512, 128, 8), (264, 384, 8), (264, 384, 6), (1000, 1024, 8), (520, 320, 5), (304, 672, 7),
                     (304, 672, 6)]:
        check(M, F, WN)
