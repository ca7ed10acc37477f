"""The MFMA GEMMs on their own (flstm_gemm_nt / flstm_gemm_tn of include/flashlstm/lstm_core.h, the counterpart of
flstm::GemmTN / GemmNN / GemmNT, reference flashlstm_v2/src/gemm.h:8-51) against a plain fp64 matrix product of the
same fp16 operands, on shapes that are not multiples of the 256 x 256 x 64 tiles: ragged M and N, K tails, odd
output pitches (element-wise store path), sub-matrix outputs, bias, alpha, and split-K with uneven slices.
Tolerance: fp32 accumulation of fp16 products, |err| <= 1e-5 * sum_k |a_k b_k| + (half an fp16 ulp for fp16 outputs)."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

F32, F16 = 0, 1


def lib():
    from flashlstm_poc_amd import load_library
    L = load_library()
    sz, vp = ctypes.c_size_t, ctypes.c_void_p
    L.flstm_gemm_nt.argtypes = [vp, sz, vp, sz, sz, sz, sz, vp, ctypes.c_int, sz, ctypes.c_float, vp, vp]
    L.flstm_gemm_nt.restype = ctypes.c_int
    L.flstm_gemm_tn.argtypes = [vp, sz, vp, sz, sz, sz, sz, vp, sz, ctypes.c_float, ctypes.c_int, vp, vp]
    L.flstm_gemm_tn.restype = ctypes.c_int
    L.flstm_gemm_tn_workspace_bytes.argtypes = [sz, sz, sz, ctypes.c_int]
    L.flstm_gemm_tn_workspace_bytes.restype = sz
    return L


def rand16(g, *shape):
    return torch.randn(*shape, generator=g, device="cuda").half()


def check(got, a64, b64_t, alpha, bias, fp16_out):
    """got ~ alpha * a64 @ b64_t (+ bias) with the error bound of fp32 accumulation."""
    ref = alpha * (a64 @ b64_t)
    mag = abs(alpha) * (a64.abs() @ b64_t.abs())
    if bias is not None:
        ref = ref + bias.double()
        mag = mag + bias.double().abs()
    tol = 1e-5 * mag + 1e-30
    if fp16_out:
        tol = tol + ref.abs() * 2.0 ** -11 + 2.0 ** -24
    bad = ((got.double() - ref).abs() > tol)
    assert not bad.any(), f"{int(bad.sum())} of {bad.numel()} elements off, worst {((got.double() - ref).abs() / tol).max().item():.2f}x the bound"


@pytest.mark.parametrize("M,N,K,ldc_extra,dtype,use_bias,alpha", [
    (256, 256, 64, 0, F16, False, 1.0),       # exactly one tile, one slab
    (1, 1, 64, 0, F32, False, 1.0),           # a single element
    (37, 53, 128, 0, F16, True, 1.0),         # ragged edge tile, N and ldc odd -> element-wise stores
    (300, 520, 192, 0, F16, True, 0.5),       # several tiles, ragged in both directions
    (513, 260, 64, 4, F32, False, -2.0),      # fp32 out with a padded pitch
    (260, 1028, 320, 3, F32, True, 1.0),      # odd pitch: no vector stores anywhere
    (1024, 512, 1024, 8, F16, True, 1.0),     # full tiles only, whole-line store path, padded pitch
    (2048 + 16, 768, 256, 0, F16, False, 1.0)])
def test_gemm_nt_against_fp64_product(M, N, K, ldc_extra, dtype, use_bias, alpha):
    L = lib()
    g = torch.Generator(device="cuda").manual_seed(M * 7 + N * 3 + K)
    lda, ldb, ldc = K + 8, K + 16, N + ldc_extra
    A = rand16(g, M, lda); Bm = rand16(g, N, ldb)
    bias = torch.randn(N, generator=g, device="cuda") if use_bias else None
    C = torch.full((M, ldc), 123.0, device="cuda", dtype=torch.float16 if dtype == F16 else torch.float32)
    rc = L.flstm_gemm_nt(A.data_ptr(), lda, Bm.data_ptr(), ldb, M, N, K, C.data_ptr(), dtype, ldc, alpha,
                         bias.data_ptr() if use_bias else None, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    check(C[:, :N], A[:, :K].double(), Bm[:, :K].double().T, alpha, bias, dtype == F16)
    if ldc_extra:
        assert (C[:, N:] == 123.0).all()      # nothing written beyond column N


def test_gemm_nt_into_a_sub_matrix_that_starts_at_an_odd_element():
    # output rows of a larger matrix starting at an odd column: unaligned for vector stores -> element path
    L = lib()
    g = torch.Generator(device="cuda").manual_seed(5)
    M, N, K = 70, 96, 64
    A = rand16(g, M, K); Bm = rand16(g, N, K)
    big = torch.zeros(M, 200, device="cuda", dtype=torch.float16)
    view = big[:, 3:3 + N]
    rc = L.flstm_gemm_nt(A.data_ptr(), K, Bm.data_ptr(), K, M, N, K, view.data_ptr(), F16, 200, 1.0, None,
                         torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    check(view, A.double(), Bm.double().T, 1.0, None, True)
    assert (big[:, :3] == 0).all() and (big[:, 3 + N:] == 0).all()


@pytest.mark.parametrize("M,N,K,splits,ldc_extra", [
    (256, 256, 64, 1, 0),
    (8, 8, 1, 1, 0),             # smallest legal problem, K far below one slab
    (264, 72, 100, 1, 4),        # ragged tiles, K tail inside the only slab
    (520, 264, 1000, 4, 0),      # split-K with a masked last slab (1000 = 15 slabs + 40)
    (1024, 256, 64 * 7 + 5, 3, 8),   # 8 slabs in 3 slices -> slices of 3, 3, 2 slabs; tail of 5 rows
    (512, 768, 4096, 16, 0),
    (128, 136, 64 * 3, 64, 0)])  # more slices asked for than slabs exist
def test_gemm_tn_against_fp64_product(M, N, K, splits, ldc_extra):
    L = lib()
    g = torch.Generator(device="cuda").manual_seed(M + N * 5 + K * 11 + splits)
    lda, ldb, ldc = M + 8, N + 24, N + ldc_extra
    A = rand16(g, K, lda); Bm = rand16(g, K, ldb)
    C = torch.full((M, ldc), -5.0, device="cuda")
    ws_bytes = L.flstm_gemm_tn_workspace_bytes(M, N, K, splits)
    ws = torch.empty(max(ws_bytes, 16) // 4, device="cuda")
    rc = L.flstm_gemm_tn(A.data_ptr(), lda, Bm.data_ptr(), ldb, M, N, K, C.data_ptr(), ldc, 0.25, splits,
                         ws.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    check(C[:, :N], A[:, :M].double().T, Bm[:, :N].double(), 0.25, None, False)
    if ldc_extra:
        assert (C[:, N:] == -5.0).all()


def test_gemm_argument_checks():
    L = lib()
    t = torch.zeros(64, 64, device="cuda", dtype=torch.float16)
    c = torch.zeros(64, 64, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    assert L.flstm_gemm_nt(t.data_ptr(), 64, t.data_ptr(), 64, 64, 64, 48, c.data_ptr(), F32, 64, 1.0, None, s) == 1   # K % 64
    assert L.flstm_gemm_nt(t.data_ptr(), 32, t.data_ptr(), 64, 64, 64, 64, c.data_ptr(), F32, 64, 1.0, None, s) == 1   # lda < K
    assert L.flstm_gemm_nt(None, 64, t.data_ptr(), 64, 64, 64, 64, c.data_ptr(), F32, 64, 1.0, None, s) == 1
    assert L.flstm_gemm_tn(t.data_ptr(), 64, t.data_ptr(), 64, 60, 64, 64, c.data_ptr(), 64, 1.0, 1, None, s) == 1     # M % 8
    assert L.flstm_gemm_tn(t.data_ptr(), 64, t.data_ptr(), 64, 64, 64, 64, c.data_ptr(), 64, 1.0, 4, None, s) in (0, 1)  # 1 slab -> no split
    assert L.flstm_gemm_tn(t.data_ptr(), 64, t.data_ptr(), 64, 64, 64, 256, c.data_ptr(), 64, 1.0, 4, None, s) == 1    # split without workspace
    torch.cuda.synchronize()


def test_the_comparison_tool_runs_both_libraries_on_the_same_operands_and_they_agree():
    """python -m flashlstm_poc_amd.gemm_compare at a small size: the three products through this library's C ABI and
    through torch.matmul (the vendor GEMM library), outputs within fp16 rounding of each other."""
    from flashlstm_poc_amd.gemm_compare import compare
    rows = compare(rows=4096, hidden=256, inputs=320, reps=1)
    assert [r["product"].split()[0] for r in rows] == ["projection", "dX", "dW"]
    for r in rows:
        assert r["own_ms"] > 0 and r["vendor_ms"] > 0
        assert r["max_rel_diff"] < 2e-3, r


def test_gemm_kernels_on_seeded_random_shapes():
    """Twenty-four seeded random shapes per kernel -- tile counts from one to a few dozen (several rounds of the
    persistent kernels' work lists, workgroups with and without work), K tails, split-K -- against the fp64 product."""
    L = lib()
    rng = np.random.default_rng(20240607)
    s = torch.cuda.current_stream().cuda_stream
    for case in range(24):
        g = torch.Generator(device="cuda").manual_seed(1000 + case)
        # NT: any M, N; K a multiple of 64
        M, N, K = int(rng.integers(1, 1500)), int(rng.integers(1, 1100)), 64 * int(rng.integers(1, 9))
        lda, ldb = K + 8 * int(rng.integers(0, 3)), K + 8 * int(rng.integers(0, 3))
        ldc = N + 4 * int(rng.integers(0, 3))
        A = rand16(g, M, lda); Bm = rand16(g, N, ldb)
        f16 = bool(rng.integers(0, 2))
        bias = torch.randn(N, generator=g, device="cuda") if rng.integers(0, 2) else None
        C = torch.full((M, ldc), 7.0, device="cuda", dtype=torch.float16 if f16 else torch.float32)
        rc = L.flstm_gemm_nt(A.data_ptr(), lda, Bm.data_ptr(), ldb, M, N, K, C.data_ptr(), F16 if f16 else F32, ldc, 1.0,
                             bias.data_ptr() if bias is not None else None, s)
        assert rc == 0, (case, M, N, K)
        torch.cuda.synchronize()
        check(C[:, :N], A[:, :K].double(), Bm[:, :K].double().T, 1.0, bias, f16)
        assert (C[:, N:] == 7.0).all()
        # TN: M, N multiples of 8; any K
        M, N, K = 8 * int(rng.integers(1, 160)), 8 * int(rng.integers(1, 130)), int(rng.integers(1, 1200))
        splits = int(rng.integers(1, 6))
        lda, ldb, ldc = M + 8 * int(rng.integers(0, 3)), N + 8 * int(rng.integers(0, 3)), N + 4 * int(rng.integers(0, 2))
        A = rand16(g, K, lda); Bm = rand16(g, K, ldb)
        C = torch.full((M, ldc), -3.0, device="cuda")
        ws = torch.empty(max(L.flstm_gemm_tn_workspace_bytes(M, N, K, splits), 16) // 4, device="cuda")
        rc = L.flstm_gemm_tn(A.data_ptr(), lda, Bm.data_ptr(), ldb, M, N, K, C.data_ptr(), ldc, 1.0, splits, ws.data_ptr(), s)
        assert rc == 0, (case, M, N, K, splits)
        torch.cuda.synchronize()
        check(C[:, :N], A[:, :M].double().T, Bm[:, :N].double(), 1.0, None, False)
        assert (C[:, N:] == -3.0).all()
