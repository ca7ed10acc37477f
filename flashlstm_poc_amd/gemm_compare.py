"""This library's MFMA GEMMs and the vendor GEMM library side by side, on the three products of a training pass.

    python -m flashlstm_poc_amd.gemm_compare [--rows 262144] [--hidden 1024] [--input 1024] [--reps 10] [--json FILE]

For T*B = rows, 4H gate columns and I inputs the pass multiplies
    projection   G  = X  * W_ih^T      (rows x 4H x I,    both operands K-contiguous:   flstm_gemm_nt)
    dX           dX = dG * W_ih        (rows x I  x 4H,   W_ih^T K-contiguous:          flstm_gemm_nt)
    dW           dW = dG^T * [X | H]   (4H x (I+H) x rows, operands k-major:            flstm_gemm_tn, one launch
                                        for both halves; the vendor library gets two matmuls of the same size)
Both sides see the same normally distributed fp16 operands (the part throttles under MFMA load by an amount that
depends on the data, so constant or zero operands flatter every GEMM), are called through their public entry
points (the C ABI of include/flashlstm/lstm_core.h here, torch.matmul -> hipBLASLt / rocBLAS there), are warmed up
and then timed back to back over `reps` calls with HIP events on the current stream.  Outputs are compared so
that a fast wrong answer cannot win."""
import argparse
import ctypes
import json

import torch


def _bind():
    from flashlstm_poc_amd import load_library
    L = load_library()
    sz, vp = ctypes.c_size_t, ctypes.c_void_p
    L.flstm_gemm_nt.argtypes = [vp, sz, vp, sz, sz, sz, sz, vp, ctypes.c_int, sz, ctypes.c_float, vp, vp]
    L.flstm_gemm_nt.restype = ctypes.c_int
    L.flstm_gemm_tn.argtypes = [vp, sz, vp, sz, sz, sz, sz, vp, sz, ctypes.c_float, ctypes.c_int, vp, vp]
    L.flstm_gemm_tn.restype = ctypes.c_int
    L.flstm_gemm_tn_workspace_bytes.argtypes = [sz, sz, sz, ctypes.c_int]
    L.flstm_gemm_tn_workspace_bytes.restype = sz
    L.flstm_gemm_tn_auto_splits.argtypes = [sz, sz, sz, ctypes.c_int]
    L.flstm_gemm_tn_auto_splits.restype = ctypes.c_int
    return L


def _time(fn, reps):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def _worst(got, ref):
    return float((got.float() - ref.float()).abs().max() / ref.float().abs().max().clamp_min(1e-30))


def compare(rows, hidden, inputs, reps):
    L = _bind()
    F32, F16 = 0, 1
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(1234)
    H4 = 4 * hidden
    x = torch.randn(rows, inputs, generator=g, device=dev).half()
    h = torch.randn(rows, hidden, generator=g, device=dev).half()
    w = (torch.randn(H4, inputs, generator=g, device=dev) * 0.03).half()
    w_t = w.t().contiguous()
    dg = torch.randn(rows, H4, generator=g, device=dev).half()
    stream = torch.cuda.current_stream().cuda_stream
    out = []

    def record(name, shape, flop, own, vendor, err):
        ms_own, ms_vendor = _time(own, reps), _time(vendor, reps)
        out.append({"product": name, "shape_m_n_k": shape, "tflop": flop / 1e12,
                    "own_ms": ms_own, "own_tflops": flop / ms_own / 1e9,
                    "vendor_ms": ms_vendor, "vendor_tflops": flop / ms_vendor / 1e9,
                    "own_over_vendor_time": ms_own / ms_vendor, "max_rel_diff": err()})

    # projection
    G_own = torch.empty(rows, H4, device=dev, dtype=torch.half)
    G_ven = torch.empty_like(G_own)

    def proj_own():
        rc = L.flstm_gemm_nt(x.data_ptr(), inputs, w.data_ptr(), inputs, rows, H4, inputs, G_own.data_ptr(), F16, H4,
                             1.0, None, stream)
        assert rc == 0, rc
    record("projection X*W_ih^T", [rows, H4, inputs], 2.0 * rows * H4 * inputs, proj_own,
           lambda: torch.matmul(x, w.t(), out=G_ven), lambda: _worst(G_own, G_ven))
    del G_own, G_ven

    # dX
    dx_own = torch.empty(rows, inputs, device=dev, dtype=torch.half)
    dx_ven = torch.empty_like(dx_own)

    def dx_own_fn():
        rc = L.flstm_gemm_nt(dg.data_ptr(), H4, w_t.data_ptr(), H4, rows, inputs, H4, dx_own.data_ptr(), F16, inputs,
                             1.0, None, stream)
        assert rc == 0, rc
    record("dX = dG*W_ih", [rows, inputs, H4], 2.0 * rows * H4 * inputs, dx_own_fn,
           lambda: torch.matmul(dg, w, out=dx_ven), lambda: _worst(dx_own, dx_ven))

    # dW_ih | dW_hh: [X | H] side by side as one k-major operand of pitch I + H for this library's single launch
    xh = torch.cat([x, h], dim=1).contiguous()
    N = inputs + hidden
    splits = L.flstm_gemm_tn_auto_splits(H4, N, rows, 64)
    ws = torch.empty(max(1, L.flstm_gemm_tn_workspace_bytes(H4, N, rows, splits)), device=dev, dtype=torch.uint8)
    dw_own = torch.empty(H4, N, device=dev, dtype=torch.float32)
    dwi_ven = torch.empty(H4, inputs, device=dev, dtype=torch.half)
    dwh_ven = torch.empty(H4, hidden, device=dev, dtype=torch.half)

    def dw_own_fn():
        rc = L.flstm_gemm_tn(dg.data_ptr(), H4, xh.data_ptr(), N, H4, N, rows, dw_own.data_ptr(), N, 1.0, splits,
                             ws.data_ptr(), stream)
        assert rc == 0, rc

    def dw_vendor():
        torch.matmul(dg.t(), x, out=dwi_ven)
        torch.matmul(dg.t(), h, out=dwh_ven)
    record("dW = dG^T*[X|H]", [H4, N, rows], 2.0 * rows * H4 * N, dw_own_fn, dw_vendor,
           lambda: max(_worst(dw_own[:, :inputs], dwi_ven), _worst(dw_own[:, inputs:], dwh_ven)))
    out[-1]["own_splits"] = splits
    return out


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--rows", type=int, default=262144, help="T*B")
    ap.add_argument("--hidden", type=int, default=1024)
    ap.add_argument("--input", type=int, default=1024)
    ap.add_argument("--reps", type=int, default=10)
    ap.add_argument("--json", default=None, help="also write the table to this file")
    a = ap.parse_args()
    rows = compare(a.rows, a.hidden, a.input, a.reps)
    print(f"{'product':24s} {'M x N x K':>24s} {'own ms':>8s} {'TFLOP/s':>8s} {'vendor ms':>10s} {'TFLOP/s':>8s} "
          f"{'own/vendor':>10s} {'max rel diff':>12s}")
    for r in rows:
        shape = " x ".join(str(v) for v in r["shape_m_n_k"])
        print(f"{r['product']:24s} {shape:>24s} {r['own_ms']:8.3f} {r['own_tflops']:8.0f} {r['vendor_ms']:10.3f} "
              f"{r['vendor_tflops']:8.0f} {r['own_over_vendor_time']:10.3f} {r['max_rel_diff']:12.2e}")
    tot_o, tot_v = sum(r["own_ms"] for r in rows), sum(r["vendor_ms"] for r in rows)
    print(f"{'sum':24s} {'':>24s} {tot_o:8.3f} {'':8s} {tot_v:10.3f} {'':8s} {tot_o / tot_v:10.3f}")
    print("torch", torch.__version__, "| device", torch.cuda.get_device_name(0))
    if a.json:
        with open(a.json, "w") as f:
            json.dump({"rows": rows, "torch": torch.__version__, "device": torch.cuda.get_device_name(0)}, f, indent=1)


if __name__ == "__main__":
    main()
