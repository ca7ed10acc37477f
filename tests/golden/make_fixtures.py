"""Writes tests/golden/lstm_golden.npz: seeded torch.nn.LSTM (CPU, float64) inputs, outputs and autograd
gradients on small shapes taken from the reference's own test lists.

The reference ships no golden vectors (its tests compare against torch.nn.LSTM at run time:
python/test_lstm.py:280-302, flashlstm_v2/scripts/validate_lstm_fwd.py:243-250,
flashlstm_v2/python/tests/test_streaming_lstm.py:17-20, playground/simple_lstm_bwd.py shape (5,3,4,6)),
so the vectors are generated from the same third-party oracle, torch.nn.LSTM, on those shapes.
Run:  python tests/golden/make_fixtures.py
"""
import os

import numpy as np
import torch

CASES = {  # name: (T, B, I, H, seed)
    "v2_pytest": (4, 2, 3, 5, 1234),
    "v1_quick": (7, 2, 32, 24, 1234),
    "playground_bwd": (5, 3, 4, 6, 0),
    "validate_small": (16, 8, 64, 32, 0),
}


def main():
    out = {}
    for name, (T, B, I, H, seed) in CASES.items():
        torch.manual_seed(seed)
        m = torch.nn.LSTM(I, H).double()
        x = torch.randn(T, B, I, dtype=torch.float64, requires_grad=True)
        h0 = torch.randn(1, B, H, dtype=torch.float64, requires_grad=True)
        c0 = torch.randn(1, B, H, dtype=torch.float64, requires_grad=True)
        dy = torch.randn(T, B, H, dtype=torch.float64)
        d_hn = torch.randn(1, B, H, dtype=torch.float64)
        d_cn = torch.randn(1, B, H, dtype=torch.float64)
        y, (hn, cn) = m(x, (h0, c0))
        ((y * dy).sum() + (hn * d_hn).sum() + (cn * d_cn).sum()).backward()
        t = dict(x=x, h0=h0[0], c0=c0[0], dy=dy, d_hn=d_hn[0], d_cn=d_cn[0], w_ih=m.weight_ih_l0,
                 w_hh=m.weight_hh_l0, b_ih=m.bias_ih_l0, b_hh=m.bias_hh_l0, y=y, hn=hn[0], cn=cn[0], dx=x.grad,
                 dh0=h0.grad[0], dc0=c0.grad[0], dw_ih=m.weight_ih_l0.grad, dw_hh=m.weight_hh_l0.grad,
                 db_ih=m.bias_ih_l0.grad, db_hh=m.bias_hh_l0.grad)
        for k, v in t.items():
            out[f"{name}/{k}"] = v.detach().numpy().astype(np.float64)
        out[f"{name}/shape"] = np.array([T, B, I, H], dtype=np.int64)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lstm_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
