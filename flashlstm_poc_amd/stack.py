"""Stacked LSTM on top of the single-layer core: layer l's outputs are layer l+1's inputs, and in the backward
pass layer l+1's input gradient is layer l's upstream gradient.  The reference is single-layer only
(flashlstm_v2/python/flashlstm/streaming_lstm.py:380-430); this is the thin layer loop a multi-layer workload
needs, with everything resident on the GPU in fp16 between layers."""
from typing import List, Optional, Sequence, Tuple

from .core import LstmCore


class LstmStack:
    """num_layers LSTM layers of equal hidden size; layer 0 takes `input_size` features."""

    def __init__(self, batch: int, input_size: int, hidden_size: int, num_layers: int):
        if num_layers < 1:
            raise ValueError("num_layers must be >= 1")
        self.B, self.I, self.H, self.L = int(batch), int(input_size), int(hidden_size), int(num_layers)
        self.layers: List[LstmCore] = [LstmCore(self.B, self.I if l == 0 else self.H, self.H) for l in range(self.L)]
        self._inputs: List = []
        self.last_loss_scale = 1.0

    def close(self) -> None:
        for layer in self.layers:
            layer.close()
        self._inputs = []

    def pack(self, params: Sequence[Tuple]) -> None:
        """params[l] = (w_ih, w_hh, b_ih, b_hh) of layer l (fp32 CUDA tensors, torch.nn.LSTM layout)."""
        if len(params) != self.L:
            raise ValueError(f"expected parameters for {self.L} layers")
        for layer, (w_ih, w_hh, b_ih, b_hh) in zip(self.layers, params):
            layer.pack(w_ih, w_hh, b_ih, b_hh)

    def forward(self, x, h0: Optional[Sequence] = None, c0: Optional[Sequence] = None):
        """x (T,B,I) fp16 on the GPU -> (y of the top layer (T,B,H) fp16, [hy per layer], [cy per layer])."""
        import torch
        if x.dtype != torch.float16:
            raise ValueError("x must be fp16 (activations travel between layers in fp16)")
        self._inputs = []
        hys, cys = [], []
        cur = x
        for l, layer in enumerate(self.layers):
            self._inputs.append(cur)
            cur, hy, cy = layer.forward(cur, None if h0 is None else h0[l], None if c0 is None else c0[l])
            hys.append(hy)
            cys.append(cy)
        return cur, hys, cys

    def backward(self, dy_top, *, loss_scale="auto", d_hn: Optional[Sequence] = None,
                 d_cn: Optional[Sequence] = None, want_dx: bool = True):
        """dy_top (T,B,H): gradient wrt the top layer's outputs.  loss_scale (a power of two) multiplies it before
        it is rounded to fp16 and stays on every inter-layer gradient, so that small gradients survive the fp16
        hand-over between layers; it is divided out of everything returned.  "auto" (the default) picks the power
        of two that brings the largest |dy_top| to about 64: far enough from the fp16 maximum (65504) for the
        gradients to grow a thousandfold on the way down, and far enough from the smallest normal fp16 number
        (6e-5) for them to shrink a few hundredfold per layer (the mean-squared-error gradient of a 4096 x 128 x
        2048 output is ~2e-9 per element: with a scale of 2^12 the bottom layer of a 4-layer stack loses all of
        its gradient).  The scale used is kept in self.last_loss_scale.
        Returns (dx of layer 0 (fp32 when a loss scale is in use) or None, [(dW_ih, dW_hh, db) per layer], [dh0 per layer], [dc0 per layer])."""
        import math
        import torch
        if not self._inputs:
            raise RuntimeError("backward needs a forward pass first")
        if isinstance(loss_scale, str):
            if loss_scale != "auto":
                raise ValueError("loss_scale must be a positive number or 'auto'")
            amax = float(dy_top.abs().max())
            S = 2.0 ** min(60, max(-14, math.floor(math.log2(64.0 / amax)))) if 0.0 < amax < float("inf") else 1.0
        else:
            S = float(loss_scale) if loss_scale and loss_scale > 0 else 1.0
        self.last_loss_scale = S
        cur = (dy_top.float() * S).half() if S != 1.0 else dy_top.half()
        grads: List = [None] * self.L
        dh0s: List = [None] * self.L
        dc0s: List = [None] * self.L
        for l in range(self.L - 1, -1, -1):
            dhn = None if d_hn is None or d_hn[l] is None else (d_hn[l].float() * S)
            dcn = None if d_cn is None or d_cn[l] is None else (d_cn[l].float() * S)
            need_dx = want_dx or l > 0
            dx, dW_ih, dW_hh, db, dh0, dc0 = self.layers[l].backward(self._inputs[l], cur, dhn, dcn, want_dx=need_dx,
                                                                     dx_dtype=torch.float16)
            if S != 1.0:
                for t in (dW_ih, dW_hh, db, dh0, dc0):
                    t.mul_(1.0 / S)
            grads[l] = (dW_ih, dW_hh, db)
            dh0s[l], dc0s[l] = dh0, dc0
            cur = dx
        if cur is not None and S != 1.0:
            cur = cur.float() * (1.0 / S)   # fp32: the unscaled values may lie below the fp16 range
        return cur, grads, dh0s, dc0s
