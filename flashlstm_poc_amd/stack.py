"""Stacked LSTM on top of the single-layer core: layer l's outputs are layer l+1's inputs, and in the backward
pass layer l+1's input gradient is layer l's upstream gradient.  The reference is single-layer only
(flashlstm_v2/python/flashlstm/streaming_lstm.py:380-430); this is the thin layer loop a multi-layer workload
needs, with everything resident on the GPU in fp16 between layers."""
from typing import List, Optional, Sequence, Tuple

import torch

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
                 d_cn: Optional[Sequence] = None, want_dx: bool = True, dy_factor: float = 1.0):
        """dy_top (T,B,H): gradient wrt the top layer's outputs, times 1 / dy_factor: the gradient is dy_factor * dy_top
        (a loss that averages over many elements has a gradient of the form tiny_constant * tensor_of_order_one; handing
        the two over apart keeps the tensor in fp16 range and saves the fp32 passes that would form their product).  loss_scale (a power of two) multiplies it before
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
            lo, hi = torch.aminmax(dy_top)
            amax = max(-float(lo), float(hi)) * abs(float(dy_factor))
            S = 2.0 ** min(60, max(-14, math.floor(math.log2(64.0 / amax)))) if 0.0 < amax < float("inf") else 1.0
        else:
            S = float(loss_scale) if loss_scale and loss_scale > 0 else 1.0
        self.last_loss_scale = S
        k = S * float(dy_factor)
        if dy_top.dtype == torch.float16:
            cur = dy_top * k if k != 1.0 else dy_top     # one pass: the product is formed in fp32 and rounded once
        else:
            cur = (dy_top.float() * k).half()
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

    def backward_mse(self, y_top, target, **kwargs):
        """backward() for the loss mean((y_top - target)^2) over all elements: its gradient 2 / N * (y_top - target) is
        handed over as the fp16 difference and the factor 2 / N (see dy_factor).  y_top: what forward() returned."""
        import torch
        if y_top.dtype != torch.float16 or target.dtype != torch.float16:
            return self.backward((y_top.float() - target.float()), dy_factor=2.0 / y_top.numel(), **kwargs)
        return self.backward(torch.sub(y_top, target), dy_factor=2.0 / y_top.numel(), **kwargs)


class _StackFunction(torch.autograd.Function):
    """Autograd node around LstmStack: inputs (x, h0 (L,B,H) or None, c0 or None, 4 * L parameters)."""

    @staticmethod
    def forward(ctx, module, x, h0, c0, y_dtype, loss_scale, *params):
        L = module.num_layers
        stack = module._stack_for(x.shape[1])
        stack.pack([tuple(p.detach() for p in params[4 * l:4 * l + 4]) for l in range(L)])
        y, hys, cys = stack.forward(x.detach(), None if h0 is None else list(h0.detach().half()),
                                    None if c0 is None else list(c0.detach().half()))
        module._generation += 1
        ctx.module, ctx.stack, ctx.generation, ctx.loss_scale = module, stack, module._generation, loss_scale
        ctx.has_state = (h0 is not None, c0 is not None)
        ctx.x_dtype = x.dtype
        if y_dtype != y.dtype:
            y = y.to(y_dtype)
        return y, torch.stack(hys), torch.stack(cys)

    @staticmethod
    def backward(ctx, dy, dhn, dcn):
        if ctx.generation != ctx.module._generation:
            raise RuntimeError("StackedLSTM keeps the caches of its most recent forward pass only: call backward "
                               "before the next forward pass of the same module")
        L = ctx.module.num_layers
        zero_state = lambda g: None if g is None else list(g)
        if dy is None:
            dy = torch.zeros((ctx.stack._inputs[0].shape[0], ctx.stack.B, ctx.stack.H), device=dhn.device, dtype=torch.float16)
        dx, grads, dh0s, dc0s = ctx.stack.backward(dy, loss_scale=ctx.loss_scale, d_hn=zero_state(dhn), d_cn=zero_state(dcn),
                                                   want_dx=ctx.needs_input_grad[1])
        flat = []
        for l in range(L):
            dW_ih, dW_hh, db = grads[l]
            flat += [dW_ih, dW_hh, db, db.clone()]
        gx = None if dx is None else dx.to(ctx.x_dtype)
        gh0 = torch.stack(dh0s).half() if ctx.has_state[0] and ctx.needs_input_grad[2] else None
        gc0 = torch.stack(dc0s).half() if ctx.has_state[1] and ctx.needs_input_grad[3] else None
        return (None, gx, gh0, gc0, None, None, *flat)


class StackedLSTM(torch.nn.Module):
    """Multi-layer LSTM as an nn.Module with autograd, on the device-resident core: the training surface for a
    stacked workload (BASELINE config 5).  The reference's module is single-layer and host-streaming
    (flashlstm_v2/python/flashlstm/streaming_lstm.py:380-430, mirrored by flashlstm.StreamingLSTM); this one keeps
    every sequence on the GPU.  Parameters carry torch.nn.LSTM's names (weight_ih_l0, weight_hh_l0, bias_ih_l0,
    bias_hh_l0, ...), layout and initialisation (U(-1/sqrt(H), 1/sqrt(H)), fp32, on the GPU), so a state_dict moves
    between the two.

    forward(x, (h0, c0)=None) -> (y, (h_n, c_n)):  x (T,B,I) fp16 CUDA; h0 / c0 (L,B,H) fp16 or None (zeros);
    y (T,B,H) in `output_dtype` (fp16, or fp32 for losses whose gradient per element lies below the fp16 range: the
    gradient arrives in y's dtype); h_n, c_n (L,B,H) fp16.  Differentiable in x, h0, c0 and all parameters.  Inside,
    gradients pass from layer to layer in fp16 under a power-of-two loss scale (`loss_scale`, default "auto").
    The module keeps the caches of its MOST RECENT forward pass only; backward must run before the next forward."""

    def __init__(self, input_size: int, hidden_size: int, num_layers: int = 1, *, output_dtype=torch.float16,
                 loss_scale="auto", device="cuda"):
        super().__init__()
        if num_layers < 1:
            raise ValueError("num_layers must be >= 1")
        self.input_size, self.hidden_size, self.num_layers = int(input_size), int(hidden_size), int(num_layers)
        self.output_dtype, self.loss_scale = output_dtype, loss_scale
        H = self.hidden_size
        for l in range(self.num_layers):
            I = self.input_size if l == 0 else H
            for name, shape in ((f"weight_ih_l{l}", (4 * H, I)), (f"weight_hh_l{l}", (4 * H, H)),
                                (f"bias_ih_l{l}", (4 * H,)), (f"bias_hh_l{l}", (4 * H,))):
                self.register_parameter(name, torch.nn.Parameter(torch.empty(shape, device=device, dtype=torch.float32)))
        self.reset_parameters()
        self._stacks = {}       # batch size -> LstmStack
        self._generation = 0

    def reset_parameters(self) -> None:
        k = 1.0 / self.hidden_size ** 0.5
        for p in self.parameters():     # same order as torch.nn.LSTM.reset_parameters
            torch.nn.init.uniform_(p, -k, k)

    def _stack_for(self, batch: int) -> LstmStack:
        st = self._stacks.get(batch)
        if st is None:
            for old in self._stacks.values():   # one batch size at a time: the caches are large
                old.close()
            self._stacks = {}
            st = self._stacks[batch] = LstmStack(batch, self.input_size, self.hidden_size, self.num_layers)
        return st

    def forward(self, x, state=None):
        if not x.is_cuda or x.dtype != torch.float16 or x.dim() != 3 or x.shape[2] != self.input_size:
            raise ValueError(f"x must be a CUDA float16 tensor of shape (T, B, {self.input_size})")
        h0 = c0 = None
        if state is not None:
            h0, c0 = state
            for name, t in (("h0", h0), ("c0", c0)):
                if t is not None and (not t.is_cuda or tuple(t.shape) != (self.num_layers, x.shape[1], self.hidden_size)):
                    raise ValueError(f"{name} must be a CUDA tensor of shape ({self.num_layers}, {x.shape[1]}, {self.hidden_size})")
        params = [getattr(self, f"{n}_l{l}") for l in range(self.num_layers) for n in ("weight_ih", "weight_hh", "bias_ih", "bias_hh")]
        y, h_n, c_n = _StackFunction.apply(self, x.contiguous(), h0, c0, self.output_dtype, self.loss_scale, *params)
        return y, (h_n, c_n)

    def release(self) -> None:
        """Frees the device caches (plans are rebuilt on the next forward pass)."""
        for st in self._stacks.values():
            st.close()
        self._stacks = {}
