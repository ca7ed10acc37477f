"""Autograd wrapper and nn.Module over the streaming LSTM extension functions.

Mirrors the interface of the reference's flashlstm_v2/python/flashlstm/streaming_lstm.py:
`GateCache` (:14-16), the argument checks (:19-58, 75-112), `streaming_lstm` (:347-376) and
`StreamingLSTM` (:379-430): sequences live in pinned host memory as fp16, states are fp16 CUDA
tensors, parameters are fp32 CUDA tensors, and the h/c checkpoint tensors returned next to the
outputs are not differentiable.  On PyTorch-ROCm "cuda" is the HIP device and
`torch.cuda.Stream().cuda_stream` is the hipStream_t handed to the library.
"""
from __future__ import annotations

import math
from typing import NamedTuple, Optional, Tuple

import torch
from torch import nn

from . import _flashlstm


class GateCache(NamedTuple):
    """Host checkpoints of the recurrent state, one entry per `recompute_interval` steps."""
    h: torch.Tensor
    c: torch.Tensor


_CACHE_DTYPE_CODES = {torch.float32: 0, torch.float16: 1}


def _cache_dtype_code(dtype: torch.dtype) -> int:
    try:
        return _CACHE_DTYPE_CODES[dtype]
    except KeyError:
        raise ValueError(f"gate cache dtype must be float16 or float32, got {dtype}") from None


def _require_pinned_host(t: torch.Tensor, name: str, dtype: torch.dtype) -> None:
    if t.device.type != "cpu":
        raise ValueError(f"{name} must reside on the CPU (pinned host memory).")
    if t.dtype != dtype:
        raise ValueError(f"{name} must use dtype {dtype}, got {t.dtype}.")
    if not t.is_pinned():
        raise ValueError(f"{name} must be allocated in pinned memory (tensor.pin_memory()).")


def _state_or_zeros(t: Optional[torch.Tensor], shape: Tuple[int, int], name: str) -> torch.Tensor:
    if t is None:
        return torch.zeros(shape, device="cuda", dtype=torch.float16)
    if t.device.type != "cuda":
        raise ValueError(f"{name} must reside on CUDA, got device {t.device}.")
    if t.dtype != torch.float16:
        raise ValueError(f"{name} must use dtype torch.float16, got {t.dtype}.")
    return t if t.is_contiguous() else t.contiguous()


def _three_streams():
    return torch.cuda.Stream(), torch.cuda.Stream(), torch.cuda.Stream()


def _join(streams) -> None:
    for s in streams:
        s.synchronize()
    torch.cuda.current_stream().wait_stream(streams[0])


def _half_cuda_grad(g: Optional[torch.Tensor], name: str) -> Optional[torch.Tensor]:
    if g is None:
        return None
    if g.device.type != "cuda":
        raise ValueError(f"{name} must reside on CUDA.")
    if g.dtype != torch.float16:
        g = g.to(dtype=torch.float16)
    return g if g.is_contiguous() else g.contiguous()


class _StreamingLSTMFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x_host, h0, c0, weight_ih, weight_hh, bias_ih, bias_hh, recompute_interval,
                gate_cache_dtypes):
        _require_pinned_host(x_host, "x_host", torch.float16)
        if not x_host.is_contiguous():
            x_host = x_host.contiguous()
        if recompute_interval <= 0:
            raise ValueError(f"recompute_interval must be >= 1, got {recompute_interval}")
        params = {"weight_ih": weight_ih, "weight_hh": weight_hh, "bias_ih": bias_ih, "bias_hh": bias_hh}
        for name, p in params.items():
            if p.device.type != "cuda":
                raise ValueError(f"{name} must reside on CUDA.")
            if p.dtype != torch.float32:
                raise ValueError(f"{name} must use dtype torch.float32.")

        T, B, I = x_host.shape
        H = weight_hh.size(1)
        h0 = _state_or_zeros(h0, (B, H), "h0")
        c0 = _state_or_zeros(c0, (B, H), "c0")
        if tuple(weight_ih.shape) != (4 * H, I):
            raise ValueError(f"weight_ih must have shape {(4 * H, I)}, got {tuple(weight_ih.shape)}")
        if tuple(weight_hh.shape) != (4 * H, H):
            raise ValueError(f"weight_hh must have shape {(4 * H, H)}, got {tuple(weight_hh.shape)}")
        if bias_ih.numel() != 4 * H or bias_hh.numel() != 4 * H:
            raise ValueError("Bias tensors must have length 4 * hidden_size.")
        weight_ih, weight_hh = weight_ih.contiguous(), weight_hh.contiguous()
        bias_ih, bias_hh = bias_ih.contiguous(), bias_hh.contiguous()

        h_dtype, c_dtype = gate_cache_dtypes
        h_code, c_code = _cache_dtype_code(h_dtype), _cache_dtype_code(c_dtype)
        n_ckpt = (T + recompute_interval - 1) // recompute_interval

        y_host = torch.empty((T, B, H), dtype=torch.float16, pin_memory=True)
        cache_h = torch.empty((n_ckpt, B, H), dtype=h_dtype, pin_memory=True)
        cache_c = torch.empty((n_ckpt, B, H), dtype=c_dtype, pin_memory=True)
        hy = torch.empty((B, H), device="cuda", dtype=torch.float16)
        cy = torch.empty_like(hy)

        # inputs produced on the current stream must be complete before the library's streams read them
        torch.cuda.current_stream().synchronize()
        streams = _three_streams()
        _flashlstm.streaming_lstm_forward(
            T, B, I, H, recompute_interval,
            x_host.data_ptr(), h0.data_ptr(), c0.data_ptr(),
            weight_ih.data_ptr(), weight_hh.data_ptr(), bias_ih.data_ptr(), bias_hh.data_ptr(),
            y_host.data_ptr(), cache_h.data_ptr(), cache_c.data_ptr(), h_code, c_code,
            hy.data_ptr(), cy.data_ptr(),
            streams[0].cuda_stream, streams[1].cuda_stream, streams[2].cuda_stream)
        _join(streams)

        ctx.save_for_backward(x_host, h0, c0, weight_ih, weight_hh, bias_ih, bias_hh, y_host, cache_h, cache_c)
        ctx.meta = (T, B, I, H, recompute_interval, h_code, c_code)
        ctx.mark_non_differentiable(cache_h, cache_c)
        return y_host, cache_h, cache_c, hy, cy

    @staticmethod
    def backward(ctx, grad_y_host, _grad_cache_h, _grad_cache_c, grad_hy, grad_cy):
        x_host, h0, c0, weight_ih, weight_hh, bias_ih, bias_hh, y_host, cache_h, cache_c = ctx.saved_tensors
        T, B, I, H, recompute_interval, h_code, c_code = ctx.meta
        for name, cache in (("gate_cache_h", cache_h), ("gate_cache_c", cache_c)):
            if cache.dtype not in _CACHE_DTYPE_CODES:
                raise ValueError(f"Unsupported dtype for {name}: {cache.dtype}")
            _require_pinned_host(cache, name, cache.dtype)

        if grad_y_host is None:
            grad_y_host = torch.zeros_like(y_host)
        else:
            if grad_y_host.device.type != "cpu":
                raise ValueError("grad_y_host must reside on the CPU.")
            if grad_y_host.dtype != torch.float16:
                grad_y_host = grad_y_host.to(dtype=torch.float16)
            if not grad_y_host.is_contiguous():
                grad_y_host = grad_y_host.contiguous()
            if not grad_y_host.is_pinned():
                grad_y_host = grad_y_host.pin_memory()
        _require_pinned_host(grad_y_host, "grad_y_host", torch.float16)

        grad_hy = _half_cuda_grad(grad_hy, "grad_hy")
        grad_cy = _half_cuda_grad(grad_cy, "grad_cy")

        dx_host = torch.empty_like(x_host)
        if not dx_host.is_pinned():
            dx_host = torch.empty(x_host.shape, dtype=torch.float16, pin_memory=True)
        dW_ih = torch.zeros_like(weight_ih)
        dW_hh = torch.zeros_like(weight_hh)
        db_ih = torch.zeros_like(bias_ih)
        db_hh = torch.zeros_like(bias_hh)
        dh0 = torch.empty((B, H), device="cuda", dtype=torch.float32)
        dc0 = torch.empty_like(dh0)

        torch.cuda.current_stream().synchronize()
        streams = _three_streams()
        _flashlstm.streaming_lstm_backward(
            T, B, I, H, recompute_interval,
            x_host.data_ptr(), y_host.data_ptr(), cache_h.data_ptr(), cache_c.data_ptr(), h_code, c_code,
            grad_y_host.data_ptr(),
            0 if grad_hy is None else grad_hy.data_ptr(),
            0 if grad_cy is None else grad_cy.data_ptr(),
            h0.data_ptr(), c0.data_ptr(),
            weight_ih.data_ptr(), weight_hh.data_ptr(), bias_ih.data_ptr(), bias_hh.data_ptr(),
            dx_host.data_ptr(), dW_ih.data_ptr(), dW_hh.data_ptr(), db_ih.data_ptr(), db_hh.data_ptr(),
            dh0.data_ptr(), dc0.data_ptr(),
            streams[0].cuda_stream, streams[1].cuda_stream, streams[2].cuda_stream)
        _join(streams)

        return (dx_host, dh0.to(dtype=h0.dtype), dc0.to(dtype=c0.dtype), dW_ih, dW_hh, db_ih, db_hh, None, None)


def streaming_lstm(
    x_host: torch.Tensor,
    h0: Optional[torch.Tensor],
    c0: Optional[torch.Tensor],
    weight_ih: torch.Tensor,
    weight_hh: torch.Tensor,
    bias_ih: torch.Tensor,
    bias_hh: torch.Tensor,
    *,
    recompute_interval: int = 1,
    gate_cache_dtypes: Tuple[torch.dtype, torch.dtype] = (torch.float32, torch.float32),
) -> Tuple[torch.Tensor, GateCache, torch.Tensor, torch.Tensor]:
    """Single-layer LSTM over a pinned host sequence.

    Returns `(y_host, GateCache(h, c), hy, cy)`: pinned fp16 outputs (T,B,H), the pinned checkpoint
    tensors (ceil(T/recompute_interval), B, H) in the requested dtypes, and the final fp16 CUDA states.
    """
    y_host, cache_h, cache_c, hy, cy = _StreamingLSTMFunction.apply(
        x_host, h0, c0, weight_ih, weight_hh, bias_ih, bias_hh, recompute_interval, gate_cache_dtypes)
    return y_host, GateCache(cache_h, cache_c), hy, cy


class StreamingLSTM(nn.Module):
    """nn.LSTM-compatible parameters (single layer, unidirectional) on the GPU, host-resident sequences."""

    def __init__(self, input_size: int, hidden_size: int) -> None:
        super().__init__()
        self.input_size = int(input_size)
        self.hidden_size = int(hidden_size)
        g = 4 * self.hidden_size
        # creation order matches nn.LSTM (weight_ih, weight_hh, bias_ih, bias_hh) so that equal seeds
        # give equal parameters
        self.weight_ih = nn.Parameter(torch.empty(g, self.input_size, device="cuda", dtype=torch.float32))
        self.weight_hh = nn.Parameter(torch.empty(g, self.hidden_size, device="cuda", dtype=torch.float32))
        self.bias_ih = nn.Parameter(torch.zeros(g, device="cuda", dtype=torch.float32))
        self.bias_hh = nn.Parameter(torch.zeros(g, device="cuda", dtype=torch.float32))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        bound = 1.0 / math.sqrt(self.hidden_size) if self.hidden_size > 0 else 0.0
        for p in self.parameters():
            nn.init.uniform_(p, -bound, bound)

    def forward(
        self,
        x_host: torch.Tensor,
        h0: Optional[torch.Tensor] = None,
        c0: Optional[torch.Tensor] = None,
        *,
        recompute_interval: int = 1,
        gate_cache_dtypes: Tuple[torch.dtype, torch.dtype] = (torch.float32, torch.float32),
    ) -> Tuple[torch.Tensor, GateCache, Tuple[torch.Tensor, torch.Tensor]]:
        _require_pinned_host(x_host, "x_host", torch.float16)
        B = x_host.size(1)
        h0 = _state_or_zeros(h0, (B, self.hidden_size), "h0")
        c0 = _state_or_zeros(c0, (B, self.hidden_size), "c0")
        y_host, cache, hy, cy = streaming_lstm(
            x_host, h0, c0, self.weight_ih, self.weight_hh, self.bias_ih, self.bias_hh,
            recompute_interval=recompute_interval, gate_cache_dtypes=gate_cache_dtypes)
        return y_host, cache, (hy, cy)

    def extra_repr(self) -> str:
        return f"input_size={self.input_size}, hidden_size={self.hidden_size}"
