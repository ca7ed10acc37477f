"""ctypes binding of the device-resident C ABI (include/flashlstm/lstm_core.h).

torch is used for device memory and streams only; every computation happens inside
libflashlstm.so.  There is no fallback: if the library is missing, loading raises.
"""
from __future__ import annotations

import ctypes
import os
import sys
from typing import Optional, Tuple

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

F32, F16 = 0, 1


class LibraryMissing(RuntimeError):
    pass


def library_path() -> str:
    return os.path.join(_HERE, "libflashlstm.so")


def add_flashlstm_to_path() -> str:
    """Puts the drop-in `flashlstm` package (StreamingLSTM & co.) on sys.path and returns its parent dir."""
    p = os.path.join(_HERE, "python")
    if p not in sys.path:
        sys.path.insert(0, p)
    return p


def load_library() -> ctypes.CDLL:
    global _LIB
    if _LIB is not None:
        return _LIB
    path = library_path()
    if not os.path.exists(path):
        raise LibraryMissing(
            f"{path} not found: build it with `make -C flashlstm_poc_amd/csrc` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`)")
    lib = ctypes.CDLL(path)
    c = ctypes
    vp, sz, i32 = c.c_void_p, c.c_size_t, c.c_int
    lib.flstm_core_create.argtypes = [sz, sz, sz, c.POINTER(vp)]
    lib.flstm_core_destroy.argtypes = [vp]
    lib.flstm_core_set_option.argtypes = [vp, c.c_char_p, c.c_long]
    lib.flstm_core_get_info.argtypes = [vp, c.c_char_p]
    lib.flstm_core_get_info.restype = c.c_long
    lib.flstm_core_pack_weights.argtypes = [vp, vp, vp, vp]
    lib.flstm_core_pack_bias.argtypes = [vp, vp, vp, vp]
    lib.flstm_core_forward.argtypes = [vp, sz, vp, i32, vp, vp, i32, vp, i32, vp, vp, i32, i32, vp]
    lib.flstm_core_forward_static.argtypes = [vp, sz, vp, i32, vp, vp, i32, vp, i32, vp, vp, i32, vp]
    lib.flstm_core_forward_static.restype = i32
    lib.flstm_core_tune.argtypes = [vp, sz, i32, i32, vp]
    lib.flstm_core_tune.restype = i32
    lib.flstm_core_tuned_ms.argtypes = [vp, sz, c.c_char_p]
    lib.flstm_core_tuned_ms.restype = c.c_double
    ip = c.POINTER(i32)
    lib.flstm_core_get_tuned.argtypes = [vp, sz, c.POINTER(sz), ip, ip, ip, ip, ip, ip]
    lib.flstm_core_get_tuned.restype = i32
    lib.flstm_core_set_tuned.argtypes = [vp, sz, i32, i32, i32, i32, i32, i32]
    lib.flstm_core_set_tuned.restype = i32
    lib.flstm_core_backward.argtypes = [vp, sz, vp, i32, vp, i32, vp, vp, i32, c.c_float, vp, i32,
                                        vp, vp, vp, vp, vp, vp, vp]
    # the passes fed in ranges of steps
    lib.flstm_core_forward_begin.argtypes = [vp, sz, vp, i32, vp, vp, i32, vp]
    lib.flstm_core_forward_steps.argtypes = [vp, sz, sz, vp]
    lib.flstm_core_forward_end.argtypes = [vp, vp, vp, i32, i32, vp]
    lib.flstm_core_backward_begin.argtypes = [vp, sz, vp, i32, vp, vp, i32, c.c_float, vp, i32, vp]
    lib.flstm_core_backward_steps.argtypes = [vp, sz, sz, vp]
    lib.flstm_core_backward_end.argtypes = [vp, vp, i32, vp, vp, vp, vp, vp, vp, vp]
    for name in ("flstm_core_forward_begin", "flstm_core_forward_steps", "flstm_core_forward_end",
                 "flstm_core_backward_begin", "flstm_core_backward_steps", "flstm_core_backward_end"):
        getattr(lib, name).restype = i32
    lib.flstm_core_cache_ptr.argtypes = [vp, i32, c.POINTER(vp), c.POINTER(sz)]
    lib.flstm_core_last_ms.argtypes = [vp, c.c_char_p]
    lib.flstm_core_last_ms.restype = c.c_double
    for name in ("flstm_core_create", "flstm_core_destroy", "flstm_core_set_option", "flstm_core_pack_weights",
                 "flstm_core_pack_bias", "flstm_core_forward", "flstm_core_backward", "flstm_core_cache_ptr"):
        getattr(lib, name).restype = i32
    _LIB = lib
    return lib


def _dtype_code(t) -> int:
    import torch
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.float16:
        return F16
    raise ValueError(f"unsupported dtype {t.dtype}: tensors must be float16 or float32")


def _ptr(t) -> Optional[int]:
    return None if t is None else t.data_ptr()


class LstmCore:
    """One single-layer LSTM of fixed (batch, input, hidden) on the current GPU."""

    def __init__(self, batch: int, input_size: int, hidden_size: int):
        self.lib = load_library()
        self.B, self.I, self.H = int(batch), int(input_size), int(hidden_size)
        h = ctypes.c_void_p()
        rc = self.lib.flstm_core_create(self.B, self.I, self.H, ctypes.byref(h))
        if rc != 0:
            raise RuntimeError(f"flstm_core_create failed with status {rc}")
        self._h = h

    def close(self) -> None:
        if getattr(self, "_h", None) is not None and self._h:
            self.lib.flstm_core_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @staticmethod
    def _stream() -> int:
        import torch
        return torch.cuda.current_stream().cuda_stream

    def set_option(self, name: str, value: int) -> None:
        rc = self.lib.flstm_core_set_option(self._h, name.encode(), int(value))
        if rc != 0:
            raise ValueError(f"option {name}={value} rejected (status {rc})")

    def info(self, name: str) -> int:
        return int(self.lib.flstm_core_get_info(self._h, name.encode()))

    def last_ms(self, phase: str) -> float:
        return float(self.lib.flstm_core_last_ms(self._h, phase.encode()))

    def tune(self, seq_len: int, repeats: int = 3, try_stepwise: bool = False) -> dict:
        """flstm_core_tune: times the launch choices for this sequence length on synthetic data, caches the best in
        the plan (later passes of similar length use them) and returns them with the best time found per phase."""
        rc = self.lib.flstm_core_tune(self._h, int(seq_len), int(repeats), 1 if try_stepwise else 0, self._stream())
        if rc != 0:
            raise RuntimeError(f"flstm_core_tune failed with status {rc}")
        out = {k: self.info("tuned_" + k) for k in ("T", "row_tiles_fwd", "row_tiles_bwd", "stepwise_fwd", "stepwise_bwd",
                                                    "dw_splits", "bwd_two_d")}
        for ph in ("fwd_rec", "bwd_rec", "bwd_dw"):
            out[ph + "_ms"] = float(self.lib.flstm_core_tuned_ms(self._h, int(seq_len), ph.encode()))
        return out

    _TUNED_KEYS = ("row_tiles_fwd", "row_tiles_bwd", "stepwise_fwd", "stepwise_bwd", "dw_splits", "bwd_two_d")

    def tuned_table(self) -> list:
        """The plan's tuned entries (flstm_core_get_tuned) as a list of dicts, JSON-serialisable: keep it between
        processes and hand it to set_tuned_table of a plan of the same sizes."""
        import ctypes as c
        rows = []
        for i in range(self.info("tuned_entries")):
            T = c.c_size_t()
            v = [c.c_int32() for _ in self._TUNED_KEYS]
            rc = self.lib.flstm_core_get_tuned(self._h, i, c.byref(T), *[c.byref(x) for x in v])
            if rc != 0:
                raise RuntimeError(f"flstm_core_get_tuned failed with status {rc}")
            rows.append({"T": int(T.value), "B": self.B, "I": self.I, "H": self.H,
                         **{k: int(x.value) for k, x in zip(self._TUNED_KEYS, v)}})
        return rows

    def set_tuned_table(self, rows) -> int:
        """Writes tuned entries (as tuned_table returns them) into the plan; rows of other sizes are skipped.  Returns
        the number of entries taken."""
        taken = 0
        for r in rows:
            if (r.get("B"), r.get("I"), r.get("H")) != (self.B, self.I, self.H):
                continue
            rc = self.lib.flstm_core_set_tuned(self._h, int(r["T"]), *[int(r[k]) for k in self._TUNED_KEYS])
            if rc != 0:
                raise RuntimeError(f"flstm_core_set_tuned failed with status {rc}")
            taken += 1
        return taken

    def pack(self, w_ih, w_hh, b_ih=None, b_hh=None) -> None:
        import torch
        for name, t, shape in (("w_ih", w_ih, (4 * self.H, self.I)), ("w_hh", w_hh, (4 * self.H, self.H))):
            if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous() or tuple(t.shape) != shape:
                raise ValueError(f"{name} must be a contiguous CUDA float32 tensor of shape {shape}")
        for name, t in (("b_ih", b_ih), ("b_hh", b_hh)):
            if t is not None and (t.dtype != torch.float32 or not t.is_cuda or t.numel() != 4 * self.H):
                raise ValueError(f"{name} must be a CUDA float32 tensor with 4*hidden elements")
        rc = self.lib.flstm_core_pack_weights(self._h, w_ih.data_ptr(), w_hh.data_ptr(), self._stream())
        if rc == 0:
            rc = self.lib.flstm_core_pack_bias(self._h, _ptr(b_ih), _ptr(b_hh), self._stream())
        if rc != 0:
            raise RuntimeError(f"weight packing failed with status {rc}")

    def forward(self, x, h0=None, c0=None, *, out_dtype=None, save_for_backward: bool = True,
                want_y: bool = True) -> Tuple:
        """x (T,B,I) fp16/fp32 on the GPU -> (y (T,B,H), hy, cy) in out_dtype (default: x.dtype)."""
        import torch
        if not x.is_cuda or x.dim() != 3 or x.shape[1] != self.B or x.shape[2] != self.I:
            raise ValueError(f"x must be a CUDA tensor of shape (T, {self.B}, {self.I})")
        x = x.contiguous()
        T = x.shape[0]
        out_dtype = out_dtype or x.dtype
        st_code = F16
        for name, t in (("h0", h0), ("c0", c0)):
            if t is not None:
                if not t.is_cuda or tuple(t.shape) != (self.B, self.H) or not t.is_contiguous():
                    raise ValueError(f"{name} must be a contiguous CUDA tensor of shape ({self.B}, {self.H})")
        if h0 is not None and c0 is not None and h0.dtype != c0.dtype:
            raise ValueError("h0 and c0 must share a dtype")
        if h0 is not None:
            st_code = _dtype_code(h0)
        elif c0 is not None:
            st_code = _dtype_code(c0)
        y = torch.empty((T, self.B, self.H), device=x.device, dtype=out_dtype) if want_y else None
        hy = torch.empty((self.B, self.H), device=x.device, dtype=out_dtype)
        cy = torch.empty_like(hy)
        rc = self.lib.flstm_core_forward(self._h, T, x.data_ptr(), _dtype_code(x), _ptr(h0), _ptr(c0), st_code,
                                         _ptr(y), _dtype_code(hy), hy.data_ptr(), cy.data_ptr(), _dtype_code(hy),
                                         1 if save_for_backward else 0, self._stream())
        if rc != 0:
            raise RuntimeError(f"flstm_core_forward failed with status {rc}")
        return y, hy, cy

    def forward_static(self, x, h0, c0, y, hy, cy) -> None:
        """flstm_core_forward_static: the forward pass into caller-provided outputs (y (T,B,H), hy, cy (B,H), all
        of one dtype), with the library's fixed scratch array instead of plan-owned buffers -- the call allocates
        nothing.  h0 / c0 may be None (zeros).  Raises MemoryError when the pass does not fit the array."""
        T = x.shape[0]
        if not x.is_cuda or not x.is_contiguous() or tuple(x.shape[1:]) != (self.B, self.I):
            raise ValueError(f"x must be a contiguous CUDA tensor of shape (T, {self.B}, {self.I})")
        if tuple(y.shape) != (T, self.B, self.H) or tuple(hy.shape) != (self.B, self.H) or tuple(cy.shape) != (self.B, self.H):
            raise ValueError("outputs must have shapes (T,B,H), (B,H), (B,H)")
        if hy.dtype != cy.dtype or not (y.is_contiguous() and hy.is_contiguous() and cy.is_contiguous()):
            raise ValueError("hy and cy must share a dtype; outputs must be contiguous")
        st = h0 if h0 is not None else c0
        rc = self.lib.flstm_core_forward_static(self._h, T, x.data_ptr(), _dtype_code(x), _ptr(h0), _ptr(c0),
                                                _dtype_code(st) if st is not None else F16, y.data_ptr(),
                                                _dtype_code(y), hy.data_ptr(), cy.data_ptr(), _dtype_code(hy),
                                                self._stream())
        if rc == 2004:
            raise MemoryError("the pass needs more scratch memory than flstm_core_forward_static's fixed array holds")
        if rc != 0:
            raise RuntimeError(f"flstm_core_forward_static failed with status {rc}")

    def backward(self, x, dy, d_hn=None, d_cn=None, *, grad_scale: float = 1.0, dx_dtype=None,
                 want_dx: bool = True, accumulate_into=None):
        """Returns (dx, dW_ih, dW_hh, db, dh0, dc0); db is the gradient of both bias vectors.

        accumulate_into=(dW_ih, dW_hh, db): add this call's parameter gradients to these fp32 tensors (and return
        them) instead of writing fresh ones -- a sequence run as consecutive segments, last segment first, with
        each call's dh0 / dc0 passed to the next one as d_hn / d_cn."""
        import torch
        x = x.contiguous()
        dy = dy.contiguous()
        T = x.shape[0]
        if tuple(dy.shape) != (T, self.B, self.H):
            raise ValueError(f"dy must have shape ({T}, {self.B}, {self.H})")
        dev = x.device
        dst_code = F16
        if d_hn is not None and d_cn is not None and d_hn.dtype != d_cn.dtype:
            raise ValueError("d_hn and d_cn must share a dtype")
        if d_hn is not None:
            d_hn = d_hn.contiguous(); dst_code = _dtype_code(d_hn)
        if d_cn is not None:
            d_cn = d_cn.contiguous(); dst_code = _dtype_code(d_cn)
        dx_dtype = dx_dtype or x.dtype
        dx = torch.empty_like(x, dtype=dx_dtype) if want_dx else None
        if accumulate_into is not None:
            dW_ih, dW_hh, db = accumulate_into
            for t, shape in ((dW_ih, (4 * self.H, self.I)), (dW_hh, (4 * self.H, self.H)), (db, (4 * self.H,))):
                if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous() or tuple(t.shape) != shape:
                    raise ValueError(f"accumulate_into tensors must be contiguous CUDA float32 of shape {shape}")
        else:
            dW_ih = torch.empty((4 * self.H, self.I), device=dev, dtype=torch.float32)
            dW_hh = torch.empty((4 * self.H, self.H), device=dev, dtype=torch.float32)
            db = torch.empty((4 * self.H,), device=dev, dtype=torch.float32)
        dh0 = torch.empty((self.B, self.H), device=dev, dtype=torch.float32)
        dc0 = torch.empty_like(dh0)
        self.set_option("accumulate_grads", 1 if accumulate_into is not None else 0)
        rc = self.lib.flstm_core_backward(self._h, T, x.data_ptr(), _dtype_code(x), dy.data_ptr(), _dtype_code(dy),
                                          _ptr(d_hn), _ptr(d_cn), dst_code, float(grad_scale), _ptr(dx),
                                          _dtype_code(dx) if dx is not None else F16, dW_ih.data_ptr(),
                                          dW_hh.data_ptr(), db.data_ptr(), None, dh0.data_ptr(), dc0.data_ptr(),
                                          self._stream())
        if rc != 0:
            raise RuntimeError(f"flstm_core_backward failed with status {rc}")
        return dx, dW_ih, dW_hh, db, dh0, dc0
