"""The fp32 C API (include/flashlstm/lstm_api.h) called through ctypes exactly like the reference's
python/test_lstm.py:44-84 binds it: presets, random shapes, handle reuse with T/2 and T+1, error codes."""
import ctypes
import random

import numpy as np
import pytest
import torch

import oracle
from helpers import TOL_OUT, make_problem, rell2, relmax, to_np

pytestmark = pytest.mark.gpu

ACC32, ACC16 = 0, 1


class Buffers(ctypes.Structure):
    _fields_ = [("impl", ctypes.c_void_p)]


def bind():
    from flashlstm_poc_amd import library_path
    lib = ctypes.CDLL(library_path())
    sz, vp, i32 = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int
    lib.lstm_create_buffers.argtypes = [i32, sz, sz, sz, sz, i32, ctypes.POINTER(Buffers)]
    lib.lstm_destroy_buffers.argtypes = [ctypes.POINTER(Buffers)]
    lib.lstm_set_execution_mode.argtypes = [ctypes.POINTER(Buffers), i32]
    lib.lstm_pack_weights.argtypes = [i32, vp, vp, sz, sz, ctypes.POINTER(Buffers)]
    lib.lstm_forward.argtypes = [vp] * 8 + [sz] * 4 + [ctypes.POINTER(Buffers), i32]
    lib.lstm_backward.argtypes = [vp] * 10 + [sz] * 4 + [ctypes.POINTER(Buffers)]
    return lib


def forward(lib, buf, p, T, precision):
    B, I = p["x"].shape[1:]
    H = p["w_hh"].shape[1]
    d = {k: p[k].cuda().float().contiguous() for k in ("b_ih", "b_hh", "h0", "c0")}
    x = p["x"][:T].cuda().float().contiguous()
    out = torch.empty(T, B, H, device="cuda"); hn = torch.empty(B, H, device="cuda"); cn = torch.empty(B, H, device="cuda")
    rc = lib.lstm_forward(x.data_ptr(), d["b_ih"].data_ptr(), d["b_hh"].data_ptr(), d["h0"].data_ptr(),
                          d["c0"].data_ptr(), out.data_ptr(), hn.data_ptr(), cn.data_ptr(), T, B, I, H,
                          ctypes.byref(buf), precision)
    return rc, out, hn, cn


def oracle_fwd(p, T):
    n = {k: to_np(v) for k, v in p.items()}
    return oracle.forward(n["x"][:T], n["w_ih"], n["w_hh"], n["b_ih"], n["b_hh"], n["h0"], n["c0"],
                          flags=oracle.FLAG_FP16_OPERANDS)


PRESET = [(7, 2, 32, 24), (5, 3, 48, 32), (32, 2, 128, 96), (16, 4, 64, 64), (24, 8, 96, 128)]
rng = random.Random(1234)
RANDOM = [(rng.randint(1, 24), rng.randint(1, 8), rng.randint(1, 64), rng.randint(1, 64)) for _ in range(4)]


@pytest.mark.parametrize("shape", PRESET + RANDOM)
@pytest.mark.parametrize("mode", [0, 1])
def test_forward_presets_with_sequence_shrink_and_grow(shape, mode):
    lib = bind()
    T, B, I, H = shape
    p = make_problem(T + 1, B, I, H, seed=1234 + T, state_scale=1.0, fp16_values=False)   # h0, c0 ~ N(0,1)
    buf = Buffers()
    assert lib.lstm_create_buffers(ACC16, T, B, I, H, 64, ctypes.byref(buf)) == 0
    assert lib.lstm_set_execution_mode(ctypes.byref(buf), mode) == 0
    w_ih, w_hh = p["w_ih"].cuda().contiguous(), p["w_hh"].cuda().contiguous()
    assert lib.lstm_pack_weights(ACC16, w_ih.data_ptr(), w_hh.data_ptr(), I, H, ctypes.byref(buf)) == 0
    for t in (T, max(1, T // 2), T + 1):
        rc, out, hn, cn = forward(lib, buf, p, t, ACC16)
        assert rc == 0
        f = oracle_fwd(p, t)
        assert relmax(to_np(out), f["y"]) <= TOL_OUT
        assert relmax(to_np(hn), f["hn"]) <= TOL_OUT
        assert relmax(to_np(cn), f["cn"]) <= TOL_OUT
        # the reference's own acceptance band (python/test_lstm.py:370-381)
        np.testing.assert_allclose(to_np(out), f["y"], atol=1e-3 + 2e-3, rtol=5e-2)
    assert lib.lstm_destroy_buffers(ctypes.byref(buf)) == 0
    assert buf.impl is None


def test_backward_addition_matches_oracle():
    lib = bind()
    T, B, I, H = 9, 4, 24, 40
    p = make_problem(T, B, I, H, seed=77, fp16_values=False)
    buf = Buffers()
    assert lib.lstm_create_buffers(ACC32, T, B, I, H, 0, ctypes.byref(buf)) == 0
    w_ih, w_hh = p["w_ih"].cuda().contiguous(), p["w_hh"].cuda().contiguous()
    assert lib.lstm_pack_weights(ACC32, w_ih.data_ptr(), w_hh.data_ptr(), I, H, ctypes.byref(buf)) == 0
    rc, out, hn, cn = forward(lib, buf, p, T, ACC32)
    assert rc == 0
    x = p["x"].cuda().contiguous(); dy = p["dy"].cuda().contiguous()
    d_hn = p["d_hn"].cuda().contiguous(); d_cn = p["d_cn"].cuda().contiguous()
    dx = torch.empty_like(x); dW_ih = torch.empty_like(w_ih); dW_hh = torch.empty_like(w_hh)
    db = torch.empty(4 * H, device="cuda"); dh0 = torch.empty(B, H, device="cuda"); dc0 = torch.empty(B, H, device="cuda")
    rc = lib.lstm_backward(x.data_ptr(), dy.data_ptr(), d_hn.data_ptr(), d_cn.data_ptr(), dx.data_ptr(),
                           dW_ih.data_ptr(), dW_hh.data_ptr(), db.data_ptr(), dh0.data_ptr(), dc0.data_ptr(),
                           T, B, I, H, ctypes.byref(buf))
    assert rc == 0
    n = {k: to_np(v) for k, v in p.items()}
    f = oracle_fwd(p, T)
    g = oracle.backward(n["x"], n["w_ih"], n["w_hh"], f, n["dy"], n["d_hn"], n["d_cn"], flags=oracle.FLAG_FP16_OPERANDS)
    for got, k in ((dx, "dx"), (dW_ih, "dw_ih"), (dW_hh, "dw_hh"), (db, "db"), (dh0, "dh0"), (dc0, "dc0")):
        assert rell2(to_np(got), g[k]) <= 1e-2, k
    lib.lstm_destroy_buffers(ctypes.byref(buf))


def test_cache_accessor_on_the_v1_handle():
    # lstm_get_cache: what the last lstm_forward on the handle kept for lstm_backward, read through the handle
    lib = bind()
    lib.lstm_get_cache.argtypes = [ctypes.POINTER(Buffers), ctypes.c_int, ctypes.POINTER(ctypes.c_void_p),
                                   ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]
    T, B, I, H = 6, 3, 10, 20
    p = make_problem(T, B, I, H, seed=31, fp16_values=False)
    buf = Buffers()
    assert lib.lstm_create_buffers(ACC32, T, B, I, H, 0, ctypes.byref(buf)) == 0
    ptr, ld, seq = ctypes.c_void_p(), ctypes.c_size_t(), ctypes.c_size_t()
    assert lib.lstm_get_cache(ctypes.byref(buf), 2, ctypes.byref(ptr), ctypes.byref(ld), ctypes.byref(seq)) == 1   # nothing cached
    w_ih, w_hh = p["w_ih"].cuda().contiguous(), p["w_hh"].cuda().contiguous()
    assert lib.lstm_pack_weights(ACC32, w_ih.data_ptr(), w_hh.data_ptr(), I, H, ctypes.byref(buf)) == 0
    rc, out, hn, cn = forward(lib, buf, p, T, ACC32)
    assert rc == 0
    f = oracle_fwd(p, T)

    def read(which, rows, dtype):
        assert lib.lstm_get_cache(ctypes.byref(buf), which, ctypes.byref(ptr), ctypes.byref(ld), ctypes.byref(seq)) == 0
        assert seq.value == T
        esz = 2 if dtype == torch.float16 else 4
        host = torch.empty(rows, ld.value, dtype=dtype)
        # plain device-to-host copy of the cached rows (the pointer belongs to the library)
        assert ctypes.CDLL("libamdhip64.so").hipMemcpy(ctypes.c_void_p(host.data_ptr()), ptr,
                                                       ctypes.c_size_t(rows * ld.value * esz), 2) == 0
        return host.double().numpy(), ld.value

    Hp = (H + 31) // 32 * 32
    h_all, ldh = read(0, (T + 1) * B, torch.float16)
    c_all, ldc = read(1, (T + 1) * B, torch.float32)
    gates, ldg = read(2, T * B, torch.float16)
    assert (ldh, ldc, ldg) == (Hp, Hp, 4 * Hp)
    assert relmax(h_all[:, :H].reshape(T + 1, B, H)[:T], f["h_all"][:T]) <= 1e-2
    assert relmax(c_all[:, :H].reshape(T + 1, B, H)[:T], f["c_all"][:T]) <= 1e-2
    # column 4 * unit + gate  <->  PyTorch order gate * H + unit
    packed = gates.reshape(T, B, Hp, 4)[:, :, :H, :]
    assert relmax(np.moveaxis(packed, 3, 2).reshape(T, B, 4 * H), f["gates"]) <= 1e-2
    assert lib.lstm_get_cache(ctypes.byref(buf), 9, ctypes.byref(ptr), ctypes.byref(ld), None) == 1
    lib.lstm_destroy_buffers(ctypes.byref(buf))


def test_error_codes_follow_the_reference():
    # reference src/lstm.cu:861-904,1912-1920: everything invalid returns 1
    lib = bind()
    T, B, I, H = 4, 2, 8, 8
    p = make_problem(T, B, I, H)
    buf = Buffers()
    assert lib.lstm_create_buffers(ACC32, T, B, I, H, 0, ctypes.byref(buf)) == 0
    rc, *_ = forward(lib, buf, p, T, ACC32)
    assert rc == 1                                           # weights not packed yet
    w_ih, w_hh = p["w_ih"].cuda().contiguous(), p["w_hh"].cuda().contiguous()
    assert lib.lstm_pack_weights(ACC16, w_ih.data_ptr(), w_hh.data_ptr(), I, H, ctypes.byref(buf)) == 1   # precision
    assert lib.lstm_pack_weights(ACC32, w_ih.data_ptr(), w_hh.data_ptr(), I + 1, H, ctypes.byref(buf)) == 1  # dims
    assert lib.lstm_pack_weights(ACC32, w_ih.data_ptr(), w_hh.data_ptr(), I, H, ctypes.byref(buf)) == 0
    assert forward(lib, buf, p, T, ACC16)[0] == 1            # precision differs from create
    q = make_problem(T, B + 1, I, H)
    assert forward(lib, buf, q, T, ACC32)[0] == 1            # batch differs from create
    assert lib.lstm_set_execution_mode(ctypes.byref(buf), 5) == 1
    assert forward(lib, buf, p, T, ACC32)[0] == 0
    assert lib.lstm_destroy_buffers(ctypes.byref(buf)) == 0
    assert forward(lib, buf, p, T, ACC32)[0] == 1            # destroyed handle


def test_entry_points_open_the_reference_s_range_names_when_a_tracing_library_is_there(tmp_path):
    """The reference brackets its entry points with NVTX ranges (src/lstm.cu:1898, flashlstm_v2/src/nvtx_guard.hpp);
    here they are roctx ranges, looked up at run time.  A stand-in library of that name, first on the loader's path
    of a child process, records what is pushed and popped around one forward and one backward call."""
    import os
    import subprocess
    import sys
    stub = tmp_path / "stub.c"
    stub.write_text(
        '#include <stdio.h>\n#include <stdlib.h>\n'
        'static void note(const char* what, const char* name) { FILE* f = fopen(getenv("FLSTM_RANGE_LOG"), "a");'
        ' if (f) { fprintf(f, "%s %s\\n", what, name); fclose(f); } }\n'
        'int roctxRangePushA(const char* name) { note("push", name); return 0; }\n'
        'int roctxRangePop(void) { note("pop", "-"); return 0; }\n')
    lib = tmp_path / "librocprofiler-sdk-roctx.so"
    subprocess.run(["gcc", "-shared", "-fPIC", "-o", str(lib), str(stub)], check=True)
    log = tmp_path / "ranges.log"
    here = os.path.dirname(os.path.abspath(__file__))
    child = (
        "import ctypes, sys, torch\n"
        f"sys.path.insert(0, {here!r}); sys.path.insert(0, {os.path.dirname(here)!r})\n"
        "import test_v1_api_gpu as t\n"
        "from helpers import make_problem\n"
        "lib = t.bind(); p = make_problem(6, 2, 16, 24, seed=3, fp16_values=False); buf = t.Buffers()\n"
        "assert lib.lstm_create_buffers(t.ACC16, 6, 2, 16, 24, 64, ctypes.byref(buf)) == 0\n"
        "w_ih, w_hh = p['w_ih'].cuda().contiguous(), p['w_hh'].cuda().contiguous()\n"
        "assert lib.lstm_pack_weights(t.ACC16, w_ih.data_ptr(), w_hh.data_ptr(), 16, 24, ctypes.byref(buf)) == 0\n"
        "rc, out, hn, cn = t.forward(lib, buf, p, 6, t.ACC16); assert rc == 0\n"
        "torch.cuda.synchronize(); assert lib.lstm_destroy_buffers(ctypes.byref(buf)) == 0\n")
    env = dict(os.environ, FLSTM_RANGE_LOG=str(log),
               LD_LIBRARY_PATH=str(tmp_path) + os.pathsep + os.environ.get("LD_LIBRARY_PATH", ""))
    r = subprocess.run([sys.executable, "-c", child], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = log.read_text().split("\n")
    pushed = [l.split(" ", 1)[1] for l in lines if l.startswith("push ")]
    assert "FlashLSTM::lstm_forward" in pushed and "FlashLSTM::lstm_forward::compute" in pushed
    assert sum(l.startswith("pop ") for l in lines) == len(pushed)   # every range is closed
