"""Pins the CPU oracle (oracle/lstm_oracle.c): golden vectors, torch.nn.LSTM, finite differences,
closed forms.  Each check is chosen so that a plausible slip (gate order, dropped bias, transposed
operand, wrong sign, off-by-one checkpoint) fails it.  CPU only."""
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import make_problem, torch_reference, to_np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "lstm_golden.npz")


def _case(z, name):
    keys = [k.split("/", 1)[1] for k in z.files if k.startswith(name + "/")]
    return {k: z[f"{name}/{k}"] for k in keys}


@pytest.mark.parametrize("name", ["v2_pytest", "v1_quick", "playground_bwd", "validate_small"])
def test_oracle_reproduces_golden_vectors(name):
    z = np.load(GOLDEN)
    c = _case(z, name)
    f = oracle.forward(c["x"], c["w_ih"], c["w_hh"], c["b_ih"], c["b_hh"], c["h0"], c["c0"])
    for k in ("y", "hn", "cn"):
        np.testing.assert_allclose(f[k], c[k], rtol=0, atol=1e-12, err_msg=k)
    g = oracle.backward(c["x"], c["w_ih"], c["w_hh"], f, c["dy"], c["d_hn"], c["d_cn"])
    for k, gk in (("dx", "dx"), ("dw_ih", "dw_ih"), ("dw_hh", "dw_hh"), ("db", "db_ih"), ("db", "db_hh"),
                  ("dh0", "dh0"), ("dc0", "dc0")):
        np.testing.assert_allclose(g[k], c[gk], rtol=0, atol=1e-11, err_msg=k)


# shape lists of the reference's own tests: python/test_lstm.py:280-302 (quick/standard presets),
# flashlstm_v2/scripts/validate_lstm_fwd.py:243-250 (the CPU-sized ones)
@pytest.mark.parametrize("shape", [(7, 2, 32, 24), (32, 2, 128, 96), (4, 2, 3, 5), (16, 8, 64, 32), (32, 4, 128, 16),
                                   (1, 1, 1, 1), (3, 1, 5, 2), (2, 7, 1, 3)])
def test_oracle_matches_torch_lstm_fp64(shape):
    T, B, I, H = shape
    p = make_problem(T, B, I, H, seed=11, fp16_values=False)
    ref = torch_reference(p, fp16_weights=False)
    n = {k: to_np(v) for k, v in p.items()}
    f = oracle.forward(n["x"], n["w_ih"], n["w_hh"], n["b_ih"], n["b_hh"], n["h0"], n["c0"])
    g = oracle.backward(n["x"], n["w_ih"], n["w_hh"], f, n["dy"], n["d_hn"], n["d_cn"])
    for k in ("y", "hn", "cn"):
        np.testing.assert_allclose(f[k], ref[k], rtol=0, atol=1e-11, err_msg=k)
    for k in ("dx", "dw_ih", "dw_hh", "db", "dh0", "dc0"):
        np.testing.assert_allclose(g[k], ref[k], rtol=0, atol=1e-10, err_msg=k)
    np.testing.assert_allclose(ref["db"], ref["db_hh"], rtol=0, atol=1e-13)  # db_ih == db_hh


def test_config1_cpu_case_matches_torch_lstm():
    # BASELINE config 1: I=128, H=256, B=8, T=64, seed 0, default nn.LSTM init, x ~ N(0,1), h0=c0=0,
    # loss = sum(y^2)
    torch.manual_seed(0)
    m = torch.nn.LSTM(128, 256)
    x = torch.randn(64, 8, 128, requires_grad=True)
    y, _ = m(x)
    (y ** 2).sum().backward()
    P = [to_np(t) for t in (m.weight_ih_l0, m.weight_hh_l0, m.bias_ih_l0, m.bias_hh_l0)]
    f = oracle.forward(to_np(x), *P)
    g = oracle.backward(to_np(x), P[0], P[1], f, 2.0 * f["y"])
    assert np.abs(f["y"] - to_np(y)).max() < 5e-6          # torch ran in fp32
    for k, t in (("dx", x.grad), ("dw_ih", m.weight_ih_l0.grad), ("dw_hh", m.weight_hh_l0.grad), ("db", m.bias_ih_l0.grad)):
        ref = to_np(t)
        assert np.linalg.norm(g[k] - ref) / np.linalg.norm(ref) < 1e-5, k


def test_backward_matches_central_finite_differences():
    T, B, I, H = 3, 2, 3, 4
    p = {k: to_np(v) for k, v in make_problem(T, B, I, H, seed=5, fp16_values=False).items()}

    def loss(q):
        f = oracle.forward(q["x"], q["w_ih"], q["w_hh"], q["b_ih"], q["b_hh"], q["h0"], q["c0"])
        return (f["y"] * q["dy"]).sum() + (f["hn"] * q["d_hn"]).sum() + (f["cn"] * q["d_cn"]).sum()

    f = oracle.forward(p["x"], p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"], p["h0"], p["c0"])
    g = oracle.backward(p["x"], p["w_ih"], p["w_hh"], f, p["dy"], p["d_hn"], p["d_cn"])
    eps = 1e-6
    for name, gname in (("x", "dx"), ("w_ih", "dw_ih"), ("w_hh", "dw_hh"), ("b_ih", "db"), ("b_hh", "db"),
                        ("h0", "dh0"), ("c0", "dc0")):
        a = p[name]
        num = np.zeros_like(a)
        it = np.nditer(a, flags=["multi_index"])
        for _ in it:
            idx = it.multi_index
            q = dict(p); ap = a.copy(); ap[idx] += eps; q[name] = ap
            lp = loss(q)
            am = a.copy(); am[idx] -= eps; q[name] = am
            num[idx] = (lp - loss(q)) / (2 * eps)
        np.testing.assert_allclose(g[gname], num, rtol=0, atol=2e-8, err_msg=name)


def test_zero_recurrent_weights_reduce_to_independent_cells():
    # W_hh = 0: every step is y_t = o * tanh(f * c_{t-1} + i * g) with gates from x_t only
    T, B, I, H = 4, 3, 5, 6
    p = {k: to_np(v) for k, v in make_problem(T, B, I, H, seed=2, fp16_values=False).items()}
    w_hh = np.zeros_like(p["w_hh"])
    f = oracle.forward(p["x"], p["w_ih"], w_hh, p["b_ih"], p["b_hh"], p["h0"], p["c0"])
    sig = lambda v: 1 / (1 + np.exp(-v))
    c = p["c0"].copy()
    for t in range(T):
        z = p["x"][t] @ p["w_ih"].T + p["b_ih"] + p["b_hh"]
        i, fg, g, o = sig(z[:, :H]), sig(z[:, H:2 * H]), np.tanh(z[:, 2 * H:3 * H]), sig(z[:, 3 * H:])
        c = fg * c + i * g
        np.testing.assert_allclose(f["y"][t], o * np.tanh(c), atol=1e-14)
        np.testing.assert_allclose(f["gates"][t], np.concatenate([i, fg, g, o], axis=1), atol=1e-14)
    np.testing.assert_allclose(f["cn"], c, atol=1e-14)


def test_zero_input_zero_bias_zero_state_stays_zero():
    T, B, I, H = 5, 2, 3, 4
    p = {k: to_np(v) for k, v in make_problem(T, B, I, H, seed=3).items()}
    f = oracle.forward(np.zeros_like(p["x"]), p["w_ih"], p["w_hh"], None, None, None, None)
    assert np.all(f["y"] == 0) and np.all(f["cn"] == 0)
    np.testing.assert_allclose(f["gates"][..., :H], 0.5)        # i = sigmoid(0)
    np.testing.assert_allclose(f["gates"][..., 2 * H:3 * H], 0.0)  # g = tanh(0)


def test_state_history_and_checkpoints():
    T, B, I, H = 9, 2, 3, 4
    p = {k: to_np(v) for k, v in make_problem(T, B, I, H, seed=4, fp16_values=False).items()}
    f = oracle.forward(p["x"], p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"], p["h0"], p["c0"])
    np.testing.assert_array_equal(f["h_all"][0], p["h0"])
    np.testing.assert_array_equal(f["c_all"][0], p["c0"])
    np.testing.assert_array_equal(f["h_all"][1:], f["y"])
    np.testing.assert_array_equal(f["h_all"][T], f["hn"])
    for R in (1, 2, 4, 9, 20):
        ck = oracle.checkpoints(f["h_all"], R)
        assert ck.shape[0] == (T + R - 1) // R
        for k in range(ck.shape[0]):
            np.testing.assert_array_equal(ck[k], f["h_all"][k * R])
    # restarting from checkpoint k reproduces the tail (what a recomputing backward relies on)
    R, k = 4, 1
    f2 = oracle.forward(p["x"][k * R:], p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"],
                        oracle.checkpoints(f["h_all"], R)[k], oracle.checkpoints(f["c_all"], R)[k])
    np.testing.assert_allclose(f2["y"], f["y"][k * R:], atol=1e-15)


def test_fp16_rounding_matches_numpy_half():
    rng = np.random.default_rng(0)
    vals = np.concatenate([rng.standard_normal(2000), rng.standard_normal(500) * 1e-6, rng.standard_normal(500) * 3e4,
                           [0.0, -0.0, 65504.0, 65519.9, 65520.0, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -24,
                            2.5 * 2.0 ** -24, 1.0009765625, 1.00048828125, 1.00146484375]])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float32).astype(np.float16).astype(np.float64)
    got = np.array([oracle.round_fp16(v) for v in vals])
    np.testing.assert_array_equal(got, want)


def test_fp16_flags_round_operands_and_feedback():
    T, B, I, H = 6, 2, 5, 4
    p = {k: to_np(v) for k, v in make_problem(T, B, I, H, seed=6, fp16_values=False).items()}
    f0 = oracle.forward(p["x"], p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"], p["h0"], p["c0"])
    r16 = lambda a: a.astype(np.float16).astype(np.float64)
    f1 = oracle.forward(p["x"], p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"], p["h0"], p["c0"],
                        flags=oracle.FLAG_FP16_OPERANDS)
    f1b = oracle.forward(r16(p["x"]), r16(p["w_ih"]), r16(p["w_hh"]), p["b_ih"], p["b_hh"], p["h0"], p["c0"])
    np.testing.assert_array_equal(f1["y"], f1b["y"])
    f2 = oracle.forward(p["x"], p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"], p["h0"], p["c0"],
                        flags=oracle.FLAG_FP16_FEEDBACK | oracle.FLAG_FP16_OUTPUT)
    np.testing.assert_array_equal(f2["y"], r16(f2["y"]))
    assert 0 < np.abs(f2["y"] - f0["y"]).max() < 2e-3


def test_v1_weight_pack_layout():
    # reference src/kernels.cu:57-84: row r = [W_ih[r], W_hh[r], zero pad], stride align_up(I+H, 8)
    for I, H in ((3, 5), (32, 24), (8, 8), (1, 1)):
        w_ih = np.arange(4 * H * I, dtype=np.float64).reshape(4 * H, I) / 64.0
        w_hh = -np.arange(4 * H * H, dtype=np.float64).reshape(4 * H, H) / 64.0
        packed = oracle.pack_weights_v1(w_ih, w_hh)
        stride = (I + H + 7) // 8 * 8
        assert packed.shape == (4 * H, stride)
        r16 = lambda a: a.astype(np.float16).astype(np.float64)
        np.testing.assert_array_equal(packed[:, :I], r16(w_ih))
        np.testing.assert_array_equal(packed[:, I:I + H], r16(w_hh))
        assert np.all(packed[:, I + H:] == 0)


def test_projection_chunk_semantics():
    # reference src/lstm.cu:144-153: <= 0 or larger than T means the whole sequence
    assert oracle.chunk_steps(0, 17) == 17
    assert oracle.chunk_steps(-3, 17) == 17
    assert oracle.chunk_steps(64, 17) == 17
    assert oracle.chunk_steps(17, 17) == 17
    assert oracle.chunk_steps(4, 17) == 4
    assert oracle.chunk_steps(1, 17) == 1


def _fp16_path_oracle(n, gates16=True):
    """The oracle run the way the fp16 path stores things: fp16 operands, h fed back through fp16, the activated
    gates kept as fp16 (the gate cache), dG rounded to fp16 for the products that consume it."""
    f = dict(oracle.forward(n["x"], n["w_ih"], n["w_hh"], n["b_ih"], n["b_hh"], n["h0"], n["c0"],
                            flags=oracle.FLAG_FP16_OPERANDS | oracle.FLAG_FP16_FEEDBACK))
    if gates16:
        f["gates"] = f["gates"].astype(np.float16).astype(np.float64)
    g = oracle.backward(n["x"], n["w_ih"], n["w_hh"], f, n["dy"], n["d_hn"], n["d_cn"],
                        flags=oracle.FLAG_FP16_OPERANDS | oracle.FLAG_FP16_DG)
    return f, g


def test_fp16_dg_flag_only_rounds_the_preactivation_gradients():
    # pins flag bit 3: the flagged run differs from the plain one by no more than fp16 rounding of dG can explain
    # (relative 2^-11 per element), and db -- a plain sum of dG -- is a sum of fp16-representable values
    p = make_problem(6, 3, 5, 4, seed=77)
    n = {k: to_np(v) for k, v in p.items()}
    f = oracle.forward(n["x"], n["w_ih"], n["w_hh"], n["b_ih"], n["b_hh"], n["h0"], n["c0"])
    g0 = oracle.backward(n["x"], n["w_ih"], n["w_hh"], f, n["dy"], n["d_hn"], n["d_cn"])
    g1 = oracle.backward(n["x"], n["w_ih"], n["w_hh"], f, n["dy"], n["d_hn"], n["d_cn"], flags=oracle.FLAG_FP16_DG)
    for k in ("dx", "dw_ih", "dw_hh", "db", "dh0", "dc0"):
        err = np.linalg.norm(g1[k] - g0[k]) / np.linalg.norm(g0[k])
        assert 0 < err < 2e-3, (k, err)
    # one step, one row: db IS dG, so every entry must be exactly representable in fp16
    q = make_problem(1, 1, 3, 4, seed=78)
    m = {k: to_np(v) for k, v in q.items()}
    f = oracle.forward(m["x"], m["w_ih"], m["w_hh"], m["b_ih"], m["b_hh"], m["h0"], m["c0"])
    g = oracle.backward(m["x"], m["w_ih"], m["w_hh"], f, m["dy"], m["d_hn"], m["d_cn"], flags=oracle.FLAG_FP16_DG)
    np.testing.assert_array_equal(g["db"], g["db"].astype(np.float16).astype(np.float64))
    g_plain = oracle.backward(m["x"], m["w_ih"], m["w_hh"], f, m["dy"], m["d_hn"], m["d_cn"])
    np.testing.assert_array_equal(g["db"], g_plain["db"].astype(np.float16).astype(np.float64))


def test_single_unit_dh0_is_ill_conditioned_under_an_fp16_gate_cache():
    # T=40, B=1, I=65, H=1 (seed 550): dh0 is ONE number, the sum of four products dG_0[gate] * w_hh[gate] that
    # nearly cancel.  Storing the activated gates in fp16 (the gate cache) moves it by ~10 % while every other
    # gradient stays within 1e-3: a property of the conditioning of this element, not of any code path.
    p = make_problem(40, 1, 65, 1, seed=550)
    n = {k: to_np(v) for k, v in p.items()}
    ref = torch_reference(p)
    _, g_cache = _fp16_path_oracle(n, gates16=True)
    _, g_nocache = _fp16_path_oracle(n, gates16=False)
    rel = lambda a, b: float(np.abs(a - b).max() / np.abs(b).max())
    assert 5e-2 < rel(g_cache["dh0"], ref["dh0"]) < 2e-1          # the gate cache alone explains the deviation
    assert rel(g_nocache["dh0"], ref["dh0"]) < 2e-3               # without it the element is fine
    for k in ("dx", "dw_ih", "dw_hh", "db", "dc0"):                 # and nothing else is affected
        assert np.linalg.norm(g_cache[k] - ref[k]) / np.linalg.norm(ref[k]) < 2e-3, k
