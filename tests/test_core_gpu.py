"""Parity of the device-resident core (HIP kernels through the C ABI) against the CPU oracle and
torch.nn.LSTM on the same seeded inputs.  Tolerances: max relative error <= 1e-2 on y / h_T / c_T,
relative L2 error <= 1e-2 on every gradient (fp16 storage, fp32 accumulation, fp32 cell state)."""
import numpy as np
import pytest
import torch

import oracle
from helpers import check_against, make_problem, rell2, relmax, to_np, torch_reference

pytestmark = pytest.mark.gpu


def run_core(p, *, half=True, stepwise=False, proj_chunk=0, grad_scale=1.0, state_grads=True, T=None, core=None):
    from flashlstm_poc_amd import LstmCore
    dev = "cuda"
    T_full, B, I = p["x"].shape
    H = p["w_hh"].shape[1]
    T = T or T_full
    cv = (lambda t: t.to(dev).half()) if half else (lambda t: t.to(dev).float())
    own = core is None
    if own:
        core = LstmCore(B, I, H)
        core.pack(p["w_ih"].to(dev), p["w_hh"].to(dev), p["b_ih"].to(dev), p["b_hh"].to(dev))
    core.set_option("stepwise", 1 if stepwise else 0)
    core.set_option("proj_chunk", proj_chunk)
    x = cv(p["x"][:T])
    y, hy, cy = core.forward(x, cv(p["h0"]), cv(p["c0"]))
    dx, dW_ih, dW_hh, db, dh0, dc0 = core.backward(
        x, cv(p["dy"][:T]), cv(p["d_hn"]) if state_grads else None, cv(p["d_cn"]) if state_grads else None,
        grad_scale=grad_scale)
    torch.cuda.synchronize()
    out = dict(y=to_np(y), hn=to_np(hy), cn=to_np(cy), dx=to_np(dx), dw_ih=to_np(dW_ih), dw_hh=to_np(dW_hh),
               db=to_np(db), dh0=to_np(dh0), dc0=to_np(dc0))
    info = {k: core.info(k) for k in ("persistent_fwd", "persistent_bwd", "xcd_local_fwd", "fallbacks", "bwd_two_d")}
    if own:
        core.close()
    return out, info


def oracle_reference(p, state_grads=True, T=None):
    n = {k: to_np(v) for k, v in p.items()}
    T = T or n["x"].shape[0]
    f = oracle.forward(n["x"][:T], n["w_ih"], n["w_hh"], n["b_ih"], n["b_hh"], n["h0"], n["c0"],
                       flags=oracle.FLAG_FP16_OPERANDS)
    g = oracle.backward(n["x"][:T], n["w_ih"], n["w_hh"], f, n["dy"][:T], n["d_hn"] if state_grads else None,
                        n["d_cn"] if state_grads else None, flags=oracle.FLAG_FP16_OPERANDS)
    return dict(y=f["y"], hn=f["hn"], cn=f["cn"], **g), f


# shapes of the reference's tests (python/test_lstm.py:280-302, validate_lstm_fwd.py:243-250,
# validate_lstm_bwd.py:435-443, test_streaming_lstm.py:17-20) plus ragged / odd sizes
SHAPES = [(4, 2, 3, 5), (7, 2, 32, 24), (32, 2, 128, 96), (16, 8, 64, 32), (32, 4, 128, 16), (64, 32, 256, 256),
          (1, 1, 1, 1), (3, 33, 7, 9), (5, 70, 65, 33), (9, 1, 130, 257)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("half", [True, False])
def test_forward_backward_match_oracle(shape, half):
    p = make_problem(*shape, seed=hash(shape) % 1000)
    ref, _ = oracle_reference(p)
    got, info = run_core(p, half=half)
    assert info["fallbacks"] == 0
    check_against(ref, got, label=f"{shape} half={half}")


@pytest.mark.parametrize("shape", [(4, 2, 3, 5), (16, 8, 64, 32), (64, 8, 128, 256)])
def test_matches_torch_lstm(shape):
    p = make_problem(*shape, seed=7)
    ref = torch_reference(p)  # fp64 nn.LSTM on the fp16-rounded weights
    got, _ = run_core(p)
    check_against(ref, got, label=str(shape))


def test_config1_through_fp32_io():
    # BASELINE config 1: I=128, H=256, B=8, T=64, h0 = c0 = 0, loss = sum(y^2)
    torch.manual_seed(0)
    m = torch.nn.LSTM(128, 256)
    x = torch.randn(64, 8, 128)
    from flashlstm_poc_amd import LstmCore
    core = LstmCore(8, 128, 256)
    core.pack(*(t.detach().cuda() for t in (m.weight_ih_l0, m.weight_hh_l0, m.bias_ih_l0, m.bias_hh_l0)))
    y, hy, cy = core.forward(x.cuda())
    dx, dW_ih, dW_hh, db, dh0, dc0 = core.backward(x.cuda(), 2.0 * y)
    xr = x.clone().requires_grad_(True)
    yr, (hr, cr) = m(xr)
    (yr ** 2).sum().backward()
    assert relmax(to_np(y), to_np(yr)) <= 1e-2 and relmax(to_np(cy), to_np(cr[0])) <= 1e-2
    for got, ref in ((dx, xr.grad), (dW_ih, m.weight_ih_l0.grad), (dW_hh, m.weight_hh_l0.grad), (db, m.bias_ih_l0.grad)):
        assert rell2(to_np(got), to_np(ref)) <= 1e-2
    core.close()


@pytest.mark.parametrize("shape", [(6, 300, 32, 1024), (5, 128, 32, 2048), (4, 520, 32, 512)])
def test_two_row_blocks_per_workgroup_match_torch_lstm(shape):
    # more row blocks than groups that run side by side: a workgroup walks two (or more) blocks per step and keeps
    # the cell state of the first two in registers
    p = make_problem(*shape, seed=5)
    ref = torch_reference(p, dtype=torch.float32, device="cuda")
    got, info = run_core(p)
    assert info["persistent_fwd"] == 1 and info["persistent_bwd"] == 1 and info["fallbacks"] == 0
    check_against(ref, got, label=str(shape))


@pytest.mark.parametrize("shape", [(12, 40, 32, 64), (20, 16, 64, 1024), (6, 300, 32, 1024), (5, 128, 32, 2048)])
def test_persistent_and_stepwise_agree(shape):
    p = make_problem(*shape, seed=3)
    a, ia = run_core(p, stepwise=False)
    b, ib = run_core(p, stepwise=True)
    assert ia["persistent_fwd"] == 1 and ib["persistent_fwd"] == 0
    for k in ("y", "hn", "cn"):
        np.testing.assert_array_equal(a[k], b[k])       # same arithmetic, same order
    # the backward kernels sum a product in the same order either way -- except the persistent kernel for 2048 hidden
    # units, which splits the contraction over eight workgroups (other fp32 summation order, then fp16 rounding of dG)
    tol = 2e-4 if ia["bwd_two_d"] == 1 else 1e-5
    assert ib["bwd_two_d"] == 0
    for k in ("dx", "dh0", "dc0", "dw_hh", "db"):
        assert rell2(a[k], b[k]) < tol, k


@pytest.mark.parametrize("shape", [(7, 128, 32, 2048), (6, 40, 32, 2048), (9, 5, 64, 2040), (4, 17, 32, 2048),
                                   (1, 16, 32, 2048), (2, 33, 32, 2017), (5, 96, 32, 2048), (3, 100, 64, 2048),
                                   (4, 256, 32, 2048), (3, 200, 32, 2048), (3, 150, 32, 2040), (2, 300, 32, 2048),
                                   (6, 256, 32, 1024), (5, 200, 32, 1024), (4, 130, 64, 1000), (7, 40, 32, 1024)])
def test_two_way_split_backward_for_2048_units(shape):
    # 2048 (padded) hidden units: the persistent backward kernel splits its product over column slices AND over the
    # contraction, and sums the partial products through a second ring.  One row block (8 contraction slices) and two
    # to four (4 slices, two groups taking alternate blocks, one or two passes per workgroup), ragged batches, padded
    # hidden sizes, a single step; against torch, against the one-way layout, and through the give-up path.  More than
    # 128 rows: the batch is walked in windows of 128 rows, one persistent launch each (the last one short).
    # 1024 (padded) hidden units: 16 column slices x 2 contraction slices inside every XCD, one row block per XCD.
    from flashlstm_poc_amd import LstmCore
    T, B, I, H = shape
    p = make_problem(*shape, seed=11)
    ref = torch_reference(p, dtype=torch.float32, device="cuda")
    core = LstmCore(B, I, H)
    core.pack(*(p[k].cuda() for k in ("w_ih", "w_hh", "b_ih", "b_hh")))
    if H > 1024:   # by itself the plan takes the layout where it measured faster
        assert core.info("bwd_two_d") == (0 if 32 < B <= 64 else 1)   # (two row blocks per step: a tie, the one-way layout stays)
    else:
        assert core.info("bwd_two_d") == 0   # (1024 units: measured slower than the one-way layout, only on request)
    core.set_option("bwd_two_d", 2)                           # here: wherever it can run
    got, info = run_core(p, core=core)
    assert info["persistent_bwd"] == 1 and info["bwd_two_d"] == 1 and info["fallbacks"] == 0
    check_against(ref, got, label=f"two-way {shape}")
    again, _ = run_core(p, core=core)
    for k in got:
        np.testing.assert_array_equal(again[k], got[k], err_msg=k)   # fixed summation order: run-to-run identical
    core.set_option("bwd_two_d", 0)
    one_way, info1 = run_core(p, core=core)
    assert info1["persistent_bwd"] == 1 and info1["bwd_two_d"] == 0
    for k in ("dx", "dh0", "dc0", "dw_ih", "dw_hh", "db"):
        assert rell2(got[k], one_way[k]) < 2e-4, k
    core.set_option("bwd_two_d", 2)
    core.set_option("spin_limit", 0)   # the first operand found unwritten makes the launch give up; the pass is repeated step-wise
    repaired, info2 = run_core(p, core=core)
    if T > 1 and B <= 32 and H > 1024:   # one row block per step: the next step's operand is always requested before it is complete
        assert info2["fallbacks"] >= 1
    check_against(ref, repaired, label=f"two-way, repaired {shape}")
    core.close()


@pytest.mark.parametrize("shape", [(6, 128, 32, 2048), (6, 40, 32, 1024), (5, 33, 16, 256)])
def test_a_batch_row_of_nans_stays_in_its_row(shape):
    """Values that are NaN in their own right must travel through the exchange like any others.  The forward kernel
    for 2048 units with several row blocks per workgroup validates what it fetched by its effect on the product (a
    NaN in the result sends the wave through a second, word-by-word checked pass): a NaN row takes that second pass at
    every step, must not be mistaken for unwritten data (no give-up, no fallback), and must leave every other batch
    row bit-identical to a run without it."""
    from flashlstm_poc_amd import LstmCore
    T, B, I, H = shape
    p = make_problem(T, B, I, H, seed=11)
    core = LstmCore(B, I, H)
    core.pack(p["w_ih"].cuda(), p["w_hh"].cuda(), p["b_ih"].cuda(), p["b_hh"].cuda())
    x = p["x"].cuda().half()
    h0, c0 = p["h0"].cuda().half(), p["c0"].cuda().half()
    y_clean, hn_clean, cn_clean = (t.clone() for t in core.forward(x, h0, c0))
    bad = 5
    x_bad = x.clone()
    x_bad[1:, bad, :] = float("nan")
    y, hn, cn = core.forward(x_bad, h0, c0)
    dy = p["dy"].cuda().half()
    grads = core.backward(x_bad, dy, None, None)
    torch.cuda.synchronize()
    assert core.info("fallbacks") == 0 and core.info("persistent_fwd") == 1
    keep = [b for b in range(B) if b != bad]
    assert torch.equal(y[:, keep], y_clean[:, keep]) and torch.equal(hn[keep], hn_clean[keep]) and torch.equal(cn[keep], cn_clean[keep])
    assert torch.equal(y[0, bad], y_clean[0, bad]) and bool(torch.isnan(y[1:, bad]).all())
    dx = grads[0]
    assert bool(torch.isfinite(dx[:, keep]).all()) and bool(torch.isnan(dx[1:, bad]).all())
    core.close()


def test_retry_limit_hit_is_repaired_by_stepwise_pass():
    # Failure handling of the persistent kernels, forced from the host: with a retry limit of 1 a workgroup
    # that finds an operand not yet written gives up at once, every kernel still exits normally, and the
    # library repeats the pass one launch per step.  The results must be the same either way.
    from flashlstm_poc_amd import LstmCore
    p = make_problem(24, 40, 64, 256, seed=5)
    ref, _ = oracle_reference(p)
    core = LstmCore(40, 64, 256)
    core.pack(*(p[k].cuda() for k in ("w_ih", "w_hh", "b_ih", "b_hh")))
    core.set_option("spin_limit", 1)
    for _ in range(2):
        got, info = run_core(p, core=core)
        check_against(ref, got, label=f"spin_limit=1 fallbacks={info['fallbacks']}")
    core.close()


def test_give_up_demotes_for_a_few_passes_and_then_the_persistent_kernel_returns():
    # The give-up of a persistent launch is injected from the host (no kernel waits for anything): the pass is
    # repeated step-wise with the same results, that direction stays step-wise for 8 passes, then the persistent
    # kernel is back; a second give-up holds it for 16.  The other direction is not touched.
    from flashlstm_poc_amd import LstmCore
    p = make_problem(10, 40, 64, 256, seed=6)
    ref, _ = oracle_reference(p)
    core = LstmCore(40, 64, 256)
    core.pack(*(p[k].cuda() for k in ("w_ih", "w_hh", "b_ih", "b_hh")))
    x = p["x"].cuda().half(); h0 = p["h0"].cuda().half(); c0 = p["c0"].cuda().half()
    assert core.info("persistent_fwd") == 1 and core.info("hold_fwd") == 0
    y0, _, _ = core.forward(x, h0, c0)
    core.set_option("inject_stall", 1)
    y1, _, _ = core.forward(x, h0, c0)
    assert torch.equal(y0, y1)                        # step-wise repeat: bit-identical forward results
    assert core.info("demotions_fwd") == 1 and core.info("fallbacks") == 1
    assert core.info("persistent_fwd") == 0 and core.info("hold_fwd") == 7 and core.info("persistent_bwd") == 1
    for left in range(6, -1, -1):
        y2, _, _ = core.forward(x, h0, c0)
        assert torch.equal(y0, y2) and core.info("hold_fwd") == left
    assert core.info("persistent_fwd") == 1           # back on the persistent kernel
    core.set_option("inject_stall", 1)
    core.forward(x, h0, c0)
    assert core.info("demotions_fwd") == 2 and core.info("hold_fwd") == 15
    # the same for the backward direction, checked against the oracle
    core.set_option("inject_stall", 0)
    got, _ = run_core(p, core=core)
    check_against(ref, got, label="before the injected backward give-up")
    core.forward(x, h0, c0)
    core.set_option("inject_stall", 1)                # forward is step-wise now, so the backward pass takes it
    assert core.info("persistent_fwd") == 0 and core.info("persistent_bwd") == 1
    dy = p["dy"].cuda().half()
    grads = core.backward(x, dy, p["d_hn"].cuda().half(), p["d_cn"].cuda().half())
    assert core.info("demotions_bwd") == 1 and core.info("persistent_bwd") == 0 and core.info("hold_bwd") == 7
    for k, t in zip(("dx", "dw_ih", "dw_hh", "db", "dh0", "dc0"), grads):
        assert rell2(to_np(t), ref[k]) <= 1e-2, k
    core.close()


@pytest.mark.parametrize("shape", [(24, 40, 64, 256), (12, 8, 32, 3072)])
def test_stepwise_launches_replay_from_a_captured_graph(shape):
    # Where a pass is one launch per time step (here: forced; H = 3072: weights that do not fit on chip) the launches
    # of a range are captured into a hipGraph once and replayed afterwards.  Every replay is checked against the
    # first (eager-equivalent) results, with the program's own eager work and synchronisations between the replays.
    from flashlstm_poc_amd import LstmCore
    T, B, I, H = shape
    p = make_problem(T, B, I, H, seed=8)
    dev = {k: v.cuda() for k, v in p.items()}
    x, h0, c0, dy = dev["x"].half(), dev["h0"].half(), dev["c0"].half(), dev["dy"].half()
    side = torch.cuda.Stream()      # the legacy default stream cannot be captured
    with torch.cuda.stream(side):
        plain = LstmCore(B, I, H)
        plain.pack(dev["w_ih"], dev["w_hh"], dev["b_ih"], dev["b_hh"])
        plain.set_option("stepwise", 1)
        plain.set_option("step_graphs", 0)
        y_ref, hy_ref, cy_ref = plain.forward(x, h0, c0)
        g_ref = plain.backward(x, dy)
        assert plain.info("graph_captures") == 0 and plain.info("persistent_fwd") == 0
        core = LstmCore(B, I, H)
        core.pack(dev["w_ih"], dev["w_hh"], dev["b_ih"], dev["b_hh"])
        core.set_option("stepwise", 1)
        for rep in range(4):
            y, hy, cy = core.forward(x, h0, c0)
            g = core.backward(x, dy)
            side.synchronize()
            assert torch.equal(y, y_ref) and torch.equal(cy, cy_ref), rep
            for a, b_, name in zip(g, g_ref, ("dx", "dW_ih", "dW_hh", "db", "dh0", "dc0")):
                assert torch.equal(a, b_), (rep, name)
            junk = (torch.randn(256, 256, device="cuda") @ torch.randn(256, 256, device="cuda")).sum().item()   # eager work between replays
            assert junk == junk
        assert core.info("graphs_disabled") == 0
        assert core.info("graph_captures") == 2 and core.info("graph_replays") == 6     # one graph per direction, 3 replays each
        # a different sequence length is a different graph; the old ones stay usable
        y2, _, _ = core.forward(x[:T - 2].contiguous(), h0, c0)
        assert torch.equal(y2, y_ref[:T - 2]) and core.info("graph_captures") == 3
        y3, _, _ = core.forward(x, h0, c0)
        assert torch.equal(y3, y_ref) and core.info("graph_captures") == 3
        plain.close(); core.close()
    ref, _ = oracle_reference(p, state_grads=False)
    check_against(ref, dict(y=to_np(y_ref), hn=to_np(hy_ref), cn=to_np(cy_ref), dx=to_np(g_ref[0]), dw_ih=to_np(g_ref[1]),
                            dw_hh=to_np(g_ref[2]), db=to_np(g_ref[3]), dh0=to_np(g_ref[4]), dc0=to_np(g_ref[5])))


def test_projection_chunk_size_does_not_change_results():
    p = make_problem(17, 6, 48, 40, seed=9)
    base, _ = run_core(p, proj_chunk=0)
    for chunk in (-1, 1, 2, 5, 17, 64):
        got, _ = run_core(p, proj_chunk=chunk)
        for k in ("y", "cn", "dx", "dw_ih"):
            np.testing.assert_array_equal(got[k], base[k], err_msg=f"chunk {chunk} {k}")


def test_handle_reuse_with_shorter_and_longer_sequences():
    # the reference re-runs one handle with T/2 and T+1 (python/test_lstm.py:186-271)
    from flashlstm_poc_amd import LstmCore
    T, B, I, H = 12, 3, 20, 24
    p = make_problem(T + 1, B, I, H, seed=21)
    core = LstmCore(B, I, H)
    core.pack(*(p[k].cuda() for k in ("w_ih", "w_hh", "b_ih", "b_hh")))
    for t in (T, T // 2, T + 1, 1):
        ref, _ = oracle_reference(p, T=t)
        got, _ = run_core(p, T=t, core=core)
        check_against(ref, got, label=f"T={t}")
    core.close()


def test_missing_state_gradients_equal_zero_state_gradients():
    p = make_problem(6, 4, 10, 12, seed=4)
    a, _ = run_core(p, state_grads=False)
    q = dict(p); q["d_hn"] = torch.zeros_like(p["d_hn"]); q["d_cn"] = torch.zeros_like(p["d_cn"])
    b, _ = run_core(q, state_grads=True)
    for k in a:
        np.testing.assert_array_equal(a[k], b[k], err_msg=k)
    ref, _ = oracle_reference(p, state_grads=False)
    check_against(ref, a)


def test_grad_scale_rescues_tiny_upstream_gradients():
    # dY ~ 1e-7 underflows fp16 pre-activation gradients unless scaled (power of two => exact otherwise)
    p = make_problem(8, 4, 16, 32, seed=5, fp16_values=False)
    p["dy"] = p["dy"] * 1e-7; p["d_hn"] = p["d_hn"] * 0; p["d_cn"] = p["d_cn"] * 0
    ref, _ = oracle_reference(p)
    got, _ = run_core(p, half=False, grad_scale=2.0 ** 20)
    check_against(ref, got, label="scaled")
    unscaled, _ = run_core(p, half=False, grad_scale=1.0)
    assert rell2(unscaled["dx"], ref["dx"]) > 1e-2   # the unscaled run really loses the gradient


def test_zero_recurrent_weights_and_zero_input_special_cases():
    p = make_problem(5, 3, 8, 16, seed=6)
    p["w_hh"] = torch.zeros_like(p["w_hh"])
    ref, _ = oracle_reference(p)
    got, _ = run_core(p)
    check_against(ref, got, label="W_hh=0")
    assert np.abs(got["dw_hh"] - ref["dw_hh"]).max() <= 1e-2 * np.abs(ref["dw_hh"]).max()
    q = make_problem(5, 3, 8, 16, seed=6)
    for k in ("x", "h0", "c0", "b_ih", "b_hh"):
        q[k] = torch.zeros_like(q[k])
    got, _ = run_core(q)
    assert np.all(got["y"] == 0) and np.all(got["cn"] == 0)


def test_gate_cache_and_state_arrays_hold_what_the_oracle_computes():
    import ctypes
    from flashlstm_poc_amd import LstmCore
    T, B, I, H = 6, 5, 12, 40
    p = make_problem(T, B, I, H, seed=8)
    _, f = oracle_reference(p)
    core = LstmCore(B, I, H)
    core.pack(*(p[k].cuda() for k in ("w_ih", "w_hh", "b_ih", "b_hh")))
    core.forward(p["x"].cuda().half(), p["h0"].cuda().half(), p["c0"].cuda().half())
    Hp = core.info("hidden_padded")

    def view(which, rows, cols, dtype):
        ptr, ld = ctypes.c_void_p(), ctypes.c_size_t()
        assert core.lib.flstm_core_cache_ptr(core._h, which, ctypes.byref(ptr), ctypes.byref(ld)) == 0
        t = torch.empty((rows, ld.value), dtype=dtype, device="cuda")
        nbytes = t.numel() * t.element_size()
        assert ctypes.CDLL("libamdhip64.so").hipMemcpy(ctypes.c_void_p(t.data_ptr()), ptr, ctypes.c_size_t(nbytes), 3) == 0
        return to_np(t)[:, :cols]

    h_all = view(0, (T + 1) * B, Hp, torch.float16).reshape(T + 1, B, Hp)[..., :H]
    c_all = view(1, (T + 1) * B, Hp, torch.float32).reshape(T + 1, B, Hp)[..., :H]
    gates = view(2, T * B, 4 * Hp, torch.float16).reshape(T, B, 4 * Hp)
    assert relmax(h_all, f["h_all"]) <= 1e-2 and relmax(c_all, f["c_all"]) <= 1e-2
    np.testing.assert_array_equal(h_all[0], to_np(p["h0"]))          # entry 0 is the initial state
    # packed gate order: unit j, gate g sits at column 4 * j + g
    j = np.arange(H)
    for g in range(4):
        cols = 4 * j + g
        assert relmax(gates[..., cols], f["gates"][..., g * H:(g + 1) * H]) <= 1e-2
    assert gates.min() >= -1.0 and gates.max() <= 1.0
    core.close()


@pytest.mark.parametrize("shape,cuts", [((23, 5, 12, 20), (7, 15)), ((96, 40, 64, 256), (32, 64)), ((40, 64, 128, 1024), (24,))])
def test_sequence_in_segments_equals_the_whole_sequence(shape, cuts):
    # A sequence run as consecutive segments: forward carries (h, c) from one segment to the next in fp32,
    # backward runs the segments last to first, feeds each segment's dh0 / dc0 to the next call as d_hn / d_cn
    # and adds the parameter gradients up ("accumulate_grads").  Every state and dx must come out bit-identical
    # to the single pass; dW and db are sums in another order.
    from flashlstm_poc_amd import LstmCore
    p = make_problem(*shape, seed=21)
    T, B, I, H = shape
    whole, _ = run_core(p)
    core = LstmCore(B, I, H)
    core.pack(*(p[k].cuda() for k in ("w_ih", "w_hh", "b_ih", "b_hh")))
    x, dy = p["x"].cuda().half(), p["dy"].cuda().half()
    bounds = [0, *cuts, T]
    segs = list(zip(bounds[:-1], bounds[1:]))
    h, c = p["h0"].cuda().float(), p["c0"].cuda().float()
    starts, ys = [], []
    for a, b in segs:
        starts.append((h, c))
        y, hy, cy = core.forward(x[a:b], h, c, out_dtype=torch.float32)
        ys.append(y)
        h, c = hy, cy
    np.testing.assert_array_equal(to_np(torch.cat(ys).half()), whole["y"])
    np.testing.assert_array_equal(to_np(h.half()), whole["hn"])
    assert relmax(to_np(c), whole["cn"]) < 1e-3   # the single pass returned c_T rounded to fp16
    acc = (torch.zeros(4 * H, I, device="cuda"), torch.zeros(4 * H, H, device="cuda"), torch.zeros(4 * H, device="cuda"))
    dh, dc = p["d_hn"].cuda().float(), p["d_cn"].cuda().float()
    dxs = []
    for (a, b), (h_in, c_in) in reversed(list(zip(segs, starts))):
        core.forward(x[a:b], h_in, c_in, want_y=False)   # rebuild this segment's caches
        dx, _, _, _, dh, dc = core.backward(x[a:b], dy[a:b], dh, dc, accumulate_into=acc)
        dxs.insert(0, dx)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(to_np(torch.cat(dxs)), whole["dx"])
    np.testing.assert_array_equal(to_np(dh), whole["dh0"])
    np.testing.assert_array_equal(to_np(dc), whole["dc0"])
    for got, name in zip(acc, ("dw_ih", "dw_hh", "db")):
        assert rell2(to_np(got), whole[name]) < 1e-5, name
    core.close()


def test_error_codes():
    from flashlstm_poc_amd import LstmCore
    core = LstmCore(2, 3, 5)
    x = torch.zeros(4, 2, 3, device="cuda", dtype=torch.float16)
    with pytest.raises(RuntimeError, match="2001"):     # forward before packing
        core.forward(x)
    w = make_problem(4, 2, 3, 5)
    core.pack(*(w[k].cuda() for k in ("w_ih", "w_hh", "b_ih", "b_hh")))
    with pytest.raises(RuntimeError, match="2002"):     # backward without forward
        core.backward(x, torch.zeros(4, 2, 5, device="cuda", dtype=torch.float16))
    core.forward(x, save_for_backward=False)
    with pytest.raises(RuntimeError, match="2002"):
        core.backward(x, torch.zeros(4, 2, 5, device="cuda", dtype=torch.float16))
    core.forward(x)
    with pytest.raises(RuntimeError, match="2002"):     # sequence length differs from the cached forward
        core.backward(x[:3], torch.zeros(3, 2, 5, device="cuda", dtype=torch.float16))
    with pytest.raises(ValueError):
        core.set_option("no_such_option", 1)
    with pytest.raises(ValueError):
        core.forward(torch.zeros(4, 3, 3, device="cuda", dtype=torch.float16))
    core.close()


@pytest.mark.parametrize("shape", [(9, 40, 20, 96), (6, 33, 7, 9), (12, 300, 64, 256), (5, 70, 65, 1000), (8, 520, 32, 512)])
def test_eight_wave_forward_kernel_on_ragged_shapes_ranges_and_single_steps(shape):
    # The forward kernel with eight waves per workgroup and two interleaved row tiles (option "waves_fwd" = 8: the plan
    # picks it by itself only where every workgroup has one 32-row block) on shapes it would not be chosen for --
    # ragged batches and hidden sizes, batches of several row blocks per workgroup -- against the oracle, persistent,
    # one launch per step, and fed in ranges of steps; its weights are packed for eight waves, so the option un-packs.
    from flashlstm_poc_amd import LstmCore, load_library
    p = make_problem(*shape, seed=77)
    T, B, I, H = shape
    ref, _ = oracle_reference(p)
    core = LstmCore(B, I, H)
    core.pack(*(p[k].cuda() for k in ("w_ih", "w_hh", "b_ih", "b_hh")))
    core.set_option("waves_fwd", 8)
    assert core.info("waves_fwd") == 8 and core.info("row_tiles_fwd") == 2
    x, h0, c0 = p["x"].cuda().half(), p["h0"].cuda().half(), p["c0"].cuda().half()
    with pytest.raises(RuntimeError):
        core.forward(x, h0, c0)          # the weight fragments were packed for four waves
    core.pack(*(p[k].cuda() for k in ("w_ih", "w_hh", "b_ih", "b_hh")))
    got, info = run_core(p, core=core)
    assert info["persistent_fwd"] == 1 and info["fallbacks"] == 0
    check_against(ref, got, label=f"eight waves {shape}")
    y_p = torch.from_numpy(got["y"])
    got_s, info_s = run_core(p, core=core, stepwise=True)
    assert info_s["persistent_fwd"] == 0
    assert np.array_equal(got_s["y"], got["y"]) and np.array_equal(got_s["cn"], got["cn"])   # same kernel, one step per launch
    core.set_option("stepwise", 0)
    # ranges of steps through the C ABI: [0, a), [a, b), [b, T)
    lib = load_library()
    s = torch.cuda.current_stream().cuda_stream
    hy = torch.empty(B, H, device="cuda", dtype=torch.float16); cy = torch.empty_like(hy)
    assert lib.flstm_core_forward_begin(core._h, T, x.data_ptr(), 1, h0.data_ptr(), c0.data_ptr(), 1, s) == 0
    cuts = sorted({0, max(1, T // 3), max(2, (2 * T) // 3), T})
    for a, b in zip(cuts[:-1], cuts[1:]):
        assert lib.flstm_core_forward_steps(core._h, a, b - a, s) == 0
    assert lib.flstm_core_forward_end(core._h, hy.data_ptr(), cy.data_ptr(), 1, 1, s) == 0
    torch.cuda.synchronize()
    assert np.array_equal(to_np(hy), got["hn"]) and np.array_equal(to_np(cy), got["cn"])
    core.close()


def test_eight_wave_forward_kernel_is_the_rule_where_every_workgroup_has_one_32_row_block():
    from flashlstm_poc_amd import LstmCore
    for (B, H, want) in ((256, 1024, 8), (128, 1024, 4), (512, 1024, 4), (512, 512, 8), (256, 2048, 4), (160, 768, 8)):
        core = LstmCore(B, 64, H)
        assert core.info("waves_fwd") == want, (B, H, core.info("waves_fwd"))
        core.close()
