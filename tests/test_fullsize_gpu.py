"""BASELINE-sized runs (I = H = 1024) checked through properties that do not need a CPU oracle run:
prefix consistency, batch-row independence, linearity of BPTT in the upstream gradient, persistent vs
step-wise agreement -- plus a direct comparison with torch.nn.LSTM on the GPU at a reduced length."""
import numpy as np
import pytest
import torch

from helpers import rell2, relmax, to_np

pytestmark = pytest.mark.gpu


def problem(T, B, I, H, seed=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    k = 1.0 / H ** 0.5
    u = lambda *s: (torch.rand(*s, generator=g, device="cuda") * 2 - 1) * k
    n = lambda *s: torch.randn(*s, generator=g, device="cuda")
    return dict(w_ih=u(4 * H, I), w_hh=u(4 * H, H), b_ih=u(4 * H), b_hh=u(4 * H), x=n(T, B, I).half(),
                h0=(n(B, H) * 0.1).half(), c0=(n(B, H) * 0.1).half(), dy=n(T, B, H).half())


def make_core(p):
    from flashlstm_poc_amd import LstmCore
    T, B, I = p["x"].shape
    core = LstmCore(B, I, p["w_hh"].shape[1])
    core.pack(p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"])
    return core


def test_config2_forward_prefix_and_batch_independence():
    # forward only, I = H = 1024, B = 64, T = 512
    p = problem(512, 64, 1024, 1024, seed=1)
    core = make_core(p)
    y, hy, cy = core.forward(p["x"], p["h0"], p["c0"], save_for_backward=False)
    assert core.info("persistent_fwd") == 1 and core.info("xcd_local_fwd") == 1 and core.info("fallbacks") == 0
    assert torch.isfinite(y.float()).all() and y.abs().max() <= 1.0
    assert torch.equal(y[-1], hy)
    y_half, hy_half, cy_half = core.forward(p["x"][:256], p["h0"], p["c0"], save_for_backward=False)
    assert torch.equal(y_half, y[:256])                       # causality: a prefix is a prefix
    y_rest, hy2, cy2 = core.forward(p["x"][256:], hy_half, cy_half, save_for_backward=False)
    assert relmax(to_np(y_rest), to_np(y[256:])) <= 2e-3      # restart from (h, c): c passes through fp16 here
    perm = torch.randperm(64, device="cuda")
    y_perm, _, _ = core.forward(p["x"][:, perm].contiguous(), p["h0"][perm].contiguous(), p["c0"][perm].contiguous(),
                                save_for_backward=False)
    assert torch.equal(y_perm, y[:, perm])                    # rows never mix
    core.close()


def test_config3_backward_linearity_and_mode_agreement():
    # forward + backward with the fp16 gate cache, I = H = 1024, B = 256; T reduced to 128 to bound memory/time
    p = problem(128, 256, 1024, 1024, seed=2)
    core = make_core(p)
    core.forward(p["x"], p["h0"], p["c0"])
    a = core.backward(p["x"], p["dy"])
    b = core.backward(p["x"], (2 * p["dy"].float()).half())    # BPTT is linear in dY; doubling is exact in fp16
    for ga, gb, name in zip(a, b, ("dx", "dW_ih", "dW_hh", "db", "dh0", "dc0")):
        assert rell2(to_np(gb), 2 * to_np(ga)) <= 1e-3, name
    c = core.backward(p["x"], p["dy"], grad_scale=4.0)         # a power-of-two loss scale changes nothing
    for ga, gc, name in zip(a, c, ("dx", "dW_ih", "dW_hh", "db", "dh0", "dc0")):
        assert rell2(to_np(gc), to_np(ga)) <= 1e-3, name
    assert core.info("persistent_bwd") == 1 and core.info("fallbacks") == 0
    core.set_option("stepwise", 1)
    y2, _, _ = core.forward(p["x"], p["h0"], p["c0"])
    d = core.backward(p["x"], p["dy"])
    for ga, gd, name in zip(a, d, ("dx", "dW_ih", "dW_hh", "db", "dh0", "dc0")):
        assert rell2(to_np(gd), to_np(ga)) <= 1e-4, name
    core.close()


@pytest.mark.parametrize("shape", [(64, 256, 1024, 1024), (48, 16, 2048, 2048), (24, 128, 512, 2048)])
def test_headline_shapes_against_torch_lstm_on_gpu(shape):
    # configs 3, 4 and 5 (one layer) at reduced T, against fp32 nn.LSTM on the fp16-rounded operands
    T, B, I, H = shape
    p = problem(T, B, I, H, seed=3)
    core = make_core(p)
    y, hy, cy = core.forward(p["x"], p["h0"], p["c0"])
    dx, dW_ih, dW_hh, db, dh0, dc0 = core.backward(p["x"], p["dy"])
    m = torch.nn.LSTM(I, H, device="cuda")
    with torch.no_grad():
        m.weight_ih_l0.copy_(p["w_ih"].half().float()); m.weight_hh_l0.copy_(p["w_hh"].half().float())
        m.bias_ih_l0.copy_(p["b_ih"]); m.bias_hh_l0.copy_(p["b_hh"])
    xr = p["x"].float().requires_grad_(True)
    hr = p["h0"].float().requires_grad_(True); cr = p["c0"].float().requires_grad_(True)
    yr, (hn, cn) = m(xr, (hr[None], cr[None]))
    (yr * p["dy"].float()).sum().backward()
    assert relmax(to_np(y), to_np(yr)) <= 1e-2 and relmax(to_np(hy), to_np(hn[0])) <= 1e-2
    assert relmax(to_np(cy), to_np(cn[0])) <= 1e-2
    for got, ref, name in ((dx, xr.grad, "dx"), (dW_ih, m.weight_ih_l0.grad, "dW_ih"), (dW_hh, m.weight_hh_l0.grad, "dW_hh"),
                           (db, m.bias_ih_l0.grad, "db"), (dh0, hr.grad, "dh0"), (dc0, cr.grad, "dc0")):
        assert rell2(to_np(got), to_np(ref)) <= 1e-2, name
    core.close()


def _torch_lstm_reference(p, with_grads=True):
    """fp32 nn.LSTM on the GPU with the fp16-rounded weights, called the safe way (helpers.SafeTorchLstm)."""
    from helpers import SafeTorchLstm
    m = SafeTorchLstm([(p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"])])
    xr = p["x"].float().requires_grad_(with_grads)
    hr = p["h0"].float().requires_grad_(with_grads); cr = p["c0"].float().requires_grad_(with_grads)
    yr, hn, cn = m(xr, [hr], [cr])
    grads = None
    if with_grads:
        (yr * p["dy"].float()).sum().backward()
        dW_ih, dW_hh, db = m.grads(0)
        grads = dict(dx=xr.grad, dW_ih=dW_ih, dW_hh=dW_hh, db=db, dh0=hr.grad, dc0=cr.grad)
    return yr.detach(), hn[0].detach(), cn[0].detach(), grads


def _gpu_relmax(a, b):
    return ((a.float() - b.float()).abs().max() / b.float().abs().max()).item()


def _gpu_rell2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


@pytest.mark.parametrize("name,shape,backward", [("config2", (512, 64, 1024, 1024), False),
                                                 ("config3", (1024, 256, 1024, 1024), True),
                                                 ("config4", (2048, 16, 2048, 2048), True)])
def test_full_length_configs_against_fp32_torch_lstm(name, shape, backward):
    # The BASELINE configurations at their FULL sequence length against fp32 nn.LSTM on the GPU, same fp16-rounded
    # operands: max relative error <= 1e-2 on y / h_T / c_T, relative L2 <= 1e-2 on every gradient.  The error of
    # the LAST step is reported beside the maximum: h is fed back through fp16 at every step, and this is where a
    # growth of that error over 1024 / 2048 steps would show.
    T, B, I, H = shape
    p = problem(T, B, I, H, seed=11)
    core = make_core(p)
    y, hy, cy = core.forward(p["x"], p["h0"], p["c0"], save_for_backward=backward)
    got = core.backward(p["x"], p["dy"]) if backward else None
    assert core.info("persistent_fwd") == 1 and core.info("fallbacks") == 0
    yr, hn, cn, gr = _torch_lstm_reference(p, with_grads=backward)
    errs = {"y_max": _gpu_relmax(y, yr), "y_last_step": _gpu_relmax(y[-1], yr[-1]), "y_first_step": _gpu_relmax(y[0], yr[0]),
            "h_T": _gpu_relmax(hy, hn), "c_T": _gpu_relmax(cy, cn)}
    if backward:
        for k, t in zip(("dx", "dW_ih", "dW_hh", "db", "dh0", "dc0"), got):
            errs[k] = _gpu_rell2(t, gr[k])
        # gradient of the FIRST time step's input: the end of the backward chain
        errs["dx_first_step"] = _gpu_rell2(got[0][0], gr["dx"][0])
    print(f"\n{name} T={T} B={B} I={I} H={H}: " + ", ".join(f"{k}={v:.2e}" for k, v in errs.items()))
    assert max(errs.values()) <= 1e-2, errs
    core.close()


def _cpu_lstm_reference(p):
    """fp32 torch.nn.LSTM on the host CPU -- the oracle the reference's own test uses (python/test_lstm.py:99-104) --
    with the fp16-rounded weights and inputs the kernels see; forward and autograd for the loss sum(y * dY)."""
    T, B, I = p["x"].shape
    H = p["w_hh"].shape[1]
    m = torch.nn.LSTM(I, H)
    with torch.no_grad():
        m.weight_ih_l0.copy_(p["w_ih"].half().float().cpu()); m.weight_hh_l0.copy_(p["w_hh"].half().float().cpu())
        m.bias_ih_l0.copy_(p["b_ih"].cpu()); m.bias_hh_l0.copy_(p["b_hh"].cpu())
    xr = p["x"].float().cpu().requires_grad_(True)
    hr = p["h0"].float().cpu().requires_grad_(True); cr = p["c0"].float().cpu().requires_grad_(True)
    yr, (hn, cn) = m(xr, (hr[None], cr[None]))
    (yr * p["dy"].float().cpu()).sum().backward()
    return dict(y=yr.detach(), h_T=hn[0].detach(), c_T=cn[0].detach(), dx=xr.grad, dW_ih=m.weight_ih_l0.grad,
                dW_hh=m.weight_hh_l0.grad, db=m.bias_ih_l0.grad, db_hh=m.bias_hh_l0.grad, dh0=hr.grad, dc0=cr.grad)


@pytest.mark.parametrize("name,shape", [("config3", (1024, 256, 1024, 1024)), ("config4", (2048, 16, 2048, 2048)),
                                        ("config5_layer", (4096, 128, 2048, 2048))])
def test_full_size_configs_against_cpu_fp32_torch_lstm(name, shape):
    # The headline configurations and one full layer of the stack at FULL size against torch.nn.LSTM in fp32 on the
    # CPU: all of y, h_T, c_T (max relative error <= 1e-2) and dx, dW_ih, dW_hh, db, dh0, dc0 (relative L2 <= 1e-2).
    # The GPU library's nn.LSTM is not involved; the errors are printed.
    import time
    T, B, I, H = shape
    p = problem(T, B, I, H, seed=17)
    core = make_core(p)
    y, hy, cy = core.forward(p["x"], p["h0"], p["c0"])
    got = dict(zip(("dx", "dW_ih", "dW_hh", "db", "dh0", "dc0"), core.backward(p["x"], p["dy"])))
    got.update(y=y, h_T=hy, c_T=cy)
    assert core.info("persistent_fwd") == 1 and core.info("persistent_bwd") == 1 and core.info("fallbacks") == 0
    got = {k: v.float().cpu() for k, v in got.items()}
    core.close()
    t0 = time.perf_counter()
    ref = _cpu_lstm_reference(p)
    cpu_s = time.perf_counter() - t0
    errs = {}
    for k in ("y", "h_T", "c_T"):
        errs[k] = ((got[k] - ref[k]).abs().max() / ref[k].abs().max()).item()
    errs["y_last_step"] = ((got["y"][-1] - ref["y"][-1]).abs().max() / ref["y"][-1].abs().max()).item()
    for k in ("dx", "dW_ih", "dW_hh", "db", "dh0", "dc0"):
        errs[k] = ((got[k].double() - ref[k].double()).norm() / ref[k].double().norm()).item()
    errs["db_vs_db_hh"] = ((got["db"].double() - ref["db_hh"].double()).norm() / ref["db_hh"].double().norm()).item()
    print(f"\n{name} T={T} B={B} I={I} H={H} vs CPU fp32 nn.LSTM ({cpu_s:.1f} s on {torch.get_num_threads()} threads): "
          + ", ".join(f"{k}={v:.2e}" for k, v in errs.items()))
    assert max(errs.values()) <= 1e-2, errs
