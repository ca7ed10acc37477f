"""The stacked-layer driver (flashlstm_poc_amd.LstmStack) against torch.nn.LSTM(num_layers=L) on the GPU: the loop
a multi-layer workload (BASELINE config 5: 4 layers, MSE on the top layer's outputs) puts around the single-layer
path, which is all the reference has (flashlstm_v2/python/flashlstm/streaming_lstm.py:380).  Tolerances: max
relative error <= 1e-2 on outputs, relative L2 <= 1e-2 on every gradient."""
import pytest
import torch

from helpers import SafeTorchLstm, rell2, relmax, to_np

pytestmark = pytest.mark.gpu


def _run(T, B, I, H, L, loss_scale, seed=5, safe_reference=False, max_rows=131072, mse_helper=False):
    """Our stack first (forward, MSE gradient, backward), then -- after its device memory has been given back -- the
    fp32 reference on the same inputs: nn.LSTM(num_layers=L) itself, or (safe_reference) the same function built
    from nn.LSTM calls of bounded size, helpers.SafeTorchLstm.  Returns the error of every output and gradient."""
    from flashlstm_poc_amd import LstmStack
    torch.manual_seed(seed)
    ref = torch.nn.LSTM(I, H, num_layers=L, device="cuda")
    with torch.no_grad():   # the kernels see fp16 weights: give the reference the same values
        for name, prm in ref.named_parameters():
            if name.startswith("weight"):
                prm.copy_(prm.half().float())
    x = torch.randn(T, B, I, device="cuda").half()
    target = torch.randn(T, B, H, device="cuda")
    if mse_helper:
        target = target.half().float()   # the helper takes an fp16 target: give the reference the same values
    stack = LstmStack(B, I, H, L)
    stack.pack([tuple(getattr(ref, f"{n}_l{l}").detach() for n in ("weight_ih", "weight_hh", "bias_ih", "bias_hh"))
                for l in range(L)])
    y, hys, cys = stack.forward(x)
    # MSE(y_top, target): d loss / d y = 2 (y - target) / numel
    if mse_helper:   # the same gradient handed over as fp16 difference and factor 2 / numel
        dx, grads, dh0s, dc0s = stack.backward_mse(y, target.half(), loss_scale=loss_scale)
    else:
        dy = 2.0 * (y.float() - target) / y.numel()
        dx, grads, dh0s, dc0s = stack.backward(dy, loss_scale=loss_scale)
        del dy
    stack.close()
    torch.cuda.empty_cache()

    xr = x.float().requires_grad_(True)
    if safe_reference:
        safe = SafeTorchLstm([tuple(getattr(ref, f"{n}_l{l}").detach() for n in ("weight_ih", "weight_hh", "bias_ih", "bias_hh"))
                              for l in range(L)], max_rows=max_rows)
        grad_of = lambda name, l: safe.grads(l)[("weight_ih", "weight_hh", "bias_ih").index(name)]
        yr, hn, cn = safe(xr)
    else:
        grad_of = lambda name, l: getattr(ref, f"{name}_l{l}").grad
        yr, (hn, cn) = ref(xr)
    errs = {"y": relmax_t(y, yr), "y_last_step": relmax_t(y[-1], yr[-1])}
    for l in range(L):
        errs[f"h_T{l}"] = relmax_t(hys[l], hn[l])
        errs[f"c_T{l}"] = relmax_t(cys[l], cn[l])
    loss = torch.nn.functional.mse_loss(yr, target)
    loss.backward()
    errs["dx"] = rell2_t(dx, xr.grad)
    for l in range(L):
        dW_ih, dW_hh, db = grads[l]
        errs[f"dW_ih{l}"] = rell2_t(dW_ih, grad_of("weight_ih", l))
        errs[f"dW_hh{l}"] = rell2_t(dW_hh, grad_of("weight_hh", l))
        errs[f"db{l}"] = rell2_t(db, grad_of("bias_ih", l))
    return errs


def relmax_t(a, b):   # on the GPU: the full-size tensors are too large to move to numpy for a norm
    return ((a.float() - b.float()).abs().max() / b.float().abs().max()).item()


def rell2_t(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


def test_safe_reference_is_the_multilayer_lstm():
    # the reference used at full size equals nn.LSTM(num_layers=L), outputs and gradients, where both are sound;
    # max_rows=20 forces three time segments per layer on this 12-step problem
    a = _run(12, 5, 16, 24, 3, loss_scale=2.0 ** 12)
    b = _run(12, 5, 16, 24, 3, loss_scale=2.0 ** 12, safe_reference=True, max_rows=20)
    for k in a:
        assert abs(a[k] - b[k]) <= 2e-4, (k, a[k], b[k])


@pytest.mark.parametrize("shape", [(12, 5, 16, 24, 3), (20, 33, 48, 64, 4)])
def test_stack_matches_multilayer_torch_lstm_with_loss_scale(shape):
    # the MSE gradient is ~1e-4 per element and smaller after each layer: without a loss scale it falls out of fp16
    errs = _run(*shape, loss_scale=2.0 ** 12)
    assert max(errs.values()) <= 1e-2, errs


def test_loss_scale_is_what_keeps_small_gradients():
    errs = _run(12, 5, 16, 24, 3, loss_scale=1.0)
    scaled = _run(12, 5, 16, 24, 3, loss_scale=2.0 ** 12)
    auto = _run(12, 5, 16, 24, 3, loss_scale="auto")
    assert max(scaled.values()) <= 1e-2 and max(auto.values()) <= 1e-2
    assert max(errs.values()) > max(scaled.values())   # unscaled: fp16 underflow costs accuracy


def test_mse_helper_gives_the_gradients_of_the_mse_loss():
    a = _run(12, 5, 16, 24, 3, loss_scale="auto", mse_helper=True)
    b = _run(33, 40, 64, 256, 2, loss_scale="auto", mse_helper=True)
    assert max(a.values()) <= 1e-2 and max(b.values()) <= 1e-2, (a, b)


def test_config5_stack_full_size_against_fp32_torch_lstm():
    # BASELINE config 5 as written: 4 layers, I = 512, H = 2048, B = 128, T = 4096, MSE on the top layer's outputs
    # against seeded N(0,1) targets; the reference for every output and all 13 gradients is fp32
    # nn.LSTM on the same GPU with the same fp16-rounded weights, called in pieces of at most 131072 rows
    # (helpers.SafeTorchLstm says why).
    # The automatic loss scale is part of what is tested: d MSE / d y is ~2e-9 per element here.
    errs = _run(4096, 128, 512, 2048, 4, loss_scale="auto", seed=7, safe_reference=True)
    print("\nconfig5 stack: " + ", ".join(f"{k}={v:.2e}" for k, v in errs.items()))
    assert max(errs.values()) <= 1e-2, errs


def test_stacked_module_trains_like_torch_lstm():
    # StackedLSTM as an nn.Module under autograd, the way the reference's pytest drives its single-layer module
    # (flashlstm_v2/python/tests/test_streaming_lstm.py:15-64): same state_dict as nn.LSTM(num_layers=2), loss on
    # y, h_n and c_n, gradients of x, h0, c0 and every parameter.
    from flashlstm_poc_amd import StackedLSTM
    T, B, I, H, L = 10, 6, 20, 32, 2
    torch.manual_seed(1234)
    ref = torch.nn.LSTM(I, H, num_layers=L, device="cuda")
    mod = StackedLSTM(I, H, L, output_dtype=torch.float32)
    with torch.no_grad():
        for name, prm in ref.named_parameters():
            if name.startswith("weight"):
                prm.copy_(prm.half().float())
    mod.load_state_dict(ref.state_dict())       # same parameter names and layouts
    x = torch.randn(T, B, I, device="cuda").half()
    h0 = (torch.randn(L, B, H, device="cuda") * 0.3).half()
    c0 = (torch.randn(L, B, H, device="cuda") * 0.3).half()
    xa, ha, ca = (t.clone().requires_grad_(True) for t in (x, h0, c0))
    xb, hb, cb = (t.float().clone().requires_grad_(True) for t in (x, h0, c0))
    ya, (hna, cna) = mod(xa, (ha, ca))
    yb, (hnb, cnb) = ref(xb, (hb, cb))
    assert ya.dtype == torch.float32 and relmax(to_np(ya), to_np(yb)) <= 1e-2
    assert relmax(to_np(hna), to_np(hnb)) <= 1e-2 and relmax(to_np(cna), to_np(cnb)) <= 1e-2
    loss = lambda y, hn, cn: (y.float() ** 2).mean() + (hn.float() ** 2).mean() + (cn.float() ** 2).mean()
    loss(ya, hna, cna).backward()
    loss(yb, hnb, cnb).backward()
    assert rell2(to_np(xa.grad), to_np(xb.grad)) <= 1e-2 and xa.grad.dtype == torch.float16
    assert rell2(to_np(ha.grad), to_np(hb.grad)) <= 1e-2 and rell2(to_np(ca.grad), to_np(cb.grad)) <= 1e-2
    for name, prm in ref.named_parameters():
        got = getattr(mod, name).grad
        assert got is not None and rell2(to_np(got), to_np(prm.grad)) <= 1e-2, name
    # one optimiser step on both, then a second forward/backward: repacking follows the updated weights
    with torch.no_grad():
        for name, prm in ref.named_parameters():
            prm -= 0.1 * prm.grad
            getattr(mod, name).copy_(prm)
    ya2, _ = mod(x)
    yb2, _ = ref(x.float())
    assert relmax(to_np(ya2), to_np(yb2)) <= 1e-2
    # the caches belong to the latest forward pass only
    y_old, _ = mod(xa)
    mod(xa)
    with pytest.raises(RuntimeError, match="most recent forward"):
        y_old.sum().backward()
    mod.release()
