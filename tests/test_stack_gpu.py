"""The stacked-layer driver (flashlstm_poc_amd.LstmStack) against torch.nn.LSTM(num_layers=L) on the GPU: the loop
a multi-layer workload (BASELINE config 5: 4 layers, MSE on the top layer's outputs) puts around the single-layer
path, which is all the reference has (flashlstm_v2/python/flashlstm/streaming_lstm.py:380).  Tolerances: max
relative error <= 1e-2 on outputs, relative L2 <= 1e-2 on every gradient."""
import pytest
import torch

from helpers import rell2, relmax, to_np

pytestmark = pytest.mark.gpu


def _run(T, B, I, H, L, loss_scale):
    from flashlstm_poc_amd import LstmStack
    torch.manual_seed(5)
    ref = torch.nn.LSTM(I, H, num_layers=L, device="cuda")
    with torch.no_grad():   # the kernels see fp16 weights: give the reference the same values
        for name, prm in ref.named_parameters():
            if name.startswith("weight"):
                prm.copy_(prm.half().float())
    x = torch.randn(T, B, I, device="cuda").half()
    target = torch.randn(T, B, H, device="cuda")
    stack = LstmStack(B, I, H, L)
    stack.pack([tuple(getattr(ref, f"{n}_l{l}").detach() for n in ("weight_ih", "weight_hh", "bias_ih", "bias_hh"))
                for l in range(L)])
    y, hys, cys = stack.forward(x)
    xr = x.float().requires_grad_(True)
    yr, (hn, cn) = ref(xr)
    assert relmax(to_np(y), to_np(yr)) <= 1e-2
    for l in range(L):
        assert relmax(to_np(hys[l]), to_np(hn[l])) <= 1e-2 and relmax(to_np(cys[l]), to_np(cn[l])) <= 1e-2
    # MSE(y_top, target): d loss / d y = 2 (y - target) / numel
    loss = torch.nn.functional.mse_loss(yr, target)
    loss.backward()
    dy = 2.0 * (y.float() - target) / y.numel()
    dx, grads, dh0s, dc0s = stack.backward(dy, loss_scale=loss_scale)
    errs = {"dx": rell2(to_np(dx), to_np(xr.grad))}
    for l in range(L):
        dW_ih, dW_hh, db = grads[l]
        errs[f"dW_ih{l}"] = rell2(to_np(dW_ih), to_np(getattr(ref, f"weight_ih_l{l}").grad))
        errs[f"dW_hh{l}"] = rell2(to_np(dW_hh), to_np(getattr(ref, f"weight_hh_l{l}").grad))
        errs[f"db{l}"] = rell2(to_np(db), to_np(getattr(ref, f"bias_ih_l{l}").grad))
    stack.close()
    return errs


@pytest.mark.parametrize("shape", [(12, 5, 16, 24, 3), (20, 33, 48, 64, 4)])
def test_stack_matches_multilayer_torch_lstm_with_loss_scale(shape):
    # the MSE gradient is ~1e-4 per element and smaller after each layer: without a loss scale it falls out of fp16
    errs = _run(*shape, loss_scale=2.0 ** 12)
    assert max(errs.values()) <= 1e-2, errs


def test_loss_scale_is_what_keeps_small_gradients():
    errs = _run(12, 5, 16, 24, 3, loss_scale=1.0)
    scaled = _run(12, 5, 16, 24, 3, loss_scale=2.0 ** 12)
    assert max(scaled.values()) <= 1e-2
    assert max(errs.values()) > max(scaled.values())   # unscaled: fp16 underflow costs accuracy
