"""The `flashlstm` Python package (StreamingLSTM / streaming_lstm) against torch.nn.LSTM, written the way
the reference's flashlstm_v2/python/tests/test_streaming_lstm.py:14-89 tests it, plus the argument checks
of streaming_lstm.py:27-58,79-112."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _random_pinned_half(shape):
    t = torch.empty(shape, dtype=torch.float16, pin_memory=True)
    t.copy_(torch.randn(shape).half())
    return t


@pytest.mark.parametrize("shape,kw", [((4, 2, 3, 5), {}), ((9, 3, 16, 24), dict(recompute_interval=4, gate_cache_dtypes=(torch.float16, torch.float32)))])
def test_streaming_lstm_matches_torch_lstm(shape, kw):
    from flashlstm import StreamingLSTM
    T, B, I, H = shape
    torch.manual_seed(1234)
    module = StreamingLSTM(I, H)
    torch.manual_seed(1234)
    reference = torch.nn.LSTM(I, H, batch_first=False, device="cuda")
    # equal seeds give equal parameters (creation order weight_ih, weight_hh, bias_ih, bias_hh)
    torch.testing.assert_close(module.weight_ih, reference.weight_ih_l0)
    torch.testing.assert_close(module.bias_hh, reference.bias_hh_l0)

    x_host = _random_pinned_half((T, B, I)).contiguous()
    x_ref = x_host.to(device="cuda", dtype=torch.float32)
    h0 = torch.randn(B, H, device="cuda", dtype=torch.float16)
    c0 = torch.randn(B, H, device="cuda", dtype=torch.float16)

    y_host, cache, (hy, cy) = module(x_host, h0, c0, **kw)
    assert y_host.is_pinned() and y_host.dtype == torch.float16 and tuple(y_host.shape) == (T, B, H)
    R = kw.get("recompute_interval", 1)
    assert tuple(cache.h.shape) == ((T + R - 1) // R, B, H) and cache.h.is_pinned()
    assert cache.h.dtype == kw.get("gate_cache_dtypes", (torch.float32,) * 2)[0]
    assert not cache.h.requires_grad and not cache.c.requires_grad
    y = y_host.to(device="cuda", dtype=torch.float32)
    hy_f, cy_f = hy.float(), cy.float()
    y_ref, (hy_ref, cy_ref) = reference(x_ref, (h0.float()[None], c0.float()[None]))
    torch.testing.assert_close(y, y_ref, rtol=1e-3, atol=2e-3)
    torch.testing.assert_close(hy_f, hy_ref[0], rtol=1e-3, atol=2e-3)
    torch.testing.assert_close(cy_f, cy_ref[0], rtol=1e-3, atol=2e-3)

    (y.pow(2).mean() + hy_f.pow(2).mean() + cy_f.pow(2).mean()).backward()
    (y_ref.pow(2).mean() + hy_ref.pow(2).mean() + cy_ref.pow(2).mean()).backward()
    for mine, ref in ((module.weight_ih, reference.weight_ih_l0), (module.weight_hh, reference.weight_hh_l0),
                      (module.bias_ih, reference.bias_ih_l0), (module.bias_hh, reference.bias_hh_l0)):
        torch.testing.assert_close(mine.grad, ref.grad, rtol=1e-3, atol=5e-3)


def test_functional_form_gradients_for_inputs_and_states():
    from flashlstm import streaming_lstm
    T, B, I, H = 6, 2, 8, 12
    torch.manual_seed(0)
    lstm = torch.nn.LSTM(I, H, device="cuda")
    params = [p.detach().clone().requires_grad_(True) for p in (lstm.weight_ih_l0, lstm.weight_hh_l0, lstm.bias_ih_l0, lstm.bias_hh_l0)]
    x_host = _random_pinned_half((T, B, I)).requires_grad_(True)
    h0 = torch.randn(B, H, device="cuda", dtype=torch.float16, requires_grad=True)
    c0 = torch.randn(B, H, device="cuda", dtype=torch.float16, requires_grad=True)
    y_host, cache, hy, cy = streaming_lstm(x_host, h0, c0, *params)
    w = torch.randn(T, B, H)
    ((y_host.float() * w).sum() + hy.float().sum().cpu() + (2 * cy.float()).sum().cpu()).backward()
    assert x_host.grad.dtype == torch.float16 and x_host.grad.device.type == "cpu"
    assert h0.grad.dtype == torch.float16 and h0.grad.device.type == "cuda"

    xr = x_host.detach().cuda().float().requires_grad_(True)
    hr = h0.detach().float().requires_grad_(True); cr = c0.detach().float().requires_grad_(True)
    yr, (hn, cn) = lstm(xr, (hr[None], cr[None]))
    ((yr * w.cuda()).sum() + hn.sum() + 2 * cn.sum()).backward()
    rel = lambda a, b: ((a.float().cpu() - b.float().cpu()).norm() / b.float().norm().cpu()).item()
    assert rel(x_host.grad, xr.grad) <= 1e-2 and rel(h0.grad, hr.grad) <= 1e-2 and rel(c0.grad, cr.grad) <= 1e-2
    assert rel(params[0].grad, lstm.weight_ih_l0.grad) <= 1e-2 and rel(params[3].grad, lstm.bias_hh_l0.grad) <= 1e-2


def test_default_states_are_zero_and_argument_checks():
    from flashlstm import StreamingLSTM, streaming_lstm
    m = StreamingLSTM(4, 6)
    x = _random_pinned_half((3, 2, 4))
    y0, _, _ = m(x)
    z = torch.zeros(2, 6, device="cuda", dtype=torch.float16)
    y1, _, _ = m(x, z, z)
    assert torch.equal(y0, y1)
    with pytest.raises(ValueError, match="pinned"):
        m(torch.zeros(3, 2, 4, dtype=torch.float16))
    with pytest.raises(ValueError, match="CPU"):
        m(torch.zeros(3, 2, 4, dtype=torch.float16, device="cuda"))
    with pytest.raises(ValueError, match="float16"):
        m(x, torch.zeros(2, 6, device="cuda"), None)
    with pytest.raises(ValueError, match="CUDA"):
        m(x, torch.zeros(2, 6, dtype=torch.float16), None)
    with pytest.raises(ValueError, match="recompute_interval"):
        m(x, recompute_interval=0)
    with pytest.raises(ValueError, match="gate cache dtype"):
        m(x, gate_cache_dtypes=(torch.bfloat16, torch.float32))
    with pytest.raises(ValueError, match="weight_ih must have shape"):
        streaming_lstm(x, None, None, torch.zeros(24, 5, device="cuda"), m.weight_hh, m.bias_ih, m.bias_hh)
    with pytest.raises(ValueError, match="float32"):
        streaming_lstm(x, None, None, m.weight_ih.half(), m.weight_hh, m.bias_ih, m.bias_hh)


def test_mfu_report_is_printed_when_the_environment_asks_for_it():
    # FLASHLSTM_PROFILE_MFU / FLASHLSTM_MFU_PEAK_TFLOPS as in flashlstm_v2/include/mfu_profiler.hpp:21-100:
    # one line per streaming call, labelled "forward" / "backward"
    import os
    import re
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import sys, torch; sys.path.insert(0, %r)\n"
        "import flashlstm_poc_amd; flashlstm_poc_amd.add_flashlstm_to_path()\n"
        "from flashlstm import StreamingLSTM\n"
        "m = StreamingLSTM(8, 16)\n"
        "x = torch.empty(5, 2, 8, dtype=torch.float16, pin_memory=True).copy_(torch.randn(5, 2, 8).half())\n"
        "y, cache, (hy, cy) = m(x)\n"
        "y.float().sum().backward()\n"
        "torch.cuda.synchronize()\n" % root)
    env = dict(os.environ, FLASHLSTM_PROFILE_MFU="1", FLASHLSTM_MFU_PEAK_TFLOPS="2500")
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    pat = r"\[flashlstm\]\[%s\] MFU=[0-9.]+%% HFU=[0-9.]+%% \(useful=[0-9.]+ TFLOP/s, matmul=[0-9.]+ TFLOP/s, peak=2500\.000 TFLOP/s\)"
    assert re.search(pat % "forward", out.stdout), out.stdout
    assert re.search(pat % "backward", out.stdout), out.stdout
    quiet = subprocess.run([sys.executable, "-c", code], env={k: v for k, v in os.environ.items() if not k.startswith("FLASHLSTM_")},
                           capture_output=True, text=True, timeout=300)
    assert quiet.returncode == 0 and "[flashlstm]" not in quiet.stdout
