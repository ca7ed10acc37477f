"""flstm_core_forward_static (the forward pass that allocates nothing: its scratch memory is one fixed array in the
library's device image) through the C ABI against flstm_core_forward: bit-identical outputs, on calls in a row that
shrink (a shorter sequence on the same plan, then a smaller plan) and so reuse the array with whatever the call
before left in it; device memory in use does not change across the calls; a pass beyond the array is rejected."""
import ctypes

import pytest
import torch

from helpers import make_problem

pytestmark = pytest.mark.gpu

F32, F16 = 0, 1


def _free_bytes():
    free, _ = torch.cuda.mem_get_info()
    return free


def _plan(lib, p):
    T, B, I = p["x"].shape
    H = p["w_hh"].shape[1]
    h = ctypes.c_void_p()
    assert lib.flstm_core_create(B, I, H, ctypes.byref(h)) == 0
    s = torch.cuda.current_stream().cuda_stream
    w = [p[k].cuda().float().contiguous() for k in ("w_ih", "w_hh", "b_ih", "b_hh")]
    assert lib.flstm_core_pack_weights(h, w[0].data_ptr(), w[1].data_ptr(), s) == 0
    assert lib.flstm_core_pack_bias(h, w[2].data_ptr(), w[3].data_ptr(), s) == 0
    return h, w


def _call(lib, fn_static, plan, x, h0, c0, dtype_code, out_dtype):
    T, B = x.shape[0], x.shape[1]
    H = h0.shape[1]
    y = torch.full((T, B, H), 9.0, device="cuda", dtype=out_dtype)
    hy = torch.full((B, H), 9.0, device="cuda", dtype=out_dtype); cy = torch.full((B, H), 9.0, device="cuda", dtype=out_dtype)
    s = torch.cuda.current_stream().cuda_stream
    oc = F32 if out_dtype == torch.float32 else F16
    torch.cuda.synchronize()
    if fn_static:
        before = _free_bytes()
        rc = lib.flstm_core_forward_static(plan, T, x.data_ptr(), dtype_code, h0.data_ptr(), c0.data_ptr(), dtype_code,
                                           y.data_ptr(), oc, hy.data_ptr(), cy.data_ptr(), oc, s)
        after = _free_bytes()
    else:
        before = after = 0
        rc = lib.flstm_core_forward(plan, T, x.data_ptr(), dtype_code, h0.data_ptr(), c0.data_ptr(), dtype_code,
                                    y.data_ptr(), oc, hy.data_ptr(), cy.data_ptr(), oc, 0, s)
    torch.cuda.synchronize()
    return rc, (y, hy, cy), before - after


def test_static_forward_equals_the_allocating_forward_on_shrinking_calls():
    from flashlstm_poc_amd import load_library
    lib = load_library()
    big = make_problem(24, 40, 64, 256, seed=41)       # fp16 I/O, x used in place
    small = make_problem(12, 5, 20, 40, seed=42)       # fp32 I/O, padded x rows (I % 64 != 0), ragged H
    plan_a, keep_a = _plan(lib, big)
    plan_ref_a, keep_ra = _plan(lib, big)
    plan_b, keep_b = _plan(lib, small)
    plan_ref_b, keep_rb = _plan(lib, small)
    cases = []
    for name, plan, ref, p, T, half in (("first call", plan_a, plan_ref_a, big, 24, True),
                                        ("shorter sequence, same plan", plan_a, plan_ref_a, big, 9, True),
                                        ("smaller plan, fp32 tensors", plan_b, plan_ref_b, small, 12, False),
                                        ("the first size again", plan_a, plan_ref_a, big, 24, True)):
        cv = (lambda t: t.cuda().half().contiguous()) if half else (lambda t: t.cuda().float().contiguous())
        x, h0, c0 = cv(p["x"][:T]), cv(p["h0"]), cv(p["c0"])
        code, odt = (F16, torch.float16) if half else (F32, torch.float32)
        rc, got, grew = _call(lib, True, plan, x, h0, c0, code, odt)
        assert rc == 0, (name, rc)
        rc, want, _ = _call(lib, False, ref, x, h0, c0, code, odt)
        assert rc == 0
        for g, w, what in zip(got, want, ("y", "hy", "cy")):
            assert torch.equal(g, w), (name, what, (g.float() - w.float()).abs().max().item())
        cases.append((name, grew))
    # after the first call (which may load code objects) the calls leave device memory in use unchanged
    for name, grew in cases[1:]:
        assert grew == 0, (name, grew)
    # a cache left by an allocating forward pass survives static calls on the same plan
    cvh = lambda t: t.cuda().half().contiguous()
    x, h0, c0 = cvh(big["x"]), cvh(big["h0"]), cvh(big["c0"])
    T, B, I = x.shape
    y = torch.empty(T, B, 256, device="cuda", dtype=torch.float16); hy = torch.empty(B, 256, device="cuda", dtype=torch.float16)
    cy = torch.empty_like(hy)
    s = torch.cuda.current_stream().cuda_stream
    assert lib.flstm_core_forward(plan_a, T, x.data_ptr(), F16, h0.data_ptr(), c0.data_ptr(), F16, y.data_ptr(), F16,
                                  hy.data_ptr(), cy.data_ptr(), F16, 1, s) == 0
    ptr, ld = ctypes.c_void_p(), ctypes.c_size_t()
    assert lib.flstm_core_cache_ptr(plan_a, 2, ctypes.byref(ptr), ctypes.byref(ld)) == 0
    kept = ptr.value
    rc, _, _ = _call(lib, True, plan_a, x[:5].contiguous(), h0, c0, F16, torch.float16)
    assert rc == 0
    assert lib.flstm_core_cache_ptr(plan_a, 2, ctypes.byref(ptr), ctypes.byref(ld)) == 0 and ptr.value == kept
    # too large for the fixed array: rejected up front, nothing enqueued
    limit = lib.flstm_core_get_info(plan_a, b"static_scratch_bytes")
    assert limit == 64 << 20
    T_big = limit // (40 * 14 * 256) + 8
    xl = torch.zeros(T_big, 40, 64, device="cuda", dtype=torch.float16)
    rc, _, _ = _call(lib, True, plan_a, xl, h0, c0, F16, torch.float16)
    assert rc == 2004
    for h in (plan_a, plan_ref_a, plan_b, plan_ref_b):
        assert lib.flstm_core_destroy(h) == 0


def test_static_forward_allocates_nothing_on_the_step_wise_path_and_after_a_give_up():
    """The entry point's promise holds where the pass is one launch per step -- a plan with the `stepwise` option, and
    the repeat after a persistent launch that gave up (forced from the host: `inject_stall`): plain launches, no graph
    capture, device memory in use unchanged, results bit-identical to flstm_core_forward; and a call that failed
    leaves the plan usable."""
    from flashlstm_poc_amd import load_library
    lib = load_library()
    p = make_problem(20, 40, 64, 256, seed=43)
    cvh = lambda t: t.cuda().half().contiguous()
    x, h0, c0 = cvh(p["x"]), cvh(p["h0"]), cvh(p["c0"])
    plan, keep = _plan(lib, p)
    ref, keep_r = _plan(lib, p)
    rc, want, _ = _call(lib, False, ref, x, h0, c0, F16, torch.float16)
    assert rc == 0
    # warm-up (code objects), then the measured calls
    rc, _, _ = _call(lib, True, plan, x, h0, c0, F16, torch.float16)
    assert rc == 0
    # 1) a persistent launch that gives up: the pass is repeated with one launch per step inside the same call
    assert lib.flstm_core_get_info(plan, b"persistent_fwd") == 1
    assert lib.flstm_core_set_option(plan, b"inject_stall", 1) == 0
    captures = lib.flstm_core_get_info(plan, b"graph_captures")
    rc, got, grew = _call(lib, True, plan, x, h0, c0, F16, torch.float16)
    assert rc == 0 and grew == 0, (rc, grew)
    assert lib.flstm_core_get_info(plan, b"fallbacks") == 1 and lib.flstm_core_get_info(plan, b"persistent_fwd") == 0
    assert lib.flstm_core_get_info(plan, b"graph_captures") == captures   # no graph was built
    for g, w, what in zip(got, want, ("y", "hy", "cy")):
        assert torch.equal(g, w), ("after a give-up", what)
    # 2) the demoted plan (step-wise launches) and a plan with the option: the same, still without a graph
    assert lib.flstm_core_set_option(plan, b"stepwise", 1) == 0
    for _ in range(2):
        rc, got, grew = _call(lib, True, plan, x, h0, c0, F16, torch.float16)
        assert rc == 0 and grew == 0, (rc, grew)
        for g, w, what in zip(got, want, ("y", "hy", "cy")):
            assert torch.equal(g, w), ("step-wise", what)
    assert lib.flstm_core_get_info(plan, b"graph_captures") == captures
    # 3) a pass that fails (two give-ups in a row: the step-wise repeat is treated as failed too) returns "stalled" and
    #    the next call works
    assert lib.flstm_core_set_option(plan, b"stepwise", 0) == 0
    assert lib.flstm_core_set_option(plan, b"clear_tuned", 0) == 0
    plan2, keep2 = _plan(lib, p)
    assert lib.flstm_core_set_option(plan2, b"inject_stall", 2) == 0
    rc, _, _ = _call(lib, True, plan2, x, h0, c0, F16, torch.float16)
    assert rc == 2003, rc   # FLSTM_E_STALLED
    assert lib.flstm_core_set_option(plan2, b"inject_stall", 0) == 0
    rc, got, _ = _call(lib, True, plan2, x, h0, c0, F16, torch.float16)
    assert rc == 0
    for g, w, what in zip(got, want, ("y", "hy", "cy")):
        assert torch.equal(g, w), ("after a failed call", what)
    for h in (plan, ref, plan2):
        assert lib.flstm_core_destroy(h) == 0
