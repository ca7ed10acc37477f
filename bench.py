#!/usr/bin/env python3
"""Headline benchmark: single-layer LSTM forward + backward (BPTT) with the fp16 gate cache on one MI355X.

A "step" is one forward + backward pass of the hot path over one synthetic batch with every tensor
already resident in HBM (fp16 x / dY, packed fp16 weights); weight packing and plan creation happen
before the timed region.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload config3|config2|config4|config5|config5_layer]
                  [--no-cpu-baseline] [--no-parity] [--no-engine-clock] [--no-others]

Without --workload the line is the headline workload (config 3) and carries, under "other_workloads", short runs of
the other BASELINE configurations (config 2, config 4, the config-5 stack: 1 warm-up + 3 timed steps each, with their
parity check).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0   # MI355X dense fp16 MFMA peak (2.5 PFLOP/s)
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # name: (T, B, I, H, backward?)
    "config2": (512, 64, 1024, 1024, False),
    "config3": (1024, 256, 1024, 1024, True),
    "config4": (2048, 16, 2048, 2048, True),
    # one upper layer of the config-5 stack on its own (layers 1-3: I = H = 2048, B = 128, T = 4096), for profiles
    "config5_layer": (4096, 128, 2048, 2048, True),
}
# 4-layer stack (no reference counterpart: the layer loop of flashlstm_poc_amd.LstmStack): T, B, I, H, layers
STACKS = {"config5": (4096, 128, 512, 2048, 4)}


def make_inputs(T, B, I, H, seed=0):
    import torch
    g = torch.Generator(device="cuda").manual_seed(seed)
    k = 1.0 / H ** 0.5
    u = lambda *s: (torch.rand(*s, generator=g, device="cuda") * 2 - 1) * k
    n = lambda *s: torch.randn(*s, generator=g, device="cuda")
    return dict(w_ih=u(4 * H, I), w_hh=u(4 * H, H), b_ih=u(4 * H), b_hh=u(4 * H), x=n(T, B, I).half(),
                h0=(n(B, H) * 0.1).half(), c0=(n(B, H) * 0.1).half(), dy=n(T, B, H).half())


def parity_check(p, outputs, grads):
    """The tensors that were just timed (same x, h0, c0, dY, T) through fp32 torch.nn.LSTM on the GPU with the same
    fp16-rounded weights; `outputs` / `grads` are what the last timed step produced.  Max relative error on y, h_T,
    c_T, relative L2 on the gradients; the last time step's y is listed on its own (h is fed back through fp16)."""
    import torch
    T, B, I = p["x"].shape
    H = p["w_hh"].shape[1]
    # the bias enters as the weight of an extra all-ones input column, so its gradient comes out of the
    # weight-gradient product (PyTorch-ROCm's own bias gradient of nn.LSTM is wrong at T*B = 262144 rows)
    m = torch.nn.LSTM(I + 1, H, bias=False, device="cuda")
    with torch.no_grad():
        m.weight_ih_l0[:, :I].copy_(p["w_ih"].half().float())
        m.weight_ih_l0[:, I].copy_(p["b_ih"] + p["b_hh"])
        m.weight_hh_l0.copy_(p["w_hh"].half().float())
    want_grads = grads is not None
    xr = torch.cat([p["x"].float(), torch.ones(T, B, 1, device="cuda")], dim=2).requires_grad_(want_grads)
    hr = p["h0"].float().requires_grad_(want_grads); cr = p["c0"].float().requires_grad_(want_grads)
    # (and one call of more than 131072 rows returns wrong outputs at H = 2048: the sequence goes through in
    # segments, the state carried from one call to the next inside the same autograd graph)
    seg = max(1, 131072 // B)
    ys, state = [], (hr[None], cr[None])
    for t0 in range(0, T, seg):
        y_seg, state = m(xr[t0:t0 + seg], state)
        ys.append(y_seg)
    yr, (hn, cn) = (ys[0] if len(ys) == 1 else torch.cat(ys)), state
    relmax = lambda a, b: ((a.float() - b.float()).abs().max() / b.float().abs().max()).item()
    rell2 = lambda a, b: ((a.double() - b.double()).norm() / b.double().norm()).item()
    y, hy, cy = outputs
    errs = {"y": relmax(y, yr), "y_last_step": relmax(y[-1], yr[-1]), "h_T": relmax(hy, hn[0]), "c_T": relmax(cy, cn[0])}
    if want_grads:
        (yr * p["dy"].float()).sum().backward()
        dx, dW_ih, dW_hh, db, dh0, dc0 = grads
        gw = m.weight_ih_l0.grad
        errs.update({"dx": rell2(dx, xr.grad[:, :, :I]), "dW_ih": rell2(dW_ih, gw[:, :I]),
                     "dW_hh": rell2(dW_hh, m.weight_hh_l0.grad), "db": rell2(db, gw[:, I]),
                     "dh0": rell2(dh0, hr.grad), "dc0": rell2(dc0, cr.grad)})
    worst = max(errs.values())
    return {"on": "the timed tensors", "T": T, "reference": "torch.nn.LSTM fp32 on the GPU, fp16-rounded weights, calls of at most 131072 rows",
            "errors": {k: float(f"{v:.3e}") for k, v in errs.items()}, "max_err": float(f"{worst:.3e}"),
            "tolerance": 1e-2, "ok": bool(worst <= 1e-2)}


def kernel_source_digest():
    """First 16 hex digits of the SHA-256 over the kernel sources (csrc/*.hip, csrc/*.h, sorted by name): ties a
    counter profile under profiles/ to the code it was taken from."""
    import glob
    import hashlib
    h = hashlib.sha256()
    d = os.path.join(ROOT, "flashlstm_poc_amd", "csrc")
    for f in sorted(glob.glob(os.path.join(d, "*.hip")) + glob.glob(os.path.join(d, "*.h"))):
        h.update(os.path.basename(f).encode())
        h.update(open(f, "rb").read())
    return h.hexdigest()[:16]


def measured_traffic(workload, phase):
    """HBM-side bytes per launch of a phase's kernels from the committed counter summary
    profiles/hbm_traffic_per_kernel.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, calibrated against a copy kernel).
    None unless that summary was taken from exactly the kernel sources that are running now."""
    import re
    path = os.path.join(ROOT, "profiles", "hbm_traffic_per_kernel.md")
    try:
        text = open(path).read()
        block = re.search(r"```json traffic\n(.*?)```", text, flags=re.S)
        data = json.loads(block.group(1))
    except Exception:
        return None, "no counter summary"
    if data.get("kernel_source_digest") != kernel_source_digest():
        return None, f"counter summary is from other kernel sources ({data.get('kernel_source_digest')})"
    try:
        return float(data["bytes_per_launch"][workload][phase]), data.get("taken", "")
    except Exception:
        return None, "phase not in the counter summary"


def measured_counters(workload, phase):
    """L2 request and LDS activity counters per launch of a phase's kernel from the same committed summary (rocprofv3
    --pmc TCC_REQ_sum / SQ_LDS_IDX_ACTIVE / GRBM_GUI_ACTIVE and the kernel trace's duration, taken with plain launches:
    a profiler tool and cooperative launches do not go together).  None unless the summary was taken from exactly
    the kernel sources that are running now."""
    import re
    path = os.path.join(ROOT, "profiles", "hbm_traffic_per_kernel.md")
    try:
        text = open(path).read()
        data = json.loads(re.search(r"```json traffic\n(.*?)```", text, flags=re.S).group(1))
    except Exception:
        return None, "no counter summary"
    if data.get("kernel_source_digest") != kernel_source_digest():
        return None, f"counter summary is from other kernel sources ({data.get('kernel_source_digest')})"
    try:
        return data["counters_per_launch"][workload][phase], data.get("taken", "")
    except Exception:
        return None, "phase not in the counter summary"


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(B, I, H, backward, budget_s=15.0):
    """torch.nn.LSTM (fp32, CPU) on this host's cores.  Two figures: BASELINE config 1 exactly (I=128, H=256, B=8,
    T=64, seed 0, h0=c0=0, loss = sum(y^2); 3 warm-ups, 20 repeats, forward and forward+backward), and a
    time-bounded sample of the benchmarked workload: same B, I, H and seeded inputs at reduced T (LSTM cost is
    linear in T).  `value` is the sample's rate, comparable with the GPU line."""
    import torch
    threads = torch.get_num_threads()

    def timed(fn, warm, reps):
        for _ in range(warm):
            fn()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        return (time.perf_counter() - t0) / reps

    # config 1
    torch.manual_seed(0)
    m1 = torch.nn.LSTM(128, 256)
    x1 = torch.randn(64, 8, 128, requires_grad=True)

    def c1_fwd():
        with torch.no_grad():
            m1(x1)

    def c1_fwdbwd():
        m1.zero_grad(set_to_none=True)
        x1.grad = None
        y, _ = m1(x1)
        (y ** 2).sum().backward()

    c1f = timed(c1_fwd, 3, 20)
    c1fb = timed(c1_fwdbwd, 3, 20)

    # sample of the benchmarked workload
    T = 8
    torch.manual_seed(0)
    m = torch.nn.LSTM(I, H)
    x = torch.randn(T, B, I, requires_grad=backward)
    dy = torch.randn(T, B, H)

    def once():
        y, _ = m(x)
        if backward:
            m.zero_grad(set_to_none=True)
            x.grad = None
            (y * dy).sum().backward()

    once()  # warm-up
    t0 = time.perf_counter(); once(); probe = time.perf_counter() - t0
    reps = max(3, min(20, int(budget_s / max(probe, 1e-3))))
    dt = timed(once, 2, reps)
    return {"value": round(B * T / dt, 1), "unit": "batch*timesteps/s", "cores": threads, "kind": "port",
            "impl": "torch.nn.LSTM fp32 on CPU (the oracle named for this path)",
            "cpu_model": cpu_model(), "os_cpu_count": os.cpu_count(), "torch_num_threads": threads,
            "torch_version": torch.__version__,
            "sample": f"same B={B}, I={I}, H={H}, {'fwd+bwd' if backward else 'fwd'}, T reduced to {T}, "
                      f"{reps} repeats after 4 untimed runs, {dt * 1e3:.1f} ms each",
            "config1": {"workload": "I=128, H=256, B=8, T=64, fp32, seed 0, loss=sum(y^2)", "warmups": 3, "repeats": 20,
                        "fwd_ms": round(c1f * 1e3, 3), "fwd_bwd_ms": round(c1fb * 1e3, 3),
                        "fwd_batch_timesteps_per_s": round(512 / c1f, 1),
                        "fwd_bwd_batch_timesteps_per_s": round(512 / c1fb, 1)}}


def stack_parity(params, x, target, y, grads):
    """The timed stack problem through fp32 torch.nn.LSTM on the GPU: one single-layer module per layer, the bias as
    the weight of an extra all-ones input column, every call on at most 131072 rows with (h, c) carried between the
    time segments (beyond that size PyTorch-ROCm's nn.LSTM itself goes wrong: its bias gradient from 262144 rows,
    its outputs from 524288).  `y`, `grads` = what the last timed step produced."""
    import torch
    T, B, _ = x.shape
    mods = []
    for w_ih, w_hh, b_ih, b_hh in params:
        m = torch.nn.LSTM(w_ih.shape[1] + 1, w_hh.shape[1], bias=False, device="cuda")
        with torch.no_grad():
            m.weight_ih_l0[:, :-1].copy_(w_ih.half().float()); m.weight_ih_l0[:, -1].copy_(b_ih + b_hh)
            m.weight_hh_l0.copy_(w_hh.half().float())
        mods.append(m)
    seg = max(1, 131072 // B)
    cur = x.float()
    for m in mods:
        h = c = cur.new_zeros(1, B, m.hidden_size)
        outs = []
        for t0 in range(0, T, seg):
            xs = cur[t0:t0 + seg]
            ys, (h, c) = m(torch.cat([xs, torch.ones_like(xs[:, :, :1])], dim=2), (h, c))
            outs.append(ys)
        cur = outs[0] if len(outs) == 1 else torch.cat(outs, dim=0)
    relmax = lambda a, b: ((a.float() - b.float()).abs().max() / b.float().abs().max()).item()
    rell2 = lambda a, b: ((a.double() - b.double()).norm() / b.double().norm()).item()
    errs = {"y": relmax(y, cur), "y_last_step": relmax(y[-1], cur[-1])}
    torch.nn.functional.mse_loss(cur, target.float()).backward()
    for l, (m, (dW_ih, dW_hh, db)) in enumerate(zip(mods, grads)):
        g = m.weight_ih_l0.grad
        errs[f"dW_ih{l}"] = rell2(dW_ih, g[:, :-1]); errs[f"dW_hh{l}"] = rell2(dW_hh, m.weight_hh_l0.grad)
        errs[f"db{l}"] = rell2(db, g[:, -1])
    worst = max(errs.values())
    return {"on": "the timed tensors", "T": T, "reference": "torch.nn.LSTM fp32 on the GPU per layer, fp16-rounded weights, "
            "calls of at most 131072 rows", "errors": {k: float(f"{v:.3e}") for k, v in errs.items()},
            "max_err": float(f"{worst:.3e}"), "tolerance": 1e-2, "ok": bool(worst <= 1e-2)}


def bench_stack(args, device):
    """fwd+bwd of a stack of layers with MSE on the top layer's outputs (automatic power-of-two loss scale)."""
    import torch
    from flashlstm_poc_amd import LstmStack
    T, B, I, H, L = STACKS[args.workload]
    g = torch.Generator(device="cuda").manual_seed(0)
    k = 1.0 / H ** 0.5
    u = lambda *s: (torch.rand(*s, generator=g, device="cuda") * 2 - 1) * k
    stack = LstmStack(B, I, H, L)
    params = [(u(4 * H, I if l == 0 else H), u(4 * H, H), u(4 * H), u(4 * H)) for l in range(L)]
    stack.pack(params)
    x = torch.randn(T, B, I, generator=g, device="cuda").half()
    target = torch.randn(T, B, H, generator=g, device="cuda").half()
    last = {}

    def step():
        y, _, _ = stack.forward(x)
        # d/dy of mean((y - target)^2); loss scale: automatic (a power of two from the largest |dy|)
        _, grads, _, _ = stack.backward_mse(y, target, want_dx=False)
        last["y"], last["grads"] = y, grads

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    flops = sum(24.0 * T * B * H * ((I if l == 0 else H) + H) for l in range(L))
    phases = {ph: sum(layer.last_ms(ph) for layer in stack.layers) for ph in ("fwd_proj", "fwd_rec", "bwd_rec", "bwd_dx", "bwd_dw")}
    dom = max(phases, key=phases.get)
    dom_flops = {"fwd_proj": sum(2.0 * T * B * 4 * H * (I if l == 0 else H) for l in range(L)),
                 "fwd_rec": L * 2.0 * T * B * 4 * H * H, "bwd_rec": L * 2.0 * T * B * 4 * H * H,
                 "bwd_dx": sum(2.0 * T * B * 4 * H * (I if l == 0 else H) for l in range(1, L)),
                 "bwd_dw": sum(2.0 * T * B * 4 * H * ((I if l == 0 else H) + H) for l in range(L))}[dom]
    tf = dom_flops / (phases[dom] * 1e-3) / 1e12
    out = {"metric": "fwd+bwd batch*timesteps/sec", "value": round(B * T / (ms * 1e-3), 1), "unit": "batch*timesteps/s",
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 3),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "fp16 storage, fp32 accumulate, fp32 cell state", "data": "synthetic",
           "config": {"workload": f"{args.workload}: {L}-layer LSTM stack fwd+bwd, MSE on the top outputs, I={I}, H={H}, "
                                  f"B={B}, T={T}", "T": T, "B": B, "I": I, "H": H, "layers": L},
           "mfu": round(flops / (ms * 1e-3) / (PEAK_FP16_TFLOPS * 1e12), 4), "tflops": round(flops / (ms * 1e-3) / 1e12, 1),
           "flops_per_step": flops, "phase_ms_all_layers": {k_: round(v, 3) for k_, v in phases.items()},
           "roofline": {"kernel": dom + " (summed over the layers)", "bound": "mfma", "achieved": round(tf, 1),
                        "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / PEAK_FP16_TFLOPS, 4), "traffic": None},
           "us_per_timestep": {"fwd_rec": round(phases["fwd_rec"] * 1e3 / (T * L), 3),
                               "bwd_rec": round(phases["bwd_rec"] * 1e3 / (T * L), 3)},
           "loss_scale": stack.last_loss_scale, "device": device, "cpu_baseline": None,
           "kernel_source_digest": kernel_source_digest()}
    stack.close()
    torch.cuda.empty_cache()
    if not args.no_parity:
        out["parity"] = stack_parity(params, x, target, last["y"], last["grads"])
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS) + sorted(STACKS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-parity", action="store_true")
    ap.add_argument("--no-engine-clock", action="store_true",
                    help="skip the two extra passes that read the engine clock inside the recurrence kernels (profiler runs)")
    ap.add_argument("--no-others", action="store_true", help="the headline workload only (no other_workloads block)")
    args = ap.parse_args()
    args.others = args.workload is None and not args.no_others
    args.workload = args.workload or "config3"
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU (the recurrence shards over batch; no multi-GPU path is "
              "built) -- rerun with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from flashlstm_poc_amd import LstmCore
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    props = torch.cuda.get_device_properties(0)
    probe = LstmCore(1, 8, 8)   # the library reads the engine clock from the HIP runtime
    clock_khz = probe.info("clock_khz") or getattr(props, "clock_rate", None)
    probe.close()
    device = {"name": props.name, "compute_units": props.multi_processor_count,
              "max_engine_clock_mhz": (clock_khz / 1e3) if clock_khz else None,
              # 4096 fp16 MFMA FLOP per clock and CU (CDNA4, dense)
              "derived_fp16_peak_tflops": (round(props.multi_processor_count * 4096 * clock_khz * 1e3 / 1e12, 1)
                                           if clock_khz else None),
              "peak_used_tflops": PEAK_FP16_TFLOPS, "hbm_gib": round(props.total_memory / 2 ** 30, 1)}
    if args.workload in STACKS:
        print(json.dumps(bench_stack(args, device)))
        return
    out = bench_single(args, device)
    if args.others:
        # the other BASELINE configurations, briefly: 1 warm-up + 3 timed steps each, parity on the timed tensors
        others = {}
        for wl in ("config2", "config4", "config5"):
            sub = argparse.Namespace(**vars(args))
            sub.workload, sub.steps, sub.warmup, sub.no_cpu_baseline = wl, 3, 1, True
            torch.cuda.empty_cache()
            r = bench_stack(sub, None) if wl in STACKS else bench_single(sub, None)
            others[wl] = {"workload": r["config"]["workload"], "metric": r["metric"], "value": r["value"],
                          "ms_per_step": r["ms_per_step"], "steps": 3, "warmup": 1, "mfu": r["mfu"],
                          "us_per_timestep": r.get("us_per_timestep"),
                          "phase_ms": r.get("phase_ms_all_layers") or {k["phase"]: k["ms"] for k in r.get("kernels", [])},
                          "parity": ({"max_err": r["parity"]["max_err"], "ok": r["parity"]["ok"]} if "parity" in r else None)}
        out["other_workloads"] = others
    print(json.dumps(out))


def bench_single(args, device):
    """One single-layer workload: fwd (+ bwd) steps timed with hipEvents, per-phase times from the library's own
    events on the launch stream, roofline of the dominant kernel, parity on the timed tensors."""
    import torch
    from flashlstm_poc_amd import LstmCore
    T, B, I, H, backward = WORKLOADS[args.workload]
    p = make_inputs(T, B, I, H)
    core = LstmCore(B, I, H)
    core.pack(p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"])

    last = {}

    def step():
        last["out"] = core.forward(p["x"], p["h0"], p["c0"], save_for_backward=backward)
        if backward:
            last["grads"] = core.backward(p["x"], p["dy"])

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    phases = ["fwd_proj", "fwd_rec"] + (["bwd_rec", "bwd_dx", "bwd_dw"] if backward else [])
    acc = {k: 0.0 for k in phases}
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
        for k in phases:   # device time of each phase of this step (hipEvents on the launch stream)
            acc[k] += core.last_ms(k)
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ms = e0.elapsed_time(e1) / args.steps
    phase_ms = {k: v / args.steps for k, v in acc.items()}
    # Engine clock inside the recurrence kernels, from two untimed passes with the kernels' own counters on: workgroup 0
    # reads the shader clock counter and the constant 100 MHz counter at its first and last step.  (The part lowers its
    # clock under the GEMMs and raises it again only slowly, so the recurrences that follow them run below 2.4 GHz.)
    engine_mhz = {}
    if not args.no_engine_clock:
        core.set_option("profile", 1)
        for _ in range(2):
            step()
        torch.cuda.synchronize()
        for d in ("fwd", "bwd") if backward else ("fwd",):
            ticks = core.last_ms(f"{d}_clk6")
            if ticks > 0:
                engine_mhz[f"{d}_rec"] = round(core.last_ms(f"{d}_clk5") / ticks * 100.0, 1)
        core.set_option("profile", 0)

    flops_fwd = 8.0 * T * B * H * (I + H)
    flops = flops_fwd * (3.0 if backward else 1.0)
    # algorithmic FLOPs per launch of each kernel (2*m*n*k per contraction)
    kflops = {"fwd_proj": 2.0 * T * B * 4 * H * I, "fwd_rec": 2.0 * T * B * 4 * H * H,
              "bwd_rec": 2.0 * T * B * 4 * H * H, "bwd_dx": 2.0 * T * B * 4 * H * I,
              "bwd_dw": 2.0 * T * B * 4 * H * (I + H)}
    kname = {"fwd_proj": "gemm_nt_stream (X*W_ih^T + bias)", "fwd_rec": "rec_fwd_kernel (persistent recurrence)",
             "bwd_rec": ("rec_bwd2d_kernel (persistent BPTT, product split over columns and contraction)"
                         if core.info("bwd_two_d") == 1 else "rec_bwd_kernel (persistent BPTT)"), "bwd_dx": "gemm_nt_stream (dG*W_ih)",
             "bwd_dw": "gemm_tn_stream split-K x2 (dG^T*X, dG^T*H) + reduce_dw"}
    kernels = []
    for k in phases:
        tf = kflops[k] / (phase_ms[k] * 1e-3) / 1e12 if phase_ms[k] > 0 else 0.0
        kernels.append({"phase": k, "kernel": kname[k], "ms": round(phase_ms[k], 4), "tflops": round(tf, 1),
                        "frac_of_peak": round(tf / PEAK_FP16_TFLOPS, 4)})
    dom = max(kernels, key=lambda d: d["ms"])
    traffic, traffic_note = measured_traffic(args.workload, dom["phase"])
    roofline = {"kernel": dom["kernel"], "bound": "mfma", "achieved": dom["tflops"], "peak": PEAK_FP16_TFLOPS,
                "unit": "TFLOP/s", "frac": dom["frac_of_peak"],
                "traffic": traffic, "traffic_source": traffic_note,
                "traffic_unit": "bytes per launch (fetched + written beyond the L2)",
                "launch_ms": dom["ms"], "flops_per_launch": kflops[dom["phase"]]}
    if dom["phase"] in ("fwd_rec", "bwd_rec"):
        roofline["us_per_timestep"] = round(dom["ms"] * 1e3 / T, 3)

    out = {
        "metric": "fwd+bwd batch*timesteps/sec" if backward else "fwd batch*timesteps/sec",
        "value": round(B * T / (ms * 1e-3), 1),
        "unit": "batch*timesteps/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "wall_ms_per_step": round(wall_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16 storage, fp32 accumulate, fp32 cell state", "data": "synthetic",
        "config": {"workload": f"{args.workload}: single-layer LSTM {'fwd+bwd with fp16 gate cache' if backward else 'forward'}"
                               f", I={I}, H={H}, B={B}, T={T}", "T": T, "B": B, "I": I, "H": H},
        "mfu": round(flops / (ms * 1e-3) / (PEAK_FP16_TFLOPS * 1e12), 4),
        "mfu_target": 0.40, "tflops": round(flops / (ms * 1e-3) / 1e12, 1), "flops_per_step": flops,
        "persistent": {"fwd": core.info("persistent_fwd"), "bwd": core.info("persistent_bwd"),
                       "xcd_local_fwd": core.info("xcd_local_fwd"), "xcd_local_bwd": core.info("xcd_local_bwd"),
                       "bwd_two_d": core.info("bwd_two_d"), "fallbacks": core.info("fallbacks")},
        "roofline": roofline, "kernels": kernels, "device": device,
        "us_per_timestep": {"fwd_rec": round(phase_ms["fwd_rec"] * 1e3 / T, 3),
                            **({"bwd_rec": round(phase_ms["bwd_rec"] * 1e3 / T, 3)} if backward else {})},
        "engine_mhz_in_recurrence": engine_mhz,
    }
    # What the recurrence moves between workgroups each step.  Measured: requests to the L2 (TCC_REQ, each at most one
    # 128-byte line) and the cycles the LDS address unit was busy (SQ_LDS_IDX_ACTIVE, summed over the CUs), from the
    # committed counter summary -- taken with plain launches, 5 % slower than the cooperative launches timed here --
    # divided by that profile's own kernel duration.  Beside them the byte model: every workgroup (16 or 32 batch rows x
    # one slice of hidden units) fetches the whole h_{t-1} (forward) or dG_{t+1} (backward) of its rows from the L2.
    block = 16 * core.info("row_tiles")   # batch rows per workgroup
    Hp, rows = core.info("hidden_padded"), block * ((B + block - 1) // block)
    xch = {}
    for d, k_cols in (("fwd", Hp), ("bwd", 4 * Hp)) if backward else (("fwd", Hp),):
        us = phase_ms[d + "_rec"] * 1e3 / T
        slices = Hp // core.info("slice_" + d)
        l2_bytes = rows * slices * k_cols * 2
        if d == "bwd" and core.info("bwd_two_d") == 1:
            # 256 workgroups, each fetches an eighth of dG_{t+1} of every row and passes 7/8 of its fp32 partial
            # products [rows][64 columns] once through the L2 to the slice's peers
            l2_bytes = rows * 256 * (k_cols // 8) * 2 + 2 * rows * 256 * 64 * 4
        entry = {"model_l2_fetch_bytes_per_step": l2_bytes, "model_l2_fetch_gb_per_s": round(l2_bytes / us / 1e3, 1)}
        c, note = measured_counters(args.workload, d + "_rec")
        if c:
            cus = device["compute_units"] if device else 256
            entry.update({"measured": {
                "l2_requests_per_step": round(c["TCC_REQ"] / T, 1),
                "l2_gb_per_s_at_128B_per_request": round(c["TCC_REQ"] * 128 / (c["ms"] * 1e-3) / 1e9, 1),
                "lds_busy_cycles_per_step_and_cu": round(c["SQ_LDS_IDX_ACTIVE"] / T / cus, 1),
                "lds_busy_fraction": round(c["SQ_LDS_IDX_ACTIVE"] / cus / (c["GRBM_GUI_ACTIVE"] / 8), 4),
                "profile_launch_ms": c["ms"], "launches": "plain (profiler attached)", "source": note}})
        else:
            entry["measured"] = None
            entry["measured_note"] = note
        xch[d] = entry
    out["exchange_per_step"] = xch
    core.close()
    out["kernel_source_digest"] = kernel_source_digest()
    if not args.no_parity:
        out["parity"] = parity_check(p, last["out"], last.get("grads"))
    last.clear()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(B, I, H, backward)
    return out


if __name__ == "__main__":
    main()
