"""Sequence-length sweep and tuner for the device-resident LSTM core.

    python -m flashlstm_poc_amd.sweep --batch 64 --input-size 1024 --hidden-size 1024 --seq-lens 128 512 2048
    python -m flashlstm_poc_amd.sweep --tune --seq-lens 256 1024      # tune a plan per length, then sweep with it

Counterpart of the reference's python/benchmark_lstm.py:455-620 (sequence-length sweep against torch.nn.LSTM,
here the MIOpen-backed one of PyTorch-ROCm on the same GPU) and of its tuners (src/tune_projchunksz.cu:56-226,
python/benchmark_lstm.py:203-301): --tune runs the library's own tuner (LstmCore.tune -> flstm_core_tune: 16- or
32-row blocks per recurrence, persistent or step-wise launches, split-K count of the weight-gradient GEMM) for
every length before timing it, prints what it chose, and the sweep then runs with those choices cached in the
plan.  Inputs are synthetic (seeded); every tensor is resident on the GPU before timing starts.
"""
import argparse
import csv
import json
import os
import statistics
import sys
from typing import Dict, List, Optional, Sequence

PEAK_FP16_TFLOPS = 2500.0   # MI355X dense fp16 MFMA peak


def _time_ms(fn, warmup: int, repeats: int) -> List[float]:
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    out = []
    for _ in range(repeats):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        out.append(a.elapsed_time(b))
    return out


def make_problem(T: int, B: int, I: int, H: int, seed: int):
    import torch
    g = torch.Generator(device="cuda").manual_seed(seed)
    k = 1.0 / H ** 0.5
    u = lambda *s: (torch.rand(*s, generator=g, device="cuda") * 2 - 1) * k
    return {"w_ih": u(4 * H, I), "w_hh": u(4 * H, H), "b_ih": u(4 * H), "b_hh": u(4 * H),
            "x": torch.randn(T, B, I, generator=g, device="cuda").half(),
            "dy": torch.randn(T, B, H, generator=g, device="cuda").half(),
            "h0": (torch.randn(B, H, generator=g, device="cuda") * 0.1).half(),
            "c0": (torch.randn(B, H, generator=g, device="cuda") * 0.1).half()}


def torch_lstm(p, I: int, H: int):
    """torch.nn.LSTM in fp16 on the GPU with the same weights."""
    import torch
    m = torch.nn.LSTM(I, H).cuda().half()
    with torch.no_grad():
        m.weight_ih_l0.copy_(p["w_ih"]); m.weight_hh_l0.copy_(p["w_hh"])
        m.bias_ih_l0.copy_(p["b_ih"]); m.bias_hh_l0.copy_(p["b_hh"])
    return m


def check_parity(core, p, I: int, H: int) -> Dict[str, float]:
    """Max relative error of y / h_T / c_T and relative L2 error of dx, dW against torch.nn.LSTM in fp32 on the
    fp16-rounded operands (the tolerance of both is 1e-2)."""
    import torch
    m = torch.nn.LSTM(I, H).cuda().float()
    with torch.no_grad():
        for dst, key in ((m.weight_ih_l0, "w_ih"), (m.weight_hh_l0, "w_hh"), (m.bias_ih_l0, "b_ih"), (m.bias_hh_l0, "b_hh")):
            dst.copy_(p[key].half().float() if key.startswith("w") else p[key])
    x = p["x"].float().requires_grad_(True)
    y_ref, (h_ref, c_ref) = m(x, (p["h0"].float()[None], p["c0"].float()[None]))
    (y_ref * p["dy"].float()).sum().backward()
    y, hy, cy = core.forward(p["x"], p["h0"], p["c0"])
    dx, dW_ih, dW_hh, _, _, _ = core.backward(p["x"], p["dy"])
    relmax = lambda a, b: float((a.float() - b.detach()).abs().max() / b.detach().abs().max().clamp_min(1e-30))
    rell2 = lambda a, b: float((a.float() - b.detach()).norm() / b.detach().norm().clamp_min(1e-30))
    return {"y": relmax(y, y_ref), "h_T": relmax(hy, h_ref[0]), "c_T": relmax(cy, c_ref[0]), "dx": rell2(dx, x.grad),
            "dW_ih": rell2(dW_ih, m.weight_ih_l0.grad), "dW_hh": rell2(dW_hh, m.weight_hh_l0.grad)}


def sweep(B: int, I: int, H: int, seq_lens: Sequence[int], *, warmup: int = 3, repeats: int = 10, seed: int = 2025,
          baseline: bool = True, check: bool = False, tune: bool = False, try_stepwise: bool = False,
          tuned_table: Optional[List[Dict]] = None) -> List[Dict]:
    """tuned_table: tuned entries (LstmCore.tuned_table) to start every plan from; with `tune` the entries found are
    appended to it in place, so the caller can save the table for the next process."""
    import torch
    from . import LstmCore
    rows = []
    for T in seq_lens:
        p = make_problem(T, B, I, H, seed)
        core = LstmCore(B, I, H)
        core.pack(p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"])
        row: Dict = {"T": T, "B": B, "I": I, "H": H}
        if tuned_table:
            row["tuned_entries_loaded"] = core.set_tuned_table(tuned_table)
        if tune:
            row["untuned"] = {"row_tiles_fwd": core.info("row_tiles_fwd"), "row_tiles_bwd": core.info("row_tiles_bwd")}
            row["tuned"] = core.tune(T, repeats=3, try_stepwise=try_stepwise)
            if tuned_table is not None:
                tuned_table[:] = [r for r in tuned_table if (r["T"], r["B"], r["I"], r["H"]) != (T, B, I, H)]
                tuned_table.extend(r for r in core.tuned_table() if r["T"] == T)
        if check:
            row["parity"] = check_parity(core, p, I, H)
            row["parity_ok"] = all(v <= 1e-2 for v in row["parity"].values())
        fwd = _time_ms(lambda: core.forward(p["x"], p["h0"], p["c0"], want_y=False), warmup, repeats)

        def both():
            core.forward(p["x"], p["h0"], p["c0"], want_y=False)
            core.backward(p["x"], p["dy"])
        fb = _time_ms(both, warmup, repeats)
        flops_f = 8.0 * T * B * H * (I + H)
        row.update({
            "fwd_ms": statistics.median(fwd), "fwd_ms_min": min(fwd),
            "fwd_bwd_ms": statistics.median(fb), "fwd_bwd_ms_min": min(fb),
            "fwd_mfu": flops_f / (statistics.median(fwd) * 1e-3) / (PEAK_FP16_TFLOPS * 1e12),
            "fwd_bwd_mfu": 3 * flops_f / (statistics.median(fb) * 1e-3) / (PEAK_FP16_TFLOPS * 1e12),
            "fwd_bwd_batch_timesteps_per_s": B * T / (statistics.median(fb) * 1e-3),
            "us_per_step_fwd_rec": core.last_ms("fwd_rec") * 1e3 / T,
            "us_per_step_bwd_rec": core.last_ms("bwd_rec") * 1e3 / T,
            "persistent": bool(core.info("persistent_fwd") and core.info("persistent_bwd")),
        })
        core.close()
        if baseline:
            m = torch_lstm(p, I, H)
            state = (p["h0"][None].contiguous(), p["c0"][None].contiguous())
            with torch.no_grad():
                tf = _time_ms(lambda: m(p["x"], state), warmup, repeats)
            xg = p["x"].clone().requires_grad_(True)

            def tboth():
                m.zero_grad(set_to_none=True)
                xg.grad = None
                y, _ = m(xg, state)
                y.backward(p["dy"])
            tfb = _time_ms(tboth, warmup, repeats)
            row.update({"torch_fwd_ms": statistics.median(tf), "torch_fwd_bwd_ms": statistics.median(tfb),
                        "speedup_fwd": statistics.median(tf) / row["fwd_ms"],
                        "speedup_fwd_bwd": statistics.median(tfb) / row["fwd_bwd_ms"]})
        rows.append(row)
        print(format_row(row), flush=True)
    return rows


def format_row(r: Dict) -> str:
    s = (f"T={r['T']:>6}  fwd {r['fwd_ms']:9.3f} ms ({r['fwd_mfu'] * 100:5.1f}% MFU)  "
         f"fwd+bwd {r['fwd_bwd_ms']:9.3f} ms ({r['fwd_bwd_mfu'] * 100:5.1f}% MFU, "
         f"{r['fwd_bwd_batch_timesteps_per_s'] / 1e6:7.3f} M batch*steps/s)  "
         f"step {r['us_per_step_fwd_rec']:.2f}/{r['us_per_step_bwd_rec']:.2f} us")
    if "torch_fwd_ms" in r:
        s += (f"  | nn.LSTM fwd {r['torch_fwd_ms']:9.3f} ms (x{r['speedup_fwd']:.2f})  "
              f"fwd+bwd {r['torch_fwd_bwd_ms']:9.3f} ms (x{r['speedup_fwd_bwd']:.2f})")
    if "tuned" in r:
        t = r["tuned"]
        s += (f"  | tuned: rows/block fwd {16 * t['row_tiles_fwd']} bwd {16 * t['row_tiles_bwd']}, "
              f"{'step-wise' if t['stepwise_fwd'] else 'persistent'}/{'step-wise' if t['stepwise_bwd'] else 'persistent'}, "
              f"dW split-K {t['dw_splits']}")
    if "parity_ok" in r:
        s += "  parity " + ("ok" if r["parity_ok"] else "FAILED " + json.dumps(r["parity"]))
    return s


def tune_dw_splits(B: int, I: int, H: int, T: int, *, candidates: Sequence[int] = (0, 1, 2, 4, 8, 16, 32, 64),
                   warmup: int = 2, repeats: int = 5, seed: int = 2025) -> Dict:
    """Times the weight-gradient phase for every split-K count (0 = the library's own choice) and returns the
    table and the best entry; LstmCore.set_option("dw_splits", best) pins it on a plan."""
    from . import LstmCore
    p = make_problem(T, B, I, H, seed)
    core = LstmCore(B, I, H)
    core.pack(p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"])
    table = {}
    for sp in candidates:
        core.set_option("dw_splits", sp)
        ms = []
        for i in range(warmup + repeats):
            core.forward(p["x"], p["h0"], p["c0"], want_y=False)
            core.backward(p["x"], p["dy"])
            if i >= warmup:
                ms.append(core.last_ms("bwd_dw"))
        table[sp] = statistics.median(ms)
    core.close()
    best = min((k for k in table if k != 0), key=lambda k: table[k])
    return {"T": T, "B": B, "I": I, "H": H, "dw_ms_by_splits": table, "best": best,
            "automatic_over_best": table[0] / table[best] if 0 in table else None}


def main(argv: Optional[Sequence[str]] = None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--input-size", type=int, default=1024)
    ap.add_argument("--hidden-size", type=int, default=1024)
    ap.add_argument("--seq-lens", type=int, nargs="+", default=None)
    ap.add_argument("--seq-len-min", type=int, default=64)
    ap.add_argument("--seq-len-max", type=int, default=4096)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--repeats", type=int, default=10)
    ap.add_argument("--seed", type=int, default=2025)
    ap.add_argument("--no-baseline", action="store_true", help="skip torch.nn.LSTM on the GPU")
    ap.add_argument("--check", action="store_true", help="parity against torch.nn.LSTM (fp32) at every length")
    ap.add_argument("--tune", action="store_true", help="run the library's tuner for every length first (choices are "
                    "cached in the plan and printed)")
    ap.add_argument("--tune-stepwise", action="store_true", help="with --tune: also time one launch per step")
    ap.add_argument("--tuned-table", type=str, default=None, help="JSON file of tuned entries: read (if it exists) "
                    "before the sweep, so that a fresh process starts tuned, and with --tune written back with what "
                    "the tuner found")
    ap.add_argument("--dw-splits-table", action="store_true", help="print the weight-gradient time for every "
                    "split-K count instead of sweeping")
    ap.add_argument("--side-stream", action="store_true", help="run on a stream of its own instead of the default "
                    "stream (step-wise launches can only be captured into a hipGraph off the default stream)")
    ap.add_argument("--csv", type=str, default=None)
    ap.add_argument("--json", type=str, default=None)
    args = ap.parse_args(argv)
    import torch
    if not torch.cuda.is_available():
        print("sweep: no GPU visible", file=sys.stderr)
        return 1
    lens = args.seq_lens
    if not lens:
        lens, t = [], args.seq_len_min
        while t <= args.seq_len_max:
            lens.append(t)
            t *= 2
    if args.side_stream:
        side = torch.cuda.Stream()
        torch.cuda.set_stream(side)
    if args.dw_splits_table:
        results = [tune_dw_splits(args.batch, args.input_size, args.hidden_size, T, seed=args.seed) for T in lens]
        for r in results:
            print(f"T={r['T']}: " + "  ".join(f"{k}:{v:.3f}ms" for k, v in r["dw_ms_by_splits"].items()) +
                  f"  best={r['best']}  automatic/best={r['automatic_over_best']:.3f}")
    else:
        table = None
        if args.tuned_table:
            table = []
            if os.path.exists(args.tuned_table):
                with open(args.tuned_table) as f:
                    table = json.load(f)
        results = sweep(args.batch, args.input_size, args.hidden_size, lens, warmup=args.warmup, repeats=args.repeats,
                        seed=args.seed, baseline=not args.no_baseline, check=args.check, tune=args.tune,
                        try_stepwise=args.tune_stepwise, tuned_table=table)
        if args.tuned_table and args.tune:
            with open(args.tuned_table, "w") as f:
                json.dump(table, f, indent=1)
        if args.csv:
            keys = [k for k in results[0] if k not in ("parity", "tuned", "untuned")]
            with open(args.csv, "w", newline="") as f:
                w = csv.DictWriter(f, fieldnames=keys, extrasaction="ignore")
                w.writeheader()
                w.writerows(results)
    if args.json:
        with open(args.json, "w") as f:
            json.dump(results, f, indent=1)
    return 0


if __name__ == "__main__":
    sys.exit(main())
