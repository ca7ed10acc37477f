"""The sequence-length sweep and the split-K tuner (flashlstm_poc_amd/sweep.py; counterparts of the reference's
python/benchmark_lstm.py and src/tune_projchunksz.cu) run end to end on small shapes, with parity switched on."""
import pytest

pytestmark = pytest.mark.gpu


def test_sweep_reports_every_length_with_parity(tmp_path):
    from flashlstm_poc_amd import sweep
    out = tmp_path / "sweep.csv"
    rc = sweep.main(["--batch", "8", "--input-size", "64", "--hidden-size", "96", "--seq-lens", "16", "40", "--warmup", "1",
                     "--repeats", "2", "--check", "--csv", str(out), "--json", str(tmp_path / "sweep.json")])
    assert rc == 0
    lines = out.read_text().strip().splitlines()
    assert len(lines) == 3 and lines[0].startswith("T,B,I,H")
    rows = sweep.sweep(8, 64, 96, [24], warmup=1, repeats=2, baseline=True, check=True)
    r = rows[0]
    assert r["parity_ok"], r["parity"]
    assert r["fwd_ms"] > 0 and r["fwd_bwd_ms"] > r["fwd_ms"] and r["torch_fwd_bwd_ms"] > 0
    assert 0 < r["fwd_bwd_mfu"] < 1


def test_tuner_returns_a_table_and_the_automatic_choice_is_close_to_the_best():
    from flashlstm_poc_amd import sweep
    r = sweep.tune_dw_splits(32, 256, 256, 64, candidates=(0, 1, 2, 4, 8, 16), warmup=1, repeats=3)
    assert set(r["dw_ms_by_splits"]) == {0, 1, 2, 4, 8, 16} and r["best"] in (1, 2, 4, 8, 16)
    assert r["automatic_over_best"] < 4.0   # launches of ~50 us: only a grossly wrong automatic choice fails this


def test_plan_caches_the_tuned_choice_per_sequence_length():
    # flstm_core_tune: the choice lands in the plan, is read back through get_info, applies to passes of similar
    # length only, loses against explicit options, and never changes results beyond summation order.
    import torch
    from flashlstm_poc_amd import LstmCore, sweep
    B, I, H, T = 16, 128, 256, 48          # 16 rows: both 16- and 32-row blocks are possible
    p = sweep.make_problem(T, B, I, H, seed=3)
    core = LstmCore(B, I, H)
    core.pack(p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"])
    y0, hy0, cy0 = core.forward(p["x"], p["h0"], p["c0"])
    g0 = core.backward(p["x"], p["dy"])
    assert core.info("tuned_entries") == 0 and core.info("tuned_T") == 0
    t = core.tune(T, repeats=2, try_stepwise=True)
    assert core.info("tuned_entries") == 1 and t["T"] == T
    assert t["row_tiles_fwd"] in (1, 2) and t["row_tiles_bwd"] in (1, 2) and t["dw_splits"] >= 1
    assert t["stepwise_fwd"] in (0, 1) and t["fwd_rec_ms"] > 0 and t["bwd_rec_ms"] > 0 and t["bwd_dw_ms"] > 0
    y1, hy1, cy1 = core.forward(p["x"], p["h0"], p["c0"])
    g1 = core.backward(p["x"], p["dy"])
    assert core.info("tuned_T") == T
    assert core.info("row_tiles_fwd") == t["row_tiles_fwd"] and core.info("row_tiles_bwd") == t["row_tiles_bwd"]
    assert core.info("persistent_fwd") == 1 - t["stepwise_fwd"]
    assert torch.equal(y0, y1) and torch.equal(cy0, cy1)          # the forward pass does not depend on the choice
    for a, b in zip(g0, g1):
        assert ((a.float() - b.float()).norm() / b.float().norm()).item() <= 1e-5
    # a sequence eight times longer is outside the tuned entry's range: rules of thumb again
    long = sweep.make_problem(8 * T, B, I, H, seed=4)
    core.forward(long["x"], long["h0"], long["c0"])
    assert core.info("tuned_T") == 0 and core.info("tuned_dw_splits") == 0
    # explicit options win over the tuned entry
    core.set_option("row_tiles_fwd", 3 - t["row_tiles_fwd"])
    core.forward(p["x"], p["h0"], p["c0"])
    assert core.info("row_tiles_fwd") == 3 - t["row_tiles_fwd"] and core.info("tuned_row_tiles_fwd") == t["row_tiles_fwd"]
    core.set_option("row_tiles_fwd", 0)
    core.set_option("clear_tuned", 1)
    assert core.info("tuned_entries") == 0
    core.close()


def test_sweep_with_tuning_prints_the_choices(capsys):
    from flashlstm_poc_amd import sweep
    rc = sweep.main(["--batch", "16", "--input-size", "64", "--hidden-size", "128", "--seq-lens", "32", "--warmup", "1",
                     "--repeats", "2", "--tune", "--no-baseline"])
    assert rc == 0
    assert "tuned: rows/block" in capsys.readouterr().out


def test_tuned_table_survives_the_process_through_a_file(tmp_path):
    # What the tuner found is written to a JSON file and read into a FRESH plan (flstm_core_get_tuned /
    # flstm_core_set_tuned): the new plan starts with the same choices in force, without tuning.
    import json
    from flashlstm_poc_amd import LstmCore, sweep
    B, I, H, T = 16, 128, 256, 48
    path = tmp_path / "tuned.json"
    rc = sweep.main(["--batch", str(B), "--input-size", str(I), "--hidden-size", str(H), "--seq-lens", str(T), "--warmup", "1",
                     "--repeats", "2", "--tune", "--no-baseline", "--tuned-table", str(path)])
    assert rc == 0
    table = json.loads(path.read_text())
    assert len(table) == 1 and table[0]["T"] == T and (table[0]["B"], table[0]["I"], table[0]["H"]) == (B, I, H)
    assert table[0]["row_tiles_fwd"] in (1, 2) and table[0]["dw_splits"] >= 1
    p = sweep.make_problem(T, B, I, H, seed=5)
    core = LstmCore(B, I, H)
    core.pack(p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"])
    assert core.info("tuned_entries") == 0
    assert core.set_tuned_table(table + [dict(table[0], B=B + 1)]) == 1      # rows of other sizes are skipped
    assert core.info("tuned_entries") == 1 and core.tuned_table()[0] == table[0]
    core.forward(p["x"], p["h0"], p["c0"])
    core.backward(p["x"], p["dy"])
    assert core.info("tuned_T") == T and core.info("row_tiles_fwd") == table[0]["row_tiles_fwd"]
    assert core.info("tuned_dw_splits") == table[0]["dw_splits"]
    # values out of range are refused
    assert core.lib.flstm_core_set_tuned(core._h, T, 3, 0, 0, 0, 0, -1) == 1
    core.close()


def test_tuner_tries_the_layouts_of_the_backward_recurrence_at_2048_units():
    # 2048 hidden units: the two-way split of the backward recurrence is one of the tuner's candidates (bwd_two_d 0 / 1 /
    # 2) unless the option was set explicitly; results do not depend on what it picks beyond summation order.
    import torch
    from flashlstm_poc_amd import LstmCore, sweep
    B, I, H, T = 48, 64, 2048, 12
    p = sweep.make_problem(T, B, I, H, seed=6)
    core = LstmCore(B, I, H)
    core.pack(p["w_ih"], p["w_hh"], p["b_ih"], p["b_hh"])
    core.forward(p["x"], p["h0"], p["c0"])
    g0 = core.backward(p["x"], p["dy"])
    t = core.tune(T, repeats=1)
    assert t["bwd_two_d"] in (-1, 0, 1, 2) and t["bwd_rec_ms"] > 0
    core.forward(p["x"], p["h0"], p["c0"])
    g1 = core.backward(p["x"], p["dy"])
    assert core.info("tuned_bwd_two_d") == t["bwd_two_d"]
    if t["bwd_two_d"] >= 0:
        assert core.info("bwd_two_d") == (1 if t["bwd_two_d"] > 0 and core.info("bwd_two_d") else core.info("bwd_two_d"))
    for a, b in zip(g0, g1):
        assert ((a.float() - b.float()).norm() / b.float().norm()).item() <= 2e-3
    core.set_option("bwd_two_d", 0)          # an explicit option wins over the tuned entry
    core.forward(p["x"], p["h0"], p["c0"]); core.backward(p["x"], p["dy"])
    assert core.info("bwd_two_d") == 0
    core.close()
