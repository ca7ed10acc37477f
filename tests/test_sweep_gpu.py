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
