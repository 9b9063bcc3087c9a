"""The operator benchmark on the GPU: one cell of the launch-shape sweep and one line of the
table mode run end to end (tiny problems; this checks the tool, not the numbers)."""
import csv

import pytest

pytestmark = pytest.mark.gpu


def test_one_sweep_cell_and_one_table_line(tmp_path, capsys):
    from msd_pytorch_amd import _native, benchmark_ops as bo
    out = tmp_path / "sweep.csv"
    rc = bo.main(["--sweep", "--ndim", "3", "--size", "16", "16", "64", "--channels", "5", "--dilations", "2",
                  "--ops", "forward", "backward_xkb", "--limit", "3", "--trials", "1", "--csv", str(out)])
    assert rc == 0
    rows = list(csv.DictReader(open(out)))
    assert len(rows) == 2 * 4 and rows[0]["setting"] == "default" and rows[4]["setting"] == "default"
    assert {r["op"] for r in rows} == {"forward", "backward_xkb"}
    assert all(float(r["us"]) > 0 and float(r["GBps"]) > 0 for r in rows)
    text = capsys.readouterr().out
    assert "best" in text and "[4 settings]" in text
    # the sweep leaves every knob at the library default
    lib = _native.load()
    for key in bo.SWEEP_GRID["forward"][3]:
        assert lib.msd_set_tuning(key.encode(), -1) == 0
    rc = bo.main(["--ndim", "2", "--size", "128", "--channels", "3", "--dilations", "1", "--trials", "1"])
    assert rc == 0
    assert "forward" in capsys.readouterr().out
