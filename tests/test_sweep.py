"""Sweep harness: file naming / CSV schema on the CPU, one tiny end-to-end sweep on the GPU."""
import math
import os

import pytest

from linear_cross_entropy_loss_amd import sweep


def test_csv_schema_matches_the_reference_files(tmp_path):
    # The reference's files look like  "N,provider-a,provider-b\n256.000000,67.450302,\n"  (an empty cell where a
    # provider could not run), e.g. bench/bf16 fwd-bwd-Linear+Loss Performance over N. Defaults: ....csv
    p = tmp_path / "bench" / "x.csv"
    sweep._write_csv(str(p), "N", [(256.0, [67.450302, float("nan")]), (512.0, [74.074746, 46.797293])])
    assert p.read_text() == "N,torch-baseline,hip-gfx950\n256.000000,67.450302,\n512.000000,74.074746,46.797293\n"


def test_ranges_are_the_reference_ranges():
    assert [2**i for i in sweep.RANGES["H"]] == [256, 512, 1024, 2048, 4096, 8192]
    assert [2**i for i in sweep.RANGES["V"]][0] == 256 and [2**i for i in sweep.RANGES["V"]][-1] == 131072
    assert [2**i for i in sweep.RANGES["N"]][-1] == 65536 and [2**i for i in sweep.ACC_RANGES["N"]][-1] == 32768
    assert sweep.DEFAULTS == dict(N=16384, H=2048, V=131072)


@pytest.mark.gpu
def test_tiny_sweep_end_to_end(tmp_path, monkeypatch):
    print("tiny sweep", flush=True)
    monkeypatch.setattr(sweep, "DEFAULTS", dict(N=1024, H=512, V=8192))
    monkeypatch.setattr(sweep, "RANGES", {"H": range(8, 10), "V": range(12, 14), "N": range(9, 11)})
    monkeypatch.setattr(sweep, "ACC_RANGES", {"H": range(8, 10), "V": range(12, 14), "N": range(9, 11)})
    files = sweep.run(str(tmp_path), ["speed", "mem", "acc"], ["bf16", "fp16-mixed"], ["N", "V"], quick=False,
                      log=lambda m: None)
    names = sorted(os.path.relpath(f, tmp_path) for f in files)
    assert "bench/bf16 fwd-bwd-Linear+Loss Performance over N. Defaults: N=B*S=16384, H=2048, V=131072.csv" in names
    assert "bench-mem/fp16-mixed fwd-bwd-Linear+Loss Memory Peak over V. Defaults: N=B*S=16384, H=2048, V=131072.csv" in names
    assert "bench-acc/ bwd bf16 Linear+Loss Accuracy over N. Defaults: N=B*S=16384, H=2048, V=131072.csv" in names
    assert len(files) == 2 * 2 + 2 * 2 + 2 * 1 * 2  # speed, mem: 2 modes x 2 vars; acc: fwd/bwd x bf16 x 2 vars
    for f in files:
        lines = open(f).read().strip().split("\n")
        assert lines[0].split(",")[1:] == sweep.PROVIDERS
        for line in lines[1:]:
            cells = line.split(",")
            assert len(cells) == 3 and cells[2] != "", (f, line)  # this package ran every point
            v = float(cells[2])
            assert math.isfinite(v) and v >= 0
            if "Accuracy" in f:
                assert v < 5e-2


@pytest.mark.gpu
def test_heads_and_routes_tables_end_to_end(tmp_path, monkeypatch):
    """The two tables that are not the reference's protocols, on shapes small enough for a test: one line per shape, the
    plan of each column in the routes table, finite times."""
    print("heads / routes tables", flush=True)
    monkeypatch.setattr(sweep, "HEADS", [("tiny", 1024, 256, 4096), ("odd", 1000, 264, 5000)])
    path = sweep.run_heads(str(tmp_path), chunk_sizes=(512, 4096), log=lambda m: None)
    lines = open(path).read().strip().split("\n")
    assert len(lines) == 3 and lines[1].startswith("tiny") and lines[2].startswith("odd")
    for line in lines[1:]:
        assert "nan" not in line and ("one," in line or "two passes" in line)
    monkeypatch.setattr(sweep, "ROUTE_SHAPES", [("tiny", 2048, 256, 4096, 512), ("tiny", 1024, 512, 8192, 4096)])
    path = sweep.run_routes(str(tmp_path), log=lambda m: None)
    lines = open(path).read().strip().split("\n")
    assert len(lines) == 3
    for line in lines[1:]:
        cells = line.split("|")
        assert len(cells) == 6 and cells[4].strip().startswith("(0, 0)")  # (the last route column: two passes)
        assert 1.0 <= float(cells[5]) < 3.0
