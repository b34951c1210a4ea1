"""Host-side pieces of the GEMV sweep tool: presets, byte counts, argument parsing."""
import pytest

from bitmtp_amd import gemv_bench as gb


def test_algorithmic_bytes_match_the_published_examples():
    # packed weights + bf16 group scales: T2 0.265625 N K, Q1 0.140625 N K
    assert gb.gemv_bytes("t2", 6144, 2048) == 3_342_336
    assert gb.gemv_bytes("t2", 151936, 2048) == 82_653_184
    assert gb.gemv_bytes("t2", 2560, 9728) == 6_615_040
    assert gb.gemv_bytes("q1", 9728, 9728) == 13_307_904
    assert gb.gemv_bytes("q1", 1024, 2560) == 368_640


def test_presets_cover_the_registered_layer_shapes():
    assert sum(gb.gemv_bytes("t2", n, k) * (2 if (n, k) in ((2048, 2048), (1024, 2048), (6144, 2048)) else 1)
               for n, k in gb.PRESETS["layer-1.7b"]) == 13_369_344
    assert sum(gb.gemv_bytes("t2", n, k) for n, k in gb.PRESETS["merged-1.7b"]) == 13_369_344
    assert len(gb.PRESETS["config4"]) == 6
    assert all(k % 128 == 0 for shapes in gb.PRESETS.values() for _, k in shapes)


def test_width_and_shape_parsing():
    assert gb.parse_widths("1-8") == list(range(1, 9))
    assert gb.parse_widths("1,4,8") == [1, 4, 8]
    assert gb.parse_widths("1-2,9,16-17") == [1, 2, 9, 16, 17]
    with pytest.raises(ValueError):
        gb.parse_widths("0-3")
    assert gb.parse_shapes("9728x2560,2560X9728") == [(9728, 2560), (2560, 9728)]


def test_cli_needs_exactly_one_of_preset_and_shapes(monkeypatch, capsys):
    monkeypatch.setattr("sys.argv", ["gemv_bench"])
    assert gb.main() == 2
    monkeypatch.setattr("sys.argv", ["gemv_bench", "--preset", "head", "--shapes", "128x128"])
    assert gb.main() == 2


def test_bench_refuses_more_than_one_gpu(capsys):
    """bench.py is a one-GPU measurement: any other --gpus exits with a message and status 2
    before anything touches a device."""
    import subprocess
    import sys
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode == 2 and "one GPU" in proc.stderr and proc.stdout.strip() == ""


def test_traffic_table_matches_the_layer_bytes():
    """The measured HBM traffic bench.py reports comes from profiles/traffic.json; every width's
    figure is the counters' own arithmetic and lies within 10 % above the algorithmic bytes."""
    import bench
    for width in (1, 4, 8):
        t = bench.measured_traffic(width)
        assert t is not None and bench.LAYER_BYTES <= t <= 1.10 * bench.LAYER_BYTES
    assert bench.measured_traffic(5) is None
    assert bench.LAYER_BYTES == sum(bench.t2_bytes(n, k) for _, n, k in bench.PROJECTIONS) == 13369344


def test_kernel_choices_of_the_sweep_tool():
    from bitmtp_amd import gemv_bench
    assert gemv_bench.KERNELS["auto"] == (0, 0)
    assert set(gemv_bench.KERNELS) >= {"auto", "dot4", "staged", "operand", "lean", "stream", "single-token"}
