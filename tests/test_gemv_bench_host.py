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
