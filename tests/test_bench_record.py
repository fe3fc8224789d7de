"""Host-side pieces of bench.py: the HBM traffic figures are read from the committed counter summaries, the
iteration FLOP count follows the layer list, the CPU baseline's partition count follows the reference's rule."""
import os

import pytest

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_traffic_source_exists_and_parses():
    for (workload, kind), path in bench.TRAFFIC_SOURCE.items():
        assert os.path.exists(os.path.join(ROOT, path)), path
        table = bench.parse_traffic_table(path)
        assert table, "no table with fetched / written columns in %s" % path
        assert all(v >= 0 for v in table.values()) and any(v > 0 for v in table.values())


def test_traffic_lookup_is_by_kernel_instance_and_role(tmp_path):
    text = "\n".join([
        "| kernel | calls | fetched MB | written MB |", "|---|---|---|---|",
        "| `k_one<5, 1, 2> (forward launches)` | 3 | 10.0 | 2.5 |",
        "| `k_one<5, 1, 2> (data-gradient launches)` | 3 | 20.0 | 1.0 |",
        "| `k_two<3>` | 9 | 1.5 | - |",
        "| `k_three` | 9 | 4.0 | 4.0 |", ""])
    f = tmp_path / "t.md"
    f.write_text(text)
    table = bench.parse_traffic_table(str(f))
    assert table == {("k_one<5,1,2>", "forward"): 12.5e6, ("k_one<5,1,2>", "data-gradient"): 21e6, ("k_three", ""): 8e6}
    bench.TRAFFIC_SOURCE[("t", "direct")] = str(f)
    try:
        assert bench.traffic_of("t", "direct", "GEMM", "k_one<5,1,2> splits=3") == (12.5e6, str(f))
        assert bench.traffic_of("t", "direct", "GEMM Data", "k_one<5,1,2>") == (21e6, str(f))
        assert bench.traffic_of("t", "direct", "GEMM Wghts", "k_three waves=4") == (8e6, str(f))
        assert bench.traffic_of("t", "direct", "GEMM", "k_one<5,1,4>") == (None, None)   # another instance ran
        assert bench.traffic_of("nothing", "direct", "GEMM", "k_three") == (None, None)
    finally:
        del bench.TRAFFIC_SOURCE[("t", "direct")]


def test_iteration_flop_counts():
    """CaffeNet b=256 with conv2/4/5 in two groups: 1.06e12 FLOP per iteration (conv1 without a data gradient)."""
    pytest.importorskip("numpy")
    total, per_layer = bench.net_flop(bench.net_workload("caffenet"))
    conv1 = 2.0 * 96 * 256 * 55 * 55 * 363
    conv2 = 2.0 * 256 * 256 * 27 * 27 * 25 * 48
    assert per_layer[0] == conv1 and per_layer[4] == conv2
    fc = 2.0 * 256 * (9216 * 4096 + 4096 * 4096 + 4096 * 1000)
    conv = conv1 * 2 + 3 * (conv2 + 2.0 * 256 * 169 * (384 * 9 * 256 + 384 * 9 * 192 + 256 * 9 * 192))
    assert total == pytest.approx(conv + 3 * fc, rel=1e-12)
    assert 1.05e12 < total < 1.07e12
    total_l, _ = bench.net_flop(bench.net_workload("lenet"))
    want = 2.0 * 64 * (2 * 20 * 576 * 25 + 3 * 50 * 64 * 500 + 3 * 800 * 500 + 3 * 500 * 10)
    assert total_l == pytest.approx(want, rel=1e-12)


def test_partition_rule():
    assert [bench.cct_partitions(c, 256) for c in (1, 2, 3, 8, 15, 16, 17, 100)] == [1, 2, 2, 8, 8, 16, 16, 64]
    assert bench.cct_partitions(64, 16) == 16
