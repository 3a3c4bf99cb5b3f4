"""The package's counterparts of the reference's two scripts (numeric_tests.py, bench_swiglu.py), run in-process
on reduced sweeps."""
import io

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_numeric_sweep_statistics(ext):
    import numeric_tests
    buf = io.StringIO()
    res = numeric_tests.run([1024, 2048], iterations=3, seed=0, out=buf)
    text = buf.getvalue()
    assert "MNK" in text and "Relative Diff" in text and text.count("\n") == 2 + 2 * 4
    for mnk in (1024, 2048):
        p20, p80, mean, std = res[mnk]["Relative Diff"]
        # against torch's own bf16 evaluation (three roundings of its own) the reference sees ~1e-2..1e-3 too
        assert 0 <= p20 <= p80 < 2e-2 and mean < 2e-2
        # against fp32 the only error left is our single rounding to bf16
        assert res[mnk]["Relative Diff vs fp32"][2] < 4e-3
        assert res[mnk]["Max Abs Diff"][1] < 5e-2
    # seeded runs repeat exactly
    res2 = numeric_tests.run([1024], iterations=2, seed=5, out=io.StringIO())
    res3 = numeric_tests.run([1024], iterations=2, seed=5, out=io.StringIO())
    assert res2 == res3


def test_uniform_input_law():
    import numeric_tests
    g = torch.Generator(device="cuda:0").manual_seed(1)
    t = numeric_tests.uniform_like_kaiming(512, 1024, "cuda:0", g).float()
    assert t.abs().max().item() <= 1 / 32 + 1e-3 and abs(t.std().item() - (1 / 32) / 3 ** 0.5) < 2e-3


def test_benchmark_sweep_small(ext, tmp_path):
    import bench_swiglu
    assert bench_swiglu.reference_flops(8192, 28672, 4096) == 1924615110656  # bench_swiglu.py:117
    csv = tmp_path / "r.csv"
    rows = bench_swiglu.run([512], k=1024, n=2048, out=io.StringIO(), csv=str(csv))
    assert [r[1] for r in rows] == ["hipBLASLt+eager", "Fused"]
    for r in rows:
        assert r[2] > 0 and r[4] <= r[3] <= r[5]
    assert csv.read_text().startswith("Tokens,provider,ms,tflops")
    rows = bench_swiglu.run([128], k=1024, n=2048, out=io.StringIO(), forward=True)
    assert [r[1] for r in rows] == ["hipBLASLt+eager", "Fused", "hipBLASLt forward", "Fused forward"]
    assert all(r[2] > 0 for r in rows)
