"""Host-side pieces of bench.py: the algorithmic-work formulas (SURVEY section 8d's figures) and the rule that a
recorded counter value is only printed for the kernel it was recorded on.  No GPU involved."""
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_algorithmic_flops_of_the_baseline_configs(bench):
    # 4 * D * B * H * pairs, pairs = W(W+1)/2 + (T-W) W with a window, T(T+1)/2 without
    assert bench.prefill_flops(1, 256, 4, 64, 128) == pytest.approx(2.523e7, rel=1e-3)               # config 1
    assert bench.prefill_flops(8, 4096, 8, 128, 1024) == pytest.approx(1.2028e11, rel=1e-4)          # config 2
    assert bench.prefill_flops(1, 65536, 16, 128, 2048) == pytest.approx(1.0823e12, rel=1e-4)        # config 3, window
    assert bench.prefill_flops(1, 65536, 16, 128, None) == pytest.approx(1.7592e13, rel=1e-4)        # config 3, full causal
    assert bench.prefill_flops(1, 100, 1, 64, 100) == bench.prefill_flops(1, 100, 1, 64, None)       # a window of T is no window
    import oracle.attention
    for args in ((8, 4096, 8, 128, 1024), (1, 65536, 16, 128, None), (2, 300, 3, 64, 17)):
        assert bench.prefill_flops(*args) == oracle.attention.prefill_flops(*args)


def test_recorded_traffic_is_tied_to_the_kernel_it_was_recorded_on(bench, tmp_path):
    nbytes, source = bench.recorded_traffic(bench.PREFILL_C2_TRAFFIC_FILE, bench.PREFILL_C2_KERNEL)
    assert nbytes is not None and 268_435_456 <= nbytes <= 2 * 268_435_456, (nbytes, source)     # between 1x and 2x the minimum
    assert bench.PREFILL_C2_KERNEL in source and "not measured by this run" in source
    # the kernel named in the summary must exist in the sources
    name = bench.PREFILL_C2_KERNEL.split("<")[0]
    with open(os.path.join(ROOT, "daisy_amd", "csrc", "prefill.hip")) as f:
        assert f"void {name}(" in f.read()
    # a summary of another kernel, a summary without the line, a missing file: no figure
    other, why = bench.recorded_traffic(bench.PREFILL_C2_TRAFFIC_FILE, "prefill_other_kernel<128>")
    assert other is None and "figure not used" in why
    rel = os.path.relpath(str(tmp_path / "no_line.txt"), ROOT)
    (tmp_path / "no_line.txt").write_text("FETCH_SIZE 1\n")
    assert bench.recorded_traffic(rel, bench.PREFILL_C2_KERNEL)[0] is None
    assert bench.recorded_traffic(os.path.join("profiles", "does_not_exist.txt"), bench.PREFILL_C2_KERNEL)[0] is None


def test_more_than_one_gpu_is_refused(bench, monkeypatch):
    monkeypatch.setattr("sys.argv", ["bench.py", "--gpus", "2"])
    with pytest.raises(SystemExit) as e:
        bench.main()
    assert "one GPU" in str(e.value)
