"""The device check-up programs of the package (`python -m autort.utils.memtest / fp32test / mmtest / export`,
README.md:43-55, 128-150)."""
import io
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_modules_import_and_the_fp32_kernel_compiles_without_a_gpu(tmp_path, monkeypatch):
    monkeypatch.setenv('AUTORT_CACHE_DIR', str(tmp_path / 'cache'))
    import autort.utils.export  # noqa: F401
    import autort.utils.memtest as memtest
    import autort.utils.mmtest  # noqa: F401
    from antares_amd.autort.op import compile_cached
    from antares_amd.autort.utils import fp32test
    assert len(compile_cached(fp32test.SOURCE)) > 1000
    props = {'memory_clock_khz': 2_000_000, 'memory_bus_width_bits': 8192, 'compute_units': 256, 'clock_khz': 2_400_000}
    assert abs(memtest.theoretical_gbps(props) - 8192.0) < 1e-6
    assert abs(fp32test.theoretical_tflops(props) - 157.2864) < 1e-3


@pytest.mark.gpu
def test_memtest_and_fp32test_report_plausible_rates():
    from antares_amd.autort.utils import fp32test, memtest
    out = io.StringIO()
    gbps = memtest.run(rounds=5, mib=256, out=out)
    assert 1000.0 < gbps < 8000.0 and re.search(r'\[5/5\] AutoRT Device Memory Bandwidth: \(Actual ~= [\d.]+ GB/s\)', out.getvalue())
    out = io.StringIO()
    tflops = fp32test.run(rounds=5, out=out)
    assert 20.0 < tflops < 160.0 and 'AutoRT FP32 TFLOPS' in out.getvalue()


@pytest.mark.gpu
def test_export_tunes_gemm_f32_and_mmtest_uses_the_module_file_in_a_new_process(tmp_path):
    """`autort.utils.export` writes `gemm_f32.mod` with the winning launch configuration; `autort.utils.mmtest`, started
    as a new process, finds the operator there, checks its result against a float64 product and prints its rate."""
    env = dict(os.environ, AUTORT_OPS_DIR=str(tmp_path / 'ops'), AUTORT_CACHE_DIR=str(tmp_path / 'cache'), PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, '-m', 'autort.utils.export', '-s', '3', '--size', '2048'], env=env, capture_output=True, text=True,
                       timeout=110, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    assert 'Module file for operator `gemm_f32` has been exported to' in r.stdout
    path = tmp_path / 'ops' / 'gemm_f32.mod'
    assert path.is_file() and '"tuned"' in path.read_text()[:20000]
    r = subprocess.run([sys.executable, '-m', 'autort.utils.mmtest', '--size', '2048'], env=env, capture_output=True, text=True, timeout=110,
                       cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    m = re.search(r'`MM-Perf` \(current\) = ([\d.]+) TFLOPS', r.stdout)
    assert m and float(m.group(1)) > 1.0
