"""bench.py's command line, as far as it can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    """Everything here runs on one GPU: `--gpus N` with N above 1 says so and exits before it touches a device."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, 'bench.py'), '--gpus', '2'], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert 'one GPU' in r.stderr and r.stdout.strip() == ''


def test_help_lists_the_stand_alone_legs():
    r = subprocess.run([sys.executable, os.path.join(ROOT, 'bench.py'), '--help'], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0
    for flag in ('--read-floor', '--stream-floors', '--phase-chain', '--attention', '--gemv-knobs', '--lowering', '--calibrate-copy', '--no-cpu'):
        assert flag in r.stdout, flag
