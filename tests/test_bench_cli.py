"""bench.py's command line, as far as it can be checked without a GPU: the layer does not span GPUs, and a run
asked for more than one says so instead of measuring something else."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*args, env=None):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=120, env=env)


def test_more_than_one_gpu_is_refused_with_a_message():
    out = _bench("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert out.returncode != 0
    assert "ONE GPU" in out.stderr and out.stdout.strip() == ""


def test_a_launcher_world_size_above_one_is_refused_too():
    out = _bench("--gpus", "1", env=dict(os.environ, WORLD_SIZE="2"))
    assert out.returncode != 0 and "ONE GPU" in out.stderr


def test_help_names_the_suite_and_the_contract_flags():
    out = _bench("--help")
    assert out.returncode == 0
    for word in ("--gpus", "--steps", "--warmup", "--workload", "qwen3-decode", "kimi-prefill"):
        assert word in out.stdout
