"""The files at the repository's root that other programs call: no GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_the_benchmark_says_that_it_runs_on_one_gpu_and_exits_with_2():
    for n in ("2", "8"):
        r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", n, "--steps", "3", "--warmup", "1"],
                           capture_output=True, text=True, timeout=300, cwd=ROOT)
        assert r.returncode == 2, (r.returncode, r.stderr[-500:])
        lines = [l for l in r.stdout.splitlines() if l.strip()]
        assert len(lines) == 1 and "one GPU" in lines[0] and f"--gpus {n}" in lines[0]


def test_the_benchmark_refuses_sizes_of_its_single_points_that_it_does_not_run():
    for args, said in ((["--sampling", "0"], "--sampling"), (["--sampling", "8,1.5"], "--sampling"),
                       (["--prefill-only", "--prefill-tokens", "1"], "--prefill-tokens"), (["--layers", "99"], "--layers")):
        r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300, cwd=ROOT)
        assert r.returncode == 2 and said in r.stdout, (args, r.returncode, r.stdout[-300:], r.stderr[-300:])


def test_the_entry_file_has_build_and_smoke_and_the_replay_program_explains_itself():
    sys.path.insert(0, ROOT)
    try:
        import __graft_entry__ as entry
    finally:
        sys.path.remove(ROOT)
    assert callable(entry.build) and callable(entry.smoke)
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--help"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0
    for option in ("--model", "--dtype", "--out", "--max-tokens", "bfloat16", "float32"):
        assert option in r.stdout
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", "/nonexistent", "--dtype", "float32", "--out", "/tmp/x"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 2 and "--max-tokens" in r.stderr          # an option is missing: argparse's own message


def test_without_a_gpu_the_replay_program_and_the_engine_say_so(tmp_path):
    import pytest
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible here")
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from tiny_configs import model_dir
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir("A"), "--dtype", "float32", "--out", str(tmp_path),
                        "--max-tokens", "64"], input="", capture_output=True, text=True, timeout=300)
    assert r.returncode == 1 and "trace_run: error: trace replay runs on the GPU; no GPU is visible" in r.stderr
    from pico_vllm_amd import LLM
    with pytest.raises(RuntimeError, match="no GPU is visible"):
        LLM(model=model_dir("A"), dtype="float32")
