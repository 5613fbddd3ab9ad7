"""The three example drivers end to end (CLI -> matmul.apply -> HIP kernel ->
validate_gemm), at small sizes."""

import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))


def run_example(tmp_path, example, *argv):
    out = tmp_path / "log.json"
    cmd = [sys.executable, "-u", os.path.join(ROOT, "examples", example, "benchmark.py"), "--output_file", str(out),
           "--heap_size", str(1 << 28), *argv]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300, cwd=str(tmp_path))
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    return json.loads(out.read_text()), proc.stdout


@pytest.mark.parametrize("example,extra", [
    ("07_gemm_all_scatter", ["--BLK_M", "256", "--BLK_N", "64"]),
    ("08_gemm_atomics_all_reduce", ["--BLK_M", "256", "--BLK_N", "128"]),
    ("09_gemm_one_shot_all_reduce", ["--BLK_M", "256", "--BLK_N", "256"]),
])
def test_example_validates(tmp_path, example, extra):
    data, stdout = run_example(tmp_path, example, "-m", "1024", "-n", "768", "-k", "512", "--datatype", "bf16", "-v",
                               "-d", *extra)
    assert data["success"] is True
    assert data["world_size"] == 1 and data["gemm_sms"] == 256
    assert data["gemm_registers"] > 0
    # the plain builds keep everything in registers; the build that also reduces each tile inside the program (09's
    # default phase) spills a few lane constants around that reduce on the 128-accumulator tiles
    assert data["gemm_spills"] == 0 or (example.startswith("09") and data["gemm_spills"] <= 128)
    assert "Final C validation passed." in stdout and "registers used" in stdout


@pytest.mark.parametrize("example", ["07_gemm_all_scatter", "08_gemm_atomics_all_reduce", "09_gemm_one_shot_all_reduce"])
def test_example_validates_with_fp32_operands(tmp_path, example):
    """``--datatype fp32`` of the reference scripts (09's benchmark.py:41-46): fp32 operands, fp32 C."""
    data, stdout = run_example(tmp_path, example, "-m", "512", "-n", "384", "-k", "256", "--datatype", "fp32", "-v",
                               "--virtual_ranks", "2")
    assert data["success"] is True and data["world_size"] == 2
    assert data["gemm_spills"] == 0
    assert "Final C validation passed." in stdout


def test_one_shot_example_with_virtual_ranks_and_benchmark(tmp_path):
    data, _ = run_example(tmp_path, "09_gemm_one_shot_all_reduce", "-m", "512", "-n", "512", "-k", "1024",
                          "--datatype", "fp16", "-v", "-b", "--virtual_ranks", "4", "--BLK_N", "128")
    assert data["success"] is True and data["world_size"] == 4 and data["k"] == 256
    assert data["triton_ms"] > 0 and data["triton_tflops"] > 0 and data["gemm_experiments"] == 126


@pytest.mark.parametrize("example,extra", [
    ("07_gemm_all_scatter", ["--BLK_M", "256", "--BLK_N", "64"]),
    ("08_gemm_atomics_all_reduce", ["--BLK_M", "128", "--BLK_N", "128"]),
    ("09_gemm_one_shot_all_reduce", ["--BLK_M", "256", "--BLK_N", "128"]),
])
def test_example_with_one_process_per_rank(tmp_path, example, extra):
    """The reference's way of running the examples, `mpirun -np 2 python
    benchmark.py`, with the launcher's environment in MPI's place: two
    processes, two heaps mapped over IPC, and for 09 the reference's single
    program (produce, signal, wait, reduce) on both ranks at once."""
    out = tmp_path / "log.json"
    procs = []
    for r in range(2):
        env = dict(os.environ, RANK=str(r), WORLD_SIZE="2", IRIS_AMD_RENDEZVOUS=f"file://{tmp_path / 'store'}",
                   IRIS_AMD_RENDEZVOUS_TIMEOUT="120", HSA_ENABLE_IPC_MODE_LEGACY="0")
        env.pop("IRIS_AMD_VIRTUAL_RANKS", None)
        # 07 runs with the scripts' default heap size, which one process per rank clamps to what IPC maps here
        heap = [] if example.startswith("07") else ["--heap_size", str(1 << 28)]
        cmd = [sys.executable, "-u", os.path.join(ROOT, "examples", example, "benchmark.py"), "--output_file", str(out),
               *heap, "-m", "1024", "-n", "768", "-k", "1024", "--datatype", "bf16", "-v", *extra]
        procs.append(subprocess.Popen(cmd, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                                      cwd=str(tmp_path)))
    outs = []
    try:
        for p in procs:
            outs.append(p.communicate(timeout=280)[0])
    finally:
        for p in procs:
            if p.poll() is None:
                p.kill()
    for r, (p, text) in enumerate(zip(procs, outs)):
        assert p.returncode == 0 and "Final C validation passed." in text, f"rank {r}:\n" + text[-3000:]
    data = json.loads(out.read_text())
    assert data["success"] is True and data["world_size"] == 2
    assert data["gemm_sms"] == 128  # two ranks share the 256 CUs, whatever the algorithm
    if example.startswith("07"):
        assert data["heap_size"] == (2 << 30) - (1 << 20) and "heap_size defaults to" in outs[0]
