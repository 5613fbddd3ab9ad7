"""The multi-rank bootstrap on one GPU (iris/iris.py:53-77 without MPI): the
parent starts one fresh process per rank; each allocates its heap, exchanges
IPC handles through a file store, maps its peers and runs the checks of
``multiprocess_child.py`` against the real mapped heaps."""

import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.parametrize("world", [2, 4])
def test_ranks_in_separate_processes_share_heaps_over_ipc(tmp_path, world):
    procs = []
    for r in range(world):
        env = dict(os.environ, RANK=str(r), WORLD_SIZE=str(world), IRIS_AMD_RENDEZVOUS=f"file://{tmp_path / 'store'}",
                   IRIS_AMD_RENDEZVOUS_TIMEOUT="120", HSA_ENABLE_IPC_MODE_LEGACY="0")
        env.pop("IRIS_AMD_VIRTUAL_RANKS", None)
        procs.append(subprocess.Popen([sys.executable, "-u", os.path.join(HERE, "multiprocess_child.py")], env=env,
                                      stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, cwd=str(tmp_path)))
    outs = []
    try:
        for p in procs:
            outs.append(p.communicate(timeout=280)[0])
    finally:
        for p in procs:
            if p.poll() is None:
                p.kill()
    for r, (p, out) in enumerate(zip(procs, outs)):
        assert p.returncode == 0 and f"RANK {r} OK" in out, f"rank {r}:\n" + out[-3000:]
