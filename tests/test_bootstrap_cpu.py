"""The rank bootstrap (iris_amd/_bootstrap.py) on the CPU: three processes
rendezvous through a file store or a TCP store and run the collectives the
Iris context needs, with the results the reference's MPI helpers give
(iris/_mpi_helpers.py:8-51)."""

import os
import socket
import subprocess
import sys

import numpy as np
import pytest

from iris_amd import _bootstrap

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))

CHILD = r"""
import sys
sys.path.insert(0, {root!r})
import numpy as np
from iris_amd import _bootstrap
comm = _bootstrap.init_comm()
assert comm is not None and comm.size == {world}
r = comm.rank
handles = comm.allgather(np.full(64, r + 1, dtype=np.uint8))          # the 64-byte IPC handles
assert handles.shape == ({world}, 64) and [int(h[0]) for h in handles] == list(range(1, {world} + 1))
bases = comm.allgather(np.array([0x7f0000000000 + (r << 32)], dtype=np.uint64))
assert bases.dtype == np.uint64 and [int(b[0]) for b in bases] == [0x7f0000000000 + (q << 32) for q in range({world})]
comm.barrier()
v = comm.broadcast_scalar(3.5 + r if r == 1 else None, root=1)
assert float(v) == 4.5
n = comm.broadcast_scalar(np.int64(41 + r) if r == 0 else None, root=0)
assert int(n) == 41
# one-byte element types (their dtype names start with '|')
assert bool(comm.broadcast_scalar(True if r == 0 else None, root=0)) is True
assert int(comm.broadcast_scalar(np.int8(-7) if r == 0 else None, root=0)) == -7
assert int(comm.broadcast_scalar(np.uint8(200) if r == 1 else None, root=1)) == 200
for _ in range(5):
    comm.barrier()
print("RANK", r, "OK")
"""


def run_ranks(tmp_path, world, env_extra):
    script = tmp_path / "child.py"
    script.write_text(CHILD.format(root=ROOT, world=world))
    procs = []
    for r in range(world):
        env = dict(os.environ, RANK=str(r), WORLD_SIZE=str(world), **env_extra)
        env.pop("IRIS_AMD_VIRTUAL_RANKS", None)
        procs.append(subprocess.Popen([sys.executable, "-u", str(script)], env=env, stdout=subprocess.PIPE,
                                      stderr=subprocess.STDOUT, text=True))
    outs = [p.communicate(timeout=120)[0] for p in procs]
    for r, (p, out) in enumerate(zip(procs, outs)):
        assert p.returncode == 0 and f"RANK {r} OK" in out, out[-2000:]


def test_file_rendezvous(tmp_path):
    run_ranks(tmp_path, 3, {"IRIS_AMD_RENDEZVOUS": f"file://{tmp_path / 'store'}", "IRIS_AMD_RENDEZVOUS_TIMEOUT": "60"})


def test_tcp_rendezvous_from_the_launcher_environment(tmp_path):
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
    run_ranks(tmp_path, 2, {"MASTER_ADDR": "127.0.0.1", "MASTER_PORT": str(port), "IRIS_AMD_RENDEZVOUS_TIMEOUT": "60"})


def test_a_process_on_its_own_has_no_communicator(monkeypatch):
    for k in ("RANK", "WORLD_SIZE", "IRIS_AMD_RENDEZVOUS", "OMPI_COMM_WORLD_SIZE", "PMI_SIZE", "PMIX_RANK"):
        monkeypatch.delenv(k, raising=False)
    assert _bootstrap.init_comm() is None
    monkeypatch.setenv("WORLD_SIZE", "1")
    monkeypatch.setenv("RANK", "0")
    assert _bootstrap.init_comm() is None
    monkeypatch.setenv("WORLD_SIZE", "2")
    monkeypatch.setenv("IRIS_AMD_RENDEZVOUS", "carrier-pigeon://x")
    with pytest.raises(ValueError):
        _bootstrap.init_comm()


def test_store_comm_rejects_a_rank_outside_the_world():
    with pytest.raises(ValueError):
        _bootstrap.StoreComm(None, 2, 2)
