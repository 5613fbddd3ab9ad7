"""Rank bootstrap of the symmetric heap: who am I, how many are we, and the
three host-side collectives ``Iris.__init__`` and ``Iris.barrier`` need
(all-gather of a small array, broadcast of a scalar, barrier).

The reference does this with mpi4py (iris/_mpi_helpers.py:8-51).  Here MPI is
one of two transports:

* ``MpiComm`` -- mpi4py, when it is importable and the process was started by
  an MPI launcher (the reference's path, same calls);
* ``StoreComm`` -- a ``torch.distributed`` key-value store (``TCPStore`` or
  ``FileStore``) used as a plain host-side rendezvous: no process group, no
  collective ever touches a device tensor.  Chosen by the environment
  ``torchrun`` sets (``RANK``, ``WORLD_SIZE``, ``MASTER_ADDR``,
  ``MASTER_PORT``) or by ``IRIS_AMD_RENDEZVOUS=file:///path`` /
  ``tcp://host:port`` together with ``RANK`` and ``WORLD_SIZE``.

``init_comm()`` returns ``None`` for a process that is on its own.
"""

from __future__ import annotations

import datetime
import importlib.util
import os

import numpy as np

__all__ = ["StoreComm", "MpiComm", "init_comm"]

_TIMEOUT_S = float(os.environ.get("IRIS_AMD_RENDEZVOUS_TIMEOUT", "300"))


class StoreComm:
    """Collectives over a ``torch.distributed`` store.  Every rank calls them in
    the same order; a sequence number keeps the keys of successive calls apart."""

    def __init__(self, store, rank: int, size: int):
        if not (0 <= rank < size):
            raise ValueError(f"invalid rank {rank} of {size}")
        self.store, self.rank, self.size = store, rank, size
        self._seq = 0

    def _exchange(self, payload: bytes):
        seq, self._seq = self._seq, self._seq + 1
        self.store.set(f"iris_amd/{seq}/{self.rank}", payload)
        # get() blocks until the key exists (or the store's timeout passes)
        return [bytes(self.store.get(f"iris_amd/{seq}/{r}")) for r in range(self.size)]

    def allgather(self, data) -> np.ndarray:
        """``[size, len(data)]`` of every rank's 1-D array (iris/_mpi_helpers.py:8-18)."""
        data = np.ascontiguousarray(data)
        assert data.ndim == 1, "Only 1D arrays are supported."
        parts = self._exchange(data.tobytes())
        return np.stack([np.frombuffer(p, dtype=data.dtype) for p in parts]).copy()

    def broadcast_scalar(self, value=None, root=0):
        """The root's scalar on every rank (iris/_mpi_helpers.py:21-40)."""
        seq, self._seq = self._seq, self._seq + 1
        key = f"iris_amd/{seq}/bcast"
        if self.rank == root:
            assert value is not None, "Root must provide a value."
            arr = np.array(value)
            # one length byte, the dtype's name, the value's bytes (a one-byte dtype's name itself starts with
            # '|': "|b1", "|i1", "|u1", so no separator character is safe)
            name = arr.dtype.str.encode()
            self.store.set(key, bytes([len(name)]) + name + arr.tobytes())
        blob = bytes(self.store.get(key))
        n = blob[0]
        return np.frombuffer(blob[1 + n:], dtype=np.dtype(blob[1:1 + n].decode()))[0]

    def barrier(self):
        self._exchange(b"\x01")


class MpiComm:
    """The reference's transport: mpi4py on the node-local communicator."""

    def __init__(self):
        from mpi4py import MPI

        self._MPI = MPI
        self.comm = MPI.COMM_WORLD
        self.rank, self.size = self.comm.Get_rank(), self.comm.Get_size()

    def allgather(self, data) -> np.ndarray:
        shm = self.comm.Split_type(self._MPI.COMM_TYPE_SHARED)
        data = np.ascontiguousarray(data)
        assert data.ndim == 1, "Only 1D arrays are supported."
        out = np.empty(len(data) * shm.Get_size(), dtype=data.dtype)
        shm.Allgather(sendbuf=data, recvbuf=out)
        n = shm.Get_size()
        shm.Free()
        return out.reshape(n, len(data))

    def broadcast_scalar(self, value=None, root=0):
        return self.comm.bcast(None if value is None else np.array(value)[()], root=root)

    def barrier(self):
        self.comm.Barrier()


def _under_mpi_launcher() -> bool:
    return any(k in os.environ for k in ("OMPI_COMM_WORLD_SIZE", "PMI_SIZE", "PMIX_RANK", "MV2_COMM_WORLD_SIZE"))


def launched_as_ranks() -> bool:
    """Whether this process was started as one rank of several (what
    ``init_comm`` would find), without opening a store or initialising MPI."""
    if int(os.environ.get("WORLD_SIZE", "1")) > 1:
        return True
    if os.environ.get("IRIS_AMD_RENDEZVOUS") is None and _under_mpi_launcher():
        return importlib.util.find_spec("mpi4py") is not None
    return False


def init_comm():
    """The communicator of this process, or ``None`` when it is on its own."""
    rendezvous = os.environ.get("IRIS_AMD_RENDEZVOUS")
    world = int(os.environ.get("WORLD_SIZE", "1"))
    if rendezvous is None and _under_mpi_launcher() and importlib.util.find_spec("mpi4py") is not None:
        comm = MpiComm()
        return comm if comm.size > 1 else None
    if world <= 1:
        return None
    rank = int(os.environ["RANK"])
    import torch.distributed as dist

    timeout = datetime.timedelta(seconds=_TIMEOUT_S)
    if rendezvous is None:
        host, port = os.environ.get("MASTER_ADDR", "127.0.0.1"), int(os.environ["MASTER_PORT"])
        # under torchrun the launcher's agent already serves the store on that port: every worker is a client
        agent_store = os.environ.get("TORCHELASTIC_USE_AGENT_STORE") == "True"
        store = dist.TCPStore(host, port, world, is_master=(rank == 0 and not agent_store), timeout=timeout)
    elif rendezvous.startswith("file://"):
        store = dist.FileStore(rendezvous[len("file://"):], world)
        store.set_timeout(timeout)
    elif rendezvous.startswith("tcp://"):
        host, _, port = rendezvous[len("tcp://"):].rpartition(":")
        store = dist.TCPStore(host, int(port), world, is_master=(rank == 0), timeout=timeout)
    else:
        raise ValueError(f"IRIS_AMD_RENDEZVOUS must be file://path or tcp://host:port, got {rendezvous!r}")
    return StoreComm(store, rank, world)
