"""The point-to-point microbenchmarks (examples/00_load .. 05_atomic_xchg):
command-line parity with the reference's scripts and their report formats on
the CPU; the kernels and the validation flow on the GPU with virtual ranks."""

import json

import numpy as np
import pytest
import torch

from examples.common import p2p_driver as D


def test_flags_and_defaults_follow_the_reference_scripts():
    a = D.parse_args("load", [])        # examples/00_load/load_bench.py:78-100
    assert (a["datatype"], a["buffer_size"], a["block_size"], a["heap_size"], a["num_experiments"], a["num_warmup"]) == \
        ("fp16", 1 << 32, 512, 1 << 33, 10, 1)
    a = D.parse_args("store", ["-t", "int8", "-z", "4096", "-b", "256", "-n", "3", "-w", "0", "-d", "-v", "-o", "x.json"])
    assert (a["datatype"], a["buffer_size"], a["block_size"], a["num_experiments"], a["num_warmup"]) == \
        ("int8", 4096, 256, 3, 0)
    assert a["validate"] and a["verbose"] and a["output_file"] == "x.json"
    a = D.parse_args("all_load", [])    # examples/02_all_load/all_load_bench.py:103-128
    assert (a["buffer_size_min"], a["buffer_size_max"], a["heap_size"], a["num_experiments"], a["num_warmup"],
            a["active_ranks"]) == (1 << 20, 1 << 32, 1 << 36, 20, 2, 8)
    a = D.parse_args("atomic_add", ["-x", "5"])   # examples/04_atomic_add/atomic_add_bench.py:58-81
    assert (a["datatype"], a["num_experiments"], a["num_warmup"]) == ("fp16", 5, 4)
    assert D.parse_args("atomic_xchg", [])["datatype"] == "int32"   # atomic_xchg_bench.py:66-72
    with pytest.raises(SystemExit):
        D.parse_args("atomic_add", ["-t", "int8"])  # not among that script's choices


def test_pair_matrix_report(tmp_path, capsys):
    m = np.array([[1.5, 20.25], [300.0, 4.0]], dtype=np.float32)
    out = tmp_path / "bw.json"
    D.print_pair_matrix(m, "Unidirectional LOAD bandwidth GiB/s [Remote read]", str(out))
    text = capsys.readouterr().out.splitlines()
    assert text[1] == "Unidirectional LOAD bandwidth GiB/s [Remote read]"
    assert text[2] == " SRC\\DST      GPU 00    GPU 01"   # load_bench.py:202-206: 10-wide columns
    assert text[3] == "GPU 00  ->      1.50     20.25"
    assert text[4] == "GPU 01  ->    300.00      4.00"
    rec = json.loads(out.read_text())
    assert rec[1] == {"source_gpu": "GPU_00", "destination_gpu": "GPU_01", "source_rank": 0, "destination_rank": 1,
                      "bandwidth_gbps": 20.25}
    assert len(rec) == 4
    with pytest.raises(ValueError):
        D.print_pair_matrix(m, "x", "bw.csv")


def test_size_table_report(tmp_path, capsys):
    data = [[10.0, 200.5], [11.25, 201.0]]
    out = tmp_path / "all.json"
    D.print_size_table(data, [1 << 20, 1 << 21], "Total Bandwidth (GiB/s) vs Buffer Size", str(out))
    text = capsys.readouterr().out.splitlines()
    assert text[2] == "Size (MiB) | log2(bytes) | GPU 00 | GPU 01"
    assert text[3] == "-" * len(text[2])
    assert text[4] == "       1.0 |          20 |  10.00 |  11.25"
    assert text[5] == "       2.0 |          21 | 200.50 | 201.00"
    rec = json.loads(out.read_text())
    assert rec[3] == {"buffer_size_bytes": 1 << 21, "buffer_size_mib": 2.0, "log2_bytes": 21, "gpu_rank": 1,
                      "gpu_id": "GPU_01", "bandwidth_gbps": 201.0}


@pytest.mark.gpu
@pytest.mark.parametrize("kind,dtype", [("load", "fp16"), ("load", "int8"), ("store", "bf16"), ("store", "fp32"),
                                        ("atomic_add", "fp32"), ("atomic_add", "bf16"), ("atomic_add", "int32"),
                                        ("atomic_xchg", "int32"), ("atomic_xchg", "fp16")])
def test_pairwise_benchmarks_validate_between_virtual_ranks(kind, dtype, tmp_path):
    flag = "-n" if kind in ("load", "store") else "-x"
    out = tmp_path / "m.json"
    matrix, ok = D.main(kind, ["-t", dtype, "-z", str(3 * 4096 + 8), "-b", "256", flag, "2", "-w", "1", "-d",
                               "-p", str(1 << 20), "-o", str(out), "--virtual_ranks", "3"])
    assert ok
    assert matrix.shape == (3, 3)   # (buffers this small cannot be timed: only the flow is checked)
    assert len(json.loads(out.read_text())) == 9


@pytest.mark.gpu
@pytest.mark.parametrize("kind,dtype", [("all_load", "fp32"), ("all_load", "fp16"), ("all_store", "bf16"),
                                        ("all_store", "int8")])
def test_all_to_one_benchmarks_validate_between_virtual_ranks(kind, dtype, tmp_path):
    out = tmp_path / "t.json"
    data, ok = D.main(kind, ["-t", dtype, "-m", "2048", "-M", "8192", "-b", "128", "-x", "2", "-w", "1", "-d",
                             "-p", str(1 << 20), "-a", "3", "-o", str(out), "--virtual_ranks", "4"])
    assert ok
    assert len(data) == 4 and len(data[0]) == 3
    assert all(v == 0 for v in data[3])  # rank 3 is not active
    assert len(json.loads(out.read_text())) == 12


@pytest.mark.gpu
def test_p2p_launcher_rejects_bad_arguments():
    import iris_amd
    from iris_amd import ops
    shmem = iris_amd.iris(1 << 20, virtual_ranks=2)
    buf = shmem.zeros(64, dtype=torch.int8)
    res = shmem.zeros(64, dtype=torch.int8)
    hb = shmem.get_heap_bases()
    with pytest.raises(ValueError):
        ops.p2p_bench("atomic_add", buf, res, hb, 0, 1, 2)     # int8 has no atomics
    with pytest.raises(ValueError):
        ops.p2p_bench("load", buf, res, hb, 0, 2, 2)           # peer out of range
    with pytest.raises(ValueError):
        ops.p2p_bench("load", buf, res, hb, 0, 1, 2, block_size=2048)
    with pytest.raises(ValueError):
        ops.p2p_bench("load", buf, shmem.zeros(64, dtype=torch.float16), hb, 0, 1, 2)


def test_tile_trace_json_follows_the_reference_layout(tmp_path):
    """examples/common/utils.py:66-128: ticks / gpu_freq, rebased to the
    earliest event of any kind, truncated to int; poll/comm keys alias the
    comm timestamps."""
    from examples.common.utils import JSONWriter, Timestamps
    ts = Timestamps(num_tiles=2, device="cpu")
    ts.reset()
    assert ts.mm_begin_timestamp.tolist() == [torch.iinfo(torch.int64).max] * 2
    assert ts.mm_end_timestamp.tolist() == [0, 0]
    ts.mm_begin_timestamp.copy_(torch.tensor([1000, 1250]))
    ts.mm_end_timestamp.copy_(torch.tensor([1500, 2050]))
    ts.comm_begin_timestamp.copy_(torch.tensor([1600, 2100]))
    ts.comm_middle_min_timestamp.copy_(torch.tensor([1700, 2200]))
    ts.comm_middle_max_timestamp.copy_(torch.tensor([1650, 2150]))
    ts.comm_end_timestamp.copy_(torch.tensor([1900, 2499]))
    out = tmp_path / "trace.json"
    ts.to_json(str(out), gpu_freq=100.0)  # 100 ticks per microsecond
    assert json.loads(out.read_text()) == [
        {"tile_id": 0, "gemm_begin": 0, "gemm_end": 5, "poll_begin": 6, "poll_end": 6, "op_begin": 7, "op_end": 9,
         "comm_begin": 6, "comm_end": 9},
        {"tile_id": 1, "gemm_begin": 2, "gemm_end": 10, "poll_begin": 11, "poll_end": 11, "op_begin": 12,
         "op_end": 14, "comm_begin": 11, "comm_end": 14},
    ]
    log = tmp_path / "log.json"
    w = JSONWriter(str(log))
    assert json.loads(log.read_text()) == {}        # created empty (utils.py:23-29)
    w.add_field("world_size", 8)
    w.add_field("ms", 1.5)
    w.flush()
    assert json.loads(log.read_text()) == {"world_size": 8, "ms": 1.5}
