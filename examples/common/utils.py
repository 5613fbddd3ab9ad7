"""Logging and tile-trace helpers of the examples (examples/common/utils.py:22-132)."""

import json
import os

import numpy as np
import torch


class JSONWriter:
    """Flat key/value record written as one JSON object."""

    def __init__(self, file_path):
        self.file_path = file_path
        self.data = {}
        if not os.path.exists(file_path):
            with open(file_path, "w") as f:
                json.dump({}, f)

    def add_field(self, key, value):
        self.data[key] = value

    def display(self):
        print(json.dumps(self.data, indent=4))

    def flush(self):
        with open(self.file_path, "w") as f:
            json.dump(self.data, f, indent=4)


class Timestamps:
    """Per-tile begin/end ticks of the device wall clock, written by the
    kernels with atomic min/max (gemm_*:151-153, :273-275)."""

    _FIELDS_MIN = ("mm_begin_timestamp", "comm_begin_timestamp", "comm_middle_min_timestamp")
    _FIELDS_MAX = ("mm_end_timestamp", "comm_middle_max_timestamp", "comm_end_timestamp")

    def __init__(self, num_tiles, device="cuda"):
        self.max_ts = torch.iinfo(torch.int64).max
        self.min_ts = 0
        for name in self._FIELDS_MIN:
            setattr(self, name, torch.empty(num_tiles, dtype=torch.int64, device=device))
        for name in self._FIELDS_MAX:
            setattr(self, name, torch.zeros(num_tiles, dtype=torch.int64, device=device))

    def reset(self):
        for name in self._FIELDS_MIN:
            getattr(self, name).fill_(self.max_ts)
        for name in self._FIELDS_MAX:
            getattr(self, name).fill_(self.min_ts)

    def to_json(self, filename, gpu_freq):
        """Ticks -> microseconds (``gpu_freq`` in MHz), rebased to the earliest
        event; same record layout as examples/common/utils.py:93-128."""
        us = {
            name: getattr(self, name).cpu().numpy() / gpu_freq
            for name in self._FIELDS_MIN + self._FIELDS_MAX
        }
        t0 = min(float(np.min(v)) for v in us.values())
        us = {k: v - t0 for k, v in us.items()}
        data = [
            {
                "tile_id": i,
                "gemm_begin": int(us["mm_begin_timestamp"][i]),
                "gemm_end": int(us["mm_end_timestamp"][i]),
                "poll_begin": int(us["comm_begin_timestamp"][i]),
                "poll_end": int(us["comm_middle_max_timestamp"][i]),
                "op_begin": int(us["comm_middle_min_timestamp"][i]),
                "op_end": int(us["comm_end_timestamp"][i]),
                "comm_begin": int(us["comm_begin_timestamp"][i]),
                "comm_end": int(us["comm_end_timestamp"][i]),
            }
            for i in range(len(us["mm_begin_timestamp"]))
        ]
        with open(filename, "w") as f:
            json.dump(data, f, indent=4)


def is_triton_interpret_set():
    return "TRITON_INTERPRET" in os.environ
