"""What the engine can leave behind for comparisons between runs: a digest of every sampled
logits row, or the rows themselves.

The reference's determinism harness reads two artefacts at the sampling boundary
(python/vosti_kernels/kernels.py:1020-1033, scripts/determinism_tests/logits_observer.py):

* ``VOSTI_LOGITS_DIGEST=<file>``: one line ``<row index in the step> <sha256>`` per sampled row, the
  hash taken over the row as 32-bit floats;
* ``VOSTI_LOGITS_OBSERVER_DIR=<folder>``: every sampled row as a lossless float32 ``.npy`` file
  ``row-<pid>-<call>-<row index>.npy`` plus one JSON line per row in ``observer-<pid>.jsonl`` with
  its hash, shape, argmax, the step, and the phase that ``VOSTI_LOGITS_OBSERVER_PHASE`` names.

Both cost a device-to-host copy of the rows per step; they are instrumentation, off by default.
"""
from __future__ import annotations

import hashlib
import json
import os
from pathlib import Path

import numpy as np


class LogitsObserver:
    def __init__(self):
        self.digest_path = os.environ.get("VOSTI_LOGITS_DIGEST") or None
        folder = os.environ.get("VOSTI_LOGITS_OBSERVER_DIR") or None
        self.folder = Path(folder).resolve() if folder else None
        self.calls = 0

    @property
    def active(self) -> bool:
        return bool(self.digest_path or self.folder)

    def rows(self, data: np.ndarray, row_indices: list[int], engine_step: int, source_dtype: str) -> None:
        """data: float32 [n, vocab], one row per sampled row of the step; row_indices: their places in the step."""
        call, self.calls = self.calls, self.calls + 1
        if self.folder is not None:
            self.folder.mkdir(parents=True, exist_ok=True)
        pid = os.getpid()
        for offset, index in enumerate(row_indices):
            row = np.ascontiguousarray(data[offset], dtype=np.float32)
            raw = row.tobytes()
            sha = hashlib.sha256(raw).hexdigest()
            if self.digest_path:
                with open(self.digest_path, "a") as f:
                    f.write(f"{index} {sha}\n")
            if self.folder is None:
                continue
            name = f"row-{pid}-{call:06d}-{index:04d}.npy"
            with open(self.folder / name, "xb") as f:
                np.save(f, row, allow_pickle=False)
            record = {"schema_version": 1, "pid": pid, "call_sequence": call, "batch_index": index, "row_offset": offset,
                      "batch_size": len(row_indices), "source": "vosti_amd.engine", "source_dtype": source_dtype,
                      "observed_dtype": "float32", "shape": list(row.shape), "numel": int(row.size), "byte_length": len(raw),
                      "sha256": sha, "finite": bool(np.isfinite(row).all()), "argmax": int(np.argmax(row)) if row.size else None,
                      "artifact": name, "engine_step": engine_step}
            phase = os.environ.get("VOSTI_LOGITS_OBSERVER_PHASE")
            if phase:
                record["phase"] = phase
            with open(self.folder / f"observer-{pid}.jsonl", "a") as f:
                f.write(json.dumps(record, sort_keys=True, separators=(",", ":")) + "\n")
