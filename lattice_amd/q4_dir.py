"""Loading a directory of ``quantize_q4`` output straight onto the GPU: the host logic of
``from_q4_dir`` (forward/metal_qwen35.rs:12004-12160) for the Q4 tensors.

A checkpoint directory holds one ``<sanitised tensor name>.q4`` per quantised tensor and,
optionally, ``quantize_index.json``.  Every file is validated (header, exact extent, shape
when one is expected, per-block scale/bias rule) before anything is published to the device;
a file is uploaded whole, header included, with ``payload_offset`` pointing past the header —
the layout ``mmap_q4_weight`` produces.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, Optional, Sequence, Tuple

import numpy as np

from . import q4_file, q4_manifest


@dataclass
class Q4Tensor:
    name: str
    shape: Tuple[int, ...]
    buf: object  # backend.Q4WeightBuf


class Q4Checkpoint:
    """Q4 tensors of one directory, resident on the device of ``backend``."""

    def __init__(self, backend, directory: str):
        self.backend = backend
        self.directory = directory
        self.manifest = q4_manifest.load_manifest(directory)
        self.tensors: Dict[str, Q4Tensor] = {}

    # ------------------------------------------------------------------ inventory
    def inventory(self) -> Dict[str, str]:
        """Tensor name -> ``.q4`` path.  From the manifest when there is one (entries marked
        ``quantized: false`` and non-``.q4`` files are skipped); otherwise from a directory scan,
        where the name is the file stem."""
        if self.manifest is not None:
            out = {}
            for e in self.manifest.tensors:
                if e.quantized is False or not e.file.endswith(".q4"):
                    continue
                if os.path.basename(e.file) != e.file:
                    raise q4_manifest.InvalidShape(f"manifest entry {e.name!r}: file {e.file!r} must be a plain "
                                                   f"file name inside the checkpoint directory")
                out[e.name] = os.path.join(self.directory, e.file)
            return out
        return {f[:-3]: os.path.join(self.directory, f)
                for f in sorted(os.listdir(self.directory)) if f.endswith(".q4")}

    # --------------------------------------------------------------------- loading
    def load(self, name: str, expected_shape: Optional[Sequence[int]] = None, path: Optional[str] = None) -> Q4Tensor:
        """Validates and uploads one tensor (``mmap_q4_weight``, metal_qwen35.rs:660-702)."""
        if name in self.tensors:
            return self.tensors[name]
        if path is None:
            path = self.inventory().get(name) or q4_file.q4_tensor_path(self.directory, name)
        buf = self.backend.mmap_q4_weight(path, name, expected_shape)
        data = np.memmap(path, dtype=np.uint8, mode="r")
        shape = q4_file.read_q4_header(data).shape
        t = Q4Tensor(name, shape, buf)
        self.tensors[name] = t
        return t

    def load_all(self) -> Dict[str, Q4Tensor]:
        for name, path in self.inventory().items():
            self.load(name, None, path)
        return self.tensors

    def load_fused(self, first: str, second: str, fused_name: str) -> Q4Tensor:
        """Two tensors with the same width as one buffer, first's rows then second's — the fused
        gate||up buffer of ``make_fused_q4_buf`` (metal_qwen35.rs:12137-12152).  Payload offset 0;
        the second tensor starts at byte ``rows_first * (width/32) * 20``."""
        if fused_name in self.tensors:
            return self.tensors[fused_name]
        inv = self.inventory()
        raws, shapes = [], []
        for nm in (first, second):
            path = inv.get(nm) or q4_file.q4_tensor_path(self.directory, nm)
            data = np.fromfile(path, dtype=np.uint8)
            h = q4_file.validate_q4_file(data, path)
            if len(h.shape) != 2:
                raise q4_file.Q4FileError(f"{path}: shape {list(h.shape)} is not 2-D")
            raws.append(data[h.payload_offset:])
            shapes.append(h.shape)
        if shapes[0][1] != shapes[1][1]:
            raise q4_file.Q4FileError(f"{first}/{second}: widths {shapes[0][1]} and {shapes[1][1]} differ")
        fused = q4_file.fuse_gate_up(raws[0], raws[1])
        t = Q4Tensor(fused_name, (shapes[0][0] + shapes[1][0], shapes[0][1]), self.backend.upload_q4_blocks(fused))
        self.tensors[fused_name] = t
        return t
