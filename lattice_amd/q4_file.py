"""``.q4`` (KHQ4 v2) file ingest: header parse, exact-extent and shape preflight,
tensor-name sanitiser and the fused gate||up payload — the host logic that sits
between lattice's ``quantize_q4`` output and a device upload.

Format (crates/inference/src/weights/q4_weights.rs:36-45)::

    magic "KHQ4" | u32 version (=2) | u32 ndim | u64 shape[ndim] | u64 original_len | blocks

Blocks are the flat sequence ``ceil(original_len/32)`` x 20 bytes; for a 2-D tensor
``[N, K]`` with ``K % 32 == 0`` that is exactly the row-major ``N x K/32`` block
matrix the kernels index.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Optional, Sequence, Tuple

import numpy as np

from .q4_layout import BLOCK_BYTES, BLOCK_WEIGHTS


class Q4FileError(ValueError):
    pass


@dataclass
class Q4FileHeader:
    """``Q4FileHeader { shape, original_len, payload_offset }`` (q4_weights.rs:690-700)."""
    shape: Tuple[int, ...]
    original_len: int
    payload_offset: int


def read_q4_header(data) -> Q4FileHeader:
    """``read_q4_header`` (q4_weights.rs:709-762): magic, version (1 = legacy symmetric
    18-byte blocks, rejected; only 2 accepted), ndim, dims, original_len."""
    buf = memoryview(data).cast("B") if not isinstance(data, np.ndarray) else data
    n = len(buf)
    if n < 4 or bytes(buf[:4]) != b"KHQ4":
        raise Q4FileError("invalid magic: not a .q4 file")
    if n < 12:
        raise Q4FileError("failed to fill whole buffer")  # read_exact on a short header
    ver = int.from_bytes(bytes(buf[4:8]), "little")
    if ver == 1:
        raise Q4FileError("legacy .q4 file (v1 symmetric format) — re-quantize with current "
                          "quantize_q4 to produce v2 asymmetric blocks")
    if ver != 2:
        raise Q4FileError(f"unsupported .q4 file version: {ver}")
    ndim = int.from_bytes(bytes(buf[8:12]), "little")
    if ndim * 8 > n:  # checked_alloc_bytes(ndim, 8, file_len, "shape dims")
        raise Q4FileError(f"shape dims: {ndim} entries exceed the file length {n}")
    if n < 20 + 8 * ndim:
        raise Q4FileError("failed to fill whole buffer")
    shape = tuple(int.from_bytes(bytes(buf[12 + 8 * i:20 + 8 * i]), "little") for i in range(ndim))
    olen = int.from_bytes(bytes(buf[12 + 8 * ndim:20 + 8 * ndim]), "little")
    return Q4FileHeader(shape, olen, 20 + 8 * ndim)


def validate_q4_file(data, path: str = "<memory>",
                     expected_shape: Optional[Sequence[int]] = None) -> Q4FileHeader:
    """``validate_q4_file`` (q4_weights.rs:837-868) = ``read_q4_header`` +
    ``validate_q4_header_payload_bounds`` (:768-812) + the shared geometry rule
    (weights/ingress.rs:521-540): the file must end exactly where the declared payload
    ends, ``original_len`` must equal the shape product, and the shape must equal
    ``expected_shape`` when one is given.  No block byte is read."""
    h = read_q4_header(data)
    file_len = len(data)
    payload = -(-h.original_len // BLOCK_WEIGHTS) * BLOCK_BYTES
    required = h.payload_offset + payload
    if file_len < required:
        raise Q4FileError(f"{path}: file truncated below Q4 block payload ({file_len} bytes < "
                          f"required {required})")
    if file_len > required:
        raise Q4FileError(f"{path}: file has trailing bytes after Q4 block payload ({file_len} "
                          f"bytes > expected {required})")
    numel = 1
    for d in h.shape:
        numel *= d
    name = os.path.basename(path) or "native Q4 tensor"
    if h.original_len != numel:
        raise Q4FileError(f"{path}: tensor {name} (Q4) original_len {h.original_len} does not match "
                          f"shape {list(h.shape)} (expected {numel})")
    if expected_shape is not None and tuple(int(s) for s in expected_shape) != h.shape:
        raise Q4FileError(f"{path}: tensor {name} shape {list(h.shape)} does not match expected "
                          f"{list(expected_shape)}")
    return h


def q4_tensor_path(directory: str, tensor_name: str, ext: str = "q4") -> str:
    """``q4_tensor_path`` (forward/metal_qwen35.rs:11428-11444): every character that is not
    alphanumeric or '-' becomes '_'."""
    stem = "".join(c if (c.isalnum() or c == "-") else "_" for c in tensor_name)
    return os.path.join(directory, f"{stem}.{ext}")


def load_q4_raw_bytes(path: str, expected_shape: Sequence[int]) -> np.ndarray:
    """Block payload of a validated ``.q4`` file as a u8 array (header stripped)."""
    data = np.fromfile(path, dtype=np.uint8)
    h = validate_q4_file(data, path, expected_shape)
    return data[h.payload_offset:]


def fuse_gate_up(gate_raw: np.ndarray, up_raw: np.ndarray) -> np.ndarray:
    """``make_fused_q4_buf`` (metal_qwen35.rs:12137-12152): gate blocks then up blocks in one
    buffer, payload_offset 0; ``up`` starts at byte ``inter*(hidden/32)*20``
    (metal_qwen35.rs:7403-7406)."""
    return np.concatenate([np.ascontiguousarray(gate_raw, dtype=np.uint8),
                           np.ascontiguousarray(up_raw, dtype=np.uint8)])
