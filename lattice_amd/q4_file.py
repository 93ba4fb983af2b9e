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


MAX_Q4_MERGE_PAYLOAD_LEN = 4 << 30  # cap on a source payload read for a merge


def q4_file_bytes(shape: Sequence[int], original_len: int, payload) -> bytes:
    """A KHQ4 v2 file image: header for ``shape`` / ``original_len`` followed by ``payload``."""
    out = bytearray(b"KHQ4")
    out += (2).to_bytes(4, "little") + len(shape).to_bytes(4, "little")
    for d in shape:
        out += int(d).to_bytes(8, "little")
    out += int(original_len).to_bytes(8, "little")
    out += bytes(memoryview(np.ascontiguousarray(payload, dtype=np.uint8)))
    return bytes(out)


def write_q4_file(path: str, shape: Sequence[int], payload) -> None:
    """Writes a ``.q4`` file through a temporary file and an atomic rename, so a crash in the
    middle never leaves a partial file at the final path."""
    numel = 1
    for d in shape:
        numel *= int(d)
    tmp = path + ".tmp"
    try:
        with open(tmp, "wb") as f:
            f.write(q4_file_bytes(shape, numel, payload))
        os.replace(tmp, path)
    except OSError:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise


def read_q4_payload_bounded(path: str, max_payload: int = MAX_Q4_MERGE_PAYLOAD_LEN):
    """Header and block payload of a ``.q4`` file, read with a size cap (the role of
    ``read_q4_payload_bounded`` in write_merged_qkvz, q4_weights.rs:1560-1566)."""
    size = os.stat(path).st_size
    if size > max_payload + 64:
        raise Q4FileError(f"{path}: file of {size} bytes exceeds the merge cap of {max_payload} bytes")
    data = np.fromfile(path, dtype=np.uint8)
    h = validate_q4_file(data, path)
    return h, data[h.payload_offset:]


def merge_q4_files(first_path: str, second_path: str, out_path: str) -> Q4FileHeader:
    """``write_merged_qkvz`` (q4_weights.rs:1552-1636): concatenates two 2-D ``.q4`` tensors with
    the same hidden width along the rows — payload bytes verbatim, new header with the summed
    row count and ``original_len`` — and writes the result atomically.  Both inputs must be
    exactly 2-D (a rank-0 header must not be indexed)."""
    h1, p1 = read_q4_payload_bounded(first_path)
    h2, p2 = read_q4_payload_bounded(second_path)
    if len(h1.shape) != 2:
        raise Q4FileError(f"{first_path}: qkv header shape {list(h1.shape)} is not 2-D (expected [rows, hidden])")
    if len(h2.shape) != 2:
        raise Q4FileError(f"{second_path}: z header shape {list(h2.shape)} is not 2-D (expected [rows, hidden])")
    if h1.shape[1] != h2.shape[1]:
        raise Q4FileError(f"{first_path}/{second_path}: qkv hidden dimension {h1.shape[1]} does not match "
                          f"z hidden dimension {h2.shape[1]}")
    if h1.shape[1] % BLOCK_WEIGHTS:
        raise Q4FileError(f"{first_path}: hidden dimension {h1.shape[1]} is not a multiple of {BLOCK_WEIGHTS}: "
                          f"rows are not block-aligned and cannot be concatenated")
    shape = (h1.shape[0] + h2.shape[0], h1.shape[1])
    write_q4_file(out_path, shape, np.concatenate([p1, p2]))
    return Q4FileHeader(shape, h1.original_len + h2.original_len, 36)
