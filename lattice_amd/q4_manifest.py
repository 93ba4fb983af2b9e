"""``quantize_index.json``: the per-tensor manifest written next to a Q4 checkpoint's
``.q4`` / ``.f16`` files (crates/inference/src/quant/q4_manifest.rs).

Two writers produce it with different top-level shapes:

* ``quantize_q4``: a bare array of tensor entries;
* the QuaRot converter: ``{"quarot_seed": u64 | null, "tensors": [...]}``.

The reader is bounded (16 MiB), returns ``None`` only when the manifest is genuinely absent
and fails closed on anything present but oversized, unreadable, a dangling symlink, invalid
JSON or the wrong shape (q4_manifest.rs:164-288).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import List, Optional

MAX_QUANTIZE_INDEX_LEN = 16 * 1024 * 1024  # q4_manifest.rs:48
MANIFEST_NAME = "quantize_index.json"

FLAVOR_QUANTIZE_Q4 = "QuantizeQ4"  # bare array
FLAVOR_QUAROT = "QuaRot"           # object with "tensors"


class Q4ManifestError(ValueError):
    """Base of the four failure classes of q4_manifest.rs:60-77."""


class Unreadable(Q4ManifestError):
    pass


class TooLarge(Q4ManifestError):
    pass


class InvalidJson(Q4ManifestError):
    pass


class InvalidShape(Q4ManifestError):
    pass


@dataclass
class Q4ManifestEntry:
    """One tensor entry (q4_manifest.rs:104-122): ``name`` and ``file`` are required, the rest
    is tolerated missing."""
    name: str
    file: str
    quantized: Optional[bool] = None
    shape: Optional[List[int]] = None
    numel: Optional[int] = None


@dataclass
class Q4Manifest:
    flavor: str
    quarot_seed: Optional[int]
    tensors: List[Q4ManifestEntry]


def read_manifest_bytes_bounded(path: str) -> Optional[bytes]:
    """``read_manifest_bytes_bounded`` (q4_manifest.rs:164-218): ``None`` only if the path has no
    directory entry at all; a dangling symlink, a permission error or a file above the cap
    raise.  Stat-then-bounded-read, so a file swapped for a larger one between the two cannot
    cause an unbounded allocation."""
    try:
        os.lstat(path)
    except FileNotFoundError:
        return None
    except OSError as e:
        raise Unreadable(f"{path}: failed to stat quantize_index.json: {e}") from e
    try:
        size = os.stat(path).st_size
    except OSError as e:
        raise Unreadable(f"{path}: quantize_index.json entry exists but is unreadable "
                         f"(broken symlink or permission error): {e}") from e
    if size > MAX_QUANTIZE_INDEX_LEN:
        raise TooLarge(f"{path}: quantize_index.json too large: {size} bytes exceeds cap of "
                       f"{MAX_QUANTIZE_INDEX_LEN} bytes")
    try:
        with open(path, "rb") as f:
            buf = f.read(MAX_QUANTIZE_INDEX_LEN + 1)
    except OSError as e:
        raise Unreadable(f"{path}: failed to open quantize_index.json: {e}") from e
    if len(buf) > MAX_QUANTIZE_INDEX_LEN:
        raise TooLarge(f"{path}: quantize_index.json too large: read exceeds cap of "
                       f"{MAX_QUANTIZE_INDEX_LEN} bytes")
    return buf


def _entry(obj, where: str) -> Q4ManifestEntry:
    if not isinstance(obj, dict):
        raise InvalidShape(f"{where}: invalid type: expected a tensor entry object")
    for field in ("name", "file"):
        if field not in obj:
            raise InvalidShape(f"{where}: missing field `{field}`")
        if not isinstance(obj[field], str):
            raise InvalidShape(f"{where}: invalid type for `{field}`: expected a string")
    quantized = obj.get("quantized")
    if quantized is not None and not isinstance(quantized, bool):
        raise InvalidShape(f"{where}: invalid type for `quantized`: expected a boolean")
    shape = obj.get("shape")
    if shape is not None and not (isinstance(shape, list) and
                                  all(isinstance(d, int) and not isinstance(d, bool) and d >= 0 for d in shape)):
        raise InvalidShape(f"{where}: invalid type for `shape`: expected a sequence of unsigned integers")
    numel = obj.get("numel")
    if numel is not None and not (isinstance(numel, int) and not isinstance(numel, bool) and numel >= 0):
        raise InvalidShape(f"{where}: invalid type for `numel`: expected an unsigned integer")
    return Q4ManifestEntry(obj["name"], obj["file"], quantized, shape, numel)


def parse_manifest(data: bytes, path: str = MANIFEST_NAME) -> Q4Manifest:
    """``parse_manifest`` (q4_manifest.rs:228-271): untyped parse first, then the schema that
    matches the root, so errors name the offending field instead of "no variant matched"."""
    try:
        value = json.loads(data)
    except (ValueError, UnicodeDecodeError) as e:
        raise InvalidJson(f"{path} is not valid JSON: {e}") from e
    if isinstance(value, list):
        try:
            tensors = [_entry(v, f"entry {i}") for i, v in enumerate(value)]
        except InvalidShape as e:
            raise InvalidShape(f"{path}: invalid bare-array (quantize_q4) manifest: {e}") from e
        return Q4Manifest(FLAVOR_QUANTIZE_Q4, None, tensors)
    if isinstance(value, dict):
        try:
            if "tensors" not in value:
                raise InvalidShape("missing field `tensors`")
            if not isinstance(value["tensors"], list):
                raise InvalidShape("invalid type for `tensors`: expected a sequence")
            seed = value.get("quarot_seed")
            if seed is not None and not (isinstance(seed, int) and not isinstance(seed, bool) and 0 <= seed < 2 ** 64):
                raise InvalidShape("invalid type for `quarot_seed`: expected u64 or null")
            tensors = [_entry(v, f"tensors[{i}]") for i, v in enumerate(value["tensors"])]
        except InvalidShape as e:
            raise InvalidShape(f"{path}: invalid object-form (quantize_quarot) manifest: {e}") from e
        return Q4Manifest(FLAVOR_QUAROT, seed, tensors)
    raise InvalidShape(f"{path}: expected quantize_index.json to be either a bare array of tensor "
                       f"entries (quantize_q4) or an object with a \"tensors\" array (quantize_quarot)")


def load_manifest(directory: str) -> Optional[Q4Manifest]:
    """``load_manifest`` (q4_manifest.rs:279-285)."""
    path = os.path.join(directory, MANIFEST_NAME)
    data = read_manifest_bytes_bounded(path)
    return None if data is None else parse_manifest(data, path)
