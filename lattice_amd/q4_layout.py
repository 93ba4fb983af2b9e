"""Host-side view of lattice's native Q4 block layout (numpy, no GPU).

One block = 20 bytes = ``[u16 scale (f16 bits)][u16 bias (f16 bits)][16 packed bytes]``
covering 32 weights; ``packed[b] = (q[2b+1] << 4) | q[2b]`` (low nibble = even
index); ``weight = nibble * scale + bias``
(crates/inference/src/weights/q4_weights.rs:3-25, 65-92).  A weight matrix
``[N, K]`` is ``N`` rows of ``K/32`` blocks, row stride ``(K/32)*20`` bytes.
"""
from __future__ import annotations

import numpy as np

BLOCK_BYTES = 20
BLOCK_WEIGHTS = 32
Q4_FILE_MAGIC = b"KHQ4"
Q4_FILE_VERSION = 2


def weight_nbytes(n: int, k: int) -> int:
    if k <= 0 or k % BLOCK_WEIGHTS:
        raise ValueError(f"K must be a non-zero multiple of 32, got {k}")
    return n * (k // BLOCK_WEIGHTS) * BLOCK_BYTES


def pack_blocks(scale_bits: np.ndarray, bias_bits: np.ndarray, nibbles: np.ndarray) -> np.ndarray:
    """``nibbles`` [..., 32] in 0..15, ``scale_bits``/``bias_bits`` [...] u16 -> flat u8 bytes."""
    nib = np.ascontiguousarray(nibbles, dtype=np.uint8).reshape(-1, BLOCK_WEIGHTS)
    nb = nib.shape[0]
    if nib.max(initial=0) > 15:
        raise ValueError("nibble out of range 0..15")
    out = np.empty((nb, BLOCK_BYTES), dtype=np.uint8)
    out[:, 0:2] = np.ascontiguousarray(scale_bits, dtype="<u2").reshape(nb, 1).view(np.uint8)
    out[:, 2:4] = np.ascontiguousarray(bias_bits, dtype="<u2").reshape(nb, 1).view(np.uint8)
    out[:, 4:] = nib[:, 0::2] | (nib[:, 1::2] << 4)
    return out.reshape(-1)


def unpack_blocks(data: np.ndarray):
    """Flat u8 bytes -> (scale_bits [nb] u16, bias_bits [nb] u16, nibbles [nb, 32] u8)."""
    d = np.ascontiguousarray(data, dtype=np.uint8)
    nb = d.size // BLOCK_BYTES
    blk = d[: nb * BLOCK_BYTES].reshape(nb, BLOCK_BYTES)
    scale_bits = blk[:, 0:2].copy().view("<u2").reshape(nb)
    bias_bits = blk[:, 2:4].copy().view("<u2").reshape(nb)
    nib = np.empty((nb, BLOCK_WEIGHTS), dtype=np.uint8)
    nib[:, 0::2] = blk[:, 4:] & 0x0F
    nib[:, 1::2] = blk[:, 4:] >> 4
    return scale_bits, bias_bits, nib


def dequantize_numpy(data: np.ndarray, n_weights: int | None = None) -> np.ndarray:
    """numpy twin of dequantize_row_q4_0: ``f32(nibble) * scale + bias`` with a rounded
    multiply then a rounded add, both in f32."""
    scale_bits, bias_bits, nib = unpack_blocks(data)
    scale = scale_bits.view(np.float16).astype(np.float32)[:, None]
    bias = bias_bits.view(np.float16).astype(np.float32)[:, None]
    with np.errstate(invalid="ignore", over="ignore"):
        w = (nib.astype(np.float32) * scale + bias).reshape(-1)
    return w if n_weights is None else w[:n_weights]


def q4_file_bytes(shape, blocks: np.ndarray, original_len: int | None = None) -> bytes:
    """Serialise a ``.q4`` file: magic, version 2, ndim, u64 dims, u64 original_len, blocks
    (save_q4_file, crates/inference/src/weights/q4_weights.rs:623-660)."""
    shape = [int(s) for s in shape]
    numel = int(np.prod(shape, dtype=np.int64)) if shape else 1
    olen = numel if original_len is None else int(original_len)
    head = Q4_FILE_MAGIC + np.array([Q4_FILE_VERSION, len(shape)], dtype="<u4").tobytes()
    head += np.array(shape, dtype="<u8").tobytes() + np.array([olen], dtype="<u8").tobytes()
    return head + np.ascontiguousarray(blocks, dtype=np.uint8).tobytes()
