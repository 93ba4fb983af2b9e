"""ctypes front-end for the CPU checker in ``q4_oracle.c`` / ``cpu_baseline.c``.

TEST INFRASTRUCTURE ONLY: importable from ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``.  The shipped package
(``lattice_amd``) never imports this module.

``build()`` compiles ``libq4_oracle.so`` with the Makefile beside this file;
``lib()`` loads it (building first only if no library exists yet).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libq4_oracle.so")
_lib = None

BLOCK_BYTES = 20
BLOCK_WEIGHTS = 32

_u8p = C.POINTER(C.c_uint8)
_f32p = C.POINTER(C.c_float)
_f64p = C.POINTER(C.c_double)
_i32p = C.POINTER(C.c_int32)
_u64p = C.POINTER(C.c_uint64)


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "-s", "clean"], check=True)
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _SO


def lib() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_SO):
        build()
    L = C.CDLL(_SO)
    L.lq4o_f16_to_f32.restype = C.c_float
    L.lq4o_f16_to_f32.argtypes = [C.c_uint16]
    L.lq4o_f32_to_f16.restype = C.c_uint16
    L.lq4o_f32_to_f16.argtypes = [C.c_float]
    L.lq4o_bf16_to_f32.restype = C.c_float
    L.lq4o_bf16_to_f32.argtypes = [C.c_uint16]
    L.lq4o_quantize_block.restype = C.c_int
    L.lq4o_quantize_block.argtypes = [_f32p, C.c_int, C.c_int, _u8p]
    L.lq4o_quantize_flat.restype = C.c_int
    L.lq4o_quantize_flat.argtypes = [_f32p, C.c_size_t, C.c_int, _u8p]
    L.lq4o_quantize_rows.restype = C.c_int
    L.lq4o_quantize_rows.argtypes = [_f32p, C.c_size_t, C.c_size_t, C.c_int, _u8p]
    L.lq4o_dequantize.restype = C.c_size_t
    L.lq4o_dequantize.argtypes = [_u8p, C.c_size_t, C.c_size_t, _f32p]
    L.lq4o_validate_blocks.restype = C.c_long
    L.lq4o_validate_blocks.argtypes = [_u8p, C.c_size_t, C.POINTER(C.c_int)]
    L.lq4o_gemm_f32.restype = C.c_int
    L.lq4o_gemm_f32.argtypes = [_f32p, _u8p, _f32p, C.c_size_t, C.c_size_t, C.c_size_t]
    L.lq4o_gemm_f64.restype = C.c_int
    L.lq4o_gemm_f64.argtypes = [_f32p, _u8p, _f64p, C.c_size_t, C.c_size_t, C.c_size_t]
    L.lq4o_lora_apply.restype = None
    L.lq4o_lora_apply.argtypes = [_f32p, _f32p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_float,
                                  _f32p, _f32p, C.c_size_t]
    L.lq4o_lora_apply_f64.restype = None
    L.lq4o_lora_apply_f64.argtypes = [_f32p, _f32p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_float,
                                      _f32p, _f64p, C.c_size_t]
    L.lq4o_f16_to_f32_array.restype = None
    L.lq4o_f16_to_f32_array.argtypes = [C.POINTER(C.c_uint16), C.POINTER(C.c_uint32), C.c_size_t]
    L.lq4o_f32_to_f16_array.restype = None
    L.lq4o_f32_to_f16_array.argtypes = [C.POINTER(C.c_uint32), C.POINTER(C.c_uint16), C.c_size_t]
    L.lq4o_sweep_f32_to_f16_vs_f16c.restype = C.c_uint64
    L.lq4o_sweep_f32_to_f16_vs_f16c.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32,
                                                C.POINTER(C.c_uint32)]
    L.lq4o_router_softmax.restype = None
    L.lq4o_router_softmax.argtypes = [_f32p, C.c_int, _f32p]
    L.lq4o_select_top_k.restype = None
    L.lq4o_select_top_k.argtypes = [_f32p, C.c_int, C.c_int, _i32p, _f32p]
    L.lq4o_renormalize_selected.restype = None
    L.lq4o_renormalize_selected.argtypes = [_f32p, C.c_int]
    L.lq4o_moe_route.restype = None
    L.lq4o_moe_route.argtypes = [_f32p, C.c_int, C.c_int, _f32p, _i32p, _f32p]
    for name, outp in (("lq4o_moe_ffn_f32", _f32p), ("lq4o_moe_ffn_f64", _f64p)):
        fn = getattr(L, name)
        fn.restype = C.c_int
        fn.argtypes = [_u8p, _u8p, C.c_int, C.c_int, C.c_int, _f32p, C.c_int, _i32p, _f32p,
                       C.c_int, outp]
    for name, outp in (("lq4o_moe_shared_expert_f32", _f32p), ("lq4o_moe_shared_expert_f64", _f64p)):
        fn = getattr(L, name)
        fn.restype = C.c_int
        fn.argtypes = [_u8p, _u8p, _f32p, C.c_int, C.c_int, _f32p, C.c_int, outp]
    L.lq4o_q3_quantize_block.restype = C.c_int
    L.lq4o_q3_quantize_block.argtypes = [_f32p, C.c_int, C.c_int, _u8p]
    L.lq4o_q3_quantize_row.restype = C.c_int
    L.lq4o_q3_quantize_row.argtypes = [_f32p, C.c_size_t, C.c_int, _u8p]
    L.lq4o_q3_dequantize.restype = C.c_size_t
    L.lq4o_q3_dequantize.argtypes = [_u8p, C.c_size_t, C.c_size_t, _f32p]
    L.lq4o_q3_gemm_f32.restype = C.c_int
    L.lq4o_q3_gemm_f32.argtypes = [_f32p, _u8p, _f32p, C.c_size_t, C.c_size_t, C.c_size_t]
    L.lq4o_q3_gemm_f64.restype = C.c_int
    L.lq4o_q3_gemm_f64.argtypes = [_f32p, _u8p, _f64p, C.c_size_t, C.c_size_t, C.c_size_t]
    L.lq4o_q8_quantize_row.restype = C.c_long
    L.lq4o_q8_quantize_row.argtypes = [_f32p, C.c_size_t, _u8p]
    L.lq4o_q8_dequantize.restype = C.c_size_t
    L.lq4o_q8_dequantize.argtypes = [_u8p, C.c_size_t, _f32p]
    L.lq4o_q8_gemm_f32.restype = C.c_int
    L.lq4o_q8_gemm_f32.argtypes = [_f32p, _u8p, _f32p, C.c_size_t, C.c_size_t, C.c_size_t]
    L.lq4o_q8_gemm_f64.restype = C.c_int
    L.lq4o_q8_gemm_f64.argtypes = [_f32p, _u8p, _f64p, C.c_size_t, C.c_size_t, C.c_size_t]
    L.lq4o_shifted_rms_norm.restype = None
    L.lq4o_shifted_rms_norm.argtypes = [_f32p, _f32p, C.c_size_t, C.c_size_t, C.c_float]
    L.lq4o_residual_add_norm.restype = None
    L.lq4o_residual_add_norm.argtypes = [_f32p, _f32p, _f32p, C.c_size_t, C.c_size_t, C.c_float, _f32p, _f32p]
    L.lq4o_silu_mul.restype = None
    L.lq4o_silu_mul.argtypes = [_f32p, C.c_size_t, C.c_size_t, _f32p]
    L.lq4o_add_and_copy.restype = None
    L.lq4o_add_and_copy.argtypes = [_f32p, _f32p, _f32p, C.c_size_t]
    L.lq4o_topk.restype = None
    L.lq4o_topk.argtypes = [_f32p, C.c_uint32, C.c_uint32, _f32p, C.POINTER(C.c_uint32)]
    L.lq4o_parse_q4_file.restype = C.c_int
    L.lq4o_parse_q4_file.argtypes = [_u8p, C.c_size_t, _u64p, C.c_int, C.POINTER(C.c_int), _u64p,
                                     _u64p]
    for name in ("lq4o_matmul_bt_avx2", "lq4o_matmul_bt_avx512", "lq4o_matmul_bt_tiled_avx2"):
        fn = getattr(L, name)
        fn.restype = None
        fn.argtypes = [_f32p, _f32p, _f32p, C.c_size_t, C.c_size_t, C.c_size_t]
    L.lq4o_matmul_bt.restype = C.c_int
    L.lq4o_matmul_bt.argtypes = [_f32p, _f32p, _f32p, C.c_size_t, C.c_size_t, C.c_size_t]
    L.lq4o_cpu_q4_matmul.restype = C.c_int
    L.lq4o_cpu_q4_matmul.argtypes = [_f32p, _u8p, _f32p, _f32p, C.c_size_t, C.c_size_t,
                                     C.c_size_t, C.c_int, C.c_int]
    _lib = L
    return L


def _p(a: np.ndarray, t):
    return a.ctypes.data_as(t)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    if isinstance(a, (bytes, bytearray, memoryview)):
        a = np.frombuffer(bytes(a), dtype=np.uint8)
    return np.ascontiguousarray(a, dtype=np.uint8)


# --- scalar conversions -----------------------------------------------------
def f16_to_f32(bits: int) -> float:
    return float(lib().lq4o_f16_to_f32(int(bits) & 0xFFFF))


def f32_to_f16(v: float) -> int:
    return int(lib().lq4o_f32_to_f16(C.c_float(v)))


def f32_bits_to_f16(bits: np.ndarray) -> np.ndarray:
    """f32 -> f16 over raw f32 bit patterns (bit patterns so NaN payloads survive)."""
    b = np.ascontiguousarray(bits, dtype=np.uint32).ravel()
    out = np.zeros(b.size, dtype=np.uint16)
    lib().lq4o_f32_to_f16_array(_p(b, C.POINTER(C.c_uint32)), _p(out, C.POINTER(C.c_uint16)),
                                b.size)
    return out


def f16_bits_to_f32_bits(bits: np.ndarray) -> np.ndarray:
    b = np.ascontiguousarray(bits, dtype=np.uint16).ravel()
    out = np.zeros(b.size, dtype=np.uint32)
    lib().lq4o_f16_to_f32_array(_p(b, C.POINTER(C.c_uint16)), _p(out, C.POINTER(C.c_uint32)),
                                b.size)
    return out


def sweep_f32_to_f16_vs_f16c(first: int, last: int, stride: int):
    """(mismatch count, first offending f32 bit pattern) against the CPU's vcvtps2ph."""
    bad = C.c_uint32(0)
    n = lib().lq4o_sweep_f32_to_f16_vs_f16c(first, last, stride, C.byref(bad))
    return int(n), int(bad.value)


# --- quantize / dequantize --------------------------------------------------
class QuantizeError(ValueError):
    def __init__(self, code: int):
        names = {1: "valid_len outside 1..=32", 2: "non-finite source weight",
                 3: "scale is not a finite, strictly positive f16",
                 4: "bias is not a finite f16"}
        super().__init__(names.get(code, f"code {code}"))
        self.code = code


def quantize_block(vals, valid_len: int = 32, symmetric: bool = False) -> bytes:
    v = _f32(vals)
    assert v.size == 32
    out = np.zeros(BLOCK_BYTES, dtype=np.uint8)
    rc = lib().lq4o_quantize_block(_p(v, _f32p), valid_len, int(symmetric), _p(out, _u8p))
    if rc:
        raise QuantizeError(rc)
    return out.tobytes()


def quantize_flat(src, symmetric: bool = False) -> np.ndarray:
    v = _f32(src).ravel()
    out = np.zeros(((v.size + 31) // 32) * BLOCK_BYTES, dtype=np.uint8)
    rc = lib().lq4o_quantize_flat(_p(v, _f32p), v.size, int(symmetric), _p(out, _u8p))
    if rc:
        raise QuantizeError(rc)
    return out


def quantize_rows(src, symmetric: bool = False) -> np.ndarray:
    v = _f32(src)
    rows, cols = v.shape
    out = np.zeros(rows * ((cols + 31) // 32) * BLOCK_BYTES, dtype=np.uint8)
    rc = lib().lq4o_quantize_rows(_p(v, _f32p), rows, cols, int(symmetric), _p(out, _u8p))
    if rc:
        raise QuantizeError(rc)
    return out


def dequantize(data, n_weights: int) -> np.ndarray:
    d = _u8(data)
    out = np.zeros(n_weights, dtype=np.float32)
    got = lib().lq4o_dequantize(_p(d, _u8p), d.size, n_weights, _p(out, _f32p))
    return out[:got]


def validate_blocks(payload):
    """Returns (index_of_first_bad_block or -1, reason 0/1=scale/2=bias)."""
    d = _u8(payload)
    why = C.c_int(0)
    idx = lib().lq4o_validate_blocks(_p(d, _u8p), d.size, C.byref(why))
    return int(idx), int(why.value)


# --- matmul -----------------------------------------------------------------
def gemm_f32(x, wq, n: int, k: int) -> np.ndarray:
    xx = _f32(x).reshape(-1, k)
    w = _u8(wq)
    assert w.size >= n * (k // 32) * BLOCK_BYTES
    y = np.zeros((xx.shape[0], n), dtype=np.float32)
    rc = lib().lq4o_gemm_f32(_p(xx, _f32p), _p(w, _u8p), _p(y, _f32p), xx.shape[0], n, k)
    if rc:
        raise ValueError(f"lq4o_gemm_f32 rc={rc} (k must be a non-zero multiple of 32)")
    return y


def gemm_f64(x, wq, n: int, k: int) -> np.ndarray:
    xx = _f32(x).reshape(-1, k)
    w = _u8(wq)
    assert w.size >= n * (k // 32) * BLOCK_BYTES
    y = np.zeros((xx.shape[0], n), dtype=np.float64)
    rc = lib().lq4o_gemm_f64(_p(xx, _f32p), _p(w, _u8p), _p(y, _f64p), xx.shape[0], n, k)
    if rc:
        raise ValueError(f"lq4o_gemm_f64 rc={rc}")
    return y


def lora_apply(a, b, scale: float, x, y) -> np.ndarray:
    """y[m, d_out] += scale * B.(A.x[m]) in f32; returns the updated copy."""
    aa, bb = _f32(a), _f32(b)
    rank, d_in = aa.shape
    d_out = bb.shape[0]
    xx = _f32(x).reshape(-1, d_in)
    yy = _f32(y).reshape(-1, d_out).copy()
    lib().lq4o_lora_apply(_p(aa, _f32p), _p(bb, _f32p), rank, d_in, d_out, scale, _p(xx, _f32p),
                          _p(yy, _f32p), xx.shape[0])
    return yy


def lora_apply_f64(a, b, scale: float, x, y) -> np.ndarray:
    aa, bb = _f32(a), _f32(b)
    rank, d_in = aa.shape
    d_out = bb.shape[0]
    xx = _f32(x).reshape(-1, d_in)
    yy = np.ascontiguousarray(y, dtype=np.float64).reshape(-1, d_out).copy()
    lib().lq4o_lora_apply_f64(_p(aa, _f32p), _p(bb, _f32p), rank, d_in, d_out, scale,
                              _p(xx, _f32p), _p(yy, _f64p), xx.shape[0])
    return yy


# --- MoE --------------------------------------------------------------------
def moe_route(logits, top_k: int):
    """logits [T, E] -> (ids [T, top_k] int32, weights [T, top_k] f32, probs [T, E])."""
    lg = _f32(logits)
    if lg.ndim == 1:
        lg = lg[None, :]
    t, e = lg.shape
    ids = np.zeros((t, top_k), dtype=np.int32)
    wts = np.zeros((t, top_k), dtype=np.float32)
    probs = np.zeros((t, e), dtype=np.float32)
    for i in range(t):
        lib().lq4o_moe_route(_p(lg[i], _f32p), e, top_k, _p(probs[i], _f32p), _p(ids[i], _i32p),
                             _p(wts[i], _f32p))
    return ids, wts, probs


def router_softmax(logits) -> np.ndarray:
    lg = _f32(logits).ravel()
    probs = np.zeros_like(lg)
    lib().lq4o_router_softmax(_p(lg, _f32p), lg.size, _p(probs, _f32p))
    return probs


def select_top_k(probs, top_k: int):
    pr = _f32(probs).ravel()
    ids = np.zeros(top_k, dtype=np.int32)
    vals = np.zeros(top_k, dtype=np.float32)
    lib().lq4o_select_top_k(_p(pr, _f32p), pr.size, top_k, _p(ids, _i32p), _p(vals, _f32p))
    return ids, vals


def renormalize_selected(vals) -> np.ndarray:
    v = _f32(vals).ravel().copy()
    lib().lq4o_renormalize_selected(_p(v, _f32p), v.size)
    return v


def moe_ffn(gate_up_q4, down_q4, num_experts, inter, hidden, x, ids, weights, f64=False):
    gu, dn = _u8(gate_up_q4), _u8(down_q4)
    xx = _f32(x).reshape(-1, hidden)
    ii = np.ascontiguousarray(ids, dtype=np.int32)
    ww = _f32(weights)
    t, top_k = ii.shape
    assert xx.shape[0] == t
    assert gu.size == num_experts * 2 * inter * (hidden // 32) * BLOCK_BYTES
    assert dn.size == num_experts * hidden * (inter // 32) * BLOCK_BYTES
    out = np.zeros((t, hidden), dtype=np.float64 if f64 else np.float32)
    fn = lib().lq4o_moe_ffn_f64 if f64 else lib().lq4o_moe_ffn_f32
    rc = fn(_p(gu, _u8p), _p(dn, _u8p), num_experts, inter, hidden, _p(xx, _f32p), t,
            _p(ii, _i32p), _p(ww, _f32p), top_k, _p(out, _f64p if f64 else _f32p))
    if rc:
        raise ValueError(f"moe_ffn rc={rc}")
    return out


def moe_shared_expert(gate_up_q4, down_q4, shared_gate, shared_inter, hidden, x, out, f64=False):
    """apply_shared_expert (moe.rs:194-250) over Q4 tensors; returns ``out`` plus the gated
    shared-expert FFN of every row of ``x`` (``out`` itself is left untouched)."""
    gu, dn = _u8(gate_up_q4), _u8(down_q4)
    xx = _f32(x).reshape(-1, hidden)
    sg = _f32(shared_gate).ravel()
    assert sg.size == hidden
    assert gu.size == 2 * shared_inter * (hidden // 32) * BLOCK_BYTES
    assert dn.size == hidden * (shared_inter // 32) * BLOCK_BYTES
    acc = np.array(out, dtype=np.float64 if f64 else np.float32).reshape(xx.shape[0], hidden).copy()
    fn = lib().lq4o_moe_shared_expert_f64 if f64 else lib().lq4o_moe_shared_expert_f32
    rc = fn(_p(gu, _u8p), _p(dn, _u8p), _p(sg, _f32p), shared_inter, hidden, _p(xx, _f32p),
            xx.shape[0], _p(acc, _f64p if f64 else _f32p))
    if rc:
        raise ValueError(f"moe_shared_expert rc={rc}")
    return acc


# --- .q4 file ---------------------------------------------------------------
Q4_FILE_ERRORS = {1: "invalid magic: not a .q4 file", 2: "legacy .q4 file (v1)",
                  3: "unsupported .q4 file version", 4: "header truncated",
                  5: "file truncated below Q4 block payload",
                  6: "file has trailing bytes after Q4 block payload",
                  7: "original_len does not match shape"}


def q3_quantize_block(vals, valid_len: int = 32, symmetric: bool = False) -> bytes:
    """One 16-byte Q3 block (quantize_block_with_mode_len, weights/q3_weights.rs:199-262)."""
    v = np.zeros(32, dtype=np.float32)
    vals = _f32(vals).reshape(-1)
    v[:vals.size] = vals
    out = np.empty(16, dtype=np.uint8)
    rc = lib().lq4o_q3_quantize_block(_p(v, _f32p), valid_len, int(symmetric), _p(out, _u8p))
    if rc:
        raise ValueError("Q3 weight block: bad valid_len" if rc == 1 else "Q3 weight block contains a non-finite value")
    return out.tobytes()


def q3_quantize_rows(src, symmetric: bool = False) -> np.ndarray:
    """Q3 blocks of every row of src [rows, cols] (quantize_tensor_q3_0, q3_weights.rs:321-345);
    a row whose length is not a multiple of 32 ends in a zero-padded block."""
    src = _f32(src)
    rows = src.reshape(-1, src.shape[-1])
    nb = (rows.shape[1] + 31) // 32
    out = np.empty((rows.shape[0], nb * 16), dtype=np.uint8)
    for r in range(rows.shape[0]):
        rc = lib().lq4o_q3_quantize_row(_p(rows[r], _f32p), rows.shape[1], int(symmetric), _p(out[r], _u8p))
        if rc:
            raise ValueError("Q3 weight block contains a non-finite value")
    return out.reshape(-1)


def q3_dequantize(data, n_weights: int) -> np.ndarray:
    data = _u8(data)
    out = np.empty(n_weights, dtype=np.float32)
    done = lib().lq4o_q3_dequantize(_p(data, _u8p), data.size, n_weights, _p(out, _f32p))
    return out[:done]


def q3_gemm_f32(x, wq, n: int, k: int) -> np.ndarray:
    x, wq = _f32(x), _u8(wq)
    m = x.size // k
    assert wq.size >= n * (k // 32) * 16
    y = np.empty((m, n), dtype=np.float32)
    rc = lib().lq4o_q3_gemm_f32(_p(x, _f32p), _p(wq, _u8p), _p(y, _f32p), m, n, k)
    assert rc == 0, rc
    return y


def q3_gemm_f64(x, wq, n: int, k: int) -> np.ndarray:
    x, wq = _f32(x), _u8(wq)
    m = x.size // k
    y = np.empty((m, n), dtype=np.float64)
    rc = lib().lq4o_q3_gemm_f64(_p(x, _f32p), _p(wq, _u8p), _p(y, _f64p), m, n, k)
    assert rc == 0, rc
    return y


def q8_quantize_rows(src) -> np.ndarray:
    """Q8_0 blocks (34 bytes per 32 weights) of every row of src [rows, k]
    (quantize_row_q8_0, forward/metal_qwen35.rs:2323-2346); ValueError on a non-finite value."""
    src = _f32(src)
    rows = src.reshape(-1, src.shape[-1])
    k = rows.shape[1]
    assert k % 32 == 0
    out = np.empty((rows.shape[0], (k // 32) * 34), dtype=np.uint8)
    for r in range(rows.shape[0]):
        rc = lib().lq4o_q8_quantize_row(_p(rows[r], _f32p), k, _p(out[r], _u8p))
        if rc != 0:
            raise ValueError(f"Q8_0 weight block {-rc - 1} of row {r} contains a non-finite value")
    return out.reshape(-1)


def q8_dequantize(data, n_weights: int) -> np.ndarray:
    data = _u8(data)
    assert data.size >= (n_weights // 32) * 34
    out = np.empty(n_weights, dtype=np.float32)
    lib().lq4o_q8_dequantize(_p(data, _u8p), n_weights, _p(out, _f32p))
    return out


def q8_gemm_f32(x, wq, n: int, k: int) -> np.ndarray:
    x, wq = _f32(x), _u8(wq)
    m = x.size // k
    assert wq.size >= n * (k // 32) * 34
    y = np.empty((m, n), dtype=np.float32)
    rc = lib().lq4o_q8_gemm_f32(_p(x, _f32p), _p(wq, _u8p), _p(y, _f32p), m, n, k)
    assert rc == 0, rc
    return y


def q8_gemm_f64(x, wq, n: int, k: int) -> np.ndarray:
    x, wq = _f32(x), _u8(wq)
    m = x.size // k
    y = np.empty((m, n), dtype=np.float64)
    rc = lib().lq4o_q8_gemm_f64(_p(x, _f32p), _p(wq, _u8p), _p(y, _f64p), m, n, k)
    assert rc == 0, rc
    return y


def shifted_rms_norm(x, gamma, eps: float) -> np.ndarray:
    """Qwen3.5 shifted RMSNorm of every row of x [rows, hidden] (model/qwen35/norm.rs:6-23)."""
    x = np.array(_f32(x), copy=True)
    x2 = x.reshape(-1, x.shape[-1])
    gamma = _f32(gamma)
    assert gamma.size == x2.shape[1]
    lib().lq4o_shifted_rms_norm(_p(x2, _f32p), _p(gamma, _f32p), x2.shape[1], x2.shape[0], eps)
    return x


def residual_add_norm(base, delta, gamma, eps: float):
    """(residual_out, normed_out) of fused_residual_add_norm (qwen35.metal:739-767)."""
    base, delta, gamma = _f32(base), _f32(delta), _f32(gamma)
    assert base.shape == delta.shape and gamma.size == base.shape[-1]
    rows = base.size // base.shape[-1]
    res, normed = np.empty_like(base), np.empty_like(base)
    lib().lq4o_residual_add_norm(_p(base, _f32p), _p(delta, _f32p), _p(gamma, _f32p), base.shape[-1],
                                 rows, eps, _p(res, _f32p), _p(normed, _f32p))
    return res, normed


def silu_mul(gate_up) -> np.ndarray:
    """silu(gate) * up for rows of [gate | up] (qwen35.metal:712-722)."""
    gate_up = _f32(gate_up)
    g2 = gate_up.reshape(-1, gate_up.shape[-1])
    count = g2.shape[1] // 2
    assert g2.shape[1] == 2 * count
    out = np.empty((g2.shape[0], count), dtype=np.float32)
    lib().lq4o_silu_mul(_p(g2, _f32p), count, g2.shape[0], _p(out, _f32p))
    return out.reshape(gate_up.shape[:-1] + (count,))


def add_and_copy(src, residual):
    """(updated residual, copy) of add_and_copy (qwen35.metal:2255-2266)."""
    src = _f32(src)
    res = np.array(_f32(residual), copy=True)
    dst = np.empty_like(res)
    lib().lq4o_add_and_copy(_p(src, _f32p), _p(res, _f32p), _p(dst, _f32p), res.size)
    return res, dst


def topk(logits, k: int):
    """(logits[k], ids[k]) of the k best entries in the reference's top-k order (higher logit
    first, ties to the lower id, NaN last as the (-inf, 0xFFFFFFFF) sentinel)."""
    lg = _f32(logits).reshape(-1)
    out_l = np.empty(k, dtype=np.float32)
    out_i = np.empty(k, dtype=np.uint32)
    lib().lq4o_topk(_p(lg, _f32p), lg.size, k, _p(out_l, _f32p), _p(out_i, C.POINTER(C.c_uint32)))
    return out_l, out_i


def parse_q4_file(data):
    """Returns (shape tuple, original_len, payload_offset); raises ValueError."""
    d = _u8(data)
    shape = np.zeros(8, dtype=np.uint64)
    ndim = C.c_int(0)
    olen = C.c_uint64(0)
    off = C.c_uint64(0)
    rc = lib().lq4o_parse_q4_file(_p(d, _u8p), d.size, _p(shape, _u64p), 8, C.byref(ndim),
                                  C.byref(olen), C.byref(off))
    if rc:
        raise ValueError(Q4_FILE_ERRORS.get(rc, f"code {rc}"))
    return tuple(int(s) for s in shape[: ndim.value]), int(olen.value), int(off.value)


# --- CPU baseline (timed by bench.py) ----------------------------------------
KERNEL_NAMES = {0: "tiled(4x8 AVX2 micro-kernel / scalar edge tiles)", 1: "avx512f dot",
                2: "avx2 dot"}


def matmul_bt(a, b, m: int, k: int, n: int, kernel: str = "dispatch"):
    aa, bb = _f32(a), _f32(b)
    c = np.zeros((m, n), dtype=np.float32)
    L = lib()
    if kernel == "dispatch":
        kid = L.lq4o_matmul_bt(_p(aa, _f32p), _p(bb, _f32p), _p(c, _f32p), m, k, n)
        return c, kid
    fn = {"avx2": L.lq4o_matmul_bt_avx2, "avx512": L.lq4o_matmul_bt_avx512,
          "tiled": L.lq4o_matmul_bt_tiled_avx2}[kernel]
    fn(_p(aa, _f32p), _p(bb, _f32p), _p(c, _f32p), m, k, n)
    return c, {"avx2": 2, "avx512": 1, "tiled": 0}[kernel]


def cpu_q4_matmul(x, wq, w_scratch, m, n, k, mode=0, skip_dequant=False):
    xx, w = _f32(x), _u8(wq)
    y = np.zeros((m, n), dtype=np.float32)
    kid = lib().lq4o_cpu_q4_matmul(_p(xx, _f32p), _p(w, _u8p), _p(w_scratch, _f32p),
                                   _p(y, _f32p), m, n, k, mode, int(skip_dequant))
    return y, kid
