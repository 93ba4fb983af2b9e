"""Host-side mirror of the reference's Q4 dispatch contract, over the C ABI.

The reference exposes this path as inherent methods of ``MetalQwen35State``
(crates/inference/src/forward/metal_qwen35/inner/dispatch.rs and layers/mod.rs);
:class:`HipQ4Backend` keeps the same method names, argument order, byte-offset
convention and error behaviour so a parity test reads like the reference's own:

=====================================  ===========================================
reference                              here
=====================================  ===========================================
``Q4WeightBuf`` (metal_qwen35.rs:599)  :class:`Q4WeightBuf`
``mmap_q4_weight`` (:660)              :meth:`HipQ4Backend.mmap_q4_weight`
``make_buffer_q4_0`` (:2362)           :meth:`HipQ4Backend.upload_q4_blocks`
``dispatch_matmul`` (dispatch.rs:231)  :meth:`HipQ4Backend.dispatch_matmul`
``dispatch_gemm`` (:507)               :meth:`HipQ4Backend.dispatch_gemm`
``dispatch_gemm_at`` (:935)            :meth:`HipQ4Backend.dispatch_gemm_at`
``load_lora_adapter`` (mq35.rs:3806)   :meth:`HipQ4Backend.load_lora_adapter`
``dispatch_lora_if_active`` (mod.rs:15) :meth:`HipQ4Backend.dispatch_lora_if_active`
=====================================  ===========================================

Device buffers are torch CUDA tensors (torch is only the allocator and stream
provider); every computation goes through ``liblattice_hip_q4.so``.  There is no CPU
fallback: a missing library raises :class:`Q4LibraryMissing` at first use.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import q4_file
from .q4_layout import BLOCK_BYTES, BLOCK_WEIGHTS

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblattice_hip_q4.so")

LQ4_F32, LQ4_F16 = 0, 1
MAX_GEMV_BATCH = 16

EXPORTS = [
    "lq4_last_error", "lq4_version", "lq4_ctx_create", "lq4_ctx_destroy", "lq4_sync",
    "lq4_validate_blocks", "lq4_weight_upload", "lq4_weight_wrap", "lq4_weight_free",
    "lq4_weight_info", "lq4_lora_upload", "lq4_lora_free", "lq4_lora_apply", "lq4_gemv",
    "lq4_gemm", "lq4_moe_route", "lq4_moe_grouped_gemv", "lq4_moe_shared_expert", "lq4_moe_ffn", "lq4_dequant",
    "lq4_topk",
    "lq4_lm_head_topk",
    "lq4_probe_read",
    "lq4_probe_read_config",
    "lq4_probe_copy",
    "lq4_gemv_multi",
    "lq4_set_gemv_kernel",
    "lq4_set_gemm_kernel",
    "lq4_residual_add_rmsnorm", "lq4_silu_mul", "lq4_add_and_copy", "lq4_gemv_fused", "lq4_gemv_fused_batch",
    "lq4_lm_head_topk_static",
    "lq4_gemv_chain", "lq4_ctx_reserve_scratch",
    "lq4_gemv_q8", "lq4_gemm_q8", "lq4_gemv_q3", "lq4_gemm_q3",
    "lq4_get_path_counters", "lq4_malloc", "lq4_free", "lq4_memcpy_h2d", "lq4_memcpy_d2h",
]


class Q4LibraryMissing(RuntimeError):
    pass


class Q4Error(RuntimeError):
    """A C-ABI call returned a negative code; ``code`` is the LQ4_E_* value."""

    def __init__(self, code: int, message: str):
        super().__init__(f"[{code}] {message}")
        self.code = code
        self.message = message


class PathCounters(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("gemv", "gemm", "lora_a", "moe_route", "moe_gate_up",
                                         "moe_down", "dequant", "topk", "gemv_fused", "elementwise",
                                         "gemv_chain", "lora_t_fallback", "gemv_multi")]


MAX_PROJECTIONS = 8


class Projection(C.Structure):
    """lq4_projection: one weight view of lq4_gemv_multi with its output and optional adapter."""
    _fields_ = [("w", C.c_void_p), ("w_extra_offset", C.c_uint64), ("n", C.c_uint32), ("y_dev", C.c_void_p),
                ("lora", C.c_void_p), ("lora_scale", C.c_float)]


LQ4_PRO_NONE, LQ4_PRO_ADD_RMSNORM, LQ4_PRO_SILU_MUL = 0, 1, 2
LQ4_EPI_NONE, LQ4_EPI_ADD_RESIDUAL, LQ4_EPI_SILU_MUL_PAIRS = 0, 1, 2
CHAIN_MAX_STEPS = 16
GEMV_KERNEL_AUTO, GEMV_KERNEL_LANE_BLOCKS, GEMV_KERNEL_LDS_RING = 0, 1, 2  # lq4_set_gemv_kernel


class GemvFusion(C.Structure):
    """``lq4_gemv_fusion``: elementwise steps fused into the batch-1 GEMV."""
    _fields_ = [("prologue", C.c_int), ("base", C.c_void_p), ("delta", C.c_void_p), ("gamma", C.c_void_p),
                ("eps", C.c_float), ("residual_out", C.c_void_p), ("epilogue", C.c_int),
                ("residual", C.c_void_p), ("copy_dst", C.c_void_p)]


class ChainStep(C.Structure):
    """``lq4_chain_step``: one batch-1 GEMV of a chain that runs as a single launch."""
    _fields_ = [("w", C.c_void_p), ("w_extra_offset", C.c_uint64), ("n", C.c_uint32), ("k", C.c_uint32),
                ("from_previous", C.c_int),
                ("x_dev", C.c_void_p), ("prologue", C.c_int), ("base", C.c_void_p), ("delta", C.c_void_p),
                ("gamma", C.c_void_p), ("eps", C.c_float), ("residual_out", C.c_void_p), ("epilogue", C.c_int),
                ("residual", C.c_void_p), ("y_dev", C.c_void_p)]


_lib = None


def load_library() -> C.CDLL:
    """Loads the in-tree shared library (after torch, so both share one HIP runtime)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise Q4LibraryMissing(
            f"{LIB_PATH} is not built; run `python -m lattice_amd.build` (there is no CPU fallback)")
    import torch  # noqa: F401  (loads libamdhip64 first)
    L = C.CDLL(LIB_PATH)
    vp, u32, u64, f32 = C.c_void_p, C.c_uint32, C.c_uint64, C.c_float
    sig = {
        "lq4_last_error": (C.c_char_p, []),
        "lq4_version": (C.c_char_p, []),
        "lq4_ctx_create": (C.c_int, [C.c_int, C.POINTER(vp)]),
        "lq4_ctx_destroy": (C.c_int, [vp]),
        "lq4_sync": (C.c_int, [vp, vp]),
        "lq4_validate_blocks": (C.c_int, [vp, C.c_size_t, C.POINTER(C.c_int64), C.POINTER(C.c_int)]),
        "lq4_weight_upload": (C.c_int, [vp, vp, C.c_size_t, u64, C.c_int, C.POINTER(vp)]),
        "lq4_weight_wrap": (C.c_int, [vp, vp, C.c_size_t, u64, C.POINTER(vp)]),
        "lq4_weight_free": (C.c_int, [vp]),
        "lq4_weight_info": (C.c_int, [vp, C.POINTER(vp), C.POINTER(C.c_size_t), C.POINTER(u64)]),
        "lq4_lora_upload": (C.c_int, [vp, vp, vp, C.c_int, u32, u32, u32, C.POINTER(vp)]),
        "lq4_lora_free": (C.c_int, [vp]),
        "lq4_lora_apply": (C.c_int, [vp, vp, f32, vp, C.c_int, u32, vp, vp]),
        "lq4_gemv": (C.c_int, [vp, vp, u64, u32, u32, vp, u32, vp, vp, f32, vp]),
        "lq4_gemm": (C.c_int, [vp, vp, u64, u32, u32, vp, C.c_int, u32, vp, vp, f32, vp]),
        "lq4_moe_route": (C.c_int, [vp, vp, u32, u32, u32, vp, vp, vp]),
        "lq4_moe_grouped_gemv": (C.c_int, [vp, vp, vp, u32, u32, u32, vp, u32, vp, vp, u32, vp, vp]),
        "lq4_moe_shared_expert": (C.c_int, [vp, vp, vp, vp, u32, u32, vp, u32, vp, vp]),
        "lq4_moe_ffn": (C.c_int, [vp, vp, vp, vp, u32, u32, u32, vp, vp, vp, u32, u32, vp, u32, vp, vp]),
        "lq4_dequant": (C.c_int, [vp, vp, u64, u32, u32, vp, vp]),
        "lq4_topk": (C.c_int, [vp, vp, C.c_uint32, C.c_uint32, vp, vp, vp]),
        "lq4_lm_head_topk": (C.c_int, [vp, vp, C.c_uint64, C.c_uint32, C.c_uint32, vp, C.c_uint32, vp, vp, vp]),
        "lq4_lm_head_topk_static": (C.c_int, [vp, vp, C.c_uint64, C.c_uint32, C.c_uint32, vp, C.c_uint32, vp, vp, vp]),
        "lq4_probe_read": (C.c_int, [vp, vp, C.c_size_t, vp]),
        "lq4_probe_read_config": (C.c_int, [vp, vp, C.c_size_t, C.c_uint32, C.c_uint32, C.c_int, C.c_int, vp]),
        "lq4_probe_copy": (C.c_int, [vp, vp, vp, C.c_size_t, vp]),
        "lq4_gemv_multi": (C.c_int, [vp, C.POINTER(Projection), C.c_uint32, C.c_uint32, vp, C.c_uint32, vp]),
        "lq4_set_gemv_kernel": (C.c_int, [vp, C.c_int]),
        "lq4_set_gemm_kernel": (C.c_int, [vp, C.c_int]),
        "lq4_residual_add_rmsnorm": (C.c_int, [vp, vp, vp, vp, C.c_uint32, C.c_uint32, C.c_float, vp, vp, vp]),
        "lq4_silu_mul": (C.c_int, [vp, vp, C.c_uint32, C.c_uint32, vp, C.c_uint32, vp]),
        "lq4_add_and_copy": (C.c_int, [vp, vp, vp, vp, C.c_size_t, vp]),
        "lq4_gemv_q8": (C.c_int, [vp, vp, C.c_uint64, C.c_uint32, C.c_uint32, vp, C.c_uint32, vp, vp]),
        "lq4_gemm_q8": (C.c_int, [vp, vp, C.c_uint64, C.c_uint32, C.c_uint32, vp, C.c_int, C.c_uint32, vp, vp]),
        "lq4_gemv_q3": (C.c_int, [vp, vp, C.c_uint64, C.c_uint32, C.c_uint32, vp, C.c_uint32, vp, vp]),
        "lq4_gemm_q3": (C.c_int, [vp, vp, C.c_uint64, C.c_uint32, C.c_uint32, vp, C.c_int, C.c_uint32, vp, vp]),
        "lq4_gemv_fused": (C.c_int, [vp, vp, C.c_uint64, C.c_uint32, C.c_uint32, vp, vp, C.POINTER(GemvFusion), vp,
                                     C.c_float, vp]),
        "lq4_gemv_fused_batch": (C.c_int, [vp, vp, C.c_uint64, C.c_uint32, C.c_uint32, vp, C.c_uint32, vp,
                                           C.POINTER(GemvFusion), vp, C.c_float, vp]),
        "lq4_gemv_chain": (C.c_int, [vp, C.POINTER(ChainStep), C.c_uint32, vp]),
        "lq4_ctx_reserve_scratch": (C.c_int, [vp, C.c_size_t]),
        "lq4_get_path_counters": (C.c_int, [vp, C.POINTER(PathCounters)]),
        "lq4_malloc": (C.c_int, [vp, C.c_size_t, C.POINTER(vp)]),
        "lq4_free": (C.c_int, [vp, vp]),
        "lq4_memcpy_h2d": (C.c_int, [vp, vp, vp, C.c_size_t]),
        "lq4_memcpy_d2h": (C.c_int, [vp, vp, vp, C.c_size_t]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    _lib = L
    return L


def _check(rc: int):
    if rc != 0:
        raise Q4Error(rc, load_library().lq4_last_error().decode(errors="replace"))


def validate_blocks(payload) -> None:
    """Host-side ``Q4BlockCheck::Now`` (q4_weights.rs:907-947): raises :class:`Q4Error`
    naming the first block whose scale is non-finite or non-positive or whose bias is
    non-finite.  Needs no GPU."""
    buf = np.ascontiguousarray(np.frombuffer(payload, dtype=np.uint8) if isinstance(
        payload, (bytes, bytearray, memoryview)) else payload, dtype=np.uint8)
    _check(load_library().lq4_validate_blocks(buf.ctypes.data, buf.size, None, None))


@dataclass
class Q4WeightBuf:
    """Device-resident Q4 buffer plus the byte offset of its block payload
    (``Q4WeightBuf { buffer, payload_offset, .. }``, metal_qwen35.rs:599-636)."""
    handle: int
    nbytes: int
    payload_offset: int
    _backend: "HipQ4Backend"
    _keepalive: object = None

    def free(self):
        if self.handle:
            _check(load_library().lq4_weight_free(self.handle))
            self.handle = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


@dataclass
class LoraLayerData:
    """One layer's adapter factors (metal_qwen35.rs:1701-1716): ``modules`` maps a
    projection name ("q_proj", "v_proj", ...) to ``(A [rank, d_in], B [d_out, rank])``."""
    layer_idx: int
    modules: Dict[str, Tuple[np.ndarray, np.ndarray]]


@dataclass
class ModelShapes:
    """What ``load_lora_adapter`` reads from the engine's model configuration in the reference
    (``self.engine.config``, metal_qwen35.rs:3832, 3852, 3746-3768): the layer count, the hidden size and
    the projection shape of a ``(layer_idx, module)`` pair.  ``projection_shape`` returns ``(d_in, d_out)``
    or raises ``ValueError`` with the reference's message ("unknown LoRA module ...").  ``quarot_rotate``
    is the host crate's ``rotate_adapter_for_quarot`` (quant/quarot/lora.rs): it rotates the layers' factors in
    place for a QuaRot-converted base, ``quarot_rotate(layers, seed, hidden_size)``."""
    num_hidden_layers: int
    hidden_size: int
    projection_shape: Callable[[int, str], Tuple[int, int]]
    quarot_rotate: Optional[Callable] = None


class _LoraProjection:
    def __init__(self, handle, rank, d_in, d_out):
        self.handle, self.rank, self.d_in, self.d_out = handle, rank, d_in, d_out


def _dtype_code(t) -> int:
    import torch
    if t.dtype == torch.float32:
        return LQ4_F32
    if t.dtype == torch.float16:
        return LQ4_F16
    raise TypeError(f"activations must be float32 or float16, got {t.dtype}")


class HipQ4Backend:
    """One GPU's Q4 matmul backend: owns a ``lq4_ctx`` and the loaded LoRA adapter."""

    def __init__(self, device: int = 0, model: Optional["ModelShapes"] = None):
        """``model``: the engine's model configuration as far as this path reads it (adapter checks); without
        it ``load_lora_adapter`` checks everything that does not need the model."""
        import torch
        if not torch.cuda.is_available():
            raise RuntimeError("HipQ4Backend needs a HIP device; there is no CPU fallback")
        self.lib = load_library()
        self.device = device
        self.torch_device = torch.device("cuda", device)
        ctx = C.c_void_p()
        _check(self.lib.lq4_ctx_create(device, C.byref(ctx)))
        self.ctx = ctx
        self.model = model
        self._lora: Dict[Tuple[int, str], _LoraProjection] = {}
        self._lora_scale = 0.0

    def close(self):
        self.unload_lora_adapter()
        if self.ctx:
            self.lib.lq4_ctx_destroy(self.ctx)
            self.ctx = None

    # ------------------------------------------------------------------ helpers
    def _stream(self):
        import torch
        return C.c_void_p(torch.cuda.current_stream(self.torch_device).cuda_stream)

    def synchronize(self):
        _check(self.lib.lq4_sync(self.ctx, self._stream()))

    def path_counters(self) -> Dict[str, int]:
        pc = PathCounters()
        _check(self.lib.lq4_get_path_counters(self.ctx, C.byref(pc)))
        return {n: int(getattr(pc, n)) for n, _ in PathCounters._fields_}

    def probe_read(self, t):
        """One read-only streaming launch over tensor ``t`` (bandwidth-ceiling calibration)."""
        _check(self.lib.lq4_probe_read(self.ctx, t.data_ptr(), t.numel() * t.element_size(), self._stream()))

    def probe_read_config(self, t, nbytes: int, workgroups: int, bytes_in_flight: int, strided: bool,
                          nontemporal: bool, offset: int = 0):
        """The read probe with its launch spelled out, over ``nbytes`` of ``t`` from byte ``offset``."""
        _check(self.lib.lq4_probe_read_config(self.ctx, t.data_ptr() + offset, nbytes, workgroups, bytes_in_flight,
                                              int(strided), int(nontemporal), self._stream()))

    def reserve_scratch(self, nbytes: int):
        """Grows the context's scratch ahead of time (growing it allocates, which a call under HIP
        graph capture refuses to do)."""
        _check(self.lib.lq4_ctx_reserve_scratch(self.ctx, int(nbytes)))

    def set_gemv_kernel(self, which: int):
        """Which kernel serves a one-token GEMV without LoRA: 0 = by shape, 1 = each lane loads its own
        blocks, 2 = weights streamed into a per-wave ring of LDS slots wherever the shape fits."""
        _check(self.lib.lq4_set_gemv_kernel(self.ctx, int(which)))

    def set_gemm_kernel(self, which: int):
        """0 = pick the prefill kernel by shape, 1 = LDS-staged tile, 2 = weights in registers,
        3 = few-token kernel, 4 = weights in registers at two workgroups per CU."""
        _check(self.lib.lq4_set_gemm_kernel(self.ctx, int(which)))

    def probe_copy(self, src, dst):
        """One plain copy launch src -> dst (equal-sized tensors): traffic-counter calibration."""
        nbytes = src.numel() * src.element_size()
        if dst.numel() * dst.element_size() != nbytes:
            raise Q4Error(-1, "probe_copy needs equal-sized buffers")
        _check(self.lib.lq4_probe_copy(self.ctx, src.data_ptr(), dst.data_ptr(), nbytes, self._stream()))

    # ------------------------------------------------------- weights / residency
    def upload_q4_blocks(self, blocks, payload_offset: int = 0, validate: bool = True) -> Q4WeightBuf:
        """Uploads host bytes verbatim (``make_buffer_q4_0``, metal_qwen35.rs:2362-2378, for raw
        blocks; the whole-file no-copy buffer of ``mmap_q4_weight`` when ``payload_offset`` > 0)."""
        buf = np.ascontiguousarray(np.frombuffer(blocks, dtype=np.uint8) if isinstance(
            blocks, (bytes, bytearray, memoryview)) else blocks, dtype=np.uint8)
        h = C.c_void_p()
        _check(self.lib.lq4_weight_upload(self.ctx, buf.ctypes.data, buf.size, payload_offset,
                                          int(validate), C.byref(h)))
        return Q4WeightBuf(h.value, buf.size, payload_offset, self)

    def wrap_device_blocks(self, t, payload_offset: int = 0) -> Q4WeightBuf:
        """Adopts a uint8 CUDA tensor that already holds native blocks (kept alive by the
        returned buffer); e.g. a fused gate||up buffer (metal_qwen35.rs:12137-12152)."""
        import torch
        assert t.is_cuda and t.dtype == torch.uint8 and t.is_contiguous()
        h = C.c_void_p()
        _check(self.lib.lq4_weight_wrap(self.ctx, t.data_ptr(), t.numel(), payload_offset, C.byref(h)))
        return Q4WeightBuf(h.value, t.numel(), payload_offset, self, _keepalive=t)

    def mmap_q4_weight(self, path: str, label: str, expected_shape: Sequence[int]) -> Q4WeightBuf:
        """``mmap_q4_weight(device, path, label, expected_shape)`` (metal_qwen35.rs:660-702):
        header + exact-extent + shape preflight, per-block scale/bias scan, then the whole
        file becomes one resident buffer with ``payload_offset`` past the header."""
        data = np.memmap(path, dtype=np.uint8, mode="r")
        try:
            header = q4_file.validate_q4_file(data, path, expected_shape)
        except q4_file.Q4FileError as e:
            raise Q4Error(-1, f"failed to validate Q4 payload {path}: {e}") from None
        try:
            return self.upload_q4_blocks(data, payload_offset=header.payload_offset, validate=True)
        except Q4Error as e:
            raise Q4Error(e.code, f"{path}: tensor {label} (Q4): {e.message}") from None

    # ---------------------------------------------------------------- dispatch
    @staticmethod
    def _assert_k(k: int, who: str):
        # the reference panics here (dispatch.rs:185-188)
        assert k > 0 and k % BLOCK_WEIGHTS == 0, \
            f"{who} requires K to be non-zero and divisible by 32, got {k}"

    def _lora_for(self, layer_idx, module, n, k):
        if layer_idx is None or module is None:
            return None
        proj = self._lora.get((layer_idx, module))
        if proj is None:
            return None
        assert (proj.d_in, proj.d_out) == (k, n), "LoRA projection shape does not match the GEMV"
        return proj.handle

    def dispatch_matmul(self, x, qw: Q4WeightBuf, y, m: int, n: int, k: int, *, layer_idx=None,
                        module=None):
        """``dispatch_matmul(enc, x, qw, y, m, n, k)`` (dispatch.rs:231-245): decode GEMV
        ``y[0..n) = W . x[0..k)``; ``m`` is ignored as in the reference.  Passing
        ``layer_idx``/``module`` fuses that projection's LoRA delta into the same pass."""
        if n == 0:
            return
        self._assert_k(k, "dispatch_matmul_q4")
        lora = self._lora_for(layer_idx, module, n, k)
        _check(self.lib.lq4_gemv(self.ctx, qw.handle, 0, n, k, x.data_ptr(), 1, y.data_ptr(), lora,
                                 self._lora_scale, self._stream()))

    # ---- Q8_0 sibling format ------------------------------------------------------------------
    def upload_q8_blocks(self, blocks) -> Q4WeightBuf:
        """Uploads Q8_0 blocks (34 bytes per 32 weights, metal_qwen35.rs:2310-2346); the handle is
        the same byte-buffer type as for Q4 (the reference also keeps Q8_0 in a ``Q4WeightBuf``)."""
        return self.upload_q4_blocks(blocks, validate=False)

    def dispatch_matmul_q8(self, x, qw: Q4WeightBuf, y, m: int, n: int, k: int):
        """``dispatch_matmul_q8`` (dispatch.rs:61-84): decode GEMV over Q8_0 blocks, ``m`` ignored."""
        if n == 0:
            return
        self._assert_k(k, "dispatch_matmul_q8")
        _check(self.lib.lq4_gemv_q8(self.ctx, qw.handle, 0, n, k, x.data_ptr(), 1, y.data_ptr(), self._stream()))

    def dispatch_gemm_q8(self, x, x_offset: int, qw: Q4WeightBuf, y, y_offset: int, m: int, n: int, k: int):
        """``dispatch_gemm_q8`` (dispatch.rs:86-146): byte offsets into x and y; ``m == 0 or n == 0``
        is a no-op; ``m <= 1`` takes the GEMV."""
        if m == 0 or n == 0:
            return
        self._assert_k(k, "dispatch_gemm_q8")
        dt = _dtype_code(x)
        _check(self.lib.lq4_gemm_q8(self.ctx, qw.handle, 0, n, k, x.data_ptr() + x_offset, dt, m,
                                    y.data_ptr() + y_offset, self._stream()))

    # ---- Q3 sibling format --------------------------------------------------------------------
    def upload_q3_blocks(self, blocks, payload_offset: int = 0) -> Q4WeightBuf:
        """Uploads Q3 blocks (16 bytes per 32 weights, weights/q3_weights.rs:13-52)."""
        return self.upload_q4_blocks(blocks, payload_offset=payload_offset, validate=False)

    def dispatch_matmul_q3(self, x, qw: Q4WeightBuf, y, m: int, n: int, k: int):
        """Decode GEMV over Q3 blocks (the ``m <= 1`` arm of ``dispatch_gemm_q3``, dispatch.rs:269-325)."""
        if n == 0:
            return
        self._assert_k(k, "dispatch_gemm_q3")
        _check(self.lib.lq4_gemv_q3(self.ctx, qw.handle, 0, n, k, x.data_ptr(), 1, y.data_ptr(), self._stream()))

    def dispatch_gemm_q3(self, x, x_offset: int, qw: Q4WeightBuf, y, y_offset: int, m: int, n: int, k: int):
        """``dispatch_gemm_q3`` (dispatch.rs:269-325): byte offsets into x and y; ``m == 0 or n == 0``
        is a no-op; ``m <= 1`` takes the GEMV."""
        if m == 0 or n == 0:
            return
        self._assert_k(k, "dispatch_gemm_q3")
        _check(self.lib.lq4_gemm_q3(self.ctx, qw.handle, 0, n, k, x.data_ptr() + x_offset, _dtype_code(x), m,
                                    y.data_ptr() + y_offset, self._stream()))

    # ---- elementwise steps either side of the decode GEMVs -----------------------------------
    @staticmethod
    def _ptr(t):
        return None if t is None else t.data_ptr()

    def dispatch_fused_residual_add_norm(self, base, delta, residual_out, normed_out, gamma, row_len: int,
                                         eps: float, num_rows: int = 1):
        """``dispatch_fused_residual_add_norm`` / ``_batch`` (dispatch.rs:1171-1266):
        ``residual_out = base + delta``, ``normed_out`` = shifted RMSNorm of it.  ``delta=None`` is
        the plain ``dispatch_rms_norm`` (dispatch.rs:525); ``residual_out=None`` skips that store."""
        _check(self.lib.lq4_residual_add_rmsnorm(self.ctx, base.data_ptr(), self._ptr(delta), gamma.data_ptr(),
                                                 row_len, num_rows, eps, self._ptr(residual_out),
                                                 normed_out.data_ptr(), self._stream()))

    def dispatch_silu_mul_fused(self, data, count: int, rows: int = 1, out=None, out_stride=None):
        """``dispatch_silu_mul_fused`` (dispatch.rs:916-930): ``data[i] = silu(data[i]) *
        data[i + count]`` in place, or into ``out`` (rows ``out_stride`` floats apart)."""
        dst = data if out is None else out
        stride = (2 * count if out is None else count) if out_stride is None else out_stride
        _check(self.lib.lq4_silu_mul(self.ctx, data.data_ptr(), count, rows, dst.data_ptr(), stride, self._stream()))

    def dispatch_add_and_copy(self, src, residual, dst, count: int):
        """``dispatch_add_and_copy`` (dispatch.rs:1268-1290): ``residual += src; dst = residual``."""
        _check(self.lib.lq4_add_and_copy(self.ctx, src.data_ptr(), residual.data_ptr(), self._ptr(dst), count,
                                         self._stream()))

    def dispatch_matmul_fused(self, x, qw: Q4WeightBuf, y, n: int, k: int, *, norm=None, silu_mul=False,
                              add_residual=None, silu_mul_pairs=False, qw_extra_offset: int = 0, layer_idx=None,
                              module=None, batch: int = 1):
        """``dispatch_matmul`` for 1..16 activation rows with the neighbouring elementwise dispatches
        folded in.  ``norm=(base, delta, gamma, eps, residual_out)`` replaces a preceding
        ``dispatch_fused_residual_add_norm`` / ``_batch`` (``x`` is then unused); ``silu_mul=True``
        replaces a preceding ``dispatch_silu_mul_fused`` (``x`` holds gate | up, 2k floats per row);
        ``add_residual=(residual, dst)`` replaces a following ``dispatch_add_and_copy``;
        ``silu_mul_pairs=True`` (one row): the weight is gate rows then up rows and ``y`` receives the
        ``n / 2`` values ``silu(gate) * up``, i.e. the following ``dispatch_silu_mul_fused`` as well.  With
        ``batch`` rows every per-row tensor is ``[batch, ...]`` and dense."""
        if n == 0:
            return
        self._assert_k(k, "dispatch_matmul_q4")
        assert not (norm is not None and silu_mul), "one prologue at a time"
        f = GemvFusion()
        f.prologue = LQ4_PRO_ADD_RMSNORM if norm is not None else LQ4_PRO_SILU_MUL if silu_mul else LQ4_PRO_NONE
        keep = []
        if norm is not None:
            base, delta, gamma, eps, residual_out = norm
            f.base, f.delta, f.gamma = base.data_ptr(), self._ptr(delta), gamma.data_ptr()
            f.eps, f.residual_out = eps, self._ptr(residual_out)
            keep += [base, delta, gamma, residual_out]
        f.epilogue = LQ4_EPI_NONE
        if add_residual is not None:
            residual, dst = add_residual
            f.epilogue, f.residual, f.copy_dst = LQ4_EPI_ADD_RESIDUAL, residual.data_ptr(), self._ptr(dst)
        if silu_mul_pairs:
            assert add_residual is None, "one epilogue at a time"
            f.epilogue = LQ4_EPI_SILU_MUL_PAIRS
        lora = self._lora_for(layer_idx, module, n, k)
        _check(self.lib.lq4_gemv_fused_batch(self.ctx, qw.handle, qw_extra_offset, n, k, self._ptr(x), batch,
                                             self._ptr(y), C.byref(f), lora, self._lora_scale, self._stream()))

    def chain_step(self, qw: Q4WeightBuf, n: int, k: int, *, x=None, from_previous=False, norm=None, silu_mul=False,
                   add_residual=None, silu_mul_pairs=False, y=None, qw_extra_offset: int = 0) -> ChainStep:
        """One step of :meth:`dispatch_chain`.  ``from_previous=True`` feeds the step with the previous
        step's result (in the place of ``x``, or of ``delta`` under ``norm``).
        ``norm=(base, delta, gamma, eps, residual_out)`` as in :meth:`dispatch_matmul_fused`
        (``base`` / ``delta`` may be ``None``); ``silu_mul=True``: ``x`` holds gate | up;
        ``add_residual=residual``: the result is ``residual + W.x``, written back;
        ``silu_mul_pairs=True``: W is gate rows then up rows and the result is ``silu(gate) * up``
        (n/2 values); ``y`` receives the result."""
        self._assert_k(k, "dispatch_matmul_q4")
        assert not (norm is not None and silu_mul), "one prologue at a time"
        assert not (add_residual is not None and silu_mul_pairs), "one epilogue at a time"
        st = ChainStep()
        st.w, st.w_extra_offset, st.n, st.k = qw.handle, qw_extra_offset, n, k
        st.from_previous = int(bool(from_previous))
        st.x_dev = self._ptr(x)
        st.prologue = LQ4_PRO_ADD_RMSNORM if norm is not None else LQ4_PRO_SILU_MUL if silu_mul else LQ4_PRO_NONE
        keep = [qw, x, y, add_residual]
        if norm is not None:
            base, delta, gamma, eps, residual_out = norm
            st.base, st.delta, st.gamma = self._ptr(base), self._ptr(delta), gamma.data_ptr()
            st.eps, st.residual_out = eps, self._ptr(residual_out)
            keep += [base, delta, gamma, residual_out]
        st.epilogue = (LQ4_EPI_ADD_RESIDUAL if add_residual is not None else
                       LQ4_EPI_SILU_MUL_PAIRS if silu_mul_pairs else LQ4_EPI_NONE)
        st.residual = self._ptr(add_residual)
        st.y_dev = self._ptr(y)
        st._keep = keep
        return st

    def dispatch_chain(self, steps: Sequence[ChainStep]):
        """The dispatches of one token between two points where the host must look at the result
        (``forward_step`` encodes them into one command buffer, metal_qwen35.rs:6943), as one library call."""
        arr = (ChainStep * len(steps))(*steps)
        _check(self.lib.lq4_gemv_chain(self.ctx, arr, len(steps), self._stream()))

    def dispatch_gemm(self, x, x_offset: int, qw: Q4WeightBuf, y, y_offset: int, m: int, n: int,
                      k: int, *, layer_idx=None, module=None):
        """``dispatch_gemm`` (dispatch.rs:507-525 -> dispatch_gemm_q4 :170-229)."""
        self.dispatch_gemm_at(x, x_offset, qw, 0, y, y_offset, m, n, k, layer_idx=layer_idx,
                              module=module)

    def dispatch_gemm_at(self, x, x_offset: int, qw: Q4WeightBuf, qw_extra_offset: int, y,
                         y_offset: int, m: int, n: int, k: int, *, layer_idx=None, module=None):
        """``dispatch_gemm_at`` (dispatch.rs:935-1097): offsets are bytes into ``x``, the weight
        buffer (on top of ``payload_offset``) and ``y``; ``m == 0 or n == 0`` is a no-op;
        small ``m`` with f32 activations takes the GEMV kernel (m == 1 in the reference)."""
        if m == 0 or n == 0:
            return
        self._assert_k(k, "dispatch_gemm_q4")
        lora = self._lora_for(layer_idx, module, n, k)
        _check(self.lib.lq4_gemm(self.ctx, qw.handle, qw_extra_offset, n, k, x.data_ptr() + x_offset,
                                 _dtype_code(x), m, y.data_ptr() + y_offset, lora, self._lora_scale,
                                 self._stream()))

    def gemv_batch(self, x, qw: Q4WeightBuf, y, batch: int, n: int, k: int, qw_extra_offset: int = 0,
                   *, layer_idx=None, module=None):
        """Small-batch decode: ``y[b] = W . x[b]`` for ``b < batch <= 16`` in one pass over W."""
        if batch == 0 or n == 0:
            return
        self._assert_k(k, "dispatch_matmul_q4")
        lora = self._lora_for(layer_idx, module, n, k)
        _check(self.lib.lq4_gemv(self.ctx, qw.handle, qw_extra_offset, n, k, x.data_ptr(), batch,
                                 y.data_ptr(), lora, self._lora_scale, self._stream()))

    def gemv_multi(self, x, projections, batch: int, k: int, *, layer_idx=None):
        """Several projections of the same activations in one call (one launch at batch 1): ``projections`` is a
        list of ``(qw, n, y)`` or ``(qw, n, y, module)`` or ``(qw, n, y, module, qw_extra_offset)``; with
        ``layer_idx`` and a module name the loaded adapter's delta for that projection is fused in, as
        ``gemv_batch`` does.  The q/k/v run of dispatch_matmul calls on one input (inner/layers/gqa.rs:72-127)."""
        if batch == 0 or not projections:
            return
        self._assert_k(k, "dispatch_matmul_q4")
        if len(projections) > MAX_PROJECTIONS:
            raise ValueError(f"{len(projections)} projections, at most {MAX_PROJECTIONS} a call")
        arr = (Projection * len(projections))()
        for i, p in enumerate(projections):
            qw, n, y = p[0], p[1], p[2]
            module = p[3] if len(p) > 3 else None
            lora = self._lora_for(layer_idx, module, n, k) if module is not None else None
            arr[i].w = qw.handle
            arr[i].w_extra_offset = p[4] if len(p) > 4 else 0
            arr[i].n = n
            arr[i].y_dev = y.data_ptr()
            arr[i].lora = lora
            arr[i].lora_scale = self._lora_scale
        _check(self.lib.lq4_gemv_multi(self.ctx, arr, len(projections), k, x.data_ptr(), batch, self._stream()))

    def dequantize(self, qw: Q4WeightBuf, n: int, k: int, qw_extra_offset: int = 0):
        """f32 [n, k] tensor of ``f32(nibble)*scale + bias`` (bit-exactness probe)."""
        import torch
        self._assert_k(k, "dequantize")
        out = torch.empty((n, k), dtype=torch.float32, device=self.torch_device)
        _check(self.lib.lq4_dequant(self.ctx, qw.handle, qw_extra_offset, n, k, out.data_ptr(),
                                    self._stream()))
        return out

    # ------------------------------------------------------------ lm_head top-k
    def topk(self, logits, k: int):
        """Exact top-k of a device logits vector: ``(logits[k], token_ids[k])`` in the reference's
        rank order (dispatch_topk_enc, inner/dispatch.rs:1425-1500)."""
        import torch
        out_l = torch.empty(k, dtype=torch.float32, device=self.torch_device)
        out_i = torch.empty(k, dtype=torch.int32, device=self.torch_device)  # u32 bit patterns
        _check(self.lib.lq4_topk(self.ctx, logits.data_ptr(), logits.numel(), k, out_l.data_ptr(),
                                 out_i.data_ptr(), self._stream()))
        return out_l, out_i

    def lm_head_topk(self, x, qw: Q4WeightBuf, vocab: int, k: int, top_k: int, qw_extra_offset: int = 0,
                     out=None, static_scratch: bool = False):
        """lm_head projection fused with top-k selection (dispatch_lm_head_block_stage1_enc +
        dispatch_block_topk_merge_enc, inner/dispatch.rs:1317-1421): the full logits vector is
        never returned.  ``static_scratch=True`` takes the entry point that allocates nothing
        (pass ``out=(logits, ids)`` tensors as well and the call touches no allocator at all)."""
        import torch
        self._assert_k(k, "lm_head_topk")
        if out is None:
            out = (torch.empty(top_k, dtype=torch.float32, device=self.torch_device),
                   torch.empty(top_k, dtype=torch.int32, device=self.torch_device))
        out_l, out_i = out
        fn = self.lib.lq4_lm_head_topk_static if static_scratch else self.lib.lq4_lm_head_topk
        _check(fn(self.ctx, qw.handle, qw_extra_offset, vocab, k, x.data_ptr(), top_k,
                  out_l.data_ptr(), out_i.data_ptr(), self._stream()))
        return out_l, out_i

    # -------------------------------------------------------------------- LoRA
    def load_lora_adapter(self, layers: List[LoraLayerData], scale: float,
                          quarot_seed: Optional[int] = None):
        """``load_lora_adapter(layers, scale, quarot_seed)`` (metal_qwen35.rs:3806-3986): the reference's
        checks in the reference's order with its messages, then every projection's A/B to the device;
        ``scale`` (= alpha/rank, crates/fann/src/lora.rs:110-117) is applied verbatim.  With
        ``quarot_seed`` the factors are first rotated on the host by the model's ``quarot_rotate`` (the
        reference calls ``rotate_adapter_for_quarot`` at the same point, :3834-3849)."""
        if self._lora:
            raise Q4Error(-1, "LoRA adapter already loaded; call unload_lora_adapter first")
        if not layers:
            raise Q4Error(-1, "load_lora_adapter: layers must not be empty")
        if not np.isfinite(scale):
            raise Q4Error(-1, f"load_lora_adapter: scale must be finite, got {scale}")
        if quarot_seed is not None:
            if self.model is None or self.model.quarot_rotate is None:
                raise Q4Error(-5, "load_lora_adapter: quarot_seed needs the host crate's rotate_adapter_for_quarot "
                                  "(ModelShapes.quarot_rotate) and the model's hidden size")
            self.model.quarot_rotate(layers, int(quarot_seed), self.model.hidden_size)
        staged: Dict[Tuple[int, str], _LoraProjection] = {}
        try:
            for layer in layers:
                for module, (a, b) in layer.modules.items():
                    a = np.ascontiguousarray(a)
                    b = np.ascontiguousarray(b)
                    if a.ndim != 2 or b.ndim != 2:
                        raise Q4Error(-1, f"load_lora_adapter: layer {layer.layer_idx} module '{module}': A {a.shape} / "
                                          f"B {b.shape} are not [rank, d_in] / [d_out, rank]")
                    rank, d_in = a.shape
                    d_out = b.shape[0]
                    if rank == 0:
                        raise Q4Error(-1, f"load_lora_adapter: layer {layer.layer_idx} module '{module}' has rank=0")
                    if d_in == 0 or d_out == 0:
                        raise Q4Error(-1, f"load_lora_adapter: layer {layer.layer_idx} module '{module}' has zero "
                                          f"dimension (d_in={d_in}, d_out={d_out})")
                    if self.model is not None:
                        if not 0 <= layer.layer_idx < self.model.num_hidden_layers:
                            raise Q4Error(-1, f"load_lora_adapter: layer_idx {layer.layer_idx} >= num_hidden_layers "
                                              f"{self.model.num_hidden_layers}")
                        try:
                            exp_in, exp_out = self.model.projection_shape(layer.layer_idx, module)
                        except ValueError as e:
                            raise Q4Error(-1, str(e)) from None
                        if (d_in, d_out) != (exp_in, exp_out):
                            raise Q4Error(-1, f"load_lora_adapter: layer {layer.layer_idx} module '{module}' has "
                                              f"(d_in={d_in}, d_out={d_out}) but model expects "
                                              f"(d_in={exp_in}, d_out={exp_out})")
                    if b.shape[1] != rank:
                        raise Q4Error(-1, f"load_lora_adapter: layer {layer.layer_idx} module '{module}' B length "
                                          f"{b.size} != d_out*rank {d_out * rank}")
                    if a.dtype != b.dtype or a.dtype not in (np.float32, np.float16):
                        raise Q4Error(-1, f"load_lora_adapter: layer {layer.layer_idx} module '{module}': A and B "
                                          "must both be float32 or float16")
                    if (layer.layer_idx, module) in staged:
                        raise Q4Error(-1, f"load_lora_adapter: duplicate projection for layer {layer.layer_idx} "
                                          f"module '{module}'")
                    h = C.c_void_p()
                    _check(self.lib.lq4_lora_upload(self.ctx, a.ctypes.data, b.ctypes.data,
                                                    LQ4_F16 if a.dtype == np.float16 else LQ4_F32,
                                                    rank, d_in, d_out, C.byref(h)))
                    staged[(layer.layer_idx, module)] = _LoraProjection(h.value, rank, d_in, d_out)
        except Exception:
            for p in staged.values():
                self.lib.lq4_lora_free(p.handle)
            raise
        self._lora, self._lora_scale = staged, float(scale)

    def unload_lora_adapter(self):
        for p in self._lora.values():
            self.lib.lq4_lora_free(p.handle)
        self._lora, self._lora_scale = {}, 0.0

    def dispatch_lora_if_active(self, x, x_byte_offset: int, y, y_byte_offset: int, layer_idx: int,
                                module: str, rows: int = 1):
        """``dispatch_lora_if_active`` (layers/mod.rs:15-51): ``y += scale * B.(A.x)``; a no-op
        when no adapter is loaded or it has no projection for ``(layer_idx, module)``."""
        proj = self._lora.get((layer_idx, module))
        if proj is None:
            return
        _check(self.lib.lq4_lora_apply(self.ctx, proj.handle, self._lora_scale,
                                       x.data_ptr() + x_byte_offset, _dtype_code(x), rows,
                                       y.data_ptr() + y_byte_offset, self._stream()))

    # --------------------------------------------------------------------- MoE
    def moe_route(self, logits, top_k: int):
        """Router softmax + top-k + renormalise on the device (moe.rs:39-125); returns
        ``(ids int32 [T, top_k], weights f32 [T, top_k])``."""
        import torch
        t, e = logits.shape
        ids = torch.empty((t, top_k), dtype=torch.int32, device=self.torch_device)
        wts = torch.empty((t, top_k), dtype=torch.float32, device=self.torch_device)
        _check(self.lib.lq4_moe_route(self.ctx, logits.data_ptr(), t, e, top_k, ids.data_ptr(),
                                      wts.data_ptr(), self._stream()))
        return ids, wts

    def moe_shared_expert(self, gate_up: Q4WeightBuf, down: Q4WeightBuf, shared_gate, shared_inter: int,
                          hidden: int, x, y):
        """``apply_shared_expert`` (moe.rs:194-250): ``y += sigmoid(x . shared_gate) * FFN_shared(x)``
        per token; ``y`` normally holds the routed experts' sum already."""
        tokens = x.shape[0] if x.dim() > 1 else 1
        _check(self.lib.lq4_moe_shared_expert(self.ctx, gate_up.handle, down.handle, shared_gate.data_ptr(),
                                              shared_inter, hidden, x.data_ptr(), tokens, y.data_ptr(),
                                              self._stream()))

    def moe_ffn(self, router_logits, gate_up: Q4WeightBuf, down: Q4WeightBuf, num_experts: int, top_k: int,
                inter: int, shared_gate_up: Q4WeightBuf, shared_down: Q4WeightBuf, shared_gate, shared_inter: int,
                hidden: int, x, y):
        """``moe_ffn_step`` (moe.rs:8-36) from the router logits on: route, routed experts, shared expert;
        ``y`` is overwritten."""
        tokens = x.shape[0] if x.dim() > 1 else 1
        _check(self.lib.lq4_moe_ffn(self.ctx, router_logits.data_ptr(), gate_up.handle, down.handle, num_experts,
                                    top_k, inter, shared_gate_up.handle, shared_down.handle, shared_gate.data_ptr(),
                                    shared_inter, hidden, x.data_ptr(), tokens, y.data_ptr(), self._stream()))

    def moe_experts(self, gate_up: Q4WeightBuf, down: Q4WeightBuf, num_experts: int, inter: int,
                    hidden: int, x, ids, weights, y):
        """Routed-expert FFN over Q4 expert tensors (moe.rs:127-190); ``y`` is overwritten."""
        tokens, top_k = ids.shape
        _check(self.lib.lq4_moe_grouped_gemv(self.ctx, gate_up.handle, down.handle, num_experts, inter,
                                             hidden, x.data_ptr(), tokens, ids.data_ptr(),
                                             weights.data_ptr(), top_k, y.data_ptr(), self._stream()))
