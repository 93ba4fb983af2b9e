"""CPU-only checks of the shipped host logic: the C-ABI library loads and exports every
symbol the header declares, the host-side block rule agrees with the oracle, and the
`.q4` ingest helpers reproduce the reference's behaviour on its golden files."""
import ctypes
import os
import re

import numpy as np
import pytest

import oracle
from lattice_amd import backend, q4_file, q4_layout, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "lattice_hip_q4.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lq4_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(backend.LIB_PATH)
    names = _declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    assert sorted(backend.EXPORTS) == names


def test_version_and_error_string():
    lib = backend.load_library()
    assert b"gfx950" in lib.lq4_version()
    with pytest.raises(backend.Q4Error) as e:
        backend.validate_blocks(q4_layout.pack_blocks(np.array([0x7C00], np.uint16),
                                                      np.array([0], np.uint16),
                                                      np.zeros((1, 32), np.uint8)))
    assert e.value.code == -3 and "scale" in e.value.message


def test_host_block_rule_matches_oracle():
    # weights/ingress.rs:542-559 through the C ABI's host-side scan (no GPU involved)
    lib = backend.load_library()
    rng = np.random.default_rng(0)
    for trial in range(200):
        nb = 8
        sb = rng.integers(1, 0x7C00, size=nb, dtype=np.uint16)
        bb = rng.integers(0, 0x7C00, size=nb, dtype=np.uint16)
        which = rng.integers(0, nb)
        kind = trial % 4
        if kind == 1:
            sb[which] = rng.choice([0x0000, 0x8000, 0x7C00, 0xFC00, 0x7E01, 0xB800])
        elif kind == 2:
            bb[which] = rng.choice([0x7C00, 0xFC00, 0x7FFF, 0xFE00])
        data = q4_layout.pack_blocks(sb, bb, np.zeros((nb, 32), np.uint8))
        bad, why = ctypes.c_int64(0), ctypes.c_int(0)
        rc = lib.lq4_validate_blocks(data.ctypes.data, data.size, ctypes.byref(bad), ctypes.byref(why))
        o_idx, o_why = oracle.validate_blocks(data)
        assert (bad.value, why.value) == (o_idx, o_why)
        assert (rc == 0) == (o_idx == -1)


def test_validate_q4_file_on_reference_goldens(golden_dir):
    for name, shape in (("k_proj_golden.q4", (1, 32)), ("gate_proj_golden.q4", (2, 33))):
        raw = np.fromfile(os.path.join(golden_dir, name), dtype=np.uint8)
        h = q4_file.validate_q4_file(raw, name, shape)
        assert (h.shape, h.original_len, h.payload_offset) == (shape, shape[0] * shape[1], 36)
        assert oracle.parse_q4_file(raw) == (h.shape, h.original_len, h.payload_offset)
        with pytest.raises(q4_file.Q4FileError, match="does not match expected"):
            q4_file.validate_q4_file(raw, name, (shape[1], shape[0]))
        backend.validate_blocks(raw[36:])


def test_validate_q4_file_errors_agree_with_oracle():
    blocks = oracle.quantize_flat(np.arange(64, dtype=np.float32))
    good = q4_layout.q4_file_bytes((2, 32), blocks)
    bad_files = [b"XXXX" + good[4:], good[:4] + b"\x01\x00\x00\x00" + good[8:],
                 good[:4] + b"\x07\x00\x00\x00" + good[8:], good[:-3], good + b"\x00\x00",
                 q4_layout.q4_file_bytes((2, 31), blocks, original_len=64)]
    for data in bad_files:
        with pytest.raises(ValueError):
            oracle.parse_q4_file(data)
        with pytest.raises(q4_file.Q4FileError):
            q4_file.validate_q4_file(np.frombuffer(data, dtype=np.uint8))
    assert q4_file.validate_q4_file(np.frombuffer(good, dtype=np.uint8)).payload_offset == 36


def test_tensor_path_sanitiser_and_fused_gate_up():
    # forward/metal_qwen35.rs:11428-11444
    p = q4_file.q4_tensor_path("/m", "model.layers.0.mlp.gate_proj.weight")
    assert p == "/m/model_layers_0_mlp_gate_proj_weight.q4"
    assert q4_file.q4_tensor_path("/m", "a-b/c d", "f16") == "/m/a-b_c_d.f16"
    gate = synth.q4_weight(4, 64, tag="g")
    up = synth.q4_weight(4, 64, tag="u")
    fused = q4_file.fuse_gate_up(gate, up)
    gate_bytes = 4 * (64 // 32) * 20  # metal_qwen35.rs:7403-7406
    assert np.array_equal(fused[:gate_bytes], gate) and np.array_equal(fused[gate_bytes:], up)


def test_synth_weights_are_deterministic_and_valid():
    a = synth.q4_weight(64, 256, seed=0)
    b = synth.q4_weight(64, 256, seed=0)
    assert np.array_equal(a, b) and a.size == q4_layout.weight_nbytes(64, 256)
    assert not np.array_equal(a, synth.q4_weight(64, 256, seed=1))
    backend.validate_blocks(a)
    sb, bb, nib = q4_layout.unpack_blocks(a)
    assert nib.min() == 0 and nib.max() == 15
    s = sb.view(np.float16).astype(np.float32)
    assert 0.5 * 0.02 / 7 < s.mean() / np.sqrt(2 / np.pi) < 2 * 0.02 / 7  # E|N(0,s)| = s*sqrt(2/pi)


def test_backend_refuses_to_run_without_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        backend.HipQ4Backend(0)
