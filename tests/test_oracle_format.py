"""Pins the oracle's scalar conversions, block quantizer, dequantizer and `.q4`
header parser against vectors the reference's own tests hold and against
independent implementations (numpy float16, the CPU's F16C instruction).

Reference sources of each vector are cited per test (paths relative to the
lattice repository root)."""
import os

import numpy as np
import pytest

import oracle
from lattice_amd import q4_layout


# --------------------------------------------------------------------------- f16
def test_f16_widen_all_patterns_vs_numpy():
    # weights/half_bits.rs:230-255 checks every non-signalling pattern against an
    # independent library; numpy.float16 plays that part here.
    bits = np.arange(65536, dtype=np.uint16)
    exp, frac = (bits >> 10) & 0x1F, bits & 0x3FF
    snan = (exp == 0x1F) & (frac != 0) & ((frac & 0x200) == 0)
    got = oracle.f16_bits_to_f32_bits(bits)
    want = bits.view(np.float16).astype(np.float32).view(np.uint32)
    assert np.array_equal(got[~snan], want[~snan])
    # weights/half_bits.rs:267-302: signalling NaNs keep their payload un-quieted.
    s = bits[snan].astype(np.uint32)
    closed = ((s >> 15) << 31) | 0x7F800000 | ((s & 0x3FF) << 13)
    assert np.array_equal(got[snan], closed)


def test_f16_special_values():
    # weights/q4_weights.rs:1862-1887
    assert oracle.f32_to_f16(0.0) == 0x0000
    assert oracle.f32_to_f16(-0.0) == 0x8000
    assert oracle.f16_to_f32(0x0000) == 0.0
    assert oracle.f32_to_f16(float("inf")) == 0x7C00
    assert oracle.f32_to_f16(float("-inf")) == 0xFC00
    assert np.isnan(oracle.f16_to_f32(oracle.f32_to_f16(float("nan"))))
    assert oracle.f32_to_f16(1.0e10) == 0x7C00
    assert oracle.f16_to_f32(0x7C00) == float("inf")
    assert oracle.f16_to_f32(0x0001) == 2.0 ** -24
    assert oracle.f16_to_f32(0x03FF) == 1023 * 2.0 ** -24
    assert oracle.f16_to_f32(0x7BFF) == 65504.0


def test_f32_narrow_vs_hardware_f16c_sweep():
    # Every 257th f32 pattern over the whole space (16.7M cases) plus dense windows
    # around every binade edge f16 cares about, against vcvtps2ph.
    assert oracle.sweep_f32_to_f16_vs_f16c(0, 0xFFFFFFFF, 257) == (0, 0)
    for sign in (0, 0x80000000):
        for exp in (0, 1, 101, 102, 103, 112, 113, 114, 126, 127, 141, 142, 143, 144, 254):
            lo = sign | (exp << 23)
            assert oracle.sweep_f32_to_f16_vs_f16c(lo, lo + 0x1FFFF, 1)[0] == 0
            assert oracle.sweep_f32_to_f16_vs_f16c(lo + 0x7E0000, lo + 0x7FFFFF, 1)[0] == 0


def test_f32_narrow_ties_and_nan_payload():
    # Round-half-to-even at the f16 ulp: 1 + 2^-11 ties down to 1.0, 1 + 3*2^-11 ties up.
    assert oracle.f32_to_f16(1.0 + 2.0 ** -11) == 0x3C00
    assert oracle.f32_to_f16(1.0 + 3 * 2.0 ** -11) == 0x3C02
    assert oracle.f32_to_f16(65520.0) == 0x7C00  # ties to even -> overflow
    assert oracle.f32_to_f16(65519.0) == 0x7BFF
    assert oracle.f32_to_f16(2.0 ** -25) == 0x0000  # tie to even (zero)
    assert oracle.f32_to_f16(2.0 ** -25 * 1.0001) == 0x0001
    # weights/f16_encode.rs:35-44: payload = frac >> 13, forced non-zero, quiet bit set.
    got = oracle.f32_bits_to_f16(np.array([0x7F800001, 0xFFC12000, 0x7FA00000], dtype=np.uint32))
    assert list(got) == [0x7E01, 0xFE09, 0x7F00]
    # f32 subnormals flush to a signed zero (f16_encode.rs:47-49)
    assert list(oracle.f32_bits_to_f16(np.array([0x00000001, 0x807FFFFF], dtype=np.uint32))) == [0, 0x8000]


# ------------------------------------------------------------------ golden bytes
def gen_values(n, seed):
    # crates/inference/tests/quantize_q4_reader_refactor.rs:35-39, then truncated to bf16
    # (:27-29) which is what the converter quantizes.
    i = np.arange(n, dtype=np.int64)
    v = (((i * 37 + seed * 13) % 200) - 100).astype(np.float32) / np.float32(4.0)
    return ((v.view(np.uint32) >> 16) << 16).astype(np.uint32).view(np.float32)


@pytest.mark.parametrize("name,shape,seed", [("k_proj_golden.q4", (1, 32), 2),
                                             ("gate_proj_golden.q4", (2, 33), 1)])
def test_quantizer_reproduces_reference_golden_files(golden_dir, name, shape, seed):
    # Byte goldens written by the reference's own converter
    # (crates/inference/tests/fixtures/quantize_q4_reader_refactor/*.q4; fixture_tensors
    # in quantize_q4_reader_refactor.rs:117-136).  gate_proj [2,33] pins flat (not per-row)
    # blocking and the partial-tail statistics; both pin layout, nibble order and rounding.
    raw = open(os.path.join(golden_dir, name), "rb").read()
    got_shape, olen, off = oracle.parse_q4_file(raw)
    n = shape[0] * shape[1]
    assert got_shape == shape and olen == n and off == 36
    blocks = oracle.quantize_flat(gen_values(n, seed), symmetric=False)
    assert blocks.tobytes() == raw[off:]
    assert q4_layout.q4_file_bytes(shape, blocks) == raw


def test_golden_k_proj_hand_checked_bytes(golden_dir):
    raw = open(os.path.join(golden_dir, "k_proj_golden.q4"), "rb").read()
    blk = np.frombuffer(raw[36:], dtype=np.uint8)
    sb, bb, nib = q4_layout.unpack_blocks(blk)
    assert (sb[0], bb[0]) == (0x426F, 0xCE10)  # scale 3.2168, bias -24.25
    assert (nib[0, 0], nib[0, 1]) == (2, 5)  # v0=-18.5 -> round(5.75/3.21667)=2 ; v1=-9.25 -> 5
    w = oracle.dequantize(blk, 32)
    assert w[0] == np.float32(2) * np.float32(3.216796875) + np.float32(-24.25)


# ------------------------------------------------------- quantizer known answers
def _u16(buf, off):
    return int(buf[off]) | (int(buf[off + 1]) << 8)


def _row(**kv):
    v = np.zeros(32, dtype=np.float32)
    for i, x in kv.items():
        v[int(i[1:])] = x
    return v


def test_nibble_packing_order():
    # weights/q4_weights.rs:1893-1924
    data = oracle.quantize_flat(_row(_0=0.0, _1=7.0))
    assert data[4] == 0xF0
    out = oracle.dequantize(data, 32)
    assert abs(out[0]) < 1e-3 and abs(out[1] - 7.0) < 0.05


def test_quantize_max_range():
    # weights/q4_weights.rs:1755-1777
    data = oracle.quantize_flat(_row(_0=7.0, _1=-7.0))
    assert data[4] & 0x0F == 15 and data[4] >> 4 == 0


def test_symmetric_max_value_clamps_to_15():
    # weights/q4_weights.rs:2025-2033 (100 -> scale 100/7 -> round(7)+8 = 15)
    blk = oracle.quantize_block(_row(_0=100.0), symmetric=True)
    assert blk[4] & 0x0F == 15
    assert blk[4] >> 4 == 8 and all(b == 0x88 for b in blk[5:])
    scale = oracle.f16_to_f32(_u16(blk, 0))
    bias = oracle.f16_to_f32(_u16(blk, 2))
    assert bias == -8.0 * scale


def test_partial_tail_uses_real_min_max():
    # weights/q4_weights.rs:2184-2208
    data = oracle.quantize_flat(np.array([5.0, 6.0, 7.0], dtype=np.float32))
    assert data.size == 20
    assert _u16(data, 0) == oracle.f32_to_f16(np.float32(2.0) / np.float32(15.0))
    assert _u16(data, 2) == oracle.f32_to_f16(5.0)
    assert _u16(data, 0) != oracle.f32_to_f16(np.float32(7.0) / np.float32(15.0))


def test_underflowing_scale_takes_degenerate_fallback():
    # weights/q4_weights.rs:2239-2280 (symmetric) and the asymmetric sibling above it.
    tiny = np.float32(1e-12)
    assert oracle.f16_to_f32(oracle.f32_to_f16(tiny / np.float32(7))) == 0.0
    blk = oracle.quantize_block(_row(_0=tiny, _7=-tiny / 3), symmetric=True)
    assert oracle.f16_to_f32(_u16(blk, 0)) == 1.0
    out = oracle.dequantize(blk, 32)
    assert np.all(np.abs(out) <= 2 * tiny)
    blk = oracle.quantize_block(_row(_0=tiny), symmetric=False)
    assert oracle.f16_to_f32(_u16(blk, 0)) == 1.0
    # exactly-zero block: same fallback
    blk = oracle.quantize_block(np.zeros(32, np.float32), symmetric=False)
    assert oracle.f16_to_f32(_u16(blk, 0)) == 1.0 and set(blk[4:]) == {0}


def test_unrepresentable_metadata_is_rejected():
    # weights/q4_weights.rs:2345-2371
    with pytest.raises(oracle.QuantizeError) as e:
        oracle.quantize_block(_row(_0=1.0e7), symmetric=True)
    assert "strictly positive f16" in str(e.value)
    v = np.full(32, 1.0e5, dtype=np.float32)
    v[0] += 1.0
    with pytest.raises(oracle.QuantizeError) as e:
        oracle.quantize_block(v, symmetric=False)
    assert "finite f16" in str(e.value)


@pytest.mark.parametrize("bad", [np.nan, np.inf, -np.inf])
def test_non_finite_source_is_rejected(bad):
    # weights/q4_weights.rs:250-258
    with pytest.raises(oracle.QuantizeError):
        oracle.quantize_block(_row(_5=bad))
    with pytest.raises(oracle.QuantizeError):
        oracle.quantize_block(np.zeros(32, np.float32), valid_len=0)
    with pytest.raises(oracle.QuantizeError):
        oracle.quantize_block(np.zeros(32, np.float32), valid_len=33)


def test_rows_are_blocked_independently():
    # quantize_tensor_q4_0 (weights/q4_weights.rs:364-388) vs flat blocking
    rng = np.random.default_rng(3)
    w = rng.normal(size=(3, 40)).astype(np.float32)
    rows = oracle.quantize_rows(w)
    assert rows.size == 3 * 2 * 20
    for r in range(3):
        assert np.array_equal(rows[r * 40:(r + 1) * 40], oracle.quantize_flat(w[r]))
    assert not np.array_equal(rows[:120], oracle.quantize_flat(w.ravel())[:120])


def test_symmetric_round_trip_error_bound():
    rng = np.random.default_rng(5)
    w = rng.normal(scale=0.05, size=(64, 32)).astype(np.float32)
    q = oracle.quantize_rows(w, symmetric=True)
    d = oracle.dequantize(q, w.size).reshape(w.shape)
    sb, _, _ = q4_layout.unpack_blocks(q)
    scale = sb.view(np.float16).astype(np.float32)[:, None]
    # half a step, plus the clamp of +7.x*scale to nibble 15 at the positive end, plus f16
    # rounding of the scale spread over up to 8 steps
    assert np.all(np.abs(d - w) <= 0.5 * scale * 1.01 + 8 * scale * 2.0 ** -11)


# -------------------------------------------------------------------- dequantize
def test_dequantize_matches_independent_numpy_restatement():
    # weights/q4_weights.rs:2543-2567 keeps an independent re-implementation for this check.
    rng = np.random.default_rng(11)
    nb = 4096
    sb = rng.integers(0, 0x7C00, size=nb, dtype=np.uint16)  # any finite positive f16 incl. subnormals
    bb = rng.integers(0, 0x7C00, size=nb, dtype=np.uint16) | (rng.integers(0, 2, size=nb, dtype=np.uint16) << 15)
    nib = rng.integers(0, 16, size=(nb, 32), dtype=np.uint8)
    data = q4_layout.pack_blocks(sb, bb, nib)
    got = oracle.dequantize(data, nb * 32)
    want = q4_layout.dequantize_numpy(data)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequantize_all_nibbles_closed_form():
    # n*scale is exact in f32 (4 bits x 11 bits), so w is one rounding of the real
    # number n*scale + bias; f64 evaluates that number exactly before rounding.
    rng = np.random.default_rng(12)
    sb = rng.integers(1, 0x7C00, size=512, dtype=np.uint16)
    bb = rng.integers(0, 0x7C00, size=512, dtype=np.uint16) | 0x8000
    nib = np.tile(np.arange(16, dtype=np.uint8), 2)[None, :].repeat(512, 0)
    data = q4_layout.pack_blocks(sb, bb, nib)
    got = oracle.dequantize(data, 512 * 32).reshape(512, 32)
    s64 = sb.view(np.float16).astype(np.float64)[:, None]
    b64 = bb.view(np.float16).astype(np.float64)[:, None]
    want = (nib.astype(np.float64) * s64 + b64).astype(np.float32)
    assert np.array_equal(got, want)


def test_symmetric_dequant_is_exactly_n_minus_8_times_scale():
    from lattice_amd import synth
    data = synth.q4_weight(64, 256, seed=0)
    sb, bb, nib = q4_layout.unpack_blocks(data)
    scale = sb.view(np.float16).astype(np.float32)[:, None]
    bias = bb.view(np.float16).astype(np.float32)[:, None]
    got = oracle.dequantize(data, 64 * 256).reshape(-1, 32)
    # bias = f16(-8*s) equals -8*f16(s) whenever f16(s) is a normal number (power-of-two
    # scaling commutes with rounding); the few blocks whose scale is an f16 subnormal differ.
    exact = (bias == -8 * scale)[:, 0]
    assert exact.mean() > 0.9
    assert np.array_equal(got[exact], ((nib.astype(np.float32) - 8) * scale)[exact])


def test_dequantize_truncation_and_short_input():
    # weights/q4_weights.rs:330-353: trailing partial block ignored, output truncated, never panics
    data = oracle.quantize_flat(np.arange(64, dtype=np.float32))
    assert oracle.dequantize(data[:39], 64).size == 32
    assert oracle.dequantize(data[:19], 64).size == 0
    assert oracle.dequantize(data, 40).size == 40


# ----------------------------------------------------------- block metadata rule
def test_block_metadata_rule():
    # weights/ingress.rs:542-559: scale finite and > 0, bias finite
    good = q4_layout.pack_blocks(np.array([0x3C00] * 3, np.uint16), np.array([0xC000] * 3, np.uint16),
                                 np.zeros((3, 32), np.uint8))
    assert oracle.validate_blocks(good) == (-1, 0)
    for bad_scale in (0x0000, 0x8000, 0xBC00, 0x7C00, 0x7E00, 0xFC00):
        d = good.copy()
        d[20:22] = np.array([bad_scale], dtype="<u2").view(np.uint8)
        assert oracle.validate_blocks(d) == (1, 1), hex(bad_scale)
    for bad_bias in (0x7C00, 0xFC00, 0x7E00):
        d = good.copy()
        d[42:44] = np.array([bad_bias], dtype="<u2").view(np.uint8)
        assert oracle.validate_blocks(d) == (2, 2), hex(bad_bias)
    d = good.copy()
    d[0:2] = np.array([0x0001], dtype="<u2").view(np.uint8)  # smallest subnormal is a legal scale
    assert oracle.validate_blocks(d) == (-1, 0)


# ------------------------------------------------------------------ .q4 header
def test_q4_file_header_errors():
    # weights/q4_weights.rs:709-812 and the header tests at :2810-3250
    blocks = oracle.quantize_flat(np.arange(64, dtype=np.float32))
    good = q4_layout.q4_file_bytes((2, 32), blocks)
    assert oracle.parse_q4_file(good) == ((2, 32), 64, 36)
    cases = {
        b"XXXX" + good[4:]: "invalid magic",
        good[:4] + b"\x01\x00\x00\x00" + good[8:]: "legacy",
        good[:4] + b"\x03\x00\x00\x00" + good[8:]: "unsupported",
        good[:-1]: "truncated",
        good + b"\x00": "trailing",
        q4_layout.q4_file_bytes((2, 31), blocks, original_len=64): "does not match shape",
        good[:8]: "invalid magic",
    }
    for data, msg in cases.items():
        with pytest.raises(ValueError, match=msg):
            oracle.parse_q4_file(data)
    # 1-D tensor: header is 28 bytes
    one_d = q4_layout.q4_file_bytes((40,), oracle.quantize_flat(np.arange(40, dtype=np.float32)))
    assert oracle.parse_q4_file(one_d) == ((40,), 40, 28)
