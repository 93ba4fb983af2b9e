"""Q3 sibling format: 16-byte plane-split blocks (weights/q3_weights.rs:13-52), decode GEMV and
tile GEMM (inner/dispatch.rs:269-325).

Oracle pins follow the reference's own unit tests (weights/q3_weights.rs:852-975, 1199-1250):
pack/unpack of every 3-bit level in every slot, the bytes and bits the high plane must set, the
round-trip bounds of both encode modes, the partial tail block that must ignore its padding, the
exact constant block, rejection of non-finite input, 4.0 bits per weight, and the GEMV reference
being the dequantise-then-dot product, sensitive to one flipped high-plane bit."""
import numpy as np
import pytest

import oracle
from lattice_amd import synth
from util import REL_TOL, rel_err


def _unpack(packed12, i):
    low2 = (packed12[i // 4] >> ((i % 4) * 2)) & 3
    hi = (packed12[8 + i // 8] >> (i % 8)) & 1
    return low2 | (hi << 2)


def _block_of_levels(q):
    """A block whose asymmetric quantisation yields exactly the levels q (scale 1, bias 0)."""
    q = np.asarray(q, np.float32)
    assert q.min() == 0 and q.max() == 7
    return np.frombuffer(oracle.q3_quantize_block(q), np.uint8)


def test_plane_split_layout():
    for base in range(8):
        q = np.array([(base + i) % 8 for i in range(32)], np.uint8)
        blk = _block_of_levels(q)
        assert blk[:2].view(np.float16)[0] == 1.0 and blk[2:4].view(np.float16)[0] == 0.0
        assert [_unpack(blk[4:], i) for i in range(32)] == q.tolist()
        assert np.array_equal(oracle.q3_dequantize(blk, 32), q.astype(np.float32))
    q = np.zeros(32, np.uint8)
    q[0], q[5], q[17] = 7, 6, 7            # 7 so that the range is 0..7; value 5 = 0b110, value 17 = 0b111
    blk = _block_of_levels(q)
    packed = blk[4:]
    assert packed[8] & (1 << 5) and packed[10] & (1 << 1)          # q3_weights.rs:888-894
    assert (packed[1] >> 2) & 3 == 2 and (packed[4] >> 2) & 3 == 3  # low planes of values 5 and 17
    assert len(blk) == 16 and 16 * 8 / 32 == 4.0                    # four bits per weight


def test_round_trip_bounds_and_special_blocks():
    src = ((np.arange(32) - 12.0) * 0.37).astype(np.float32)       # q3_weights.rs:898-913
    back = oracle.q3_dequantize(oracle.q3_quantize_rows(src[None]), 32)
    scale = (src.max() - src.min()) / 7.0
    assert np.all(np.abs(back - src) <= scale / 2 + abs(scale) * 1e-3 + 1e-6)
    sym = ((np.arange(32) - 15.5) * 0.1).astype(np.float32)         # :916-931
    back = oracle.q3_dequantize(oracle.q3_quantize_rows(sym[None], symmetric=True), 32)
    amax = np.abs(sym).max()
    assert np.all(np.abs(back - sym) <= (amax / 3.5) / 2 + amax * 1e-3 + 1e-6)
    tail = np.array([10.0, 10.5, 11.0], np.float32)                  # :934-951: padding must not widen the range
    blk = oracle.q3_quantize_rows(tail[None])
    assert blk.size == 16
    back = oracle.q3_dequantize(blk, 3)
    assert back.size == 3 and np.all(np.abs(back - tail) <= (1.0 / 7.0) / 2 + (1.0 / 7.0) * 1e-3 + 1e-6)
    const = oracle.q3_dequantize(oracle.q3_quantize_rows(np.full((1, 32), 3.5, np.float32)), 32)
    assert np.all(const == 3.5)                                      # :954-963
    bad = np.full(32, 0.1, np.float32)
    for v in (np.nan, np.inf):                                       # :966-973
        bad[7] = v
        with pytest.raises(ValueError):
            oracle.q3_quantize_rows(bad[None])
    # symmetric mode: dequant reduces to (q - 4) * scale
    blk = np.frombuffer(oracle.q3_quantize_block(sym, symmetric=True), np.uint8)
    s, b = blk[:2].view(np.float16)[0].astype(np.float32), blk[2:4].view(np.float16)[0].astype(np.float32)
    assert abs(b + 4 * s) <= 4 * abs(s) * 2.0 ** -10


def test_gemm_reference_properties():
    g = np.random.default_rng(0x1234)
    n, k, m = 6, 128, 3
    w = (g.normal(size=(n, k))).astype(np.float32)
    wq = oracle.q3_quantize_rows(w)
    deq = oracle.q3_dequantize(wq, n * k).reshape(n, k)
    x = g.normal(size=(m, k)).astype(np.float32)
    y32, y64 = oracle.q3_gemm_f32(x, wq, n, k), oracle.q3_gemm_f64(x, wq, n, k)
    assert rel_err(y64, x.astype(np.float64) @ deq.astype(np.float64).T) < 1e-12    # dequantise then dot
    assert rel_err(y32, y64) < 1e-5
    assert np.array_equal(oracle.q3_gemm_f32(x[1:2], wq, n, k)[0], y32[1])           # GEMM row == GEMV
    flipped = wq.copy()
    flipped[12] ^= 0x01                                                              # :1227-1250: weight 0 of row 0 gains or loses 4
    d = oracle.q3_gemm_f64(x, flipped, n, k) - y64
    s0 = flipped[:2].view(np.float16)[0].astype(np.float64)
    assert np.allclose(np.abs(d[:, 0]), 4.0 * s0 * np.abs(x[:, 0].astype(np.float64)), rtol=1e-6) and not d[:, 1:].any()


# ---- GPU ------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def be():
    from lattice_amd import backend
    b = backend.HipQ4Backend(0)
    yield b
    b.close()


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def _q3_weight(n, k, seed, symmetric=False):
    g = np.random.default_rng(seed)
    w = (g.normal(size=(n, k)) * 0.02).astype(np.float32)
    return oracle.q3_quantize_rows(w, symmetric=symmetric)


GEMV_CASES = [(4096, 1024, False), (2048, 2048, True), (12288, 2048, False), (2048, 6144, False), (37, 96, False),
              (5, 32, True), (1000, 4160, False), (20000, 256, False),
              (30011, 2080, True)]  # many units per wave: steady-state loop and peeled tail


@pytest.mark.gpu
@pytest.mark.parametrize("n,k,sym", GEMV_CASES)
def test_q3_gemv_matches_oracle(be, n, k, sym):
    import torch
    print(f"q3 gemv n={n} k={k} sym={sym}", flush=True)
    wq = _q3_weight(n, k, seed=n + k, symmetric=sym)
    x = synth.activations(1, k, seed=1)
    qw = be.upload_q3_blocks(wq)
    y = torch.full((n + 1,), float("nan"), device="cuda")
    be.dispatch_matmul_q3(dev(x), qw, y, 1, n, k)
    got = host(y)
    assert np.isnan(got[n])
    e = rel_err(got[:n], oracle.q3_gemm_f32(x, wq, n, k)[0])
    print(f"  rel err {e:.2e}", flush=True)
    assert e <= REL_TOL
    # plane indexing is exact: a one-hot activation (exact in f16 at every field scale) returns
    # one dequantised column bit for bit up to the f32 scale-and-bias arithmetic
    for col in (0, 5, 13, 17, k - 1, k - 22):
        e1 = np.zeros((1, k), np.float32)
        e1[0, col] = 1.0
        be.dispatch_matmul_q3(dev(e1), qw, y, 1, n, k)
        want = oracle.q3_dequantize(wq, n * k).reshape(n, k)[:, col]
        assert np.allclose(host(y)[:n], want, rtol=0, atol=1e-9 + 2e-7 * np.abs(want).max()), col


GEMM_CASES = [(2, 64, 64, "f32"), (8, 2048, 2048, "f32"), (16, 37, 96, "f32"), (130, 300, 256, "f16"),
              (512, 256, 1024, "f16"), (33, 129, 4160, "f32"),
              (200, 300, 2080, "f32"), (96, 130, 1056, "f16"), (257, 128, 4096, "f16")]


@pytest.mark.gpu
@pytest.mark.parametrize("kernel", [0, 1, 2])  # by shape / tile kernel / weights-in-registers kernel
@pytest.mark.parametrize("m,n,k,xdt", GEMM_CASES)
def test_q3_gemm_matches_oracle(be, m, n, k, xdt, kernel):
    import torch
    print(f"q3 gemm m={m} n={n} k={k} x={xdt} kernel={kernel}", flush=True)
    wq = _q3_weight(n, k, seed=m + n + k, symmetric=(m % 2 == 0))
    x = synth.activations(m, k, seed=2, dtype=np.float16 if xdt == "f16" else np.float32)
    qw = be.upload_q3_blocks(wq)
    y = torch.full((m + 1, n), float("nan"), device="cuda")
    be.set_gemm_kernel(kernel)  # few rows take the few-token kernel whatever is chosen
    try:
        be.dispatch_gemm_q3(dev(x), 0, qw, y, 0, m, n, k)
    finally:
        be.set_gemm_kernel(0)
    got = host(y)
    assert np.all(np.isnan(got[m])) and np.all(np.isfinite(got[:m]))
    e = rel_err(got[:m], oracle.q3_gemm_f32(x.astype(np.float32), wq, n, k))
    print(f"  rel err {e:.2e}", flush=True)
    assert e <= REL_TOL


@pytest.mark.gpu
def test_q3_payload_offset_and_argument_checks(be):
    import torch
    from lattice_amd import backend
    n, k = 8, 64
    wq = _q3_weight(n, k, seed=0)
    header = np.zeros(36, np.uint8)  # a 2-D .q3 file header is 36 bytes: blocks end up 4-byte aligned only
    qw = be.upload_q3_blocks(np.concatenate([header, wq]), payload_offset=36)
    x = synth.activations(1, k, seed=3)
    y = torch.zeros(n + 1, device="cuda")
    be.dispatch_matmul_q3(dev(x), qw, y, 1, n, k)
    assert rel_err(host(y)[:n], oracle.q3_gemm_f32(x, wq, n, k)[0]) <= REL_TOL
    with pytest.raises(AssertionError):
        be.dispatch_matmul_q3(dev(x), qw, y, 1, n, 48)
    with pytest.raises(backend.Q4Error):
        be.dispatch_matmul_q3(dev(x), qw, y, 1, n + 1, k)
    be.dispatch_gemm_q3(dev(x), 0, qw, y, 0, 0, n, k)
