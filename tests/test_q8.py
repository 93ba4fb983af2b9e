"""Q8_0 sibling format: 34-byte blocks [f16 scale][32 x i8] (forward/metal_qwen35.rs:2310-2346),
decode GEMV (shaders/qwen35.metal:133-190) and tile GEMM (inner/dispatch.rs:61-146).

The reference holds no byte goldens for Q8_0, so the oracle is pinned by what fixes it: blocks
whose quantised values are known in closed form, the rounding rule at exact halves, the clamp,
the f16 scale word, rejection of non-finite input (metal_qwen35.rs:15906-15921, 32856-32870),
an independent numpy restatement, and the f64 twin of the matmul."""
import numpy as np
import pytest

import oracle
from lattice_amd import synth
from util import REL_TOL, rel_err


def _np_quantize(row):
    """Independent restatement with numpy only."""
    row = np.asarray(row, np.float32).reshape(-1, 32)
    out = bytearray()
    for blk in row:
        amax = np.float32(np.max(np.abs(blk)))
        d = np.float32(amax / np.float32(127.0))
        inv = np.float32(1.0) / d if d != 0 else np.float32(0.0)
        t = (blk * inv).astype(np.float32)
        q = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), -127, 127).astype(np.int8)  # half away from zero
        out += np.float16(d).tobytes() + q.tobytes()
    return np.frombuffer(bytes(out), np.uint8)


def test_oracle_closed_form_blocks():
    # values j * (amax / 127): every quotient is an exact integer
    blk = (np.arange(-16, 16, dtype=np.float32) * np.float32(254.0 / 127.0))
    blk[-1] = 254.0  # amax = 254 -> d = 2, q = v / 2
    q = oracle.q8_quantize_rows(blk[None])
    assert q.size == 34
    assert q[:2].view(np.float16)[0] == np.float16(2.0)
    assert np.array_equal(q[2:].view(np.int8)[:-1], np.arange(-16, 15, dtype=np.int8)) and q[2:].view(np.int8)[-1] == 127
    assert np.array_equal(oracle.q8_dequantize(q, 32)[:-1], blk[:-1])
    # all zeros: d = 0, every q = 0, dequantises to zeros
    z = oracle.q8_quantize_rows(np.zeros((1, 32), np.float32))
    assert not z.any() and not oracle.q8_dequantize(z, 32).any()
    # exact halves round away from zero; the most negative value maps to -127, never -128
    blk = np.zeros(32, np.float32)
    blk[0], blk[1], blk[2], blk[3], blk[4] = 127.0, 0.5, -0.5, 2.5, -127.0
    q = oracle.q8_quantize_rows(blk[None])[2:].view(np.int8)
    assert q[:5].tolist() == [127, 1, -1, 3, -127]
    # the stored scale is f16(d) although the quotient used the f32 d
    blk = np.zeros(32, np.float32)
    blk[0] = 0.1
    qb = oracle.q8_quantize_rows(blk[None])
    assert qb[:2].view(np.float16)[0] == np.float16(np.float32(0.1) / np.float32(127.0)) and qb[2:].view(np.int8)[0] == 127


def test_oracle_rejects_non_finite_and_matches_numpy():
    for bad in (np.nan, np.inf, -np.inf):
        row = np.ones(64, np.float32)
        row[40] = bad
        with pytest.raises(ValueError, match="block 1"):
            oracle.q8_quantize_rows(row[None])
    g = np.random.default_rng(3)
    w = (g.normal(size=(7, 96)) * g.uniform(0.01, 3.0, size=(7, 1))).astype(np.float32)
    got = oracle.q8_quantize_rows(w).reshape(7, -1)
    for r in range(7):
        assert np.array_equal(got[r], _np_quantize(w[r]))
    deq = oracle.q8_dequantize(got.reshape(-1), 7 * 96).reshape(7, 96)
    step = np.abs(w).reshape(7, 3, 32).max(axis=2, keepdims=True) / 127.0
    # half a quantisation step, plus the f16 rounding of the stored scale (2^-11 relative)
    w3 = w.reshape(7, 3, 32)
    assert np.all(np.abs(deq.reshape(7, 3, 32) - w3) <= 0.5 * step + np.abs(w3) * 2.0 ** -10 + 1e-9)


def test_oracle_gemm_properties():
    g = np.random.default_rng(4)
    n, k, m = 9, 128, 3
    w = g.normal(size=(n, k)).astype(np.float32)
    wq = oracle.q8_quantize_rows(w)
    deq = oracle.q8_dequantize(wq, n * k).reshape(n, k)
    x = g.normal(size=(m, k)).astype(np.float32)
    y32, y64 = oracle.q8_gemm_f32(x, wq, n, k), oracle.q8_gemm_f64(x, wq, n, k)
    assert rel_err(y64, x.astype(np.float64) @ deq.astype(np.float64).T) < 1e-12
    assert rel_err(y32, y64) < 1e-5
    eye = np.eye(k, dtype=np.float32)[:5]
    assert np.array_equal(oracle.q8_gemm_f32(eye, wq, n, k), deq[:, :5].T)  # one-hot picks a column exactly


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


def _q8_weight(n, k, seed):
    g = np.random.default_rng(seed)
    w = (g.normal(size=(n, k)) * 0.02).astype(np.float32)
    return oracle.q8_quantize_rows(w)


GEMV_CASES = [(4096, 1024), (2048, 2048), (12288, 2048), (2048, 6144), (37, 96), (5, 32), (1000, 4160), (20000, 256),
              (30011, 2080)]  # many units per wave: steady-state loop and peeled tail


@pytest.mark.gpu
@pytest.mark.parametrize("n,k", GEMV_CASES)
def test_q8_gemv_matches_oracle(be, n, k):
    import torch
    print(f"q8 gemv n={n} k={k}", flush=True)
    wq = _q8_weight(n, k, seed=n + k)
    x = synth.activations(1, k, seed=1)
    qw = be.upload_q8_blocks(wq)
    y = torch.full((n + 1,), float("nan"), device="cuda")
    be.dispatch_matmul_q8(dev(x), qw, y, 1, n, k)
    got = host(y)
    assert np.isnan(got[n])
    e = rel_err(got[:n], oracle.q8_gemm_f64(x, wq, n, k)[0])
    print(f"  rel err vs f64 {e:.2e}", flush=True)
    assert e <= 1e-5          # f32 activations, exact integer weights: f32-faithful
    assert rel_err(got[:n], oracle.q8_gemm_f32(x, wq, n, k)[0]) <= REL_TOL
    # one-hot activations reproduce a dequantised column
    e5 = np.zeros((1, k), np.float32)
    e5[0, k - 5] = 1.0
    be.dispatch_matmul_q8(dev(e5), qw, y, 1, n, k)
    col = oracle.q8_dequantize(wq, n * k).reshape(n, k)[:, k - 5]
    assert np.allclose(host(y)[:n], col, rtol=0, atol=1e-9 + 1e-6 * np.abs(col).max())


GEMM_CASES = [(2, 64, 64, "f32"), (8, 2048, 2048, "f32"), (16, 37, 96, "f32"), (130, 300, 256, "f16"),
              (512, 256, 1024, "f16"), (33, 129, 4160, "f32"),
              (200, 300, 2080, "f32"), (96, 130, 1056, "f16"), (257, 128, 4096, "f16")]


@pytest.mark.gpu
@pytest.mark.parametrize("kernel", [0, 1, 2])  # by shape / tile kernel / weights-in-registers kernel
@pytest.mark.parametrize("m,n,k,xdt", GEMM_CASES)
def test_q8_gemm_matches_oracle(be, m, n, k, xdt, kernel):
    import torch
    print(f"q8 gemm m={m} n={n} k={k} x={xdt} kernel={kernel}", flush=True)
    wq = _q8_weight(n, k, seed=m + n + k)
    x = synth.activations(m, k, seed=2, dtype=np.float16 if xdt == "f16" else np.float32)
    qw = be.upload_q8_blocks(wq)
    y = torch.full((m + 1, n), float("nan"), device="cuda")
    be.set_gemm_kernel(kernel)  # few rows take the few-token kernel whatever is chosen
    try:
        be.dispatch_gemm_q8(dev(x), 0, qw, y, 0, m, n, k)
    finally:
        be.set_gemm_kernel(0)
    got = host(y)
    assert np.all(np.isnan(got[m])) and np.all(np.isfinite(got[:m]))
    e = rel_err(got[:m], oracle.q8_gemm_f32(x.astype(np.float32), wq, n, k))
    print(f"  rel err {e:.2e}", flush=True)
    assert e <= REL_TOL


@pytest.mark.gpu
def test_q8_argument_checks(be):
    import torch
    from lattice_amd import backend
    wq = _q8_weight(8, 64, seed=0)
    qw = be.upload_q8_blocks(wq)
    x, y = torch.zeros(64, device="cuda"), torch.zeros(9, device="cuda")
    with pytest.raises(AssertionError):
        be.dispatch_matmul_q8(x, qw, y, 1, 8, 48)
    with pytest.raises(backend.Q4Error):
        be.dispatch_matmul_q8(x, qw, y, 1, 9, 64)   # one row more than the buffer holds
    be.dispatch_gemm_q8(x, 0, qw, y, 0, 0, 8, 64)    # m == 0: silent no-op
