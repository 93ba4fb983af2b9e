"""GPU parity of the integer matrix-core small-batch GEMV (lq4_gemv at 2..8 rows), through the C ABI, against the CPU
oracle.

By default the kernel serves 3..8 rows of matrices up to 4096 x 2048; a context created with LQ4_GEMV_I8=2 sends
every shape it can hold to it, which is how the shapes below reach it: rows of one to 24 chunks of eight blocks, a
short last chunk, fewer rows than one tile, rows that end inside a tile, many tiles a workgroup, every batch size.

Bars: max|delta| / max|y_ref| against the f32-accumulated oracle <= 5e-6 up to four rows (activations kept to 24 bits
below their block's maximum: an f32 GEMV, as the reference's gemm_q4 is) and <= 1e-4 for five to eight (16 bits); the
contract's bar is 1e-3 (tests/util.py).  Achieved errors are printed.
"""
import os

import numpy as np
import pytest

import oracle
from lattice_amd import backend, synth
from util import REL_TOL, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def i8():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    old = os.environ.get("LQ4_GEMV_I8")
    os.environ["LQ4_GEMV_I8"] = "2"
    try:
        b = backend.HipQ4Backend(0)
    finally:
        if old is None:
            del os.environ["LQ4_GEMV_I8"]
        else:
            os.environ["LQ4_GEMV_I8"] = old
    yield b
    b.close()


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def run(be, w, x, n, k, batch, **kw):
    import torch
    q = be.upload_q4_blocks(w)
    y = torch.full((batch, n), float("nan"), dtype=torch.float32, device="cuda")
    be.gemv_batch(dev(x), q, y, batch, n, k, **kw)
    be.synchronize()
    return host(y)


I8_SHAPES = [(16, 32, 2), (16, 512, 8), (64, 2048, 8), (5, 96, 3), (33, 32, 7), (300, 2048, 4), (2048, 2048, 8),
             (1000, 1024, 5), (12288, 2048, 8), (2048, 6144, 8), (2048, 6144, 3), (700, 4160, 6), (4099, 5120, 2),
             (70000, 256, 8), (1, 64, 1 + 1), (17, 2080, 4), (8200, 2048, 6)]


@pytest.mark.parametrize("n,k,batch", I8_SHAPES)
def test_i8_gemv_against_the_oracle(i8, n, k, batch):
    print(f"i8 gemv n={n} k={k} batch={batch}", flush=True)
    w = synth.q4_weight(n, k, seed=n + k, symmetric_bias=(n % 2 == 0))
    x = synth.activations(batch, k, seed=n)
    got = run(i8, w, x, n, k, batch)
    want = oracle.gemm_f32(x, w, n, k)
    e = rel_err(got, want)
    print(f"  rel err {e:.2e}", flush=True)
    assert e <= (5e-6 if batch <= 4 else 1e-4)


@pytest.mark.parametrize("batch", [3, 8])
def test_i8_gemv_one_hot_rows_return_dequantised_columns(i8, batch):
    # activation row b = 0.5 e_j(b): the products are single weights (any mistake in nibble order, operand byte order
    # or digit weight shows); the block scale 0.5 / 32639 is not a power of two, hence a few ulps instead of none
    n, k = 48, 320
    w = synth.q4_weight(n, k, seed=5, symmetric_bias=False)
    deq = oracle.dequantize(w, n * k).reshape(n, k)
    cols = [0, 1, 7, 8, 31, 32, 255, 319][:batch]
    x = np.zeros((batch, k), np.float32)
    for b, j in enumerate(cols):
        x[b, j] = 0.5
    got = run(i8, w, x, n, k, batch)
    for b, j in enumerate(cols):
        want = 0.5 * deq[:, j]
        assert np.max(np.abs(got[b] - want)) <= 2e-6 * np.max(np.abs(want)), (b, j)


def test_i8_gemv_activation_range_and_non_finite_rows(i8):
    # any finite f32 is in range (the scale is per block); a row with an infinity or a NaN comes back NaN and
    # leaves the other rows alone
    n, k, batch = 64, 256, 6
    w = synth.q4_weight(n, k, seed=9)
    x = synth.activations(batch, k, seed=10)
    x[1] *= 1e30
    x[2] *= 1e-30
    x[3, 17] = np.inf
    x[4, 200] = np.nan
    got = run(i8, w, x, n, k, batch)
    want = oracle.gemm_f64(x[[0, 1, 2, 5]], w, n, k)
    for i, b in enumerate((0, 1, 2, 5)):
        assert np.all(np.isfinite(got[b]))
        assert rel_err(got[b], want[i].astype(np.float32)) <= 1e-4, b
    assert np.all(np.isnan(got[3])) and np.all(np.isnan(got[4]))


@pytest.mark.parametrize("batch", [3, 8])
def test_i8_gemv_with_lora(i8, batch):
    n, k = 512, 2048
    w = synth.q4_weight(n, k, seed=2)
    a, b = synth.lora_pair(16, k, n, seed=3)
    x = synth.activations(batch, k, seed=4)
    i8.load_lora_adapter([backend.LoraLayerData(0, {"v_proj": (a, b)})], scale=2.0)
    try:
        got = run(i8, w, x, n, k, batch, layer_idx=0, module="v_proj")
        plain = run(i8, w, x, n, k, batch)
    finally:
        i8.unload_lora_adapter()
    base = oracle.gemm_f32(x, w, n, k)
    want = oracle.lora_apply(a.astype(np.float32), b.astype(np.float32), 2.0, x, base)
    assert rel_err(got, want) <= (5e-6 if batch <= 4 else 1e-4)
    assert rel_err(got - plain, want - base) <= 2e-3


def test_default_routing_serves_small_matrices_within_the_contract():
    # a context with the default setting: 512 x 2048 at four rows goes to the integer kernel (f32-grade result),
    # 2048 x 6144 stays with the 4x4x4 kernel (activations rounded to f16); the contract's bar holds for both
    import torch
    be = backend.HipQ4Backend(0)
    try:
        for (n, k, tol) in ((512, 2048, 5e-6), (2048, 6144, REL_TOL)):
            w = synth.q4_weight(n, k, seed=n)
            x = synth.activations(4, k, seed=k)
            e = rel_err(run(be, w, x, n, k, 4), oracle.gemm_f32(x, w, n, k))
            print(f"  default routing {n} x {k}: rel err {e:.2e}", flush=True)
            assert e <= tol
    finally:
        be.close()
