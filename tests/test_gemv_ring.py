"""GPU parity of the LDS-ring one-token GEMV (lq4_set_gemv_kernel(LDS_RING)), through the C ABI, against the CPU
oracle and against the lane-owns-block kernel.

Bars: one-hot activations return dequantised columns bit-exactly; max|delta| / max|y_ref| <= 1e-3 against the
f32-accumulated oracle (tests/util.py; achieved ~2e-6, printed); rows of at most one slab (K <= 2048) are
bit-identical to the lane-owns-block kernel, which adds a row's blocks in the same order.

Shapes cover what the kernels branch on: rows shorter than a slab, a short last slab, two and three slabs with the
activations in registers, more slabs with the activations read from LDS, K above 8192 (three activation pieces a
wave) up to the kernel's limit 24576, fewer rows than CUs, rows that straddle waves and workgroups, a vocabulary-
sized matrix, and rows of one, two and three slabs with more rows a workgroup than the waves' first ring fillings
hold (96, 48, 32; full and short last slabs), where the waves take rows from the workgroup's counter.
"""
import numpy as np
import pytest

import oracle
from lattice_amd import backend, synth
from util import REL_TOL, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ring():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    b = backend.HipQ4Backend(0)
    b.set_gemv_kernel(backend.GEMV_KERNEL_LDS_RING)
    yield b
    b.close()


@pytest.fixture(scope="module")
def lanes():
    b = backend.HipQ4Backend(0)
    b.set_gemv_kernel(backend.GEMV_KERNEL_LANE_BLOCKS)
    yield b
    b.close()


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def run(be, w, x, n, k):
    import torch
    q = be.upload_q4_blocks(w)
    y = torch.full((1, n), float("nan"), dtype=torch.float32, device="cuda")
    be.gemv_batch(dev(x), q, y, 1, n, k)
    be.synchronize()
    return y.cpu().numpy()[0]


RING_SHAPES = [(1, 32), (64, 64), (5, 96), (33, 32), (300, 2048), (2048, 2048), (1000, 1024), (12288, 2048),
               (2048, 6144), (700, 8160), (300, 17408), (4099, 5120), (70000, 256), (9, 24576), (255, 4096),
               (257, 4128), (513, 10240), (30001, 2048), (25000, 1056), (13001, 4096), (9000, 5152)]


@pytest.mark.parametrize("n,k", RING_SHAPES)
def test_ring_gemv_against_the_oracle_and_the_other_kernel(ring, lanes, n, k):
    print(f"ring gemv n={n} k={k}", flush=True)
    w = synth.q4_weight(n, k, seed=n + k, symmetric_bias=(n % 2 == 0))
    x = synth.activations(1, k, seed=n)
    before = ring.path_counters()["gemv"]
    got = run(ring, w, x, n, k)
    assert ring.path_counters()["gemv"] == before + 1
    want = oracle.gemm_f32(x, w, n, k)[0]
    err = rel_err(got, want)
    other = run(lanes, w, x, n, k)
    same = np.array_equal(got.view(np.uint32), other.view(np.uint32))
    print(f"  rel err {err:.2e}, bit-equal to the lane-owns-block kernel: {same}", flush=True)
    assert err <= REL_TOL
    assert rel_err(got, other) <= 1e-5
    if k <= 2048:
        assert same


@pytest.fixture(scope="module")
def routed():
    b = backend.HipQ4Backend(0)  # the library's own choice between the two kernels
    yield b
    b.close()


@pytest.mark.parametrize("n,k", [(4100, 2560), (6200, 4096), (10300, 3072), (3072, 8192), (20500, 2048), (2048, 17408)])
def test_one_token_gemv_as_the_library_routes_it(routed, lanes, n, k):
    """Matrices on either side of the rule that sends a one-token GEMV to the ring kernel (size, rows that are not
    whole slabs, rows of two slabs): the call as routed agrees with the oracle and with the lane-owns-block kernel."""
    print(f"routed one-token gemv n={n} k={k}", flush=True)
    w = synth.q4_weight(n, k, seed=n ^ k)
    x = synth.activations(1, k, seed=k)
    got = run(routed, w, x, n, k)
    assert rel_err(got, oracle.gemm_f32(x, w, n, k)[0]) <= REL_TOL
    assert rel_err(got, run(lanes, w, x, n, k)) <= 1e-5


def test_ring_gemv_one_hot_columns_are_bit_exact(ring):
    # 65 blocks a row: one full slab and a last slab of a single block; 257 rows straddle waves and workgroups
    import torch
    n, k = 257, 2080
    w = synth.q4_weight(n, k, seed=3, symmetric_bias=False)
    q = ring.upload_q4_blocks(w)
    deq = oracle.dequantize(w, n * k).reshape(n, k)
    for j in (0, 1, 7, 8, 31, 32, 2047, 2048, 2079):
        x = np.zeros((1, k), np.float32)
        x[0, j] = 1.0
        y = torch.empty((1, n), dtype=torch.float32, device="cuda")
        ring.gemv_batch(dev(x), q, y, 1, n, k)
        ring.synchronize()
        assert np.array_equal(y.cpu().numpy()[0].view(np.uint32), deq[:, j].view(np.uint32)), j


def test_ring_gemv_writes_only_its_rows(ring):
    # the output sits inside a larger buffer of sentinels: nothing before or behind it may change
    import torch
    n, k = 777, 2048
    w = synth.q4_weight(n, k, seed=11)
    x = synth.activations(1, k, seed=12)
    q = ring.upload_q4_blocks(w)
    buf = torch.full((n + 512,), -7.0, dtype=torch.float32, device="cuda")
    y = buf[256:256 + n].view(1, n)
    ring.gemv_batch(dev(x), q, y, 1, n, k)
    ring.synchronize()
    h = buf.cpu().numpy()
    assert np.all(h[:256] == -7.0) and np.all(h[256 + n:] == -7.0)
    assert rel_err(h[256:256 + n], oracle.gemm_f32(x, w, n, k)[0]) <= REL_TOL


def test_default_choice_by_shape_keeps_results_within_the_contract(lanes):
    # a fresh context picks by shape: 4096 x 14336 (37 MB, long rows) takes the ring kernel, 2048 x 2048 does not;
    # the caller sees the same contract either way
    import torch
    auto = backend.HipQ4Backend(0)
    try:
        gen = np.random.default_rng(5)
        for (n, k) in ((4096, 14336), (2048, 2048)):
            w = synth.q4_weight(n, k, seed=n)
            x = synth.activations(1, k, seed=k)
            got = run(auto, w, x, n, k)
            other = run(lanes, w, x, n, k)
            rows = gen.choice(n, size=64, replace=False)
            want = oracle.gemm_f32(x, w.reshape(n, -1)[rows].reshape(-1), 64, k)[0]
            assert rel_err(got[rows], want) <= REL_TOL
            assert rel_err(got, other) <= 1e-5
    finally:
        auto.close()


def test_ring_choice_leaves_lora_and_batches_to_the_other_kernels(ring):
    # forcing the ring kernel changes nothing for calls it does not serve: K beyond its limit, several rows, LoRA
    import torch
    n, k = 64, 24608
    w = synth.q4_weight(n, k, seed=1)
    x = synth.activations(1, k, seed=2)
    assert rel_err(run(ring, w, x, n, k), oracle.gemm_f32(x, w, n, k)[0]) <= REL_TOL
    n, k, b = 96, 256, 3
    w = synth.q4_weight(n, k, seed=3)
    x = synth.activations(b, k, seed=4)
    q = ring.upload_q4_blocks(w)
    y = torch.empty((b, n), dtype=torch.float32, device="cuda")
    ring.gemv_batch(dev(x), q, y, b, n, k)
    ring.synchronize()
    assert rel_err(y.cpu().numpy(), oracle.gemm_f32(x, w, n, k)) <= REL_TOL
    with pytest.raises(backend.Q4Error):
        ring.set_gemv_kernel(3)
