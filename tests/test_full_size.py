"""GPU parity at the benchmark configurations' full sizes, and on the kernels that only unusual
shapes reach.

Prefill GEMM (benchmark config 2) is too large for the CPU oracle in seconds: the check is torch f32
matmul over the dequantisation probe's output (tied bit for bit to the oracle by
test_dequant_probe_is_bit_exact) plus a strip of the result against the oracle proper.  Every
schedule of the tile scheduler occurs among the four shapes: whole rounds only, whole rounds plus
K-sliced tail tiles, and tail tiles only.
"""
import numpy as np
import pytest

import oracle
from lattice_amd import backend, synth
from util import REL_TOL, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    b = backend.HipQ4Backend(0)
    yield b
    b.close()


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def _gemm_full(be, m, n, k, seed, lora_rank=0):
    import torch
    torch.backends.cuda.matmul.allow_tf32 = False
    wq = synth.q4_weight(n, k, seed=seed)
    x = synth.activations(m, k, seed=seed, dtype=np.float16)
    qw = be.upload_q4_blocks(wq)
    xd = dev(x)
    y = torch.full((m + 1, n), float("nan"), dtype=torch.float32, device="cuda")
    wd = be.dequantize(qw, n, k)
    ref = xd.float() @ wd.t()
    del wd
    if lora_rank:
        a, b = synth.lora_pair(lora_rank, k, n, seed=seed)
        be.load_lora_adapter([backend.LoraLayerData(0, {"proj": (a, b)})], scale=2.0)
        try:
            be.dispatch_gemm(xd, 0, qw, y, 0, m, n, k, layer_idx=0, module="proj")
        finally:
            be.unload_lora_adapter()
        delta = 2.0 * ((xd.float() @ dev(a.astype(np.float32)).t()) @ dev(b.astype(np.float32)).t())
        plain = torch.empty((m, n), dtype=torch.float32, device="cuda")
        be.dispatch_gemm(xd, 0, qw, plain, 0, m, n, k)
        derr = ((y[:m] - plain) - delta).abs().max().item() / delta.abs().max().item()
        print(f"  delta rel err {derr:.2e}", flush=True)
        assert derr <= 5e-3  # y - plain cancels the base product: its f32 rounding is the floor here
        ref = ref + delta
    else:
        be.dispatch_gemm(xd, 0, qw, y, 0, m, n, k)
    assert bool(torch.isnan(y[m]).all()) and bool(torch.isfinite(y[:m]).all())
    err = (y[:m] - ref).abs().max().item() / ref.abs().max().item()
    print(f"  rel err vs torch f32 {err:.2e}", flush=True)
    assert err <= REL_TOL
    if not lora_rank:
        # a strip of rows, first and last weight rows, against the oracle
        rows = slice(m - 3, m)
        for n0 in (0, n - 256):
            strip = wq[n0 * (k // 32) * 20:(n0 + 256) * (k // 32) * 20]
            ref_o = oracle.gemm_f32(x[rows].astype(np.float32), strip, 256, k)
            assert rel_err(host(y[rows, n0:n0 + 256]), ref_o) <= REL_TOL


@pytest.mark.parametrize("m,n,k", [(2048, 17408, 5120), (2048, 5120, 17408), (512, 5120, 17408)])
def test_prefill_gemm_config2_full_size(be, m, n, k):
    print(f"gemm full m={m} n={n} k={k}", flush=True)
    _gemm_full(be, m, n, k, seed=3)


@pytest.mark.parametrize("kernel", [2, 4])
@pytest.mark.parametrize("m,n,k", [(2048, 17408, 5120), (2048, 5120, 17408)])
def test_prefill_gemm_config2_full_size_either_register_kernel(be, kernel, m, n, k):
    # whichever of the two weights-in-registers kernels the shape rule does not pick is checked too
    print(f"gemm full kernel={kernel} m={m} n={n} k={k}", flush=True)
    be.set_gemm_kernel(kernel)
    try:
        _gemm_full(be, m, n, k, seed=6)
    finally:
        be.set_gemm_kernel(0)


@pytest.mark.parametrize("m,n,k", [(512, 5120, 17408), (2048, 5120, 17408)])
def test_prefill_gemm_config2_full_size_with_lora(be, m, n, k):
    # the down projection: at M = 512 every tile of it is a K-sliced tail tile
    print(f"gemm full + lora m={m} n={n} k={k}", flush=True)
    _gemm_full(be, m, n, k, seed=4, lora_rank=16)


@pytest.mark.parametrize("batch", [2, 8, 16])
def test_decode_gate_up_small_batch_full_size(be, batch):
    # benchmark config 1 at batch 8: the fused gate||up matrix
    import torch
    n, k = 12288, 2048
    print(f"gemv gate||up batch={batch}", flush=True)
    wq = synth.q4_weight(n, k, seed=5, symmetric_bias=False)
    x = synth.activations(batch, k, seed=5)
    qw = be.upload_q4_blocks(wq)
    y = torch.full((batch, n), float("nan"), dtype=torch.float32, device="cuda")
    be.gemv_batch(dev(x), qw, y, batch, n, k)
    e32 = rel_err(host(y), oracle.gemm_f32(x, wq, n, k))
    e64 = rel_err(host(y), oracle.gemm_f64(x, wq, n, k))
    print(f"  rel err vs f32 {e32:.2e}, vs f64 {e64:.2e}", flush=True)
    assert e32 <= REL_TOL and e64 <= REL_TOL


def test_lm_head_topk_at_the_reference_vocabulary(be):
    # vocabulary 248 320 x hidden 2048: the persistent-grid form of the batch-1 GEMV, then the
    # selection over its logits in library scratch
    import torch
    vocab, k = 248320, 2048
    print("lm_head top-k at vocab 248320", flush=True)
    wq = synth.q4_weight(vocab, k, seed=7)
    x = synth.activations(1, k, seed=7)
    qw = be.upload_q4_blocks(wq)
    xd = dev(x)
    # the logits themselves, through the same GEMV: close to the oracle's
    y = torch.empty((1, vocab), dtype=torch.float32, device="cuda")
    be.gemv_batch(xd, qw, y, 1, vocab, k)
    logits = host(y)[0]
    assert rel_err(logits, oracle.gemm_f32(x, wq, vocab, k)[0]) <= REL_TOL
    for top_k in (1, 50, 64, 65, 256):
        got_l, got_i = be.lm_head_topk(xd, qw, vocab, k, top_k)
        got_l, got_i = host(got_l), host(got_i).view(np.uint32)
        # the selection is the oracle's exact top-k of those logits
        want_l, want_i = oracle.topk(logits, top_k)
        assert np.array_equal(got_i, want_i), top_k
        assert np.array_equal(got_l.view(np.uint32), want_l.view(np.uint32)), top_k


@pytest.mark.parametrize("batch", [1, 2, 3, 4, 7, 8, 11])
def test_gemv_rows_kernel_for_activations_beyond_lds(be, batch):
    # K = 32 768: the staged activations of neither the batch-1 kernel nor the matrix-core kernel fit
    # in LDS, so the plain row kernel runs (1, 2, 4 or 8 activation rows per pass)
    import torch
    n, k = 72, 32768
    print(f"gemv rows kernel batch={batch}", flush=True)
    wq = synth.q4_weight(n, k, seed=8, symmetric_bias=False)
    x = synth.activations(batch, k, seed=8)
    qw = be.upload_q4_blocks(wq)
    y = torch.full((batch + 1, n), float("nan"), dtype=torch.float32, device="cuda")
    be.gemv_batch(dev(x), qw, y, batch, n, k)
    got = host(y)
    assert np.all(np.isnan(got[batch]))
    e = rel_err(got[:batch], oracle.gemm_f32(x, wq, n, k))
    print(f"  rel err {e:.2e}", flush=True)
    assert e <= REL_TOL


@pytest.mark.parametrize("cfg", [dict(e=4, inter=64, hidden=9600, tokens=5, top_k=2),    # gate||up: scalar kernel
                                 dict(e=3, inter=9600, hidden=96, tokens=6, top_k=3),    # down: scalar kernel
                                 dict(e=2, inter=9632, hidden=9664, tokens=3, top_k=2)])  # both
def test_moe_scalar_kernels_for_reductions_beyond_lds(be, cfg):
    import torch
    e_, inter, hidden, tokens, top_k = cfg["e"], cfg["inter"], cfg["hidden"], cfg["tokens"], cfg["top_k"]
    print(f"moe scalar {cfg}", flush=True)
    gu = synth.q4_weight(e_ * 2 * inter, hidden, seed=9, tag="moe_gu")
    dn = synth.q4_weight(e_ * hidden, inter, seed=9, tag="moe_dn")
    x = synth.activations(tokens, hidden, seed=9, tag="moe_x")
    ids, wts, _ = oracle.moe_route(synth.router_logits(tokens, e_, seed=9), top_k)
    qgu, qdn = be.upload_q4_blocks(gu), be.upload_q4_blocks(dn)
    y = torch.full((tokens, hidden), float("nan"), dtype=torch.float32, device="cuda")
    be.moe_experts(qgu, qdn, e_, inter, hidden, dev(x), dev(ids), dev(wts), y)
    ref32 = oracle.moe_ffn(gu, dn, e_, inter, hidden, x, ids, wts)
    ref64 = oracle.moe_ffn(gu, dn, e_, inter, hidden, x, ids, wts, f64=True)
    e32, e64 = rel_err(host(y), ref32), rel_err(host(y), ref64)
    print(f"  rel err vs f32 {e32:.2e}, vs f64 {e64:.2e}", flush=True)
    assert e32 <= REL_TOL and e64 <= REL_TOL


@pytest.mark.parametrize("magnitude", [1e5, 3e38 / 2048, 1e-7, 1e-30])
def test_gemv_batch1_takes_any_finite_f32_activation(be, magnitude):
    # the reference's one-token kernel reads f32 activations (shaders/qwen35.metal:800-847); here they
    # are staged as fixed point scaled by a power of two per block, so their range is f32's
    import torch
    n, k = 96, 2048
    rng = np.random.default_rng(11)
    wq = synth.q4_weight(n, k, seed=11, symmetric_bias=False)
    x = (rng.normal(size=(1, k)) * magnitude).astype(np.float32)
    x[0, 5::64] *= 1e-3          # a wide range inside blocks
    x[0, 64:96] = 0.0            # an all-zero block
    x[0, 96:128] *= 1e-4 if magnitude > 1 else 1e4  # a block far from its neighbours
    qw = be.upload_q4_blocks(wq)
    y = torch.empty((1, n), dtype=torch.float32, device="cuda")
    be.gemv_batch(dev(x), qw, y, 1, n, k)
    got = host(y)
    assert np.all(np.isfinite(got))
    ref = oracle.gemm_f64(x, wq, n, k)
    e = rel_err(got, ref)
    print(f"  |x| ~ {magnitude:g}: rel err vs f64 {e:.2e}", flush=True)
    assert e <= 2e-5


@pytest.mark.parametrize("bad", [float("nan"), float("inf"), -float("inf")])
def test_gemv_batch1_non_finite_activation_reaches_every_row(be, bad):
    # every row has a weight against every activation, so in f32 arithmetic a NaN or infinite activation
    # leaves no finite output; the fixed-point staging must not turn it into a finite garbage value
    import torch
    n, k = 70, 2048
    wq = synth.q4_weight(n, k, seed=12, symmetric_bias=False)
    x = np.random.default_rng(12).normal(size=(1, k)).astype(np.float32)
    x[0, 777] = bad
    qw = be.upload_q4_blocks(wq)
    y = torch.zeros((1, n), dtype=torch.float32, device="cuda")
    be.gemv_batch(dev(x), qw, y, 1, n, k)
    assert not np.any(np.isfinite(host(y)))


@pytest.mark.parametrize("n,k", [(70001, 2048), (33333, 1024), (40000, 512), (25000, 6144)])
def test_gemv_batch1_tall_matrix_with_waves_over_several_chunks(be, n, k):
    # more rows than one chunk per resident wave covers: the grid is persistent, every wave walks several chunks
    # whose rows lie next to each other in memory, and the last chunk is ragged; rows of 64, 32 and 16 blocks
    # (one, two and four rows side by side in a wave) and of three slabs
    import torch
    print(f"tall gemv n={n} k={k}", flush=True)
    wq = synth.q4_weight(n, k, seed=13, tag="tall")
    x = synth.activations(1, k, seed=13, tag="tall")
    qw = be.upload_q4_blocks(wq)
    y = torch.full((1, n), float("nan"), dtype=torch.float32, device="cuda")
    be.gemv_batch(dev(x), qw, y, 1, n, k)
    ref = oracle.gemm_f64(x, wq, n, k)
    e = rel_err(host(y), ref)
    print(f"  rel err vs f64 {e:.2e}", flush=True)
    assert e <= 2e-5
    # every row against its own reference (a row written to another row's place would still be "small" above)
    assert np.max(np.abs(host(y) - ref)) <= 1e-4 * np.max(np.abs(ref))
