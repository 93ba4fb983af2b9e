"""The elementwise steps either side of the decode GEMVs: residual add + shifted RMSNorm
(shaders/qwen35.metal:739-767, model/qwen35/norm.rs:6-23), silu(gate) * up
(shaders/qwen35.metal:712-722), add-and-copy (shaders/qwen35.metal:2255-2266), stand-alone and
fused into the batch-1 Q4 GEMV.

Oracle pins: the norm against the HF RMSNorm goldens the reference's tests hold
(tests/fixtures/gemma4/stage3/rms_norm*.bin, standard gamma: the shifted norm with gamma - 1 must
reproduce them), closed forms, and an f64 restatement; silu against its identities and the value
the reference's MoE test uses (model/qwen35/tests.rs:298-299, 355)."""
import os

import numpy as np
import pytest

import oracle
from lattice_amd import synth
from util import REL_TOL, rel_err

GOLD = os.path.join(os.path.dirname(__file__), "golden", "rms_norm")
ELT_TOL = 2e-6  # f32 rounding: summation order of the mean square, one ulp of expf


def _bin(name):
    return np.fromfile(os.path.join(GOLD, name), dtype="<f4")


@pytest.mark.parametrize("prefix,hidden,tol", [("rms_norm", 64, 1e-6), ("rms_norm_wide", 1536, 5e-5)])
def test_oracle_norm_reproduces_hf_goldens(prefix, hidden, tol):
    # tolerances: the fixtures' own manifest (1e-6 at width 64, 5e-5 at width 1536), eps 1e-6
    x = _bin(prefix + "_input.bin").reshape(-1, hidden)
    w = _bin(prefix + "_weight.bin")
    want = _bin(prefix + "_output.bin").reshape(-1, hidden)
    got = oracle.shifted_rms_norm(x, w - np.float32(1.0), 1e-6)
    assert np.max(np.abs(got - want)) <= tol + 2e-7 * np.max(np.abs(want))  # (1 + (w - 1)) rounds once more
    # and the shift matters: plain gamma fed to the shifted norm misses the golden by far
    assert np.max(np.abs(oracle.shifted_rms_norm(x, w, 1e-6) - want)) > 1e-2


def test_oracle_norm_closed_forms():
    h = 96
    gamma = np.linspace(-0.5, 0.5, h).astype(np.float32)
    const = np.full((1, h), 3.0, np.float32)
    got = oracle.shifted_rms_norm(const, gamma, 1e-6)
    want = 3.0 / np.sqrt(9.0 + 1e-6) * (1.0 + gamma.astype(np.float64))
    assert np.max(np.abs(got[0] - want)) < 1e-6
    assert np.all(oracle.shifted_rms_norm(np.zeros((2, h), np.float32), gamma, 1e-6) == 0.0)
    g = np.random.default_rng(0)
    x = g.normal(size=(5, h)).astype(np.float32)
    a = oracle.shifted_rms_norm(x, gamma, 0.0)
    b = oracle.shifted_rms_norm(4.0 * x, gamma, 0.0)  # scale invariance without eps
    assert rel_err(a, b) < 1e-6
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt(np.mean(x64 * x64, axis=1, keepdims=True) + 1e-5) * (1.0 + gamma.astype(np.float64))
    assert rel_err(oracle.shifted_rms_norm(x, gamma, 1e-5), want) < 1e-6
    # rows are independent
    assert np.array_equal(oracle.shifted_rms_norm(x, gamma, 1e-5)[2], oracle.shifted_rms_norm(x[2:3], gamma, 1e-5)[0])


def test_oracle_residual_add_norm_silu_and_add():
    g = np.random.default_rng(1)
    base, delta = g.normal(size=(3, 64)).astype(np.float32), g.normal(size=(3, 64)).astype(np.float32)
    gamma = g.normal(size=64).astype(np.float32) * 0.1
    res, normed = oracle.residual_add_norm(base, delta, gamma, 1e-6)
    assert np.array_equal(res, base + delta)
    assert np.array_equal(normed, oracle.shifted_rms_norm(res, gamma, 1e-6))

    gu = np.array([[0.5, 0.0, -3.0, 20.0, 2.0, 7.0, 1.0, 1.0]], np.float32)  # gate(4) | up(4)
    out = oracle.silu_mul(gu)[0]
    silu_half = np.float32(0.5) / (np.float32(1.0) + np.exp(np.float32(-0.5)))
    assert abs(out[0] - silu_half * 2.0) < 1e-7 and abs(out[0] - 0.62244) < 5e-5  # the reference quotes ~0.62244
    assert abs(out[0] - 2.0 * 0.5 / (1.0 + np.exp(-0.5))) < 1e-7
    assert out[1] == 0.0
    x = g.normal(size=200).astype(np.float32) * 4
    pos = oracle.silu_mul(np.concatenate([x, np.ones_like(x)])[None])[0]
    neg = oracle.silu_mul(np.concatenate([-x, np.ones_like(x)])[None])[0]
    assert np.max(np.abs((pos - neg) - x)) < 1e-6          # silu(x) - silu(-x) = x
    x64 = x.astype(np.float64)
    assert np.max(np.abs(pos - x64 / (1.0 + np.exp(-x64)))) < 1e-6
    rows = g.normal(size=(3, 10)).astype(np.float32)
    assert np.array_equal(oracle.silu_mul(rows)[1], oracle.silu_mul(rows[1:2])[0])

    src, res0 = g.normal(size=33).astype(np.float32), g.normal(size=33).astype(np.float32)
    res1, dst = oracle.add_and_copy(src, res0)
    assert np.array_equal(res1, res0 + src) and np.array_equal(dst, res1)


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


@pytest.mark.gpu
@pytest.mark.parametrize("rows,hidden", [(1, 2048), (5, 96), (3, 5120), (2, 100), (3, 70)])  # 70: rows that are not whole float4s
def test_standalone_kernels_match_oracle(be, rows, hidden):
    import torch
    g = np.random.default_rng(rows * 1000 + hidden)
    base, delta = g.normal(size=(rows, hidden)).astype(np.float32), g.normal(size=(rows, hidden)).astype(np.float32)
    gamma = (g.normal(size=hidden) * 0.2).astype(np.float32)
    res_ref, normed_ref = oracle.residual_add_norm(base, delta, gamma, 1e-6)
    res = torch.empty((rows, hidden), device="cuda")
    normed = torch.empty((rows, hidden), device="cuda")
    be.dispatch_fused_residual_add_norm(dev(base), dev(delta), res, normed, dev(gamma), hidden, 1e-6, rows)
    assert np.array_equal(host(res), res_ref)
    assert rel_err(host(normed), normed_ref) <= ELT_TOL
    # plain norm: no delta, no residual store
    be.dispatch_fused_residual_add_norm(dev(base), None, None, normed, dev(gamma), hidden, 1e-6, rows)
    assert rel_err(host(normed), oracle.shifted_rms_norm(base, gamma, 1e-6)) <= ELT_TOL

    count = hidden // 2
    gu = (g.normal(size=(rows, 2 * count)) * 3).astype(np.float32)
    want = oracle.silu_mul(gu)
    out = torch.empty((rows, count), device="cuda")
    be.dispatch_silu_mul_fused(dev(gu), count, rows, out=out)
    assert rel_err(host(out), want) <= ELT_TOL
    inplace = dev(gu)
    be.dispatch_silu_mul_fused(inplace, count, rows)  # the reference's in-place form
    got = host(inplace)
    assert rel_err(got[:, :count], want) <= ELT_TOL and np.array_equal(got[:, count:], gu[:, count:])

    src, r0 = g.normal(size=rows * hidden).astype(np.float32), g.normal(size=rows * hidden).astype(np.float32)
    r_ref, d_ref = oracle.add_and_copy(src, r0)
    r, d = dev(r0), torch.empty(rows * hidden, device="cuda")
    be.dispatch_add_and_copy(dev(src), r, d, rows * hidden)
    assert np.array_equal(host(r), r_ref) and np.array_equal(host(d), d_ref)


def _mlp_inputs(hidden, inter, seed):
    g = np.random.default_rng(seed)
    gate_up = synth.q4_weight(2 * inter, hidden, seed=seed)
    down = synth.q4_weight(hidden, inter, seed=seed + 1)
    base = g.normal(size=hidden).astype(np.float32)
    delta = g.normal(size=hidden).astype(np.float32)
    gamma = (g.normal(size=hidden) * 0.2).astype(np.float32)
    return gate_up, down, base, delta, gamma


@pytest.mark.gpu
@pytest.mark.parametrize("hidden,inter", [(2048, 6144), (1024, 512), (512, 96), (160, 352),
                                          (5120, 544)])  # norm prologue in an eight-wave workgroup
def test_fused_decode_mlp_matches_oracle_and_unfused(be, hidden, inter):
    """norm + gate||up GEMV, then silu*up + down GEMV + residual add: two fused launches against
    the oracle's five steps and against the same five steps run one by one on the GPU."""
    import torch
    gate_up, down, base, delta, gamma = _mlp_inputs(hidden, inter, 11)
    eps = 1e-6
    # oracle
    res_ref, normed_ref = oracle.residual_add_norm(base[None], delta[None], gamma, eps)
    gu_ref = oracle.gemm_f32(normed_ref, gate_up, 2 * inter, hidden)
    h_ref = oracle.silu_mul(gu_ref)
    ffn_ref = oracle.gemm_f32(h_ref, down, hidden, inter)
    final_ref, copy_ref = oracle.add_and_copy(ffn_ref[0], res_ref[0])

    qgu, qd = be.upload_q4_blocks(gate_up), be.upload_q4_blocks(down)
    d_base, d_delta, d_gamma = dev(base), dev(delta), dev(gamma)
    # fused: two launches
    residual = torch.full((hidden,), float("nan"), device="cuda")
    gu = torch.full((2 * inter + 1,), float("nan"), device="cuda")
    be.dispatch_matmul_fused(None, qgu, gu, 2 * inter, hidden, norm=(d_base, d_delta, d_gamma, eps, residual))
    assert np.array_equal(host(residual), res_ref[0])
    got_gu = host(gu)
    assert np.isnan(got_gu[-1]) and rel_err(got_gu[:-1], gu_ref[0]) <= REL_TOL
    hidden_out = torch.full((hidden,), float("nan"), device="cuda")
    ffn = torch.full((hidden,), float("nan"), device="cuda")
    be.dispatch_matmul_fused(gu, qd, ffn, hidden, inter, silu_mul=True, add_residual=(residual, hidden_out))
    assert rel_err(host(ffn), ffn_ref[0]) <= REL_TOL
    assert rel_err(host(residual), final_ref) <= REL_TOL
    assert np.array_equal(host(hidden_out), host(residual))
    assert np.array_equal(host(residual), res_ref[0] + host(ffn))  # the add itself is exact

    # unfused on the GPU: same kernels' arithmetic, so agreement is at f32 rounding level
    res2 = torch.empty(hidden, device="cuda")
    normed = torch.empty(hidden, device="cuda")
    be.dispatch_fused_residual_add_norm(d_base, d_delta, res2, normed, d_gamma, hidden, eps)
    gu2 = torch.empty(2 * inter, device="cuda")
    be.dispatch_matmul(normed, qgu, gu2, 1, 2 * inter, hidden)
    assert rel_err(got_gu[:-1], host(gu2)) <= 1e-5
    be.dispatch_silu_mul_fused(gu2, inter)
    ffn2 = torch.empty(hidden, device="cuda")
    be.dispatch_matmul(gu2, qd, ffn2, 1, hidden, inter)
    assert rel_err(host(ffn), host(ffn2)) <= 1e-5
    hid2 = torch.empty(hidden, device="cuda")
    be.dispatch_add_and_copy(ffn2, res2, hid2, hidden)
    assert rel_err(host(hidden_out), host(hid2)) <= 1e-5
    c = be.path_counters()
    assert c["gemv_fused"] >= 2


@pytest.mark.gpu
@pytest.mark.parametrize("hidden,inter", [(2048, 6144),   # three rows per wave rounded up to four
                                          (2048, 20000),  # a persistent grid: waves walk several pairs
                                          (160, 352), (96, 32), (4096, 64), (8192, 96),
                                          (1024, 512), (512, 96)])  # rows side by side in a wave: the steps one by one
def test_fused_decode_mlp_with_silu_in_the_first_launch(be, hidden, inter):
    """norm + gate||up GEMV + silu(gate) * up in one launch (a wave takes the gate and the up row of a pair), then
    down GEMV + residual add: against the oracle's five steps and against the form that leaves silu * up to
    the second launch's prologue."""
    import torch
    gate_up, down, base, delta, gamma = _mlp_inputs(hidden, inter, 12)
    eps = 1e-6
    res_ref, normed_ref = oracle.residual_add_norm(base[None], delta[None], gamma, eps)
    gu_ref = oracle.gemm_f32(normed_ref, gate_up, 2 * inter, hidden)
    h_ref = oracle.silu_mul(gu_ref)
    qgu = be.upload_q4_blocks(gate_up)
    d_base, d_delta, d_gamma = dev(base), dev(delta), dev(gamma)
    residual = torch.full((hidden,), float("nan"), device="cuda")
    act = torch.full((inter + 1,), float("nan"), device="cuda")
    before = be.path_counters()
    be.dispatch_matmul_fused(None, qgu, act, 2 * inter, hidden, norm=(d_base, d_delta, d_gamma, eps, residual),
                             silu_mul_pairs=True)
    after = be.path_counters()
    assert np.array_equal(host(residual), res_ref[0])
    got = host(act)
    assert np.isnan(got[-1]), "wrote past inter values"
    e = rel_err(got[:-1], h_ref[0])
    print(f"fused silu pairs hidden={hidden} inter={inter}: rel err {e:.2e}", flush=True)
    assert e <= REL_TOL
    one_launch = hidden // 32 not in (16, 32)
    assert after["gemv_fused"] - before["gemv_fused"] == (1 if one_launch else 0)
    assert after["elementwise"] - before["elementwise"] == (0 if one_launch else 2)
    # the two-step form: [gate | up] out of the first launch, silu * up where the second one stages it
    gu = torch.empty(2 * inter, device="cuda")
    be.dispatch_matmul_fused(None, qgu, gu, 2 * inter, hidden, norm=(d_base, d_delta, d_gamma, eps, residual))
    be.dispatch_silu_mul_fused(gu, inter)
    assert rel_err(got[:-1], host(gu)[:inter]) <= 2e-6  # same sums; silu through exp2/rcp against expf and a divide
    if inter % 32 == 0:  # the whole MLP: the second launch is then a plain GEMV with the residual add
        ffn = torch.full((hidden,), float("nan"), device="cuda")
        hidden_out = torch.full((hidden,), float("nan"), device="cuda")
        qd = be.upload_q4_blocks(down)
        be.dispatch_matmul_fused(act, qd, ffn, hidden, inter, add_residual=(residual, hidden_out))
        ffn_ref = oracle.gemm_f32(h_ref, down, hidden, inter)
        final_ref, _ = oracle.add_and_copy(ffn_ref[0], res_ref[0])
        assert rel_err(host(ffn), ffn_ref[0]) <= REL_TOL
        assert rel_err(host(hidden_out), final_ref) <= REL_TOL


@pytest.mark.gpu
@pytest.mark.parametrize("hidden,inter,batch", [(2048, 6144, 8), (2048, 6144, 2), (1024, 512, 5), (160, 352, 3),
                                                (512, 96, 16), (2048, 1024, 11), (5120, 544, 4),
                                                (29184, 32, 3)])  # rows too long for LDS: the unfused sequence
def test_fused_decode_mlp_for_several_rows(be, hidden, inter, batch):
    """The decode MLP of `batch` sequences at once, two launches (norm + gate||up, silu*up + down + residual
    add), against the oracle's five steps row by row and against the stand-alone kernels on the GPU."""
    import torch
    g = np.random.default_rng(21)
    gate_up = synth.q4_weight(2 * inter, hidden, seed=21)
    down = synth.q4_weight(hidden, inter, seed=22)
    base = g.normal(size=(batch, hidden)).astype(np.float32)
    base *= (1.0 + np.arange(batch, dtype=np.float32))[:, None]  # rows with different rms
    delta = g.normal(size=(batch, hidden)).astype(np.float32)
    gamma = (g.normal(size=hidden) * 0.2).astype(np.float32)
    eps = 1e-6
    print(f"fused MLP hidden={hidden} inter={inter} batch={batch}", flush=True)
    res_ref, normed_ref = oracle.residual_add_norm(base, delta, gamma, eps)
    gu_ref = oracle.gemm_f32(normed_ref, gate_up, 2 * inter, hidden)
    h_ref = oracle.silu_mul(gu_ref)
    ffn_ref = oracle.gemm_f32(h_ref, down, hidden, inter)
    final_ref = res_ref + ffn_ref

    qgu, qd = be.upload_q4_blocks(gate_up), be.upload_q4_blocks(down)
    d_base, d_delta, d_gamma = dev(base), dev(delta), dev(gamma)
    before = be.path_counters()
    residual = torch.full((batch, hidden), float("nan"), device="cuda")
    gu = torch.full((batch * 2 * inter + 1,), float("nan"), device="cuda")
    be.dispatch_matmul_fused(None, qgu, gu, 2 * inter, hidden, norm=(d_base, d_delta, d_gamma, eps, residual),
                             batch=batch)
    assert np.array_equal(host(residual), res_ref)
    got_gu = host(gu)
    assert np.isnan(got_gu[-1])
    got_gu = got_gu[:-1].reshape(batch, 2 * inter)
    for b in range(batch):  # per row: rows differ in scale
        assert rel_err(got_gu[b], gu_ref[b]) <= REL_TOL, b
    hidden_out = torch.full((batch, hidden), float("nan"), device="cuda")
    ffn = torch.full((batch, hidden), float("nan"), device="cuda")
    be.dispatch_matmul_fused(gu, qd, ffn, hidden, inter, silu_mul=True, add_residual=(residual, hidden_out), batch=batch)
    for b in range(batch):
        # two dependent GEMVs, each rounding its activations to f16 above two rows: REL_TOL apiece
        assert rel_err(host(ffn)[b], ffn_ref[b]) <= 2 * REL_TOL, b
        assert rel_err(host(residual)[b], final_ref[b]) <= 2 * REL_TOL, b
    assert np.array_equal(host(hidden_out), host(residual))
    assert np.array_equal(host(residual), res_ref + host(ffn))  # the add itself is exact
    after = be.path_counters()
    # Routing: up to 8 rows whose staged form fits in LDS run in the fused kernel, with the prologue inside
    # while its input is at most 64 KB and as a launch of its own beyond; otherwise the steps run one by one.
    def stage(k, pro_bytes, steps):
        if batch <= 8 and k <= 8192:
            return 1, (1 if pro_bytes > 64 * 1024 else 0)
        return 0, steps
    f1, e1 = stage(hidden, batch * hidden * 4 * 2, 1)      # base + delta
    f2, e2 = stage(inter, batch * inter * 4 * 2, 2)        # gate + up; silu and the residual add
    assert after["gemv_fused"] - before["gemv_fused"] == f1 + f2
    assert after["elementwise"] - before["elementwise"] == e1 + e2

    # the stand-alone kernels and the plain GEMV on the GPU: the same arithmetic but for the order of the
    # sum of squares and the silu's exp, so agreement is far inside the GEMV tolerance
    res2 = torch.empty((batch, hidden), device="cuda")
    normed = torch.empty((batch, hidden), device="cuda")
    be.dispatch_fused_residual_add_norm(d_base, d_delta, res2, normed, d_gamma, hidden, eps, num_rows=batch)
    gu2 = torch.empty((batch, 2 * inter), device="cuda")
    be.gemv_batch(normed, qgu, gu2, batch, 2 * inter, hidden)
    # (three to eight rows of a small matrix: the plain call takes the integer matrix-core kernel, which keeps 16 or
    # 24 bits of an activation, while the fused call rounds it to f16 - each is within the contract of the oracle)
    same_kernel = 2e-5 if batch <= 2 else REL_TOL
    assert rel_err(got_gu, host(gu2)) <= same_kernel
    # (the second stage from the fused first stage's own output, so that only this stage is compared)
    gu2 = dev(got_gu)
    act = torch.empty((batch, inter), device="cuda")
    be.dispatch_silu_mul_fused(gu2, inter, batch, out=act, out_stride=inter)
    ffn2 = torch.empty((batch, hidden), device="cuda")
    be.gemv_batch(act, qd, ffn2, batch, hidden, inter)
    assert rel_err(host(ffn), host(ffn2)) <= same_kernel


@pytest.mark.gpu
@pytest.mark.parametrize("batch", [3, 8, 12])
def test_fused_rows_with_a_lora_adapter_run_step_by_step(be, batch):
    """lq4_gemv_fused_batch with an adapter on the projection: the prologue, the GEMV with its LoRA delta
    (A.x of the normalised rows) and the residual add run one after the other; same result as the oracle."""
    import torch
    from lattice_amd import backend
    n, k, rank = 96, 1024, 8
    g = np.random.default_rng(31)
    wq = synth.q4_weight(n, k, seed=31)
    qw = be.upload_q4_blocks(wq)
    base = g.normal(size=(batch, k)).astype(np.float32)
    gamma = (g.normal(size=k) * 0.1).astype(np.float32)
    res0 = g.normal(size=(batch, n)).astype(np.float32)
    a, b = synth.lora_pair(rank, k, n, seed=31)
    be.load_lora_adapter([backend.LoraLayerData(0, {"o_proj": (a, b)})], scale=1.5)
    try:
        before = be.path_counters()
        y = torch.full((batch, n), float("nan"), device="cuda")
        residual = dev(res0)
        be.dispatch_matmul_fused(None, qw, y, n, k, norm=(dev(base), None, dev(gamma), 1e-6, None),
                                 add_residual=(residual, None), layer_idx=0, module="o_proj", batch=batch)
        after = be.path_counters()
        assert after["gemv_fused"] == before["gemv_fused"] and after["elementwise"] == before["elementwise"] + 2
        # (no launch for A.x: at three and eight rows the integer matrix-core kernel computes it in producer workgroups
        # of its own launch, from nine rows on the few-token GEMM computes it for its token tile)
        assert after["lora_a"] == before["lora_a"]
        xn = oracle.shifted_rms_norm(base, gamma, 1e-6)
        want = oracle.lora_apply(a, b, 1.5, xn, oracle.gemm_f32(xn, wq, n, k))
        for r in range(batch):
            assert rel_err(host(y)[r], want[r]) <= REL_TOL, r
        assert np.array_equal(host(residual), res0 + host(y))
    finally:
        be.unload_lora_adapter()


@pytest.mark.gpu
def test_fused_gemv_options_and_fallbacks(be):
    import torch
    from lattice_amd import backend
    n, k = 37, 1024
    g = np.random.default_rng(5)
    wq = synth.q4_weight(n, k, seed=5)
    qw = be.upload_q4_blocks(wq)
    x = g.normal(size=k).astype(np.float32)
    res0 = g.normal(size=n).astype(np.float32)
    y_ref = oracle.gemm_f32(x[None], wq, n, k)[0]
    # epilogue only, no y wanted
    residual = dev(res0)
    be.dispatch_matmul_fused(dev(x), qw, None, n, k, add_residual=(residual, None))
    assert rel_err(host(residual), res0 + y_ref) <= REL_TOL
    # prologue only, norm without delta and without residual store
    gamma = (g.normal(size=k) * 0.1).astype(np.float32)
    y = torch.empty(n, device="cuda")
    be.dispatch_matmul_fused(None, qw, y, n, k, norm=(dev(x), None, dev(gamma), 1e-5, None))
    want = oracle.gemm_f32(oracle.shifted_rms_norm(x[None], gamma, 1e-5), wq, n, k)[0]
    assert rel_err(host(y), want) <= REL_TOL
    # LoRA + prologue runs as the unfused sequence; LoRA + epilogue stays fused
    a, b = synth.lora_pair(8, k, n, seed=5)
    be.load_lora_adapter([backend.LoraLayerData(0, {"q_proj": (a, b)})], scale=2.0)
    try:
        before = be.path_counters()
        be.dispatch_matmul_fused(None, qw, y, n, k, norm=(dev(x), None, dev(gamma), 1e-5, None), layer_idx=0,
                                 module="q_proj")
        mid = be.path_counters()
        assert mid["gemv_fused"] == before["gemv_fused"] and mid["elementwise"] == before["elementwise"] + 1
        xn = oracle.shifted_rms_norm(x[None], gamma, 1e-5)
        assert rel_err(host(y), oracle.lora_apply(a, b, 2.0, xn, oracle.gemm_f32(xn, wq, n, k))[0]) <= REL_TOL
        residual = dev(res0)
        be.dispatch_matmul_fused(dev(x), qw, y, n, k, add_residual=(residual, None), layer_idx=0, module="q_proj")
        assert be.path_counters()["gemv_fused"] == mid["gemv_fused"] + 1
        y_l = oracle.lora_apply(a, b, 2.0, x[None], y_ref[None].copy())[0]
        assert rel_err(host(y), y_l) <= REL_TOL and rel_err(host(residual), res0 + y_l) <= REL_TOL
    finally:
        be.unload_lora_adapter()
    # K too long for the staged kernel: the unfused sequence through scratch
    kk = 29184
    wl = synth.q4_weight(4, kk, seed=6)
    ql = be.upload_q4_blocks(wl)
    gul = (g.normal(size=2 * kk)).astype(np.float32)
    yl = torch.empty(4, device="cuda")
    rl = dev(np.ones(4, np.float32))
    be.dispatch_matmul_fused(dev(gul), ql, yl, 4, kk, silu_mul=True, add_residual=(rl, None))
    want = oracle.gemm_f32(oracle.silu_mul(gul[None]), wl, 4, kk)[0]
    assert rel_err(host(yl), want) <= REL_TOL and rel_err(host(rl), 1.0 + want) <= REL_TOL
    # rejected calls: residual_out over base, missing y without an epilogue
    xb = dev(x)
    with pytest.raises(backend.Q4Error):
        be.dispatch_matmul_fused(None, qw, y, n, k, norm=(xb, None, dev(gamma), 1e-5, xb))
    with pytest.raises(backend.Q4Error):
        be.dispatch_matmul_fused(xb, qw, None, n, k, silu_mul=False, add_residual=None, norm=(xb, None, dev(gamma), 1e-5, None))
