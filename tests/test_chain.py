"""The chain of dependent batch-1 GEMVs behind one call (`lq4_gemv_chain`): the decode steps the
reference encodes into one command buffer per token (forward/metal_qwen35.rs:6943, :6447):
o -> residual add -> shifted RMSNorm -> gate||up -> silu * up -> down -> residual add -> next layer's
RMSNorm -> qkv.  Checked against the oracle's unfused sequence (f32 GEMV after dequantisation, the
elementwise restatements)."""

import numpy as np
import pytest

import oracle
from lattice_amd import synth
from util import REL_TOL, rel_err

EPS = 1e-6


def _oracle_layer(x_attn, r0, g1, g2, w_o, w_gu, w_down, w_qkv, hidden, inter, qkv_rows):
    """o(+residual) -> norm -> gate||up -> silu*up -> down(+residual) -> norm -> qkv, step by step."""
    y_o = oracle.gemm_f32(x_attn[None, :], w_o, hidden, hidden)[0]
    r1, _ = oracle.add_and_copy(y_o, r0)
    xn = oracle.shifted_rms_norm(r1[None, :], g1, EPS)[0]
    gu = oracle.gemm_f32(xn[None, :], w_gu, 2 * inter, hidden)[0]
    h = oracle.silu_mul(gu[None, :])[0]
    y_d = oracle.gemm_f32(h[None, :], w_down, hidden, inter)[0]
    r2, _ = oracle.add_and_copy(y_d, r1)
    xn2 = oracle.shifted_rms_norm(r2[None, :], g2, EPS)[0]
    qkv = oracle.gemm_f32(xn2[None, :], w_qkv, qkv_rows, hidden)[0]
    return r1, h, r2, qkv


def _layer_inputs(hidden, inter, qkv_rows, seed):
    g = np.random.default_rng(seed)
    w = dict(o=synth.q4_weight(hidden, hidden, seed=seed, tag="o"),
             gu=synth.q4_weight(2 * inter, hidden, seed=seed, tag="gu"),
             down=synth.q4_weight(hidden, inter, seed=seed, tag="down"),
             qkv=synth.q4_weight(qkv_rows, hidden, seed=seed, tag="qkv"))
    x_attn = synth.activations(1, hidden, seed=seed, tag="attn")[0]
    r0 = synth.activations(1, hidden, seed=seed, tag="res")[0]
    g1 = (0.1 * g.normal(size=hidden)).astype(np.float32)
    g2 = (0.1 * g.normal(size=hidden)).astype(np.float32)
    return w, x_attn, r0, g1, g2


def _layer_steps(be, qw, xd, r0d, r1d, r2d, g1d, g2d, hidden, inter, qkv_rows, qkv, h=None):
    return [
        be.chain_step(qw["o"], hidden, hidden, x=xd),
        be.chain_step(qw["gu"], 2 * inter, hidden, from_previous=True, norm=(r0d, None, g1d, EPS, r1d),
                      silu_mul_pairs=True, y=h),
        be.chain_step(qw["down"], hidden, inter, from_previous=True),
        be.chain_step(qw["qkv"], qkv_rows, hidden, from_previous=True, norm=(r1d, None, g2d, EPS, r2d), y=qkv),
    ]


def _run_layer_chain(be, qw, x_attn, r0, g1, g2, hidden, inter, qkv_rows, want_h=False):
    import torch
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    xd, r0d, g1d, g2d = dev(x_attn), dev(r0), dev(g1), dev(g2)
    r1d, r2d = (torch.full((hidden,), float("nan"), dtype=torch.float32, device="cuda") for _ in range(2))
    qkv = torch.full((qkv_rows,), float("nan"), dtype=torch.float32, device="cuda")
    h = torch.full((inter,), float("nan"), dtype=torch.float32, device="cuda") if want_h else None
    be.dispatch_chain(_layer_steps(be, qw, xd, r0d, r1d, r2d, g1d, g2d, hidden, inter, qkv_rows, qkv, h))
    be.synchronize()
    assert np.array_equal(r0d.cpu().numpy(), r0), "the incoming residual stream must stay untouched"
    return r2d.cpu().numpy(), qkv.cpu().numpy(), (h.cpu().numpy() if want_h else None), r1d.cpu().numpy()


@pytest.mark.gpu
@pytest.mark.parametrize("hidden,inter,qkv_rows", [(2048, 6144, 3072), (64, 96, 40), (1024, 512, 6), (4096, 2048, 1000)])
def test_decode_layer_chain_matches_oracle_sequence(hidden, inter, qkv_rows):
    from lattice_amd import backend
    be = backend.HipQ4Backend(0)
    w, x_attn, r0, g1, g2 = _layer_inputs(hidden, inter, qkv_rows, seed=3)
    qw = {k: be.upload_q4_blocks(v) for k, v in w.items()}
    want_r1, want_h, want_r2, want_qkv = _oracle_layer(x_attn, r0, g1, g2, w["o"], w["gu"], w["down"], w["qkv"], hidden, inter, qkv_rows)

    before = be.path_counters()["gemv_chain"]
    got_r, got_qkv, got_h, got_r1 = _run_layer_chain(be, qw, x_attn, r0, g1, g2, hidden, inter, qkv_rows, want_h=True)
    assert be.path_counters()["gemv_chain"] == before + 1
    assert rel_err(got_r1, want_r1) <= 2e-5
    assert rel_err(got_h, want_h) <= REL_TOL
    assert rel_err(got_r, want_r2) <= REL_TOL
    assert rel_err(got_qkv, want_qkv) <= REL_TOL
    # in fact f32-faithful
    assert rel_err(got_r, want_r2) <= 2e-5 and rel_err(got_qkv, want_qkv) <= 2e-5

    # a second run of the same chain: the same bits (every sum has a fixed order)
    got_r_again, got_qkv_again, _, _ = _run_layer_chain(be, qw, x_attn, r0, g1, g2, hidden, inter, qkv_rows, want_h=True)
    assert be.path_counters()["gemv_chain"] == before + 2
    assert np.array_equal(got_r, got_r_again) and np.array_equal(got_qkv, got_qkv_again)
    be.close()


@pytest.mark.gpu
def test_chain_of_independent_steps_and_external_prologues():
    """Steps that all take external activations (no hand-over), with each external prologue, and a
    result that is only handed on (no y) next to one that is also stored."""
    import torch
    from lattice_amd import backend
    be = backend.HipQ4Backend(0)
    n, k = 300, 256
    g = np.random.default_rng(5)
    w1, w2, w3 = (synth.q4_weight(n, k, seed=s) for s in (1, 2, 3))
    x = synth.activations(1, k, seed=1)[0]
    base, delta = synth.activations(1, k, seed=2)[0], synth.activations(1, k, seed=3)[0]
    gamma = (0.2 * g.normal(size=k)).astype(np.float32)
    gate_up = synth.activations(1, 2 * k, seed=4)[0]
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    q1, q2, q3 = (be.upload_q4_blocks(w) for w in (w1, w2, w3))
    y1, y2, y3 = (torch.full((n,), float("nan"), dtype=torch.float32, device="cuda") for _ in range(3))
    res_out = torch.zeros(k, dtype=torch.float32, device="cuda")
    steps = [
        be.chain_step(q1, n, k, x=dev(x), y=y1),
        be.chain_step(q2, n, k, norm=(dev(base), dev(delta), dev(gamma), EPS, res_out), y=y2),
        be.chain_step(q3, n, k, x=dev(gate_up), silu_mul=True, y=y3),
    ]
    before = be.path_counters()["gemv_chain"]
    be.dispatch_chain(steps)
    be.synchronize()
    assert be.path_counters()["gemv_chain"] == before + 1
    res, normed = oracle.residual_add_norm(base[None, :], delta[None, :], gamma, EPS)
    assert rel_err(y1.cpu().numpy(), oracle.gemm_f32(x[None, :], w1, n, k)[0]) <= 2e-5
    assert rel_err(y2.cpu().numpy(), oracle.gemm_f32(normed, w2, n, k)[0]) <= 2e-5
    assert np.array_equal(res_out.cpu().numpy(), res[0])
    assert rel_err(y3.cpu().numpy(), oracle.gemm_f32(oracle.silu_mul(gate_up[None, :]), w3, n, k)[0]) <= 2e-5
    be.close()


@pytest.mark.gpu
def test_chain_replays_in_a_graph_and_other_routes():
    import torch
    from lattice_amd import backend
    be = backend.HipQ4Backend(0)
    hidden, inter, qkv_rows = 512, 768, 320
    w, x_attn, r0, g1, g2 = _layer_inputs(hidden, inter, qkv_rows, seed=9)
    qw = {k: be.upload_q4_blocks(v) for k, v in w.items()}
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    xd, r0d, g1d, g2d = dev(x_attn), dev(r0), dev(g1), dev(g2)
    r1d, r2d = torch.zeros(hidden, device="cuda"), torch.zeros(hidden, device="cuda")
    qkv = torch.zeros(qkv_rows, dtype=torch.float32, device="cuda")
    steps = _layer_steps(be, qw, xd, r0d, r1d, r2d, g1d, g2d, hidden, inter, qkv_rows, qkv)
    be.dispatch_chain(steps)  # warm: the scratch exists before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        be.dispatch_chain(steps)
    # every replay continues from the residual stream the previous one produced
    r_host = r0
    for rep in range(4):
        r0d.copy_(dev(r_host))
        graph.replay()
        torch.cuda.synchronize()
        _, _, want_r2, want_qkv = _oracle_layer(x_attn, r_host, g1, g2, w["o"], w["gu"], w["down"], w["qkv"], hidden, inter, qkv_rows)
        assert rel_err(r2d.cpu().numpy(), want_r2) <= 2e-5, rep
        assert rel_err(qkv.cpu().numpy(), want_qkv) <= 2e-5, rep
        r_host = r2d.cpu().numpy()
        # eager work of the same library between the replays
        y = torch.empty((1, hidden), dtype=torch.float32, device="cuda")
        be.dispatch_matmul(xd, qw["o"], y, 1, hidden, hidden)
        be.synchronize()

    # a tall step, a residual added as the result is stored, and a later step that names an earlier
    # step's y as its x
    n_big, k_big, n_tail = 8160, 2048, 96
    wb, wt = synth.q4_weight(n_big, k_big, seed=10), synth.q4_weight(n_tail, n_big, seed=11)
    qb, qt = be.upload_q4_blocks(wb), be.upload_q4_blocks(wt)
    xb = synth.activations(1, k_big, seed=10)[0]
    res = synth.activations(1, n_big, seed=12)[0]
    yb = torch.empty(n_big, dtype=torch.float32, device="cuda")
    resd = dev(res)
    yt = torch.empty(n_tail, dtype=torch.float32, device="cuda")
    before = be.path_counters()["gemv_chain"]
    be.dispatch_chain([be.chain_step(qb, n_big, k_big, x=dev(xb), add_residual=resd, y=yb),
                       be.chain_step(qt, n_tail, n_big, x=yb, y=yt)])
    be.synchronize()
    assert be.path_counters()["gemv_chain"] == before + 1
    want_b = oracle.add_and_copy(oracle.gemm_f32(xb[None, :], wb, n_big, k_big)[0], res)[0]
    assert rel_err(yb.cpu().numpy(), want_b) <= 2e-5 and np.array_equal(yb.cpu().numpy(), resd.cpu().numpy())
    assert rel_err(yt.cpu().numpy(), oracle.gemm_f32(want_b[None, :], wt, n_tail, n_big)[0]) <= 2e-5

    # K beyond what one workgroup stages in LDS: same contract
    n_l, k_l = 48, 17408
    wl = synth.q4_weight(n_l, k_l, seed=13)
    ql = be.upload_q4_blocks(wl)
    xl = synth.activations(1, k_l, seed=13)[0]
    yl = torch.empty(n_l, dtype=torch.float32, device="cuda")
    be.dispatch_chain([be.chain_step(ql, n_l, k_l, x=dev(xl), y=yl)])
    be.synchronize()
    assert rel_err(yl.cpu().numpy(), oracle.gemm_f32(xl[None, :], wl, n_l, k_l)[0]) <= 2e-5
    be.close()


@pytest.mark.gpu
def test_chain_contract_errors():
    import torch
    from lattice_amd import backend
    be = backend.HipQ4Backend(0)
    n, k = 64, 64
    qw = be.upload_q4_blocks(synth.q4_weight(n, k, seed=0))
    x = torch.zeros(k, dtype=torch.float32, device="cuda")
    y = torch.zeros(n, dtype=torch.float32, device="cuda")
    with pytest.raises(backend.Q4Error, match="step 0 needs external"):
        be.dispatch_chain([be.chain_step(qw, n, k, from_previous=True, y=y)])
    with pytest.raises(backend.Q4Error, match="nowhere to put its result"):
        be.dispatch_chain([be.chain_step(qw, n, k, x=x)])
    with pytest.raises(backend.Q4Error, match="previous step yields"):
        be.dispatch_chain([be.chain_step(qw, n, k, x=x, silu_mul_pairs=True), be.chain_step(qw, n, k, from_previous=True, y=y)])
    with pytest.raises(backend.Q4Error, match="at most 16"):
        be.dispatch_chain([be.chain_step(qw, n, k, x=x, y=y)] * 17)
    be.dispatch_chain([])  # no-op
    be.close()
