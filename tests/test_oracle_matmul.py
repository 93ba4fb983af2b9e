"""Pins the oracle's contraction, LoRA delta, MoE routing/accumulation and the CPU
baseline kernels: reference-held hand cases plus identities a dropped term, a
transposed operand or a wrong index would break."""
import numpy as np
import pytest

import oracle
from lattice_amd import q4_layout, synth


def _dense(wq, n, k):
    return q4_layout.dequantize_numpy(wq).reshape(n, k)


# ------------------------------------------------------------------------- GEMM
@pytest.mark.parametrize("m,n,k", [(1, 1, 32), (1, 5, 64), (1, 33, 96), (5, 9, 96), (8, 8, 64),
                                   (1, 6, 64), (72, 48, 64), (64, 64, 64)])
def test_gemm_matches_numpy_f64_contraction(m, n, k):
    # shapes: forward/metal_qwen35.rs:19624-19628, 19690-19705, 22937-23122
    wq = synth.q4_weight(n, k, seed=1, symmetric_bias=False)
    x = synth.activations(m, k, seed=1)
    want = x.astype(np.float64) @ _dense(wq, n, k).astype(np.float64).T
    y64 = oracle.gemm_f64(x, wq, n, k)
    assert np.allclose(y64, want, rtol=1e-12, atol=1e-14)
    y32 = oracle.gemm_f32(x, wq, n, k)
    assert y32.shape == (m, n)
    assert np.max(np.abs(y32 - want)) <= 1e-5 * max(1.0, np.max(np.abs(want)))


def test_gemm_f32_is_sequential_ascending_k():
    # forward/metal_qwen35.rs:22887-22899: acc += x*w with k ascending, no FMA.
    n, k = 3, 96
    wq = synth.q4_weight(n, k, seed=2)
    x = synth.activations(2, k, seed=2)
    w = _dense(wq, n, k)
    want = np.zeros((2, n), np.float32)
    for mi in range(2):
        for ni in range(n):
            acc = np.float32(0)
            for ki in range(k):
                acc = np.float32(acc + np.float32(x[mi, ki] * w[ni, ki]))
            want[mi, ni] = acc
    assert np.array_equal(oracle.gemm_f32(x, wq, n, k), want)


def test_gemm_one_hot_returns_dequantized_column():
    n, k = 7, 128
    wq = synth.q4_weight(n, k, seed=3, symmetric_bias=False)
    w = _dense(wq, n, k)
    x = np.eye(k, dtype=np.float32)
    y = oracle.gemm_f32(x, wq, n, k)  # [k, n]
    assert np.array_equal(y.T, w)


def test_gemm_linearity_and_constant_block():
    n, k = 4, 64
    wq = synth.q4_weight(n, k, seed=4)
    x1, x2 = synth.activations(1, k, seed=4, tag="a"), synth.activations(1, k, seed=4, tag="b")
    y = oracle.gemm_f64(2 * x1 + x2, wq, n, k)
    assert np.allclose(y, 2 * oracle.gemm_f64(x1, wq, n, k) + oracle.gemm_f64(x2, wq, n, k),
                       rtol=1e-6, atol=1e-9)
    # all nibbles 8 in symmetric mode -> every weight is exactly 0
    z = q4_layout.pack_blocks(np.full(2, 0x2E66, np.uint16), np.full(2, 0x2E66 + 0x0C00 + 0x8000, np.uint16),
                              np.full((2, 32), 8, np.uint8))
    sb, bb, _ = q4_layout.unpack_blocks(z)
    assert bb.view(np.float16)[0] == -8 * sb.view(np.float16)[0]
    assert np.all(oracle.gemm_f32(x1, z, 1, 64) == 0)
    # constant-per-row weights (forward/metal_qwen35/mtp_weights.rs:401-404): a constant block
    # quantizes to nibble 0 with bias = the constant, so y = const * sum(x)
    c = oracle.quantize_rows(np.full((1, 64), 0.375, np.float32))
    assert np.allclose(oracle.gemm_f64(x1, c, 1, 64)[0, 0], 0.375 * x1.astype(np.float64).sum())


def test_gemm_rejects_bad_k():
    with pytest.raises(ValueError):
        oracle.gemm_f32(np.zeros((1, 48), np.float32), np.zeros(40, np.uint8), 1, 48)


# ------------------------------------------------------------------------- LoRA
def test_lora_reference_hand_cases():
    # crates/tune/src/lora/apply.rs:99-148
    y = oracle.lora_apply([[1, 0, 0]], [[1], [0]], 2.0, [5, 3, 1], [100, 200])
    assert np.allclose(y, [[110, 200]], atol=1e-6)
    y = oracle.lora_apply([[1, 0], [0, 1]], [[1, 2], [3, 4]], 0.5, [1, 1], [0, 0])
    assert np.allclose(y, [[1.5, 3.5]], atol=1e-6)
    y = oracle.lora_apply([[1, 0], [0, 1]], [[1, 2], [3, 4]], 0.0, [1, 1], [7, 9])
    assert np.array_equal(y, [[7, 9]])


def test_lora_matches_dense_algebra_per_row():
    a, b = synth.lora_pair(16, 256, 96, seed=5)
    a, b = a.astype(np.float32), b.astype(np.float32)
    x = synth.activations(8, 256, seed=5)
    y0 = synth.activations(8, 96, seed=5, tag="y")
    want = y0.astype(np.float64) + 2.0 * (x.astype(np.float64) @ a.T.astype(np.float64)) @ b.T.astype(np.float64)
    assert np.allclose(oracle.lora_apply_f64(a, b, 2.0, x, y0), want, rtol=1e-12, atol=1e-15)
    assert np.allclose(oracle.lora_apply(a, b, 2.0, x, y0), want, rtol=1e-5, atol=1e-6)


# -------------------------------------------------------------------------- MoE
def test_select_top_k_reference_cases():
    # model/qwen35/moe.rs:271-300
    ids, vals = oracle.select_top_k([0.30, 0.10, 0.50, 0.10], 2)
    assert list(ids) == [2, 0] and np.allclose(vals, [0.5, 0.3])
    # :302-330 ties: unique valid ids; strict `>` keeps the lowest ids, in order
    ids, _ = oracle.select_top_k([0.125] * 8, 3)
    assert list(ids) == [0, 1, 2]
    # nothing beats -inf with NaN probabilities: slots stay unfilled
    ids, _ = oracle.select_top_k([np.nan] * 4, 2)
    assert list(ids) == [-1, -1]


def test_renormalize_and_softmax():
    # :332-360 renormalised weights sum to one
    v = oracle.renormalize_selected([0.4, 0.2, 0.1])
    assert abs(v.sum() - 1) < 1e-6 and np.allclose(v, np.array([4, 2, 1]) / 7)
    assert np.array_equal(oracle.renormalize_selected([0.0, 0.0]), [0, 0])
    lg = synth.router_logits(4, 64, seed=0)
    for row in lg:
        p = oracle.router_softmax(row)
        e = np.exp(row.astype(np.float64) - row.max())
        assert np.allclose(p, e / e.sum(), rtol=1e-6)
    # degenerate rows fail closed to all-zero (moe.rs:52-66, 76-93)
    assert np.all(oracle.router_softmax([np.nan, np.nan]) == 0)
    assert np.all(oracle.router_softmax([np.inf, 1.0]) == 0)
    assert np.all(oracle.router_softmax([1.0, np.nan, 0.5]) == 0)
    assert np.all(oracle.router_softmax([-np.inf, -np.inf]) == 0)


def test_moe_route_matches_argsort():
    lg = synth.router_logits(16, 64, seed=0)
    ids, wts, probs = oracle.moe_route(lg, 8)
    order = np.argsort(-lg, axis=1, kind="stable")[:, :8]
    assert np.array_equal(ids, order)
    assert np.allclose(wts.sum(1), 1, atol=1e-6)
    sel = np.take_along_axis(probs, ids, 1)
    assert np.allclose(wts, sel / sel.sum(1, keepdims=True), rtol=1e-6)


def test_moe_ffn_matches_dense_f64_composition():
    e_, inter, hidden, t, top_k = 4, 64, 96, 3, 2
    gu = synth.q4_weight(e_ * 2 * inter, hidden, seed=6, tag="gu", scale_std=0.2)
    dn = synth.q4_weight(e_ * hidden, inter, seed=6, tag="dn", scale_std=0.2)
    x = synth.activations(t, hidden, seed=6)
    ids = np.array([[1, 3], [0, 1], [2, -1]], dtype=np.int32)  # -1: unfilled slot, skipped
    wts = np.array([[0.7, 0.3], [0.5, 0.5], [1.0, 0.0]], dtype=np.float32)
    wgu = _dense(gu, e_ * 2 * inter, hidden).astype(np.float64).reshape(e_, 2 * inter, hidden)
    wdn = _dense(dn, e_ * hidden, inter).astype(np.float64).reshape(e_, hidden, inter)
    want = np.zeros((t, hidden))
    for ti in range(t):
        for s in range(top_k):
            e = ids[ti, s]
            if e < 0:
                continue
            g = wgu[e, :inter] @ x[ti].astype(np.float64)
            u = wgu[e, inter:] @ x[ti].astype(np.float64)
            h = g / (1 + np.exp(-g)) * u
            want[ti] += float(wts[ti, s]) * (wdn[e] @ h)
    got64 = oracle.moe_ffn(gu, dn, e_, inter, hidden, x, ids, wts, f64=True)
    assert np.allclose(got64, want, rtol=1e-10, atol=1e-12)
    got32 = oracle.moe_ffn(gu, dn, e_, inter, hidden, x, ids, wts)
    assert np.max(np.abs(got32 - want)) <= 1e-5 * np.max(np.abs(want))


def test_moe_constant_expert_closed_form():
    # forward/metal_qwen35.rs:20089-20235 builds constant-per-row expert tensors so Q4 is exact:
    # gate rows = a, up rows = b, down rows = c  ->  out = w * c * I * silu(a*S) * (b*S), S = sum(x)
    e_, inter, hidden = 2, 32, 64
    a, b, c = 0.25, -0.5, 0.125
    gu = np.concatenate([oracle.quantize_rows(np.full((inter, hidden), v, np.float32))
                         for _ in range(e_) for v in (a, b)])
    dn = np.concatenate([oracle.quantize_rows(np.full((hidden, inter), c, np.float32))
                         for _ in range(e_)])
    x = synth.activations(1, hidden, seed=7)
    s = float(x.astype(np.float64).sum())
    g, u = a * s, b * s
    want = 1.0 * c * inter * (g / (1 + np.exp(-g))) * u
    got = oracle.moe_ffn(gu, dn, e_, inter, hidden, x, np.array([[1]], np.int32),
                         np.array([[1.0]], np.float32), f64=True)
    assert np.allclose(got, want, rtol=1e-12)


def test_moe_shared_expert_matches_dense_f64_composition():
    # independent restatement in numpy f64 from the (pinned) dequantised tensors: a swapped gate/up
    # half, a transposed operand, a dropped sigmoid or an overwritten accumulator fails here
    inter, hidden, t = 96, 160, 4
    gu = synth.q4_weight(2 * inter, hidden, seed=8, tag="sh_gu", scale_std=0.2)
    dn = synth.q4_weight(hidden, inter, seed=8, tag="sh_dn", scale_std=0.2)
    x = synth.activations(t, hidden, seed=8)
    rng = np.random.default_rng(8)
    sg = (rng.normal(size=hidden) * 0.2).astype(np.float32)
    base = rng.normal(size=(t, hidden)).astype(np.float32)
    wgu = _dense(gu, 2 * inter, hidden).astype(np.float64)
    wdn = _dense(dn, hidden, inter).astype(np.float64)
    x64 = x.astype(np.float64)
    gate_val = 1 / (1 + np.exp(-(x64 @ sg.astype(np.float64))))
    assert 0.01 < gate_val.min() and gate_val.max() < 0.99 and np.ptp(gate_val) > 0.05  # not a trivial gate
    g, u = x64 @ wgu[:inter].T, x64 @ wgu[inter:].T
    want = base.astype(np.float64) + gate_val[:, None] * ((g / (1 + np.exp(-g)) * u) @ wdn.T)
    got64 = oracle.moe_shared_expert(gu, dn, sg, inter, hidden, x, base, f64=True)
    assert np.allclose(got64, want, rtol=1e-10, atol=1e-12)
    got32 = oracle.moe_shared_expert(gu, dn, sg, inter, hidden, x, base)
    assert np.max(np.abs(got32 - want)) <= 1e-5 * np.max(np.abs(want))


def test_moe_shared_expert_with_zero_gate_vector_is_half_a_routed_expert():
    # sigmoid(0) = 1/2 exactly, so the shared expert equals one routed expert of the same tensors at
    # weight 0.5, bit for bit (moe.rs:242-244 and :187-189 share the scaled add)
    inter, hidden, t = 64, 96, 3
    gu = synth.q4_weight(2 * inter, hidden, seed=9, tag="gu", scale_std=0.2)
    dn = synth.q4_weight(hidden, inter, seed=9, tag="dn", scale_std=0.2)
    x = synth.activations(t, hidden, seed=9)
    routed = oracle.moe_ffn(gu, dn, 1, inter, hidden, x, np.zeros((t, 1), np.int32), np.full((t, 1), 0.5, np.float32))
    shared = oracle.moe_shared_expert(gu, dn, np.zeros(hidden, np.float32), inter, hidden, x, np.zeros((t, hidden), np.float32))
    assert np.array_equal(shared.view(np.uint32), routed.view(np.uint32))


def test_moe_shared_expert_gate_saturates_and_constant_closed_form():
    # constant-per-row tensors are exact in Q4: out = base + g * c * I * silu(a*S) * (b*S), S = sum(x)
    inter, hidden = 32, 64
    a, b, c = 0.25, -0.5, 0.125
    gu = np.concatenate([oracle.quantize_rows(np.full((inter, hidden), v, np.float32)) for v in (a, b)])
    dn = oracle.quantize_rows(np.full((hidden, inter), c, np.float32))
    x = synth.activations(1, hidden, seed=7)
    s = float(x.astype(np.float64).sum())
    ffn = c * inter * ((a * s) / (1 + np.exp(-a * s))) * (b * s)
    base = np.full((1, hidden), 3.0, np.float32)
    for gate_scale, want_g in ((0.0, 0.5), (1e4, None), (-1e4, None)):
        sg = (gate_scale * np.sign(x[0])).astype(np.float32)  # logit = gate_scale * sum|x|
        logit = gate_scale * float(np.abs(x.astype(np.float64)).sum())
        g = 0.5 if want_g else (1.0 if logit > 0 else 0.0)
        got = oracle.moe_shared_expert(gu, dn, sg, inter, hidden, x, base, f64=True)
        assert np.allclose(got, 3.0 + g * ffn, rtol=1e-12), gate_scale
    # ln(3) as the logit: sigmoid = 3/4
    sg = np.zeros(hidden, np.float32)
    sg[0] = np.float32(np.log(3.0) / x[0, 0])
    got = oracle.moe_shared_expert(gu, dn, sg, inter, hidden, x, base, f64=True)
    g = 1 / (1 + np.exp(-float(np.float64(sg[0]) * np.float64(x[0, 0]))))
    assert abs(g - 0.75) < 1e-6 and np.allclose(got, 3.0 + g * ffn, rtol=1e-12)


# ----------------------------------------------------------------- CPU baseline
@pytest.mark.parametrize("m,k,n", [(1, 96, 7), (3, 200, 9), (4, 256, 8), (5, 1024, 300), (1, 2048, 600)])
def test_cpu_baseline_kernels_agree_with_numpy(m, k, n):
    rng = np.random.default_rng(9)
    a = rng.normal(size=(m, k)).astype(np.float32)
    b = rng.normal(size=(n, k)).astype(np.float32)
    want = a.astype(np.float64) @ b.T.astype(np.float64)
    tol = 2e-5 * np.sqrt(k) * max(1.0, np.abs(want).max())
    kernels = ["dispatch", "avx2", "tiled"]
    for kern in kernels:
        c, kid = oracle.matmul_bt(a, b, m, k, n, kernel=kern)
        assert np.max(np.abs(c - want)) < tol, kern
        if kern == "dispatch":
            # forward/cpu/matmul.rs:83-87
            assert (kid == 0) == (m * n * k >= 1 << 20 and k >= 128)


def test_cpu_q4_route_equals_oracle_within_summation_order():
    n, k, m = 64, 256, 2
    wq = synth.q4_weight(n, k, seed=8)
    x = synth.activations(m, k, seed=8)
    scratch = np.zeros(n * k, np.float32)
    y, _ = oracle.cpu_q4_matmul(x, wq, scratch, m, n, k, mode=1)
    assert np.array_equal(scratch, q4_layout.dequantize_numpy(wq))
    ref = oracle.gemm_f64(x, wq, n, k)
    assert np.max(np.abs(y - ref)) <= 1e-5 * np.abs(ref).max()
