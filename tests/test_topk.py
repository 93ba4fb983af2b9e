"""lm_head top-k: the reference's candidate order and its two-stage exact selection
(shaders/qwen35.metal:1683-1778, 1868-1985).  The oracle is pinned by brute force (numpy
lexsort on small inputs) and by hand cases; the GPU kernels are checked bit for bit against it,
including the adversarial distributions the reference names: all winners clustered in one tile,
ties, NaN and infinities."""
import numpy as np
import pytest

import oracle
from lattice_amd import synth
from util import REL_TOL


def _brute(logits, k):
    lg = np.asarray(logits, np.float32).copy()
    ids = np.arange(lg.size, dtype=np.uint32)
    nan = np.isnan(lg)
    lg[nan] = -np.inf
    ids[nan] = 0xFFFFFFFF
    order = np.lexsort((ids, -lg.astype(np.float64)))  # primary: logit descending; secondary: id ascending
    out_l = np.full(k, -np.inf, np.float32)
    out_i = np.full(k, 0xFFFFFFFF, np.uint32)
    m = min(k, lg.size)
    out_l[:m], out_i[:m] = lg[order[:m]], ids[order[:m]]
    return out_l, out_i


def test_oracle_hand_cases():
    l, i = oracle.topk(np.array([1, 5, np.nan, 5, -np.inf, 3], np.float32), 4)
    assert l.tolist() == [5, 5, 3, 1] and i.tolist() == [1, 3, 5, 0]  # tie -> lower id first
    l, i = oracle.topk(np.array([np.nan, np.nan], np.float32), 3)
    assert np.all(np.isneginf(l)) and i.tolist() == [0xFFFFFFFF] * 3  # NaN never wins a slot
    l, i = oracle.topk(np.array([-np.inf, np.nan, -np.inf], np.float32), 3)
    assert i.tolist() == [0, 2, 0xFFFFFFFF]  # a real -inf still ranks before the sentinel
    l, i = oracle.topk(np.array([2.0, 7.0], np.float32), 1)
    assert l.tolist() == [7.0] and i.tolist() == [1]


@pytest.mark.parametrize("n,k,seed", [(7, 3, 0), (1000, 50, 1), (5000, 256, 2), (300, 300 // 2, 3)])
def test_oracle_matches_brute_force(n, k, seed):
    g = np.random.default_rng(seed)
    lg = g.normal(size=n).astype(np.float32)
    lg[g.integers(0, n, n // 10)] = lg[0]          # plenty of exact ties
    lg[g.integers(0, n, max(1, n // 50))] = np.nan
    want = _brute(lg, k)
    got = oracle.topk(lg, k)
    assert np.array_equal(got[1], want[1]) and np.array_equal(got[0], want[0])


def _cases():
    g = np.random.default_rng(7)
    n = 248320
    base = g.normal(size=n).astype(np.float32)
    clustered = base.copy()
    clustered[5 * 1024 + 3: 5 * 1024 + 3 + 200] = 50.0 + np.arange(200, dtype=np.float32)  # one tile holds all winners
    ties = np.zeros(n, np.float32)
    ties[::7] = 1.0
    nans = base.copy()
    nans[::3] = np.nan
    nans[10] = np.inf
    nans[11] = -np.inf
    zeros = np.zeros(n, np.float32)
    zeros[g.integers(0, n, n // 2)] = -0.0           # -0 and +0 tie (lower id first) and keep their sign bit
    zeros[g.integers(0, n, 20)] = -1.0
    few_real = np.full(n, np.nan, np.float32)        # fewer real values than k: the rest stay sentinels
    few_real[g.integers(0, n, 30)] = g.normal(size=30).astype(np.float32)
    return {"random": base, "clustered": clustered, "ties": ties, "nan_inf": nans,
            "short": base[:777], "one_tile_exact": base[:1024], "all_nan": np.full(2000, np.nan, np.float32),
            # whole blocks survive the threshold: thousands of candidates to cut down to k
            "ascending": np.arange(n, dtype=np.float32), "descending": -np.arange(n, dtype=np.float32),
            "constant": np.full(n, 3.25, np.float32), "signed_zeros": zeros, "few_real": few_real,
            "odd_length": base[:100003],
            "small_vocabulary": base[:32000]}  # blocks of 64 logits so that there are at least k of them


@pytest.mark.gpu
@pytest.mark.parametrize("k", [1, 8, 50, 64, 256])
def test_gpu_topk_is_exact(k):
    import torch
    from lattice_amd import backend
    be = backend.HipQ4Backend(0)
    for name, lg in _cases().items():
        print(f"topk {name} n={lg.size} k={k}", flush=True)
        out_l, out_i = be.topk(torch.from_numpy(lg).cuda(), k)
        want_l, want_i = oracle.topk(lg, k)
        got_i = out_i.cpu().numpy().view(np.uint32)
        got_l = out_l.cpu().numpy()
        assert np.array_equal(got_i, want_i), name
        assert np.array_equal(got_l.view(np.uint32), want_l.view(np.uint32)), name


@pytest.mark.gpu
def test_gpu_lm_head_topk_matches_gemv_then_topk():
    import torch
    from lattice_amd import backend
    be = backend.HipQ4Backend(0)
    vocab, k, top_k = 5000, 256, 40
    wq = synth.q4_weight(vocab, k, seed=11)
    x = synth.activations(1, k, seed=11)
    qw = be.upload_q4_blocks(wq)
    xd = torch.from_numpy(x).cuda()
    out_l, out_i = be.lm_head_topk(xd, qw, vocab, k, top_k)
    # same library, two calls: logits from the GEMV, selection on them -> must agree bit for bit
    y = torch.empty((1, vocab), dtype=torch.float32, device="cuda")
    be.dispatch_matmul(xd, qw, y, 1, vocab, k)
    ref_l, ref_i = oracle.topk(y.cpu().numpy().reshape(-1), top_k)
    assert np.array_equal(out_i.cpu().numpy().view(np.uint32), ref_i)
    assert np.array_equal(out_l.cpu().numpy().view(np.uint32), ref_l.view(np.uint32))
    # against the CPU oracle's own logits: same winners wherever the gap to the next candidate
    # exceeds the GEMV tolerance (the reference's tie epsilon, metal_qwen35.rs:37365-37427)
    logits = oracle.gemm_f32(x, wq, vocab, k).reshape(-1)
    o_l, o_i = oracle.topk(logits, top_k + 1)
    eps = REL_TOL * np.abs(logits).max()
    got = out_i.cpu().numpy().view(np.uint32)
    for r in range(top_k):
        if o_l[r] - o_l[r + 1] > eps and (r == 0 or o_l[r - 1] - o_l[r] > eps):
            assert got[r] == o_i[r], r
    assert np.abs(out_l.cpu().numpy() - o_l[:top_k]).max() <= eps


def _lm_head_cases():
    """(name, vocab, k, top_k, weight blocks, x): shapes on both sides of what the one-launch form takes,
    exact ties, logits near the top of the f32 range, and all-NaN logits."""
    cases = []
    for vocab, k, top_k, seed in [(5000, 2048, 40, 1), (300, 2048, 50, 2), (100, 2048, 50, 3), (7001, 5120, 64, 4),
                                  (3000, 4096, 1, 5), (2500, 8192, 17, 6), (4099, 2112, 33, 7), (40000, 2048, 64, 8),
                                  (6000, 1024, 20, 9), (5000, 2048, 65, 10)]:
        cases.append((f"v{vocab}_k{k}_top{top_k}", vocab, k, top_k, synth.q4_weight(vocab, k, seed=seed),
                      synth.activations(1, k, seed=seed)))
    # 37 distinct rows repeated: every logit occurs 100+ times, the lower token id must win each tie
    vocab, k = 4000, 2048
    rows = synth.q4_weight(37, k, seed=12).reshape(37, -1)
    tied = np.ascontiguousarray(rows[np.arange(vocab) % 37]).reshape(-1)
    cases.append(("exact_ties", vocab, k, 50, tied, synth.activations(1, k, seed=12)))
    # logits near the top of the f32 range, and (one activation infinite: inf - inf inside every row) all NaN,
    # which the selection returns as sentinels
    x = synth.activations(1, k, seed=13)
    x[0, 5], x[0, 40] = 3.0e38, -3.0e38
    cases.append(("huge_logits", 5000, k, 60, synth.q4_weight(5000, k, seed=13), x))
    x = synth.activations(1, k, seed=14)
    x[0, 0] = np.inf
    cases.append(("all_nan_logits", 5000, k, 60, synth.q4_weight(5000, k, seed=14), x))
    return cases


@pytest.mark.gpu
def test_gpu_lm_head_topk_is_the_exact_topk_of_the_gemv_logits():
    import torch
    from lattice_amd import backend
    be = backend.HipQ4Backend(0)
    try:
        for name, vocab, k, top_k, wq, x in _lm_head_cases():
            print(f"lm_head top-k: {name}", flush=True)
            qw = be.upload_q4_blocks(wq)
            xd = torch.from_numpy(x).cuda()
            y = torch.empty((1, vocab), dtype=torch.float32, device="cuda")
            be.dispatch_matmul(xd, qw, y, 1, vocab, k)
            ref_l, ref_i = oracle.topk(y.cpu().numpy().reshape(-1), top_k)
            for rep in range(3):  # the ticket and the maxima are shared by back-to-back calls
                two_l, two_i = be.lm_head_topk(xd, qw, vocab, k, top_k)
                two_l, two_i = two_l.cpu().numpy().view(np.uint32), two_i.cpu().numpy().view(np.uint32)
                assert np.array_equal(two_i, ref_i), (name, rep)
                assert np.array_equal(two_l, ref_l.view(np.uint32)), (name, rep)
            if name == "exact_ties":
                # the best row's copies, lower token ids first
                assert np.array_equal(two_i, two_i[0] + 37 * np.arange(top_k, dtype=np.uint32)) and two_i[0] < 37
            if name == "all_nan_logits":
                assert np.all(two_i == 0xFFFFFFFF) and np.isnan(y.cpu().numpy()).all()
    finally:
        be.close()


@pytest.mark.gpu
def test_gpu_lm_head_topk_alternating_inputs():
    """Calls that alternate between two vocabularies and activations share the logits buffer, the
    maxima and the ticket: each call must select from its own launches' values."""
    import torch
    from lattice_amd import backend
    be = backend.HipQ4Backend(0)
    k = 2048
    sets = []
    for vocab, seed, gain in [(30000, 21, 1.0), (11000, 22, 1e-3)]:
        wq = synth.q4_weight(vocab, k, seed=seed)
        x = synth.activations(1, k, seed=seed) * np.float32(gain)
        qw, xd = be.upload_q4_blocks(wq), torch.from_numpy(x).cuda()
        y = torch.empty((1, vocab), dtype=torch.float32, device="cuda")
        be.dispatch_matmul(xd, qw, y, 1, vocab, k)
        sets.append((vocab, qw, xd, oracle.topk(y.cpu().numpy().reshape(-1), 50)))
    try:
        for it in range(40):
            vocab, qw, xd, (ref_l, ref_i) = sets[it % 2]
            out_l, out_i = be.lm_head_topk(xd, qw, vocab, k, 50)
            assert np.array_equal(out_i.cpu().numpy().view(np.uint32), ref_i), it
            assert np.array_equal(out_l.cpu().numpy().view(np.uint32), ref_l.view(np.uint32)), it
    finally:
        be.close()


@pytest.mark.gpu
def test_gpu_topk_back_to_back_calls_use_their_own_block_maxima():
    """The one-launch selection hands every block's best key to the workgroup that finishes last
    through device-scope atomics, in scratch memory that all calls share.  A call that picked up
    the previous call's keys would set its threshold from the wrong data: after the 'high' input
    the 'low' input would find nothing at or above it and return sentinels.  Many alternating calls,
    each checked, with lengths that move the block boundaries."""
    import torch
    from lattice_amd import backend
    be = backend.HipQ4Backend(0)
    g = np.random.default_rng(99)
    inputs = []
    for n, lo_, hi_ in [(248320, 0.0, 1.0), (248320, 100.0, 101.0), (151936, -50.0, -49.0), (200003, 7.0, 8.0)]:
        lg = g.uniform(lo_, hi_, size=n).astype(np.float32)
        inputs.append((torch.from_numpy(lg).cuda(), oracle.topk(lg, 50)))
    for r in range(150):
        outs = [be.topk(dev_lg, 50) for dev_lg, _ in inputs]  # queued back to back, checked afterwards
        for (out_l, out_i), (_, (want_l, want_i)) in zip(outs, inputs):
            assert np.array_equal(out_i.cpu().numpy().view(np.uint32), want_i), r
            assert np.array_equal(out_l.cpu().numpy().view(np.uint32), want_l.view(np.uint32)), r
