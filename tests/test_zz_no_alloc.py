"""The entry point that allocates nothing (`lq4_lm_head_topk_static`): same result as
`lq4_lm_head_topk`, bit for bit, on two calls in a row that share the library's static scratch
array, the second with a smaller input; shapes beyond the array are refused."""
import ctypes as C

import numpy as np
import pytest

from lattice_amd import synth


@pytest.mark.gpu
def test_static_scratch_lm_head_topk_matches_the_allocating_entry_point():
    import torch
    from lattice_amd import backend
    be = backend.HipQ4Backend(0)
    lib = be.lib
    stream = be._stream()

    def both(vocab, k, top_k, seed):
        wq = synth.q4_weight(vocab, k, seed=seed)
        qw = be.upload_q4_blocks(wq)
        x = torch.from_numpy(synth.activations(1, k, seed=seed)).cuda()
        outs = []
        for fn in (lib.lq4_lm_head_topk_static, lib.lq4_lm_head_topk):
            out_l = torch.full((top_k,), float("nan"), dtype=torch.float32, device="cuda")
            out_i = torch.full((top_k,), -7, dtype=torch.int32, device="cuda")
            rc = fn(be.ctx, qw.handle, 0, vocab, k, x.data_ptr(), top_k, out_l.data_ptr(), out_i.data_ptr(), stream)
            assert rc == 0, lib.lq4_last_error()
            be.synchronize()
            outs.append((out_l.cpu().numpy().view(np.uint32), out_i.cpu().numpy().view(np.uint32)))
        return outs

    # the larger input first, then a smaller one that finds the first call's logits and candidates
    # still in the array; a third, larger again
    for vocab, k, top_k, seed in [(40000, 1024, 50, 5), (9000, 512, 8, 6), (65536 + 3, 256, 200, 7),
                                  (50000, 2048, 50, 8), (7000, 2048, 8, 9)]:
        (got_l, got_i), (want_l, want_i) = both(vocab, k, top_k, seed)
        assert np.array_equal(got_i, want_i), (vocab, k, top_k)
        assert np.array_equal(got_l, want_l), (vocab, k, top_k)
        assert got_i.max() < vocab

    # beyond the static array: refused with a clear error, nothing launched
    big_vocab, k = 600000, 32
    raw = torch.zeros(big_vocab * 20, dtype=torch.uint8, device="cuda")
    qw = be.wrap_device_blocks(raw)
    x = torch.zeros(k, dtype=torch.float32, device="cuda")
    out_l = torch.zeros(4, dtype=torch.float32, device="cuda")
    out_i = torch.zeros(4, dtype=torch.int32, device="cuda")
    before = be.path_counters()
    rc = lib.lq4_lm_head_topk_static(be.ctx, qw.handle, 0, big_vocab, k, x.data_ptr(), 4, out_l.data_ptr(),
                                     out_i.data_ptr(), stream)
    assert rc == -5 and b"static" in lib.lq4_last_error()
    assert be.path_counters() == before
    be.close()


@pytest.mark.gpu
def test_static_scratch_at_its_largest_shapes_against_the_oracle():
    """The reference vocabulary (248 320 x 2048, top 50: the persistent-grid GEMV writing into the static
    array) and the largest promised shape (262 144 rows, top 256: the four-launch selection), each checked
    against the oracle's exact top-k of the same logits; then the refusal right above the array's capacity."""
    import torch
    import oracle
    from lattice_amd import backend
    from util import REL_TOL, rel_err
    be = backend.HipQ4Backend(0)
    lib = be.lib
    stream = be._stream()
    for vocab, k, top_k, seed in [(248320, 2048, 50, 11), (262144, 256, 256, 12)]:
        print(f"static lm_head top-k: vocab {vocab} k {k} top {top_k}", flush=True)
        wq = synth.q4_weight(vocab, k, seed=seed)
        qw = be.upload_q4_blocks(wq)
        x = synth.activations(1, k, seed=seed)
        xd = torch.from_numpy(x).cuda()
        y = torch.empty((1, vocab), dtype=torch.float32, device="cuda")
        be.gemv_batch(xd, qw, y, 1, vocab, k)
        logits = y.cpu().numpy()[0]
        assert rel_err(logits, oracle.gemm_f32(x, wq, vocab, k)[0]) <= REL_TOL
        want_l, want_i = oracle.topk(logits, top_k)
        for _ in range(2):  # the second call finds the first one's contents in the array
            out_l = torch.full((top_k,), float("nan"), dtype=torch.float32, device="cuda")
            out_i = torch.full((top_k,), -7, dtype=torch.int32, device="cuda")
            rc = lib.lq4_lm_head_topk_static(be.ctx, qw.handle, 0, vocab, k, xd.data_ptr(), top_k, out_l.data_ptr(),
                                             out_i.data_ptr(), stream)
            assert rc == 0, lib.lq4_last_error()
            be.synchronize()
            assert np.array_equal(out_i.cpu().numpy().view(np.uint32), want_i), (vocab, top_k)
            assert np.array_equal(out_l.cpu().numpy().view(np.uint32), want_l.view(np.uint32)), (vocab, top_k)
        del qw

    # the boundary: the largest vocabulary the array serves at top 256 is at least the promised 262 144, and one row
    # more than that largest one is refused with nothing launched
    k, top_k = 32, 256
    rows = 400000
    raw = torch.zeros(rows * 20, dtype=torch.uint8, device="cuda")
    qw = be.wrap_device_blocks(raw)
    x = torch.zeros(k, dtype=torch.float32, device="cuda")
    out_l = torch.zeros(top_k, dtype=torch.float32, device="cuda")
    out_i = torch.zeros(top_k, dtype=torch.int32, device="cuda")

    def served(vocab):
        rc = lib.lq4_lm_head_topk_static(be.ctx, qw.handle, 0, vocab, k, x.data_ptr(), top_k, out_l.data_ptr(),
                                         out_i.data_ptr(), stream)
        assert rc in (0, -5), lib.lq4_last_error()
        return rc == 0

    lo, hi = 262144, rows  # served(lo), not served(hi)
    assert served(lo) and not served(hi)
    while hi - lo > 1:
        mid = (lo + hi) // 2
        if served(mid):
            lo = mid
        else:
            hi = mid
    be.synchronize()
    before = be.path_counters()
    assert not served(lo + 1) and b"static" in lib.lq4_last_error()
    assert be.path_counters() == before
    be.close()
