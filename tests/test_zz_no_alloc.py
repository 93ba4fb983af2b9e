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
    # (the 2048-wide ones are served by the one-launch form when that mode is on: run in both modes)
    try:
        for mode in (backend.LM_HEAD_TWO_LAUNCHES, backend.LM_HEAD_ONE_LAUNCH):
            be.set_lm_head_mode(mode)
            for vocab, k, top_k, seed in [(40000, 1024, 50, 5), (9000, 512, 8, 6), (65536 + 3, 256, 200, 7),
                                          (50000, 2048, 50, 8), (7000, 2048, 8, 9)]:
                (got_l, got_i), (want_l, want_i) = both(vocab, k, top_k, seed)
                assert np.array_equal(got_i, want_i), (mode, vocab, k, top_k)
                assert np.array_equal(got_l, want_l), (mode, vocab, k, top_k)
                assert got_i.max() < vocab
    finally:
        be.set_lm_head_mode(backend.LM_HEAD_TWO_LAUNCHES)

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
