"""GPU parity of lq4_gemv_multi (several projections of one x in one call), through the C ABI, against the CPU oracle
and against the same projections as separate lq4_gemv calls.

Bars: max|delta| / max|y_ref| <= 1e-3 against the f32-accumulated oracle (tests/util.py; achieved ~1e-6, printed);
without LoRA at batch 1 the stacked launch is bit-identical to the separate calls (same kernel, same summation).
The shapes are the reference's q/k/v run (inner/layers/gqa.rs:72-127: three projections and their LoRA deltas on one
input) and what the stacked launch branches on: rows of one, two and four slabs, rows side by side in a wave
(K 1024 and 512), views that are sub-ranges of one buffer, an empty view, and the fall-backs.
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
    b.set_gemv_kernel(backend.GEMV_KERNEL_LANE_BLOCKS)  # separate calls on the kernel the stacked launch uses
    yield b
    b.close()


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def _views(be, shapes, k, seed=0):
    ws = [synth.q4_weight(n, k, seed=seed + i, tag=f"view{i}", symmetric_bias=(i % 2 == 0)) for i, n in enumerate(shapes)]
    return ws, [be.upload_q4_blocks(w) for w in ws]


@pytest.mark.parametrize("shapes,k", [((2048, 512, 512), 2048),     # q, k, v of the 2B model
                                      ((4096, 512, 512), 2048),     # 2 * q_dim with the gate
                                      ((6144, 2048), 2048),         # qkv and z of a GDN layer
                                      ((512, 256, 256), 6144),      # three slabs a row
                                      ((96, 32, 7, 1), 8192),       # four slabs: two units a row; odd sizes
                                      ((1024, 256, 254), 1024),     # two rows side by side
                                      ((64, 8, 4, 4, 4, 4, 4, 4), 512),  # four rows side by side, eight views
                                      ((40000, 30000), 2048)])      # more rows than one chunk a wave covers
def test_multi_is_one_launch_and_equals_separate_calls(be, shapes, k):
    import torch
    print(f"multi shapes={shapes} k={k}", flush=True)
    ws, qs = _views(be, shapes, k)
    x = synth.activations(1, k, seed=3)
    xd = dev(x)
    ys = [torch.full((1, n), float("nan"), dtype=torch.float32, device="cuda") for n in shapes]
    c0 = be.path_counters()
    be.gemv_multi(xd, [(q, n, y) for q, n, y in zip(qs, shapes, ys)], 1, k)
    be.synchronize()
    c1 = be.path_counters()
    assert c1["gemv_multi"] == c0["gemv_multi"] + 1 and c1["gemv"] == c0["gemv"]
    for w, q, n, y in zip(ws, qs, shapes, ys):
        want = oracle.gemm_f32(x, w, n, k)[0]
        got = host(y)[0]
        assert rel_err(got, want) <= REL_TOL
        sep = torch.empty((1, n), dtype=torch.float32, device="cuda")
        be.gemv_batch(xd, q, sep, 1, n, k)
        assert np.array_equal(got.view(np.uint32), host(sep)[0].view(np.uint32)), n


def test_multi_views_inside_one_buffer_and_an_empty_view(be):
    # q, k, v stored one after the other in one upload, addressed by byte offsets; an empty projection in between
    import torch
    k = 2048
    shapes = (1024, 256, 256)
    ws = [synth.q4_weight(n, k, seed=10 + i) for i, n in enumerate(shapes)]
    merged = be.upload_q4_blocks(np.concatenate(ws))
    row_bytes = (k // 32) * 20
    offs = [0, shapes[0] * row_bytes, (shapes[0] + shapes[1]) * row_bytes]
    x = synth.activations(1, k, seed=4)
    ys = [torch.full((1, n), float("nan"), dtype=torch.float32, device="cuda") for n in shapes]
    empty = torch.empty((1, 0), dtype=torch.float32, device="cuda")
    be.gemv_multi(dev(x), [(merged, shapes[0], ys[0], None, offs[0]), (merged, 0, empty),
                           (merged, shapes[1], ys[1], None, offs[1]), (merged, shapes[2], ys[2], None, offs[2])], 1, k)
    be.synchronize()
    for w, n, y in zip(ws, shapes, ys):
        assert rel_err(host(y)[0], oracle.gemm_f32(x, w, n, k)[0]) <= REL_TOL


@pytest.mark.parametrize("batch", [1, 3, 12])
@pytest.mark.parametrize("f16", [True, False])
def test_multi_with_lora_on_q_and_v(be, batch, f16):
    # benchmark config 3's adapter (rank 16, scale 2.0) on q and v, k without: at batch 1 one launch in all
    import torch
    print(f"multi lora batch={batch} f16={f16}", flush=True)
    k = 2048
    names, shapes = ("q_proj", "k_proj", "v_proj"), (2048, 512, 512)
    ws, qs = _views(be, shapes, k, seed=20)
    dt = np.float16 if f16 else np.float32
    mods = {"q_proj": synth.lora_pair(16, k, 2048, seed=1, tag="q", dtype=dt),
            "v_proj": synth.lora_pair(8, k, 512, seed=2, tag="v", dtype=dt)}
    x = synth.activations(batch, k, seed=5)
    xd = dev(x)
    be.load_lora_adapter([backend.LoraLayerData(2, mods)], scale=2.0)
    try:
        ys = [torch.full((batch, n), float("nan"), dtype=torch.float32, device="cuda") for n in shapes]
        c0 = be.path_counters()
        be.gemv_multi(xd, [(q, n, y, nm) for q, n, y, nm in zip(qs, shapes, ys, names)], batch, k, layer_idx=2)
        be.synchronize()
        c1 = be.path_counters()
        if batch == 1:  # one launch in all: the A . x of both adapters inside the stacked launch
            assert c1["lora_a"] == c0["lora_a"] and c1["gemv_multi"] == c0["gemv_multi"] + 1
            assert c1["lora_t_fallback"] == c0["lora_t_fallback"], "the factors were handed over, not recomputed"
        elif batch <= 8:  # one launch over the stacked rows, every adapter's A . X in producer workgroups of it
            assert c1["lora_a"] == c0["lora_a"] and c1["gemv_multi"] == c0["gemv_multi"] + 1
            assert c1["lora_t_fallback"] <= c0["lora_t_fallback"] + 16
        else:             # projection by projection through the few-token GEMM, which computes A . X itself (ranks <= 16)
            assert c1["lora_a"] == c0["lora_a"] and c1["gemv_multi"] == c0["gemv_multi"]
        for w, q, n, y, nm in zip(ws, qs, shapes, ys, names):
            base = oracle.gemm_f32(x, w, n, k)
            want = base
            if nm in mods:
                a, b = mods[nm]
                want = oracle.lora_apply(a.astype(np.float32), b.astype(np.float32), 2.0, x, base)
            e = rel_err(host(y), want)
            print(f"  {nm}: rel err {e:.2e}", flush=True)
            assert e <= REL_TOL
            # the delta is resolved: against the same projection through lq4_gemv with its own adapter launch
            sep = torch.empty((batch, n), dtype=torch.float32, device="cuda")
            be.gemv_batch(xd, q, sep, batch, n, k, layer_idx=2, module=nm)
            # (2..8 rows: the stacked launch keeps 16 to 24 bits of an activation, the separate call with an
            # adapter rounds it to f16; one row and more than eight: the same kernels either way)
            assert rel_err(host(y), host(sep)) <= (REL_TOL if 2 <= batch <= 8 else 1e-5)
            if nm in mods:
                plain = torch.empty((batch, n), dtype=torch.float32, device="cuda")
                be.gemv_batch(xd, q, plain, batch, n, k)
                assert rel_err(host(y) - host(plain), want - base) <= 2e-3
    finally:
        be.unload_lora_adapter()


def test_multi_with_lora_ranks_beyond_one_wave_and_rows_side_by_side(be):
    # ranks 48 + 32 = 80 stacked rows of A: more than the 64 lanes that hold the factors, so A . x comes from a launch
    # of its own in front of the stacked one; K = 1024 puts two rows side by side (16 + 8 in the launch itself)
    import torch
    for k, shapes, ranks in ((2048, (256, 128), (48, 32)), (1024, (512, 64, 128), (16, 0, 8)), (512, (64, 64), (0, 4))):
        print(f"multi lora k={k} ranks={ranks}", flush=True)
        names = ("q_proj", "k_proj", "v_proj")[:len(shapes)]
        ws, qs = _views(be, shapes, k, seed=50)
        mods = {nm: synth.lora_pair(r, k, n, seed=3, tag=nm) for nm, n, r in zip(names, shapes, ranks) if r}
        x = synth.activations(1, k, seed=8)
        be.load_lora_adapter([backend.LoraLayerData(0, mods)], scale=1.5)
        try:
            ys = [torch.full((1, n), float("nan"), dtype=torch.float32, device="cuda") for n in shapes]
            c0 = be.path_counters()
            be.gemv_multi(dev(x), [(q, n, y, nm) for q, n, y, nm in zip(qs, shapes, ys, names)], 1, k, layer_idx=0)
            be.synchronize()
            c1 = be.path_counters()
            assert c1["gemv_multi"] == c0["gemv_multi"] + 1
            assert c1["lora_a"] == c0["lora_a"] + (1 if sum(ranks) > 64 else 0)
            for w, n, y, nm in zip(ws, shapes, ys, names):
                want = oracle.gemm_f32(x, w, n, k)
                if nm in mods:
                    a, b = mods[nm]
                    delta = oracle.lora_apply(a.astype(np.float32), b.astype(np.float32), 1.5, x, want) - want
                    plain = torch.empty((1, n), dtype=torch.float32, device="cuda")
                    be.gemv_batch(dev(x), qs[names.index(nm)], plain, 1, n, k)
                    assert rel_err(host(y) - host(plain), delta) <= 2e-3
                    want = want + delta
                assert rel_err(host(y), want) <= REL_TOL
        finally:
            be.unload_lora_adapter()


@pytest.mark.parametrize("batch", [2, 4, 5, 8])
def test_multi_rows_stacked_on_the_integer_kernel(be, batch):
    # 2..8 rows of q, k, v (views of whole 16-row tiles, K = 2048, 3072 rows in all): one launch; a view of 40 rows
    # (not a multiple of 16) sends the call projection by projection
    import torch
    k = 2048
    for shapes, one in (((2048, 512, 512), True), ((1024, 16, 160, 48), True), ((512, 40), False)):
        print(f"multi rows batch={batch} shapes={shapes}", flush=True)
        ws, qs = _views(be, shapes, k, seed=60)
        x = synth.activations(batch, k, seed=9)
        ys = [torch.full((batch, n), float("nan"), dtype=torch.float32, device="cuda") for n in shapes]
        c0 = be.path_counters()
        be.gemv_multi(dev(x), [(q, n, y) for q, n, y in zip(qs, shapes, ys)], batch, k)
        be.synchronize()
        c1 = be.path_counters()
        assert c1["gemv_multi"] == c0["gemv_multi"] + (1 if one else 0)
        for w, n, y in zip(ws, shapes, ys):
            e = rel_err(host(y), oracle.gemm_f32(x, w, n, k))
            assert e <= ((5e-6 if batch <= 4 else 1e-4) if one else REL_TOL), (n, e)


@pytest.mark.parametrize("batch", [40, 64, 128])
def test_multi_above_sixteen_rows_goes_through_the_gemm_routing(be, batch):
    # 17..128 rows: projection by projection as lq4_gemm would, the few-token GEMM's packed activations shared;
    # adapters of rank <= 16 up to 64 rows get their A . X inside that kernel, others a launch of their own.  The
    # wide projection in the middle (more than 2^26 weights) is served by the large-tile kernel, whose partial
    # tiles overwrite the packed activations: the projection behind it packs them again.
    import torch
    print(f"multi rows={batch}", flush=True)
    k = 2048
    names, shapes = ("q_proj", "up_proj", "v_proj", "k_proj"), (2048, 33000, 512, 512)
    ws, qs = _views(be, shapes, k, seed=50)
    mods = {"q_proj": synth.lora_pair(16, k, 2048, seed=1, tag="q"),
            "v_proj": synth.lora_pair(8, k, 512, seed=2, tag="v"),
            "k_proj": synth.lora_pair(24, k, 512, seed=3, tag="k")}
    x = synth.activations(batch, k, seed=9)
    xd = dev(x)
    be.load_lora_adapter([backend.LoraLayerData(1, mods)], scale=2.0)
    try:
        ys = [torch.full((batch, n), float("nan"), dtype=torch.float32, device="cuda") for n in shapes]
        c0 = be.path_counters()
        be.gemv_multi(xd, [(q, n, y, nm) for q, n, y, nm in zip(qs, shapes, ys, names)], batch, k, layer_idx=1)
        be.synchronize()
        c1 = be.path_counters()
        assert c1["gemm"] == c0["gemm"] + 4 and c1["gemv_multi"] == c0["gemv_multi"]
        # rank 24 always has its own A . X launch; above 64 rows also the 2048-row projection (its 32-token tiles
        # would be 512 workgroups), while the 512-row one keeps computing A . X in the kernel
        assert c1["lora_a"] == c0["lora_a"] + (1 if batch <= 64 else 2)
        for w, q, n, y, nm in zip(ws, qs, shapes, ys, names):
            base = oracle.gemm_f32(x, w, n, k)
            want = base
            if nm in mods:
                a, b = mods[nm]
                want = oracle.lora_apply(a.astype(np.float32), b.astype(np.float32), 2.0, x, base)
            e = rel_err(host(y), want)
            print(f"  {nm}: rel err {e:.2e}", flush=True)
            assert e <= REL_TOL
            sep = torch.empty((batch, n), dtype=torch.float32, device="cuda")
            be.dispatch_gemm(xd, 0, q, sep, 0, batch, n, k, layer_idx=1, module=nm)
            assert np.array_equal(host(y), host(sep)), "the same kernels as a single lq4_gemm call"
    finally:
        be.unload_lora_adapter()


def test_multi_fallbacks_keep_the_contract(be):
    # K 1024 with an odd-sized view (rows side by side would straddle two views), a single view, K beyond the LDS
    # staging: served projection by projection, same results
    import torch
    for shapes, k in (((300, 7, 64), 1024), ((777,), 2048), ((64, 32), 29152)):
        ws, qs = _views(be, shapes, k, seed=30)
        x = synth.activations(1, k, seed=6)
        ys = [torch.full((1, n), float("nan"), dtype=torch.float32, device="cuda") for n in shapes]
        c0 = be.path_counters()
        be.gemv_multi(dev(x), [(q, n, y) for q, n, y in zip(qs, shapes, ys)], 1, k)
        be.synchronize()
        c1 = be.path_counters()
        assert c1["gemv_multi"] == c0["gemv_multi"] and c1["gemv"] == c0["gemv"] + len(shapes)
        for w, n, y in zip(ws, shapes, ys):
            assert rel_err(host(y)[0], oracle.gemm_f32(x, w, n, k)[0]) <= REL_TOL


def test_multi_contract_errors_launch_nothing(be):
    import torch
    k = 256
    ws, qs = _views(be, (64, 64), k, seed=40)
    x = dev(synth.activations(1, k, seed=7))
    y0 = torch.full((1, 64), -3.0, dtype=torch.float32, device="cuda")
    small = torch.empty((1, 64), dtype=torch.float32, device="cuda")
    c0 = be.path_counters()
    with pytest.raises(ValueError):
        be.gemv_multi(x, [(qs[0], 64, y0)] * 9, 1, k)
    # the second projection asks for more rows than its buffer holds: the first one is not run either
    with pytest.raises(backend.Q4Error):
        be.gemv_multi(x, [(qs[0], 64, y0), (qs[1], 65, small)], 1, k)
    with pytest.raises(backend.Q4Error):
        be.gemv_multi(x, [(qs[0], 64, y0), (qs[1], 64, small)], 129, k)
    arr = (backend.Projection * 2)()
    arr[0].w, arr[0].n, arr[0].y_dev = qs[0].handle, 64, y0.data_ptr()
    arr[1].w, arr[1].n, arr[1].y_dev = qs[1].handle, 64, None
    assert be.lib.lq4_gemv_multi(be.ctx, arr, 2, k, x.data_ptr(), 1, None) != 0
    assert be.lib.lq4_gemv_multi(be.ctx, arr, 9, k, x.data_ptr(), 1, None) != 0
    assert be.lib.lq4_gemv_multi(be.ctx, None, 0, k, x.data_ptr(), 1, None) == 0  # nothing to do
    be.synchronize()
    c1 = be.path_counters()
    assert c1["gemv_multi"] == c0["gemv_multi"] and c1["gemv"] == c0["gemv"]
    assert np.all(host(y0) == -3.0)
