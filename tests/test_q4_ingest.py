"""`.q4` checkpoint ingest: quantize_index.json reader, file merge, directory loader.

The manifest cases restate the reference's own unit tests
(crates/inference/src/quant/q4_manifest.rs:290-499); the merge cases follow write_merged_qkvz
(crates/inference/src/weights/q4_weights.rs:1552-1636).  The GPU test loads a directory written
with the oracle's quantizer and checks GEMVs on the uploaded tensors against the oracle.
"""
import json
import os

import numpy as np
import pytest

import oracle
from lattice_amd import q4_dir, q4_file, q4_manifest, synth
from util import REL_TOL, rel_err


def _write(tmp_path, text):
    p = tmp_path / "quantize_index.json"
    p.write_text(text)
    return str(tmp_path)


# ------------------------------------------------------------------------- manifest
def test_manifest_absent_file_is_none(tmp_path):
    assert q4_manifest.load_manifest(str(tmp_path)) is None


def test_manifest_bare_array_is_quantize_q4_flavor(tmp_path):
    d = _write(tmp_path, '[{"name":"foo","file":"foo.q4","quantized":true,"shape":[2,2],"numel":4}]')
    m = q4_manifest.load_manifest(d)
    assert m.flavor == q4_manifest.FLAVOR_QUANTIZE_Q4 and m.quarot_seed is None
    assert len(m.tensors) == 1 and m.tensors[0].name == "foo" and m.tensors[0].shape == [2, 2]


def test_manifest_object_form_is_quarot_flavor_with_seed(tmp_path):
    d = _write(tmp_path, '{"quarot_seed":42,"tensors":[{"name":"foo","file":"foo.q4","quantized":true,'
                         '"shape":[2],"numel":2}]}')
    m = q4_manifest.load_manifest(d)
    assert m.flavor == q4_manifest.FLAVOR_QUAROT and m.quarot_seed == 42 and len(m.tensors) == 1


def test_manifest_object_form_without_seed(tmp_path):
    m = q4_manifest.load_manifest(_write(tmp_path, '{"tensors":[]}'))
    assert m.quarot_seed is None and m.tensors == []


def test_manifest_tolerates_minimal_entries(tmp_path):
    m = q4_manifest.parse_manifest(b'[{"name":"foo","file":"foo.q4"}]')
    assert m.tensors[0].quantized is None
    m = q4_manifest.parse_manifest(b'{"quarot_seed":42,"tensors":[{"name":"foo","file":"foo.q4"}]}')
    assert m.tensors[0].shape is None and m.tensors[0].numel is None


def test_manifest_malformed_bare_array_names_the_missing_field():
    with pytest.raises(q4_manifest.InvalidShape) as e:
        q4_manifest.parse_manifest(b'[{"name": "x"}]')
    assert "file" in str(e.value) and "did not match any variant" not in str(e.value)


def test_manifest_malformed_object_names_tensors():
    with pytest.raises(q4_manifest.InvalidShape) as e:
        q4_manifest.parse_manifest(b'{"quarot_seed": 42, "tensors": "not-an-array"}')
    assert "tensors" in str(e.value) or "sequence" in str(e.value)


def test_manifest_scalar_root_explains_both_shapes():
    with pytest.raises(q4_manifest.InvalidShape) as e:
        q4_manifest.parse_manifest(b'"just a string"')
    assert "either a bare array" in str(e.value) and "tensors" in str(e.value)


def test_manifest_oversized_file_is_rejected(tmp_path):
    p = tmp_path / "quantize_index.json"
    with open(p, "wb") as f:
        f.truncate(q4_manifest.MAX_QUANTIZE_INDEX_LEN + 1)  # sparse: no real bytes on disk
    with pytest.raises(q4_manifest.TooLarge) as e:
        q4_manifest.read_manifest_bytes_bounded(str(p))
    assert "too large" in str(e.value)


def test_manifest_truncated_json_is_invalid_json(tmp_path):
    d = _write(tmp_path, '{"quarot_seed":42,"tensors":[{"name":"foo","file":"foo.q4","quant')
    with pytest.raises(q4_manifest.InvalidJson):
        q4_manifest.load_manifest(d)


def test_manifest_dangling_symlink_fails_closed(tmp_path):
    link = tmp_path / "quantize_index.json"
    os.symlink(str(tmp_path / "does-not-exist"), str(link))
    with pytest.raises(q4_manifest.Unreadable):
        q4_manifest.read_manifest_bytes_bounded(str(link))
    with pytest.raises(q4_manifest.Unreadable):
        q4_manifest.load_manifest(str(tmp_path))


# ---------------------------------------------------------------------------- merge
def _tensor(n, k, seed):
    g = np.random.default_rng(seed)
    w = (g.normal(0, 0.02, size=(n, k))).astype(np.float32)
    return w, oracle.quantize_rows(w)


def test_write_and_merge_q4_files(tmp_path):
    wa, qa = _tensor(6, 64, 1)
    wb, qb = _tensor(3, 64, 2)
    pa, pb, po = (str(tmp_path / f) for f in ("qkv.q4", "z.q4", "merged.q4"))
    q4_file.write_q4_file(pa, (6, 64), qa)
    q4_file.write_q4_file(pb, (3, 64), qb)
    assert not os.path.exists(pa + ".tmp")
    h = q4_file.merge_q4_files(pa, pb, po)
    assert h.shape == (9, 64) and h.original_len == 9 * 64
    data = np.fromfile(po, dtype=np.uint8)
    hv = q4_file.validate_q4_file(data, po, (9, 64))
    assert hv.payload_offset == 36
    assert np.array_equal(data[36:], np.concatenate([qa, qb]))
    # the reference's own parser agrees on the merged header
    shape, olen, off = oracle.parse_q4_file(data)[:3]
    assert tuple(shape) == (9, 64) and olen == 576 and off == 36


def test_merge_rejects_bad_inputs(tmp_path):
    _, qa = _tensor(4, 64, 1)
    _, qb = _tensor(4, 32, 2)
    pa, pb = str(tmp_path / "a.q4"), str(tmp_path / "b.q4")
    q4_file.write_q4_file(pa, (4, 64), qa)
    q4_file.write_q4_file(pb, (4, 32), qb)
    with pytest.raises(q4_file.Q4FileError, match="hidden dimension"):
        q4_file.merge_q4_files(pa, pb, str(tmp_path / "o.q4"))
    # a rank-0 header must be rejected, not indexed (q4_weights.rs:1568-1585)
    p0 = str(tmp_path / "rank0.q4")
    with open(p0, "wb") as f:
        f.write(q4_file.q4_file_bytes((), 1, oracle.quantize_flat(np.ones(1, np.float32))))
    with pytest.raises(q4_file.Q4FileError, match="not 2-D"):
        q4_file.merge_q4_files(p0, pa, str(tmp_path / "o.q4"))
    assert not os.path.exists(str(tmp_path / "o.q4"))


# ------------------------------------------------------------------ directory loader
class _RecordingBackend:
    """Stands in for HipQ4Backend where no GPU is needed: records what would be uploaded."""

    def __init__(self):
        self.calls = []

    def mmap_q4_weight(self, path, label, expected_shape):
        data = np.fromfile(path, dtype=np.uint8)
        h = q4_file.validate_q4_file(data, path, expected_shape)
        self.calls.append(("mmap", label, h.payload_offset, len(data)))
        return ("buf", label)

    def upload_q4_blocks(self, blocks, payload_offset=0, validate=True):
        self.calls.append(("upload", len(blocks), payload_offset))
        return ("buf", len(blocks))


def _checkpoint(tmp_path, with_manifest):
    names = {"model.layers.0.mlp.gate_proj.weight": (8, 64), "model.layers.0.mlp.up_proj.weight": (8, 64),
             "model.layers.0.self_attn.q_proj.weight": (12, 64)}
    entries, payloads = [], {}
    for i, (nm, shp) in enumerate(names.items()):
        w, q = _tensor(shp[0], shp[1], 10 + i)
        path = q4_file.q4_tensor_path(str(tmp_path), nm)
        q4_file.write_q4_file(path, shp, q)
        payloads[nm] = (w, q)
        entries.append({"name": nm, "file": os.path.basename(path), "quantized": True, "shape": list(shp),
                        "numel": shp[0] * shp[1]})
    entries.append({"name": "model.norm.weight", "file": "model_norm_weight.f16", "quantized": False,
                    "shape": [64], "numel": 64})
    if with_manifest:
        (tmp_path / "quantize_index.json").write_text(json.dumps(entries))
    return names, payloads


@pytest.mark.parametrize("with_manifest", [True, False])
def test_checkpoint_inventory_and_load(tmp_path, with_manifest):
    names, _ = _checkpoint(tmp_path, with_manifest)
    be = _RecordingBackend()
    ck = q4_dir.Q4Checkpoint(be, str(tmp_path))
    inv = ck.inventory()
    assert len(inv) == 3
    if with_manifest:
        assert set(inv) == set(names)  # the f16 entry is skipped
    else:
        assert "model_layers_0_mlp_gate_proj_weight" in inv  # directory scan: file stems
    name = next(iter(names))
    t = ck.load(name, names[name])
    assert t.shape == names[name] and be.calls[-1][0] == "mmap" and be.calls[-1][2] == 36
    with pytest.raises(q4_file.Q4FileError):
        ck.load("model.layers.0.self_attn.q_proj.weight", (13, 64))  # shape preflight
    fused = ck.load_fused("model.layers.0.mlp.gate_proj.weight", "model.layers.0.mlp.up_proj.weight", "gate_up")
    assert fused.shape == (16, 64) and be.calls[-1] == ("upload", 16 * 2 * 20, 0)


def test_checkpoint_rejects_manifest_paths_outside_the_directory(tmp_path):
    (tmp_path / "quantize_index.json").write_text('[{"name":"x","file":"../x.q4","quantized":true}]')
    with pytest.raises(q4_manifest.InvalidShape):
        q4_dir.Q4Checkpoint(_RecordingBackend(), str(tmp_path)).inventory()


@pytest.mark.gpu
def test_checkpoint_directory_to_gpu_gemv(tmp_path):
    import torch
    from lattice_amd import backend
    names, payloads = _checkpoint(tmp_path, True)
    be = backend.HipQ4Backend(0)
    ck = q4_dir.Q4Checkpoint(be, str(tmp_path))
    ck.load_all()
    x = synth.activations(1, 64, seed=3)
    xd = torch.from_numpy(x).cuda()
    for nm, (n, k) in names.items():
        y = torch.empty((1, n), dtype=torch.float32, device="cuda")
        be.dispatch_matmul(xd, ck.tensors[nm].buf, y, 1, n, k)
        assert rel_err(y.cpu().numpy(), oracle.gemm_f32(x, payloads[nm][1], n, k)) <= REL_TOL
    g, u = "model.layers.0.mlp.gate_proj.weight", "model.layers.0.mlp.up_proj.weight"
    fused = ck.load_fused(g, u, "gate_up")
    y = torch.empty((1, 16), dtype=torch.float32, device="cuda")
    be.dispatch_matmul(xd, fused.buf, y, 1, 16, 64)
    ref = np.concatenate([oracle.gemm_f32(x, payloads[g][1], 8, 64), oracle.gemm_f32(x, payloads[u][1], 8, 64)], axis=1)
    assert rel_err(y.cpu().numpy(), ref) <= REL_TOL
    # second half through the byte offset, as the reference addresses `up` inside the fused buffer
    y2 = torch.empty((1, 8), dtype=torch.float32, device="cuda")
    be.dispatch_gemm_at(xd, 0, fused.buf, 8 * 2 * 20, y2, 0, 1, 8, 64)
    assert rel_err(y2.cpu().numpy(), oracle.gemm_f32(x, payloads[u][1], 8, 64)) <= REL_TOL
