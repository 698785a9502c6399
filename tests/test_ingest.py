"""Weight ingest: the manifest's pinned form and fail-loud rules, slice identity readback, and (GPU)
a layer prepared from slice files. The cases follow the reference's own tests
(crates/mimo26-repack/tests/manifest.rs, identity_readback.rs)."""
import hashlib
import os

import numpy as np
import pytest

from mimo26f_afd_amd import ingest as G
from mimo26f_afd_amd import synth


def entry(layer, expert, rank, data):
    return G.SliceEntry.of(layer, expert, rank, data)


def test_manifest_pinned_form_and_round_trip():
    m = G.Manifest()
    data = np.full(G.QUARTER_SLICE_BYTES, 7, np.uint8)
    m.push(entry(1, 0, 1, data))
    m.push(entry(1, 0, 0, data))
    text = m.to_json()
    assert text.endswith("}\n") and text == m.to_json()
    lines = text.split("\n")
    assert lines[:5] == ["{", '  "format": "mimo26-repack-manifest",', '  "version": 2,',
                         '  "generated_by": "mimo26-repack 0.1.0",', '  "geometry": {']
    # geometry keys sorted, one per line; the numbers the reference's test names
    assert lines[5:12] == ['    "ep_ranks": 4,', '    "expert_bytes": 13369344,', '    "experts_per_layer": 256,', '    "hidden": 4096,',
                           '    "intermediate": 2048,', '    "moe_layers": 47,', '    "quarter_slice_bytes": 3342336']
    assert '    {"proj": "gate_proj", "region": "payload", "off": 0, "len": 1048576},' in lines
    assert '    {"proj": "down_proj", "region": "scales", "off": 3276800, "len": 65536}' in lines
    assert '          {"name": "model.layers.1.mlp.experts.0.down_proj.weight_scale", "shape": [4096, 64], "dtype": "U8"}' in lines
    back = G.Manifest.parse(text)
    assert back == m and [s.file for s in back.slices] == ["L01_E000_R0.slice", "L01_E000_R1.slice"]
    assert back.get("L01_E000_R1.slice") is not None and back.get("nope.slice") is None
    assert back.slices[0].sha256 == hashlib.sha256(data.tobytes()).hexdigest()


def test_source_tensors_and_names():
    t = G.source_tensors(1, 0)
    assert [x["name"] for x in t] == [f"model.layers.1.mlp.experts.0.{p}_proj.weight{s}" for p in ("gate", "up", "down") for s in ("", "_scale")]
    assert [x["shape"] for x in t] == [[2048, 2048], [2048, 128], [2048, 2048], [2048, 128], [4096, 1024], [4096, 64]]
    assert all(x["dtype"] == "U8" for x in t)
    assert G.shard_file(9) == "model_pp0_ep2_shard0.safetensors" and G.slice_file_name(2, 4, 3) == "L02_E004_R3.slice"


@pytest.mark.parametrize("old,new,kind,what", [
    ('"moe_layers": 47', '"moe_layers": 48', "GeometryMismatch", "moe_layers"),
    ('"quarter_slice_bytes": 3342336', '"quarter_slice_bytes": 3342337', "GeometryMismatch", "quarter_slice_bytes"),
    ('"off": 1048576, "len": 65536', '"off": 1048577, "len": 65536', "BadManifest", "layout row drift"),
    ("mimo26-repack-manifest", "something-else", "BadManifest", "format"),
    ('"version": 2', '"version": 1', "BadManifest", "version"),
    ('  "slices": [\n  ]\n', "", "BadManifest", ""),
    ('  "version": 2,', '  "version": 2,\n  "version": 2,', "BadManifest", "duplicate"),
    ('"hidden": 4096,', '"hidden": 4096, "extra": 1,', None, ""),  # extra geometry numbers are carried, not refused
])
def test_manifest_fail_loud_rules(old, new, kind, what):
    text = G.Manifest().to_json()
    assert old in text
    bad = text.replace(old, new)
    if kind is None:
        G.Manifest.parse(bad)
        return
    with pytest.raises((G.IngestError, ValueError)) as e:
        G.Manifest.parse(bad)
    if isinstance(e.value, G.IngestError):
        assert e.value.kind == kind and what in str(e.value)


def test_manifest_rejects_bad_sha_trailing_bytes_and_unknown_fields():
    m = G.Manifest()
    data = np.zeros(G.QUARTER_SLICE_BYTES, np.uint8)
    m.push(entry(1, 0, 0, data))
    text, sha = m.to_json(), m.slices[0].sha256
    for bad in ("z" * 64, "a" * 63, sha.upper()):
        with pytest.raises(G.IngestError, match="bad sha256"):
            G.Manifest.parse(text.replace(sha, bad))
    with pytest.raises(G.IngestError):
        G.Manifest.parse(text + "garbage")
    with pytest.raises(G.IngestError, match="unknown field"):
        G.Manifest.parse(text.replace('"bytes": 3342336,', '"bytes": 3342336,\n      "note": 1,'))
    with pytest.raises(G.IngestError, match="missing rank"):
        G.Manifest.parse(text.replace('      "rank": 0,\n', ""))


def make_dir(tmp_path, slices):
    """A slice directory with its manifest; slices = {(layer, expert, rank): bytes}."""
    m = G.Manifest()
    for (l, e, r), data in slices.items():
        data.tofile(os.path.join(tmp_path, G.slice_file_name(l, e, r)))
        m.push(entry(l, e, r, data))
    m.write(G.manifest_path(tmp_path))
    return m


def test_identity_readback_names_every_bad_slice(tmp_path):
    rng = np.random.default_rng(1)
    slices = {(1, e, 0): rng.integers(0, 256, G.QUARTER_SLICE_BYTES, dtype=np.uint8) for e in range(4)}
    m = make_dir(tmp_path, slices)
    rep = G.verify_dir(str(tmp_path), m)
    assert rep.all_match() and rep.matched_bytes == 4 * G.QUARTER_SLICE_BYTES
    assert rep.summary() == f"identity readback: 4/4 slices match ({4 * G.QUARTER_SLICE_BYTES} B), 0 failed"
    rep.raise_on_failure()
    # one flipped bit, one truncated, one missing, one unlisted: all four reported, the first raised
    flipped = slices[(1, 0, 0)].copy()
    flipped[12345] ^= 1
    flipped.tofile(tmp_path / G.slice_file_name(1, 0, 0))
    slices[(1, 1, 0)][:-1].tofile(tmp_path / G.slice_file_name(1, 1, 0))
    os.remove(tmp_path / G.slice_file_name(1, 2, 0))
    slices[(1, 3, 0)].tofile(tmp_path / "L09_E009_R0.slice")
    rep = G.verify_dir(str(tmp_path), m)
    assert [(f, s) for f, s, _ in rep.files] == [("L01_E000_R0.slice", "ShaMismatch"), ("L01_E001_R0.slice", "SizeMismatch"),
                                                 ("L01_E002_R0.slice", "Missing"), ("L01_E003_R0.slice", "Match"),
                                                 ("L09_E009_R0.slice", "Unlisted")]
    assert not rep.all_match() and rep.matched_bytes == G.QUARTER_SLICE_BYTES
    with pytest.raises(G.IngestError) as e:
        rep.raise_on_failure()
    assert e.value.kind == "ShaMismatch"
    for file, kind in (("L01_E000_R0.slice", "ShaMismatch"), ("L01_E001_R0.slice", "SliceSize"), ("L01_E002_R0.slice", "MissingSlice"),
                       ("L09_E009_R0.slice", "BadManifest")):
        with pytest.raises(G.IngestError) as e:
            G.load_slice(str(tmp_path), m, file)
        assert e.value.kind == kind, file
    assert np.array_equal(G.load_slice(str(tmp_path), m, "L01_E003_R0.slice"), slices[(1, 3, 0)])


def test_slice_identity_must_follow_from_its_coordinates(tmp_path):
    data = np.zeros(G.QUARTER_SLICE_BYTES, np.uint8)
    m = make_dir(tmp_path, {(1, 0, 0): data})
    for field, value, kind in (("shard", "model_pp0_ep1_shard0.safetensors", "BadManifest"), ("layer", 0, "BadGeometry"),
                               ("layer", 48, "BadGeometry"), ("expert", 256, "BadGeometry"), ("rank", 4, "BadGeometry"),
                               ("expert", 1, "BadManifest")):
        bad = G.Manifest.parse(m.to_json())
        setattr(bad.slices[0], field, value)
        with pytest.raises(G.IngestError) as e:
            G.load_slice(str(tmp_path), bad, "L01_E000_R0.slice")
        assert e.value.kind == kind, (field, value)
    res = G.Resident(str(tmp_path), 0)
    assert np.array_equal(res.slice(1, 0), data)
    with pytest.raises(G.IngestError, match="MissingSlice"):
        res.slice(1, 1)
    assert G.Resident(str(tmp_path), 1).files == {}


@pytest.mark.gpu
def test_layer_from_slice_files_equals_layer_from_pool(tmp_path):
    """256 slice files of one rank -> verified -> prepared on the GPU: the same prepared pool, tag
    and FFN output bits as the layer built from the in-memory pool; a corrupted slice refuses."""
    import b1_oracle as O
    from helpers import DeviceLayer, run_ffn_dev
    from mimo26f_afd_amd import b1
    wl = synth.make(1)
    pool = wl.pools(wl.touched())[0]
    images = {(3, e, 0): pool[e * synth.IMAGE_BYTES:(e + 1) * synth.IMAGE_BYTES] for e in range(256)}
    make_dir(tmp_path, images)
    layer = G.load_layer(str(tmp_path), 3, rank=0)
    ptr, image_bytes, tag = layer.prepared_view()
    assert tag == G.LAYOUT_TAG_G950_V2 and image_bytes == synth.IMAGE_BYTES and layer.all_scales_normal()
    e = int(wl.ids[0, 0])
    got = np.empty(image_bytes, np.uint8)
    assert b1.load().m26s_b1_copy_to_host(got.ctypes.data, ptr + e * image_bytes, image_bytes) == 0
    assert np.array_equal(got, O.prepared_g950([images[(3, e, 0)]]))
    scratch = b1.Scratch()
    _, bf, _ = run_ffn_dev(layer, scratch, wl)
    _, want, _ = run_ffn_dev(DeviceLayer([pool]).layer, scratch, wl)
    assert np.array_equal(bf, want)
    bad = images[(3, e, 0)].copy()
    bad[100] ^= 0x10
    bad.tofile(tmp_path / G.slice_file_name(3, e, 0))
    with pytest.raises(G.IngestError, match="ShaMismatch"):
        G.load_layer(str(tmp_path), 3, rank=0)
