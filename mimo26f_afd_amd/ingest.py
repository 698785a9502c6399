"""Weight ingest: the repack manifest, slice identity, and a layer prepared from slice files.

Mirrors the reference's loader for the expert daemon:
  crates/mimo26-repack/src/manifest.rs:46-395  the sha manifest (pinned JSON form, strict parse,
                                               geometry and layout table checked against constants)
  crates/mimo26-repack/src/identity.rs:80-271  total readback of a slice directory, single-slice load
  crates/mimo26-repack/src/geom.rs:251-260     shard and slice file names
  crates/mimo26-spark/src/resident.rs:28-69    per-rank index; 256 quarter slices in expert-id order
Every rule is fail-loud: a manifest of another version, an unknown or missing field, a malformed
sha, a drifted geometry or layout row, a slice of the wrong size or hash refuses to load.

`load_layer` is this build's end of it: the verified slices of one layer go to the GPU (one rank's
256 images, or all four ranks for a full-intermediate layer) and are permuted once into the gfx950
operand order by the library (layout tag M26S_B1_LAYOUT_G950_V2).
"""
from __future__ import annotations

import hashlib
import json
import os
from dataclasses import dataclass, field

import numpy as np

from . import b1

FORMAT, VERSION = "mimo26-repack-manifest", 2
GENERATED_BY = "mimo26-repack 0.1.0"
HIDDEN, INTERMEDIATE, EXPERTS_PER_LAYER, MOE_LAYERS, EP_RANKS, FIRST_MOE_LAYER = 4096, 2048, 256, 47, 4, 1
EXPERT_BYTES, QUARTER_SLICE_BYTES = 13369344, 3342336
GEOMETRY = {"hidden": HIDDEN, "intermediate": INTERMEDIATE, "experts_per_layer": EXPERTS_PER_LAYER,
            "moe_layers": MOE_LAYERS, "ep_ranks": EP_RANKS, "expert_bytes": EXPERT_BYTES,
            "quarter_slice_bytes": QUARTER_SLICE_BYTES}
# (projection, region, offset, length) of the quarter-slice image v2 (crates/mimo26-expert/src/slice.rs:45-53)
LAYOUT = (("gate_proj", "payload", 0, 1048576), ("gate_proj", "scales", 1048576, 65536),
          ("up_proj", "payload", 1114112, 1048576), ("up_proj", "scales", 2162688, 65536),
          ("down_proj", "payload", 2228224, 1048576), ("down_proj", "scales", 3276800, 65536))
LAYOUT_TAG_G950_V2 = 0x47393502
_PROJ = (("gate_proj", 2048, 4096), ("up_proj", 2048, 4096), ("down_proj", 4096, 2048))  # name, out rows, in cols


class IngestError(RuntimeError):
    """A manifest or slice that must not be served; `kind` names the reference's error variant."""

    def __init__(self, kind: str, message: str):
        super().__init__(f"{kind}: {message}")
        self.kind = kind


def shard_file(expert: int) -> str:
    return f"model_pp0_ep{expert // 4}_shard0.safetensors"


def slice_file_name(layer: int, expert: int, rank: int) -> str:
    return f"L{layer:02d}_E{expert:03d}_R{rank}.slice"


def source_tensors(layer: int, expert: int) -> list[dict]:
    """The six checkpoint tensors a slice was cut from: (weight, weight_scale) of gate, up, down."""
    out = []
    for name, rows, cols in _PROJ:
        for scale in (False, True):
            out.append({"name": f"model.layers.{layer}.mlp.experts.{expert}.{name}.weight" + ("_scale" if scale else ""),
                        "shape": [rows, cols // 32 if scale else cols // 2], "dtype": "U8"})
    return out


@dataclass
class SliceEntry:
    file: str
    sha256: str
    bytes: int
    layer: int
    expert: int
    rank: int
    shard: str
    tensors: list

    @classmethod
    def of(cls, layer: int, expert: int, rank: int, data) -> "SliceEntry":
        data = memoryview(data)
        return cls(slice_file_name(layer, expert, rank), hashlib.sha256(data).hexdigest(), data.nbytes, layer, expert, rank,
                   shard_file(expert), source_tensors(layer, expert))


def _check_keys(obj, wanted, where: str, optional=()) -> None:
    if not isinstance(obj, dict):
        raise IngestError("BadManifest", f"{where} is not an object")
    for k in wanted:
        if k not in obj:
            raise IngestError("BadManifest", f"{where} missing {k}")
    for k in obj:
        if k not in wanted and k not in optional:
            raise IngestError("BadManifest", f"{where} has unknown field {k}")


def _no_duplicates(pairs):
    keys = [k for k, _ in pairs]
    if len(set(keys)) != len(keys):
        raise IngestError("BadManifest", "duplicate key in an object")
    return dict(pairs)


def _uint(v, where: str) -> int:
    if isinstance(v, bool) or not isinstance(v, int) or v < 0:
        raise IngestError("BadManifest", f"{where} is not an unsigned number")
    return v


@dataclass
class Manifest:
    format: str = FORMAT
    version: int = VERSION
    generated_by: str = GENERATED_BY
    geometry: dict = field(default_factory=lambda: dict(GEOMETRY))
    layout: list = field(default_factory=lambda: [dict(proj=p, region=r, off=o, len=n) for p, r, o, n in LAYOUT])
    slices: list = field(default_factory=list)

    def push(self, entry: SliceEntry) -> None:
        self.slices.append(entry)
        self.slices.sort(key=lambda e: e.file)

    def get(self, file: str):
        return next((s for s in self.slices if s.file == file), None)

    def to_json(self) -> str:
        """The pinned form: 2-space indent, one field per line, geometry keys sorted, layout and
        tensor rows on one line each (manifest.rs:163-236)."""
        q = json.dumps
        s = ["{", f'  "format": {q(self.format)},', f'  "version": {self.version},',
             f'  "generated_by": {q(self.generated_by)},', '  "geometry": {']
        keys = sorted(self.geometry)
        s += [f"    {q(k)}: {self.geometry[k]}" + ("" if i + 1 == len(keys) else ",") for i, k in enumerate(keys)]
        s += ["  },", '  "layout": [']
        s += [f'    {{"proj": {q(r["proj"])}, "region": {q(r["region"])}, "off": {r["off"]}, "len": {r["len"]}}}'
              + ("" if i + 1 == len(self.layout) else ",") for i, r in enumerate(self.layout)]
        s += ["  ],", '  "slices": [']
        for i, e in enumerate(self.slices):
            s += ["    {", f'      "file": {q(e.file)},', f'      "sha256": {q(e.sha256)},', f'      "bytes": {e.bytes},',
                  f'      "layer": {e.layer},', f'      "expert": {e.expert},', f'      "rank": {e.rank},',
                  '      "source": {', f'        "shard": {q(e.shard)},', '        "tensors": [']
            s += [f'          {{"name": {q(t["name"])}, "shape": [{", ".join(str(d) for d in t["shape"])}], "dtype": {q(t["dtype"])}}}'
                  + ("" if j + 1 == len(e.tensors) else ",") for j, t in enumerate(e.tensors)]
            s += ["        ]", "      }", "    }" + ("" if i + 1 == len(self.slices) else ",")]
        s += ["  ]", "}"]
        return "\n".join(s) + "\n"

    @classmethod
    def parse(cls, text: str) -> "Manifest":
        try:
            obj = json.loads(text, object_pairs_hook=_no_duplicates)
        except ValueError as e:
            raise IngestError("BadManifest", f"not JSON: {e}") from None
        _check_keys(obj, ("format", "version", "geometry", "layout", "slices"), "manifest", optional=("generated_by",))
        obj.setdefault("generated_by", "")
        if obj["format"] != FORMAT:
            raise IngestError("BadManifest", f"format {obj['format']!r} != {FORMAT!r}")
        if _uint(obj["version"], "version") != VERSION:
            raise IngestError("BadManifest", f"version {obj['version']} != {VERSION}; repack required")
        if not isinstance(obj["generated_by"], str) or not isinstance(obj["geometry"], dict) \
                or not isinstance(obj["layout"], list) or not isinstance(obj["slices"], list):
            raise IngestError("BadManifest", "a top-level field has the wrong type")
        geometry = {k: _uint(v, f"geometry.{k}") for k, v in obj["geometry"].items()}
        layout = []
        for row in obj["layout"]:
            _check_keys(row, ("proj", "region", "off", "len"), "layout row")
            layout.append(dict(proj=str(row["proj"]), region=str(row["region"]), off=_uint(row["off"], "layout off"),
                               len=_uint(row["len"], "layout len")))
        slices = []
        for e in obj["slices"]:
            _check_keys(e, ("file", "sha256", "bytes", "layer", "expert", "rank", "source"), "slice entry")
            sha = e["sha256"]
            if not isinstance(sha, str) or len(sha) != 64 or any(c not in "0123456789abcdef" for c in sha):
                raise IngestError("BadManifest", f"{e['file']}: bad sha256")
            _check_keys(e["source"], ("shard", "tensors"), f"{e['file']}: source")
            tensors = []
            for t in e["source"]["tensors"]:
                _check_keys(t, ("name", "shape", "dtype"), f"{e['file']}: tensor")
                tensors.append({"name": str(t["name"]), "shape": [_uint(d, "shape") for d in t["shape"]], "dtype": str(t["dtype"])})
            slices.append(SliceEntry(str(e["file"]), sha, _uint(e["bytes"], "bytes"), _uint(e["layer"], "layer"),
                                     _uint(e["expert"], "expert"), _uint(e["rank"], "rank"), str(e["source"]["shard"]), tensors))
        m = cls(obj["format"], obj["version"], obj["generated_by"], geometry, layout, slices)
        m.validate_geometry()
        return m

    @classmethod
    def read(cls, path: str) -> "Manifest":
        with open(path, "r", encoding="utf-8") as f:
            return cls.parse(f.read())

    def write(self, path: str) -> None:
        with open(path, "w", encoding="utf-8") as f:
            f.write(self.to_json())

    def validate_geometry(self) -> None:
        if self.format != FORMAT or self.version != VERSION:
            raise IngestError("BadManifest", f"layout version {self.version} / format {self.format!r} is not v{VERSION} / {FORMAT}; repack required")
        for k, want in GEOMETRY.items():
            if k not in self.geometry:
                raise IngestError("BadManifest", f"geometry missing {k}")
            if self.geometry[k] != want:
                raise IngestError("GeometryMismatch", f"{k}: want {want}, got {self.geometry[k]}")
        if len(self.layout) != len(LAYOUT):
            raise IngestError("BadManifest", f"layout has {len(self.layout)} rows, expected {len(LAYOUT)}")
        for got, (p, r, o, n) in zip(self.layout, LAYOUT):
            if (got["proj"], got["region"], got["off"], got["len"]) != (p, r, o, n):
                raise IngestError("BadManifest", f"layout row drift: got {got['proj']} {got['region']} @{got['off']} +{got['len']}, "
                                                 f"expected {p} {r} @{o} +{n}")


def manifest_path(directory: str) -> str:
    return os.path.join(directory, "manifest.json")


def _check_identity(entry: SliceEntry) -> None:
    """The entry's name, size, shard and tensors must be the ones its (layer, expert, rank) implies."""
    if not FIRST_MOE_LAYER <= entry.layer < FIRST_MOE_LAYER + MOE_LAYERS:
        raise IngestError("BadGeometry", f"layer {entry.layer}: MoE layer must be 1..=47 (layer 0 is dense)")
    if entry.expert >= EXPERTS_PER_LAYER:
        raise IngestError("BadGeometry", f"expert {entry.expert}: expert id must be 0..256")
    if entry.rank >= EP_RANKS:
        raise IngestError("BadGeometry", f"rank {entry.rank}: EP rank must be 0..4")
    if entry.file != slice_file_name(entry.layer, entry.expert, entry.rank) or entry.bytes != QUARTER_SLICE_BYTES \
            or entry.shard != shard_file(entry.expert) or entry.tensors != source_tensors(entry.layer, entry.expert):
        raise IngestError("BadManifest", f"{entry.file}: slice identity mismatch")


def verify_bytes(data, entry: SliceEntry) -> tuple[str, str]:
    """('Match' | 'SizeMismatch' | 'ShaMismatch', detail) for bytes claimed to be `entry`."""
    n = memoryview(data).nbytes
    if n != QUARTER_SLICE_BYTES:
        return "SizeMismatch", f"{entry.file}: want {QUARTER_SLICE_BYTES} bytes, got {n}"
    got = hashlib.sha256(data).hexdigest()
    if got != entry.sha256:
        return "ShaMismatch", f"{entry.file}: want {entry.sha256}, got {got}"
    return "Match", entry.file


@dataclass
class ReadbackReport:
    files: list  # (file, status, detail), sorted by file; status as in verify_bytes plus Missing / Unlisted
    matched_bytes: int

    def all_match(self) -> bool:
        return all(s == "Match" for _, s, _ in self.files)

    def summary(self) -> str:
        ok = sum(s == "Match" for _, s, _ in self.files)
        return f"identity readback: {ok}/{len(self.files)} slices match ({self.matched_bytes} B), {len(self.files) - ok} failed"

    def raise_on_failure(self) -> "ReadbackReport":
        for _, status, detail in self.files:
            if status != "Match":
                raise IngestError({"Missing": "MissingSlice", "Unlisted": "UnlistedSlice", "SizeMismatch": "SliceSize"}.get(status, status), detail)
        return self


def verify_dir(directory: str, manifest: Manifest) -> ReadbackReport:
    """Checks every listed slice and every resident *.slice file and reports all of them."""
    manifest.validate_geometry()
    files, matched = [], 0
    for entry in manifest.slices:
        path = os.path.join(directory, entry.file)
        if not os.path.isfile(path):
            files.append((entry.file, "Missing", entry.file))
            continue
        size = os.path.getsize(path)
        if size != QUARTER_SLICE_BYTES:
            files.append((entry.file, "SizeMismatch", f"{entry.file}: want {QUARTER_SLICE_BYTES} bytes, got {size}"))
            continue
        status, detail = verify_bytes(np.fromfile(path, np.uint8), entry)
        matched += size if status == "Match" else 0
        files.append((entry.file, status, detail))
    listed = {e.file for e in manifest.slices}
    for name in sorted(os.listdir(directory)):
        if name.endswith(".slice") and name not in listed:
            files.append((name, "Unlisted", name))
    files.sort(key=lambda f: f[0])
    return ReadbackReport(files, matched)


def load_slice(directory: str, manifest: Manifest, file: str) -> np.ndarray:
    """The verified bytes of one slice; any doubt about its identity or contents raises."""
    manifest.validate_geometry()
    entries = [s for s in manifest.slices if s.file == file]
    if len(entries) != 1:
        raise IngestError("BadManifest", f"{file}: expected exactly one manifest entry")
    _check_identity(entries[0])
    path = os.path.join(directory, file)
    if not os.path.isfile(path):
        raise IngestError("MissingSlice", file)
    data = np.fromfile(path, np.uint8)
    status, detail = verify_bytes(data, entries[0])
    if status != "Match":
        raise IngestError("SliceSize" if status == "SizeMismatch" else status, detail)
    return data


class Resident:
    """One rank's slice files of a directory, indexed by (layer, expert) (resident.rs:28-69)."""

    def __init__(self, directory: str, rank: int):
        self.dir, self.rank = directory, rank
        self.manifest = Manifest.read(manifest_path(directory))
        self.files = {(e.layer, e.expert): e.file for e in self.manifest.slices if e.rank == rank}

    def slice(self, layer: int, expert: int) -> np.ndarray:
        file = self.files.get((layer, expert))
        if file is None:
            raise IngestError("MissingSlice", f"L{layer:02d}_E{expert:03d}")
        return load_slice(self.dir, self.manifest, file)

    def grouped_image(self, layer: int, experts: int = EXPERTS_PER_LAYER, out: np.ndarray | None = None) -> np.ndarray:
        """The layer's quarter slices back to back in expert-id order (expert id == slot)."""
        image = np.empty(experts * QUARTER_SLICE_BYTES, np.uint8) if out is None else out
        for e in range(experts):
            image[e * QUARTER_SLICE_BYTES:(e + 1) * QUARTER_SLICE_BYTES] = self.slice(layer, e)
        return image


def load_layer(directory: str, layer: int, rank: int | None = 0) -> b1.Layer:
    """One layer from verified slice files, prepared on the GPU in the gfx950 operand order:
    `rank` = 0..3 for that TP4 rank's share (intermediate 512), None for all four ranks fused
    (intermediate 2048). The canonical bytes are dropped once the layer holds its prepared pool."""
    ranks = range(EP_RANKS) if rank is None else (rank,)
    pools = []
    try:
        for r in ranks:
            host = Resident(directory, r).grouped_image(layer)
            pools.append(b1.DeviceBuffer.from_host(host))
            del host
        if rank is None:
            made = b1.Layer.full([p.ptr for p in pools], pools[0].nbytes)
        else:
            made = b1.Layer(pools[0].ptr, pools[0].nbytes, rank)
    finally:
        for p in pools:
            p.free()
    if made.prepared_view()[2] != LAYOUT_TAG_G950_V2:
        raise IngestError("BadLayout", "the library prepared a layout this loader does not know")
    return made
