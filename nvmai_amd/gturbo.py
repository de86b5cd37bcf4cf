"""The `.gturbo` model directory of the reference, read into HBM: `manifest.json`, the resident
index and tensors of `model_weights.bin`, `packed_experts/layout.json` and the per-layer expert
files.  Host-side format logic (no GPU needed to parse or validate); `GTurboModel.expert_pool` and
`GTurboModel.moe_layer` put one layer's experts where the decode and prefill entry points read them.

Follows sources/NVMAIFormat/GTurboFormatV1.swift, GTurboManifestV1.swift, GTurboPackedExpertsLayoutV1.swift,
GTurboResidentIndexV1.swift, sources/NVMAIRepack/Core/Format/GTurboEncoders.swift and
sources/NVMAI/Infrastructure/ModelIO/{PackedExpertsLayout,ResidentIndex,GTurboModelDirectory}.swift;
each function cites the lines it restates.  Errors carry the reference's cases: `FormatError`
(NVMAIFormatError: invalid / overflow / truncated) inside the codecs, `ModelError` (indexCorrupt,
missingFile, partialInstall) at the reader level."""
import json
import os
import struct
import unicodedata
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np

# GTurboFormatV1.swift:3-22
MAGIC = "GTURBO"
VERSION_MAJOR, VERSION_MINOR = 1, 0
ALIGNMENT_BYTES = 16384
RESIDENT_HEADER_BYTES = 24
RESIDENT_ENTRY_BYTES = 72
RESIDENT_INDEX_MAX_BYTES = 32 * 1024 * 1024
KNOWN_FLAGS = {"streamingPresent", "turboQuantKV", "aneSharedExpert"}
DTYPES = {0: "U32", 1: "BF16", 2: "FP16", 3: "FP32"}
MANIFEST_MAX_BYTES = 4 * 1024 * 1024          # ManifestReader.defaultMaxBytes, ManifestReader.swift:71
U64_MAX = (1 << 64) - 1


class FormatError(Exception):
    """NVMAIFormatError (GTurboFormatV1.swift:25-37)."""

    def __init__(self, kind, fld, reason=""):
        self.kind, self.field, self.reason = kind, fld, reason
        text = {"invalid": "%s: %s" % (fld, reason), "overflow": "%s: arithmetic overflow" % fld,
                "truncated": "%s: truncated" % fld}[kind]
        super().__init__(text)


class ModelError(Exception):
    """The cases of the reference's ModelError that the readers throw."""

    def __init__(self, kind, detail):
        self.kind, self.detail = kind, detail
        super().__init__("%s: %s" % (kind, detail))


def _invalid(fld, reason):
    return FormatError("invalid", fld, reason)


def checked_add(a, b, fld):                    # gturboCheckedAdd, GTurboFormatV1.swift:39-44
    v = a + b
    if v > U64_MAX:
        raise FormatError("overflow", fld)
    return v


def checked_multiply(a, b, fld):               # gturboCheckedMultiply, :46-51
    v = a * b
    if v > U64_MAX:
        raise FormatError("overflow", fld)
    return v


def filesystem_key(path):                      # GTurboPathValidator.appleFilesystemKey, :54-57
    return unicodedata.normalize("NFC", path).lower()


def validate_relative_path(path, fld):         # :59-71
    if not path or path.startswith("/") or "\0" in path:
        raise _invalid(fld, "unsafe relative path")
    parts = path.split("/")
    if not all(p and p not in (".", "..") for p in parts):
        raise _invalid(fld, "non-canonical path")
    if "/".join(parts) != path:
        raise _invalid(fld, "non-normalized path")


def validate_basename(name, fld):              # :73-78
    validate_relative_path(name, fld)
    if "/" in name:
        raise _invalid(fld, "expected basename")


# ------------------------------------------------------------------------------------ JSON decoding
# A Swift Codable struct: every non-optional key present with the right type, unknown keys ignored.
class _Missing(Exception):
    pass


def _get(obj, key, kind, optional=False):
    if not isinstance(obj, dict):
        raise _Missing("expected an object around %r" % key)
    if key not in obj or obj[key] is None:
        if optional:
            return None
        raise _Missing("key %r not found" % key)
    v = obj[key]
    if kind == "uint":
        ok = isinstance(v, int) and not isinstance(v, bool) and 0 <= v <= U64_MAX
    elif kind == "int":
        ok = isinstance(v, int) and not isinstance(v, bool) and -(1 << 63) <= v < (1 << 63)
    elif kind == "float":
        ok = isinstance(v, (int, float)) and not isinstance(v, bool)
    elif kind == "bool":
        ok = isinstance(v, bool)
    elif kind == "str":
        ok = isinstance(v, str)
    elif kind == "list":
        ok = isinstance(v, list)
    elif kind == "dict":
        ok = isinstance(v, dict)
    else:
        raise AssertionError(kind)
    if not ok:
        raise _Missing("key %r has the wrong type" % key)
    return float(v) if kind == "float" else v


# ------------------------------------------------------------------------------------ manifest.json
@dataclass
class QuantSlot:                               # GTurboManifestQuantSlotV1, GTurboManifestV1.swift:64-79
    weightBits: int
    scheme: str
    scaleType: str
    biasType: str
    groupSize: int


@dataclass
class Manifest:                                # GTurboManifestV1, :101-137
    magic: str
    versionMajor: int
    versionMinor: int
    flags: Dict[str, bool]
    modelID: str
    sourceSnapshotHash: Optional[str]
    arch: Dict[str, object]
    quant: Optional[Dict[str, QuantSlot]]
    files: Dict[str, Dict[str, object]]        # path -> {"size", "sha256"}
    expertsPerLayer: int
    numLayers: int
    expertStride: int
    bitWidthOverridesHonored: Optional[int] = None


_ARCH_INT = ["hiddenSize", "ffnIntermediate", "moeIntermediateSize", "numHeads", "numKVHeads", "numFullKVHeads",
             "headDim", "fullHeadDim", "vocabSize", "slidingWindow", "numLayers", "numExperts", "topKExperts"]
_ARCH_FLOAT = ["finalLogitSoftcap", "ropeTheta", "fullRopeTheta", "partialRotaryFactor"]
_QUANT_SLOTS = ["embedding", "attention", "router", "sharedExpert", "routedExpert"]


def decode_manifest(data, validate=True):
    """GTurboManifestCodec.decode (GTurboManifestV1.swift:139-157)."""
    try:
        root = json.loads(data)
        arch_in = _get(root, "arch", "dict")
        arch = {k: _get(arch_in, k, "int") for k in _ARCH_INT}
        arch.update({k: _get(arch_in, k, "float") for k in _ARCH_FLOAT})
        arch["tieWordEmbeddings"] = _get(arch_in, "tieWordEmbeddings", "bool")
        arch["attentionKEqV"] = _get(arch_in, "attentionKEqV", "bool")
        arch["hiddenActivation"] = _get(arch_in, "hiddenActivation", "str")
        mask = _get(arch_in, "fullAttentionLayerMask", "list")
        if not all(isinstance(v, int) and not isinstance(v, bool) for v in mask):
            raise _Missing("fullAttentionLayerMask holds a non-integer")
        arch["fullAttentionLayerMask"] = list(mask)
        quant_in = _get(root, "quant", "dict", optional=True)
        quant = None
        if quant_in is not None:
            quant = {}
            for name in _QUANT_SLOTS:
                s = _get(quant_in, name, "dict")
                quant[name] = QuantSlot(_get(s, "weightBits", "int"), _get(s, "scheme", "str"), _get(s, "scaleType", "str"),
                                        _get(s, "biasType", "str"), _get(s, "groupSize", "int"))
        flags = _get(root, "flags", "dict")
        if not all(isinstance(v, bool) for v in flags.values()):
            raise _Missing("flags holds a non-boolean")
        files_in = _get(root, "files", "dict")
        files = {p: {"size": _get(e, "size", "uint"), "sha256": _get(e, "sha256", "str")} for p, e in files_in.items()}
        m = Manifest(_get(root, "magic", "str"), _get(root, "versionMajor", "int"), _get(root, "versionMinor", "int"),
                     dict(flags), _get(root, "modelID", "str"), _get(root, "sourceSnapshotHash", "str", optional=True),
                     arch, quant, files, _get(root, "expertsPerLayer", "int"), _get(root, "numLayers", "int"),
                     _get(root, "expertStride", "uint"), _get(root, "bitWidthOverridesHonored", "int", optional=True))
    except (ValueError, _Missing) as e:
        raise _invalid("manifest.json", str(e))
    if validate:
        validate_manifest(m)
    return m


def validate_manifest(m):
    """GTurboManifestCodec.validate (GTurboManifestV1.swift:159-255)."""
    if m.magic != MAGIC:
        raise _invalid("manifest.magic", "expected GTURBO")
    if m.versionMajor != VERSION_MAJOR or m.versionMinor < 0:
        raise _invalid("manifest.version", "unsupported version")
    for flag in m.flags:
        if flag not in KNOWN_FLAGS:
            raise _invalid("manifest.flags.%s" % flag, "unknown v1 flag")
    if not m.modelID or m.numLayers <= 0 or m.expertsPerLayer <= 0 or m.expertStride <= 0 or \
            m.expertStride % ALIGNMENT_BYTES:
        raise _invalid("manifest", "invalid dimensions or stride")
    a = m.arch
    if a["numLayers"] != m.numLayers or a["numExperts"] != m.expertsPerLayer:
        raise _invalid("manifest.arch", "dimensions disagree with streaming metadata")
    finite = lambda x: x == x and abs(x) != float("inf")
    ok = (a["hiddenSize"] > 0 and a["ffnIntermediate"] > 0 and a["moeIntermediateSize"] > 0 and a["numHeads"] > 0 and
          a["numKVHeads"] > 0 and a["numFullKVHeads"] > 0 and a["headDim"] > 0 and a["fullHeadDim"] > 0 and
          a["vocabSize"] > 0 and a["slidingWindow"] >= 0 and 0 < a["topKExperts"] <= a["numExperts"] and
          finite(a["finalLogitSoftcap"]) and finite(a["ropeTheta"]) and a["ropeTheta"] > 0 and
          finite(a["fullRopeTheta"]) and a["fullRopeTheta"] > 0 and finite(a["partialRotaryFactor"]) and
          0 <= a["partialRotaryFactor"] <= 1 and bool(a["hiddenActivation"]) and
          len(a["fullAttentionLayerMask"]) == a["numLayers"] and all(v in (0, 1, 2) for v in a["fullAttentionLayerMask"]))
    if not ok:
        raise _invalid("manifest.arch", "invalid architecture values")
    if m.quant is not None:
        for name in _QUANT_SLOTS:
            s = m.quant[name]
            if not (0 < s.weightBits <= 32 and s.groupSize > 0 and s.scheme and s.scaleType and s.biasType):
                raise _invalid("manifest.quant.%s" % name, "invalid quantization values")
    reserved = {"manifest.json", "verified-install.json"}
    canonical = {}
    for path in sorted(m.files):
        validate_relative_path(path, "manifest.files.%s" % path)
        key = filesystem_key(path)
        if key in canonical:
            raise _invalid("manifest.files.%s" % path, "filesystem-equivalent duplicate path")
        canonical[key] = path
        if key == "tokenizer" or key in reserved or any(key.startswith(r + "/") for r in reserved):
            raise _invalid("manifest.files.%s" % path, "reserved artifact filename")
        sha = m.files[path]["sha256"]
        if len(sha) != 64 or not all(c in "0123456789abcdefABCDEF" for c in sha):
            raise _invalid("manifest.files.%s.sha256" % path, "expected 64 hexadecimal characters")
    for key, path in canonical.items():
        parts = key.split("/")
        while len(parts) > 1:
            parts.pop()
            if "/".join(parts) in canonical:
                raise _invalid("manifest.files.%s" % path, "file path collides with a directory prefix")


# ------------------------------------------------------------------------------------ layout.json
@dataclass(frozen=True)
class SubTensorEntry:                          # PackedExpertsLayout.swift:4-10
    offset: int                                # relative to the expert blob's start
    size: int
    dtype: str                                 # "U32" | "BF16"
    shape: tuple
    bits: Optional[int] = None


@dataclass
class ExpertEntry:                             # PackedExpertsLayout.swift:12-39
    expert: int                                # logical id used by the router
    physicalRank: int                          # rank inside the layer file
    offset: int                                # absolute byte offset in the layer file
    size: int
    subTensors: Dict[str, SubTensorEntry]


@dataclass
class LayerLayout:                             # PackedExpertsLayout.swift:41-45
    layer: int
    file: str
    experts: List[ExpertEntry]


@dataclass
class PackedExpertsLayout:                     # PackedExpertsLayout.swift:47-71
    expertStride: int
    numLayers: int
    expertsPerLayer: int
    layers: List[LayerLayout] = field(default_factory=list)

    def expert(self, layer, expert):
        if not 0 <= layer < len(self.layers):
            raise ModelError("indexCorrupt", "expert layout has %d layers; layer %d is out of range"
                             % (len(self.layers), layer))
        lay = self.layers[layer]
        if not 0 <= expert < len(lay.experts):
            raise ModelError("indexCorrupt", "layer %d has %d experts; expert %d is out of range"
                             % (layer, len(lay.experts), expert))
        return lay.experts[expert]


def _decode_layout_wire(data):
    """JSONDecoder().decode(GTurboPackedExpertsLayoutV1.self) (GTurboPackedExpertsLayoutV1.swift:3-72)."""
    try:
        root = json.loads(data)
        layers = []
        for lay in _get(root, "layers", "list"):
            experts = []
            for e in _get(lay, "experts", "list"):
                tensors = {}
                for name, t in _get(e, "tensors", "dict").items():
                    shape = _get(t, "shape", "list")
                    if not all(isinstance(v, int) and not isinstance(v, bool) and 0 <= v < (1 << 32) for v in shape):
                        raise _Missing("shape is not a list of UInt32")
                    tensors[name] = SubTensorEntry(_get(t, "offset", "uint"), _get(t, "size", "uint"), _get(t, "dtype", "str"),
                                                   tuple(shape), _get(t, "bits", "int", optional=True))
                experts.append(dict(expert=_get(e, "expert", "int", optional=True),
                                    physicalRank=_get(e, "physicalRank", "int", optional=True),
                                    offset=_get(e, "offset", "uint"), size=_get(e, "size", "uint"), tensors=tensors))
            layers.append(dict(layer=_get(lay, "layer", "int"), file=_get(lay, "file", "str"), experts=experts))
        return dict(expertStride=_get(root, "expertStride", "uint"), numLayers=_get(root, "numLayers", "int"),
                    expertsPerLayer=_get(root, "expertsPerLayer", "int"), layers=layers)
    except (ValueError, _Missing) as e:
        raise _invalid("packed_experts/layout.json", str(e))


def validate_layout_wire(w):
    """GTurboV1StructuralValidator.validate (GTurboPackedExpertsLayoutV1.swift:75-160)."""
    if not (w["numLayers"] > 0 and w["expertsPerLayer"] > 0 and w["expertStride"] > 0 and
            w["expertStride"] % ALIGNMENT_BYTES == 0 and len(w["layers"]) == w["numLayers"]):
        raise _invalid("layout", "invalid dimensions or stride")
    layer_ids, layer_files = set(), set()
    for lay in w["layers"]:
        L = lay["layer"]
        if not 0 <= L < w["numLayers"] or L in layer_ids:
            raise _invalid("layout.layers", "duplicate or invalid layer")
        layer_ids.add(L)
        validate_basename(lay["file"], "layout.layers[%d].file" % L)
        key = filesystem_key(lay["file"])
        if key == "layout.json":
            raise _invalid("layout.layers[%d].file" % L, "reserved packed-expert filename")
        if key in layer_files:
            raise _invalid("layout.layers[%d].file" % L, "duplicate layer filename")
        layer_files.add(key)
        if len(lay["experts"]) != w["expertsPerLayer"]:
            raise _invalid("layout.layers[%d].experts" % L, "wrong expert count")
        explicit = [e["expert"] is not None for e in lay["experts"]]
        if any(explicit) and not all(explicit):
            raise _invalid("layout.layers[%d].experts" % L, "expert ids must be either all explicit or all positional")
        logical_ids, ranks, offsets = set(), set(), set()
        for position, e in enumerate(lay["experts"]):
            logical = e["expert"] if e["expert"] is not None else position
            physical = e["physicalRank"] if e["physicalRank"] is not None else logical
            if not (0 <= logical < w["expertsPerLayer"] and 0 <= physical < w["expertsPerLayer"]) or \
                    logical in logical_ids or physical in ranks or e["offset"] in offsets:
                raise _invalid("layout.layers[%d].experts" % L, "duplicate or invalid expert mapping")
            logical_ids.add(logical); ranks.add(physical); offsets.add(e["offset"])
            expected = checked_multiply(physical, w["expertStride"], "expert.offset")
            if e["offset"] != expected or e["size"] != w["expertStride"]:
                raise _invalid("expert[%d]" % logical, "offset or size does not match physical rank")
            ranges = []
            for name, t in e["tensors"].items():
                if not (t.dtype in ("U32", "BF16") and name and t.size > 0 and t.shape and all(v > 0 for v in t.shape) and
                        (t.bits is None or 0 < t.bits <= 32)):
                    raise _invalid("expert[%d].tensors.%s" % (logical, name), "invalid dtype or shape")
                end = checked_add(t.offset, t.size, "tensor.%s.range" % name)
                if end > e["size"]:
                    raise _invalid("expert[%d].tensors.%s" % (logical, name), "range exceeds expert blob")
                ranges.append((t.offset, end, name))
            ranges.sort(key=lambda r: (r[0], r[1]))
            for a, b in zip(ranges, ranges[1:]):
                if a[1] > b[0]:
                    raise _invalid("expert[%d].tensors" % logical, "overlapping ranges %s and %s" % (a[2], b[2]))


def cross_validate(manifest_layers, manifest_experts, manifest_stride, manifest_file_sizes, w):
    """GTurboV1StructuralValidator.crossValidate (GTurboPackedExpertsLayoutV1.swift:172-196)."""
    if manifest_layers != w["numLayers"] or manifest_experts != w["expertsPerLayer"] or manifest_stride != w["expertStride"]:
        raise _invalid("manifest/layout", "dimension mismatch")
    expected = checked_multiply(w["expertsPerLayer"], w["expertStride"], "layout.layerSize")
    for lay in w["layers"]:
        path = "packed_experts/%s" % lay["file"]
        if manifest_file_sizes.get(path) != expected:
            raise _invalid("manifest.files.%s" % path, "missing or wrong layer size")


def decode_layout(data, manifest=None):
    """PackedExpertsLayoutReader.decode (PackedExpertsLayout.swift:96-130): wire decode, structural
    validation, optional cross-check against the manifest; layers sorted by id, experts by logical id."""
    try:
        w = _decode_layout_wire(data)
        validate_layout_wire(w)
        if manifest is not None:
            cross_validate(manifest.numLayers, manifest.expertsPerLayer, manifest.expertStride,
                           {p: e["size"] for p, e in manifest.files.items()}, w)
    except FormatError as e:
        raise ModelError("indexCorrupt", "layout.json: %s" % e)
    layers = []
    for lay in sorted(w["layers"], key=lambda l: l["layer"]):
        experts = []
        for position, e in enumerate(lay["experts"]):
            logical = e["expert"] if e["expert"] is not None else position
            rank = e["physicalRank"] if e["physicalRank"] is not None else logical
            experts.append(ExpertEntry(logical, rank, e["offset"], e["size"], dict(e["tensors"])))
        experts.sort(key=lambda x: x.expert)
        layers.append(LayerLayout(lay["layer"], lay["file"], experts))
    return PackedExpertsLayout(w["expertStride"], w["numLayers"], w["expertsPerLayer"], layers)


def read_metadata(root, relative_path, max_bytes):
    """GTurboModelDirectory.readMetadata (GTurboModelDirectory.swift:60-91)."""
    path = os.path.join(root, relative_path)
    try:
        size = os.stat(path).st_size
    except FileNotFoundError:
        raise ModelError("missingFile", relative_path)
    if size > max_bytes:
        raise ModelError("indexCorrupt", "%s size %d exceeds metadata cap %d" % (relative_path, size, max_bytes))
    with open(path, "rb") as f:
        return f.read()


def load_layout(directory, manifest=None, max_bytes=RESIDENT_INDEX_MAX_BYTES):
    """PackedExpertsLayoutReader.load (PackedExpertsLayout.swift:73-94)."""
    return decode_layout(read_metadata(directory, "packed_experts/layout.json", max_bytes), manifest)


def load_manifest(directory, max_bytes=MANIFEST_MAX_BYTES):
    """ManifestReader.load without the architecture comparison (ManifestReader.swift:85-97)."""
    try:
        data = read_metadata(directory, "manifest.json", max_bytes)
    except ModelError as e:
        if e.kind == "missingFile":
            raise ModelError("partialInstall", directory)
        raise
    return decode_manifest(data)


# ------------------------------------------------------------------------------------ resident index
@dataclass(frozen=True)
class ResidentEntry:                           # GTurboResidentIndexEntryV1, GTurboResidentIndexV1.swift:15-39
    name: str
    dtype: int
    fileOffset: int
    sizeBytes: int
    shape: tuple                               # four UInt32, zeros trailing
    scaleOffset: int = 0
    scaleSize: int = 0
    biasOffset: int = 0
    biasSize: int = 0


def decode_resident_header(buf):
    """GTurboResidentIndexCodec.decodeHeader (GTurboResidentIndexV1.swift:42-51): indexSize,
    residentSize, entryCount, little-endian UInt64 each."""
    if len(buf) < RESIDENT_HEADER_BYTES:
        raise FormatError("truncated", "resident.header")
    return struct.unpack_from("<QQQ", buf, 0)


def decode_resident_region(buf, header):
    """GTurboResidentIndexCodec.decodeRegion (GTurboResidentIndexV1.swift:53-150)."""
    index_size, resident_size, count = header
    if index_size > RESIDENT_INDEX_MAX_BYTES:
        raise _invalid("resident.indexSize", "exceeds v1 metadata cap")
    if index_size > len(buf) or index_size < RESIDENT_HEADER_BYTES or index_size % ALIGNMENT_BYTES:
        raise FormatError("truncated", "resident.index")
    table_bytes = checked_multiply(count, RESIDENT_ENTRY_BYTES, "resident.entryTable")
    table_end = checked_add(RESIDENT_HEADER_BYTES, table_bytes, "resident.entryTable")
    if table_end > index_size or count > (1 << 63) - 1:
        raise _invalid("resident.entryTable", "outside index")
    resident_end = checked_add(index_size, resident_size, "resident.payload")

    def contained(offset, size, fld):
        end = checked_add(offset, size, fld)
        if offset < index_size or end > resident_end:
            raise _invalid(fld, "range outside resident payload")

    def optional(offset, size, fld):
        if size == 0:
            if offset != 0:
                raise _invalid(fld, "absent payload offset must be zero")
            return
        contained(offset, size, fld)

    entries, names, ranges = [], set(), []
    for index in range(count):
        at = RESIDENT_HEADER_BYTES + index * RESIDENT_ENTRY_BYTES
        name_off, name_len, dtype, reserved, file_off, size_bytes, s0, s1, s2, s3, sc_off, sc_size, bi_off, bi_size = \
            struct.unpack_from("<IHBBQQIIIIQQQQ", buf, at)
        if reserved != 0:
            raise _invalid("resident.entries[%d].reserved" % index, "must be zero")
        name_end = checked_add(name_off, name_len, "resident.entries[%d].name" % index)
        if name_off < table_end or name_end > index_size:
            raise _invalid("resident.entries[%d].name" % index, "range outside string table")
        try:
            name = bytes(buf[name_off:name_end]).decode("utf-8")
        except UnicodeDecodeError:
            name = ""
        if not name or name in names:
            raise _invalid("resident.entries[%d].name" % index, "invalid UTF-8 or duplicate")
        names.add(name)
        if dtype not in DTYPES:
            raise _invalid("resident.entries[%d].dtype" % index, "unknown dtype")
        shape = (s0, s1, s2, s3)
        if shape[0] == 0:
            raise _invalid("resident.entries[%d].shape" % index, "first dimension must be positive")
        saw_zero = False
        for dim in shape:
            if dim == 0:
                saw_zero = True
            elif saw_zero:
                raise _invalid("resident.entries[%d].shape" % index, "zero dimensions must be trailing")
        if size_bytes == 0:
            raise _invalid("resident.entries[%d].weights" % index, "primary payload is empty")
        contained(file_off, size_bytes, "resident.entries[%d].weights" % index)
        optional(sc_off, sc_size, "resident.entries[%d].scales" % index)
        optional(bi_off, bi_size, "resident.entries[%d].biases" % index)
        ranges.append((file_off, file_off + size_bytes, "resident.entries[%d].weights" % index))
        if sc_size:
            ranges.append((sc_off, sc_off + sc_size, "resident.entries[%d].scales" % index))
        if bi_size:
            ranges.append((bi_off, bi_off + bi_size, "resident.entries[%d].biases" % index))
        entries.append(ResidentEntry(name, dtype, file_off, size_bytes, shape, sc_off, sc_size, bi_off, bi_size))
    ranges.sort(key=lambda r: (r[0], r[1]))
    for prev, cur in zip(ranges, ranges[1:]):
        if cur[0] < prev[1]:
            raise _invalid(cur[2], "overlaps %s" % prev[2])
    return entries


def encode_resident_index(entries, resident_size):
    """The writer's side (GTurboBinary.writeIndexHeader / writeIndexEntry, GTurboEncoders.swift:9-45;
    layout as ResidentWriter lays it out: header, entry table, string table, zero padding to 16 KB).
    `entries` hold offsets RELATIVE to the start of the payload; returns (index bytes, entries with
    absolute file offsets)."""
    names = [e.name.encode("utf-8") for e in entries]
    table_base = RESIDENT_HEADER_BYTES + len(entries) * RESIDENT_ENTRY_BYTES
    raw = table_base + sum(len(n) for n in names)
    index_size = (raw + ALIGNMENT_BYTES - 1) // ALIGNMENT_BYTES * ALIGNMENT_BYTES
    buf = bytearray(index_size)
    struct.pack_into("<QQQ", buf, 0, index_size, resident_size, len(entries))
    cursor, absolute = table_base, []
    for i, (e, n) in enumerate(zip(entries, names)):
        if len(n) > 0xFFFF:
            raise ValueError("resident tensor name exceeds UInt16 length")
        shape = tuple(e.shape) + (0,) * (4 - len(e.shape))
        a = ResidentEntry(e.name, e.dtype, e.fileOffset + index_size, e.sizeBytes, shape,
                          e.scaleOffset + index_size if e.scaleSize else 0, e.scaleSize,
                          e.biasOffset + index_size if e.biasSize else 0, e.biasSize)
        struct.pack_into("<IHBBQQIIIIQQQQ", buf, RESIDENT_HEADER_BYTES + i * RESIDENT_ENTRY_BYTES, cursor, len(n), a.dtype, 0,
                         a.fileOffset, a.sizeBytes, *shape, a.scaleOffset, a.scaleSize, a.biasOffset, a.biasSize)
        buf[cursor:cursor + len(n)] = n
        cursor += len(n)
        absolute.append(a)
    return bytes(buf), absolute


def load_resident_index(path, max_bytes=RESIDENT_INDEX_MAX_BYTES):
    """ResidentIndexReader.load (ResidentIndex.swift:47-120): header, then the index region; the
    tensor region is not read.  Returns (header, {name: ResidentEntry})."""
    try:
        with open(path, "rb") as f:
            head = f.read(RESIDENT_HEADER_BYTES)
            try:
                header = decode_resident_header(head)
                if header[0] > max_bytes:
                    raise _invalid("resident.indexSize", "exceeds v1 metadata cap")
                f.seek(0)
                region = f.read(header[0])
                entries = decode_resident_region(region, header)
            except FormatError as e:
                raise ModelError("indexCorrupt", str(e))
    except FileNotFoundError:
        raise ModelError("missingFile", os.path.basename(path))
    return header, {e.name: e for e in entries}


# ------------------------------------------------------------------------------------ the path's view
_ROLES = ("gate", "gate_scales", "gate_biases", "up", "up_scales", "up_biases", "down", "down_scales", "down_biases")


def routed_expert_offsets(layout, layer):
    """Model.routedExpertOffsets (ModelExpertIO.swift:66-82): the nine sub-tensor offsets of expert 0
    of the layer, in the order of MoEExpertOffsets (0 for an absent role)."""
    e = layout.expert(layer, 0)
    return tuple(e.subTensors[r].offset if r in e.subTensors else 0 for r in _ROLES)


def validate_routed_expert_layout(layout, hidden, intermediate, weight_bits, group_size):
    """Model.validateRoutedExpertLayout (Model.swift:845-905): every layer's nine roles have the
    required dtype, shape, bit width, size and alignment, identically across the experts."""
    for lay in layout.layers:
        if not lay.experts:
            raise ModelError("indexCorrupt", "routed layer %d has no experts" % lay.layer)
        ref = lay.experts[0]
        for role, rows, cols in (("gate", intermediate, hidden), ("up", intermediate, hidden), ("down", hidden, intermediate)):
            if cols % group_size:
                raise ModelError("indexCorrupt", "routed layer %d %s has an invalid quant layout (group %d, %d-bit)"
                                 % (lay.layer, role, group_size, weight_bits))
            bits_total = rows * cols * weight_bits
            if bits_total % 8:
                raise ModelError("indexCorrupt", "routed layer %d %s %d-bit layout does not pack into whole bytes"
                                 % (lay.layer, role, weight_bits))
            weight, aux = bits_total // 8, rows * (cols // group_size) * 2
            for name, dtype, shape, bits, size, align in (
                    (role, "U32", (rows, cols), weight_bits, weight, 4),
                    (role + "_scales", "BF16", (rows, cols // group_size), None, aux, 2),
                    (role + "_biases", "BF16", (rows, cols // group_size), None, aux, 2)):
                t = ref.subTensors.get(name)
                if t is None:
                    raise ModelError("indexCorrupt", "routed layer %d is missing role %s" % (lay.layer, name))
                end = t.offset + t.size
                if not (t.dtype == dtype and tuple(t.shape) == shape and t.bits == bits and t.size == size and
                        t.offset % align == 0 and end <= U64_MAX and end <= ref.size and end <= (1 << 32)):
                    raise ModelError("indexCorrupt", "routed layer %d role %s does not match the required schema"
                                     % (lay.layer, name))
                for other in lay.experts[1:]:
                    if other.subTensors.get(name) != t:
                        raise ModelError("indexCorrupt", "routed layer %d role %s metadata differs across experts"
                                         % (lay.layer, name))


class GTurboModel:
    """An opened model directory (the part of Model.load, Model.swift:540-660, this path needs):
    manifest, resident index, packed-experts layout, with the size checks that tie them together."""

    def __init__(self, directory):
        self.directory = directory
        self.manifest = load_manifest(directory)
        if "model_weights.bin" not in self.manifest.files:
            raise ModelError("missingFile", "model_weights.bin")
        self.layout = load_layout(directory, self.manifest)
        self.weights_path = os.path.join(directory, "model_weights.bin")
        self.header, self.entries = load_resident_index(self.weights_path)
        size = os.stat(self.weights_path).st_size
        if size != self.header[0] + self.header[1]:                # Model.swift:640-650
            raise ModelError("indexCorrupt", "model_weights.bin size %d != indexSize %d + residentSize %d = %d"
                             % (size, self.header[0], self.header[1], self.header[0] + self.header[1]))
        for lay in self.layout.layers:                             # ManifestReaderTests: missingLayerFile
            if not os.path.exists(os.path.join(directory, "packed_experts", lay.file)):
                raise ModelError("missingFile", "packed_experts/%s" % lay.file)
        q = self.manifest.quant
        if q is not None:
            validate_routed_expert_layout(self.layout, self.manifest.arch["hiddenSize"],
                                          self.manifest.arch["moeIntermediateSize"], q["routedExpert"].weightBits,
                                          q["routedExpert"].groupSize)
        self._weights = None

    def resident(self, name):
        """Model.resident(name:) (Model.swift:313): (weights, scales, biases) as uint8 / uint16 views
        of the memory-mapped file (scales / biases None when absent), and the entry."""
        e = self.entries.get(name)
        if e is None:
            raise ModelError("missingTensor", name)
        if self._weights is None:
            self._weights = np.memmap(self.weights_path, dtype=np.uint8, mode="r")
        w = self._weights[e.fileOffset:e.fileOffset + e.sizeBytes]
        s = self._weights[e.scaleOffset:e.scaleOffset + e.scaleSize].view(np.uint16) if e.scaleSize else None
        b = self._weights[e.biasOffset:e.biasOffset + e.biasSize].view(np.uint16) if e.biasSize else None
        return w, s, b, e

    def expert_blobs(self, layer):
        """The layer file as uint8 [experts, stride] in LOGICAL expert order (row e = the blob the
        router's index e names; the file holds it at rank physicalRank)."""
        lay = self.layout.layers[layer]
        stride = self.layout.expertStride
        path = os.path.join(self.directory, "packed_experts", lay.file)
        if os.stat(path).st_size != stride * self.layout.expertsPerLayer:
            raise ModelError("indexCorrupt", "packed_experts/%s has the wrong size" % lay.file)
        data = np.memmap(path, dtype=np.uint8, mode="r").reshape(self.layout.expertsPerLayer, stride)
        ranks = [e.physicalRank for e in lay.experts]
        return data if ranks == list(range(len(ranks))) else data[ranks]

    def shared_matches_routed(self):
        """Whether the shared expert has the routed experts' bit width and group size, so that its
        arrays fit the routed sub-tensor regions and it can sit in the pool as one more expert.  The
        reference keeps the two in separate quant slots (Model.swift:59-60; validateLayerTensors checks
        the shared projections against quant.sharedExpert), and its repacker's default profile writes
        an 8-bit shared expert beside 4-bit routed experts (RemoteStreamingRepacker.swift:678-683)."""
        q = self.manifest.quant
        return (q["sharedExpert"].weightBits == q["routedExpert"].weightBits and
                q["sharedExpert"].groupSize == q["routedExpert"].groupSize)

    def shared_expert_offsets(self, layer):
        """(nine offsets, blob bytes, bits) of the shared expert's blob: the layer's routed-expert
        offsets when the widths agree, else CPUExpertFFN.Offsets(d:f:) at the shared expert's own
        width (CPUExpertFFN.swift:42-59)."""
        a, q = self.manifest.arch, self.manifest.quant
        bits, group = q["sharedExpert"].weightBits, q["sharedExpert"].groupSize
        if bits not in (4, 8) or group != 64:
            raise ModelError("unsupportedArch", "shared expert quantization %d-bit group %d (this build runs 4 / 8-bit, group 64)"
                             % (bits, group))
        if self.shared_matches_routed():
            return routed_expert_offsets(self.layout, layer), self.layout.expertStride, bits
        d, f = a["hiddenSize"], a["moeIntermediateSize"]
        sizes = [f * d * bits // 8, f * (d // 64) * 2, f * (d // 64) * 2] * 2 + [d * f * bits // 8, d * (f // 64) * 2, d * (f // 64) * 2]
        off, at = [], 0
        for n in sizes:
            off.append(at)
            at += n
        return tuple(off), at, bits

    def shared_expert_blob(self, layer):
        """The shared expert's nine arrays gathered from the resident file into one blob at the
        offsets of shared_expert_offsets (names: Model.swift:165-177).  Every array must have the size
        its shape and the shared expert's bit width give (validateLayerTensors, Model.swift:700-760): an
        array of another width would overlap its neighbour and be decoded as the wrong codes."""
        a = self.manifest.arch
        d, f = a["hiddenSize"], a["moeIntermediateSize"]
        off, size, bits = self.shared_expert_offsets(layer)
        blob = np.zeros(size, np.uint8)
        prefix = "language_model.model.layers.%d.mlp.shared_expert." % layer
        for i, (proj, rows, cols) in enumerate((("gate_proj", f, d), ("up_proj", f, d), ("down_proj", d, f))):
            w, s, b, _ = self.resident(prefix + proj + ".weight")
            if s is None or b is None:
                raise ModelError("indexCorrupt", "%s%s.weight has no scales or biases" % (prefix, proj))
            want = (rows * cols * bits // 8, rows * (cols // 64) * 2, rows * (cols // 64) * 2)
            for arr, at, n, what in ((w, off[3 * i], want[0], "weights"), (s.view(np.uint8), off[3 * i + 1], want[1], "scales"),
                                     (b.view(np.uint8), off[3 * i + 2], want[2], "biases")):
                if arr.size != n:
                    raise ModelError("indexCorrupt", "%s%s.weight %s hold %d bytes, a %d-bit [%d, %d] matrix needs %d"
                                     % (prefix, proj, what, arr.size, bits, rows, cols, n))
                blob[at:at + n] = arr
        return blob

    def expert_pool(self, layer, device="cuda", with_shared=True):
        """One layer's experts resident in device memory: uint8 [experts (+ 1), stride]; the shared
        expert, when asked for, is the last row -- which needs a shared expert of the routed experts'
        width (shared_matches_routed); moe_block handles both kinds of model."""
        import torch
        if with_shared and not self.shared_matches_routed():
            raise ModelError("unsupportedArch", "the shared expert's quantization differs from the routed experts': it cannot "
                             "be a row of their pool (use moe_block, which runs it through the shared-expert operator)")
        rows = [torch.from_numpy(np.array(self.expert_blobs(layer)))]
        if with_shared:
            rows.append(torch.from_numpy(self.shared_expert_blob(layer))[None])
        return torch.cat(rows).to(device)

    def _rows(self, name, bits, device, keep):
        import torch

        from . import ops
        w, s, b, e = self.resident(name)
        if e.dtype == 1:                                           # dense BF16 rows
            t = torch.from_numpy(np.array(w)).to(device)          # a copy: the map is read-only
            keep.append(t)
            return ops.rows_desc(16, t)
        ts = [torch.from_numpy(np.array(x.view(np.uint8) if x.dtype != np.uint8 else x)).to(device) for x in (w, s, b)]
        keep.extend(ts)
        return ops.rows_desc(bits, *ts)

    def moe_layer(self, layer, pool, device="cuda"):
        """The nvmai_moe_layer descriptor of one layer over `pool`: router rows and the shared expert's
        scalar gate row from the resident file (Model.swift:160-182), the expert offsets from the
        layout.  A pool with one row more than the layer has experts carries the shared expert in
        that row (expert_pool with_shared); otherwise the descriptor has no shared expert.  Returns
        (descriptor, the device tensors it points into -- keep them alive)."""
        from . import ops
        a, q = self.manifest.arch, self.manifest.quant
        keep = [pool]
        n = self.layout.expertsPerLayer
        has_shared = pool.shape[0] == n + 1
        if has_shared and not self.shared_matches_routed():
            raise ModelError("unsupportedArch", "a pool row cannot hold a shared expert of another quantization")
        prefix = "language_model.model.layers.%d.mlp." % layer
        router = self._rows(prefix + "gate.weight", q["router"].weightBits, device, keep)
        gate = self._rows(prefix + "shared_expert_gate.weight", q["router"].weightBits, device, keep) if has_shared else None
        desc = ops.moe_layer_desc(a["hiddenSize"], a["moeIntermediateSize"], n, a["topKExperts"], q["routedExpert"].weightBits,
                                  router, pool[:n], pool[n] if has_shared else None, gate,
                                  offsets=routed_expert_offsets(self.layout, layer))
        return desc, keep

    def moe_block(self, layer, device="cuda"):
        """One layer's MoE block resident in device memory, whatever the shared expert's width."""
        return GTurboMoEBlock(self, layer, device)


class GTurboMoEBlock:
    """A layer's routed experts, router, shared expert and its gate row in HBM, and the decode call
    over them.  A shared expert of the routed experts' width rides in the decode layer's own launches
    (one more work-list slot).  One of another width (the reference's default 4-bit profile keeps it at
    8 bits) runs as the reference runs it: the shared-expert operator at its own width
    (SharedExpertRuntime.encode + the scalar sigmoid gate, RealForwardRunner.swift:3866-3912), its
    16-bit output added to the routed sum (the `residual` input of phase 2, RealForwardRunner.swift:4263)."""

    def __init__(self, model, layer, device="cuda"):
        import torch

        from . import ops
        self.model, self.layer = model, layer
        a, q = model.manifest.arch, model.manifest.quant
        self.d, self.f = a["hiddenSize"], a["moeIntermediateSize"]
        self.routed_bits, self.shared_bits = q["routedExpert"].weightBits, q["sharedExpert"].weightBits
        self.fused = model.shared_matches_routed()
        self.pool = model.expert_pool(layer, device, with_shared=self.fused)
        self.desc, self.keep = model.moe_layer(layer, self.pool, device)
        if not self.fused:
            off, _, _ = model.shared_expert_offsets(layer)
            self.shared_blob = torch.from_numpy(model.shared_expert_blob(layer)).to(device)
            self.shared_offsets = ops.ExpertOffsets(*[int(v) for v in off])
            self.shared_gate = model._rows("language_model.model.layers.%d.mlp.shared_expert_gate.weight" % layer,
                                           q["router"].weightBits, device, self.keep)

    def decode(self, ctx, x, want_routes=False):
        """y[t] = sigmoid(g . x[t]) * ffn_shared(x[t]) + sum over the top-k of w * ffn_expert(x[t])."""
        from . import ops
        out = ops.MoE(ctx, self.routed_bits).decode_layer(self.desc, x, want_routes=want_routes)
        y = out[0] if want_routes else out
        if not self.fused:
            h1 = ops.SharedExpertRuntime(ctx, self.shared_bits).encode(self.shared_blob, self.shared_offsets, x, self.d, self.f,
                                                                      shared_gate=self.shared_gate)
            ops.Elementwise(ctx).encode_residual_add(y, h1)
        return out


# ------------------------------------------------------------------------------------ whole-model binding
# The resident tensors of the hybrid model by the reference's names (Model.swift:137-306; the schema
# validateLayerTensors checks, Model.swift:760-840).  A full-attention layer keeps q_proj (gate-packed
# [query; gate], 2 * heads * headDim rows), k_proj, v_proj; a gated-DeltaNet layer keeps in_proj_qkv,
# in_proj_z, in_proj_a, in_proj_b: the decode step here runs each group as ONE launch, so the binder lays
# the matrices of a group out as the rows of one matrix, in this order.
LAYER_PREFIX = "language_model.model.layers.%d."
FULL_PROJECTIONS = ("self_attn.q_proj.weight", "self_attn.k_proj.weight", "self_attn.v_proj.weight")
LINEAR_PROJECTIONS = ("linear_attn.in_proj_qkv.weight", "linear_attn.in_proj_z.weight", "linear_attn.in_proj_a.weight",
                      "linear_attn.in_proj_b.weight")


def hybrid_tensor_names(layer, full):
    """Every resident tensor name of one layer, in the reference's order of lookup."""
    p = LAYER_PREFIX % layer
    names = [p + "input_layernorm.weight", p + "post_attention_layernorm.weight", p + "mlp.gate.weight",
             p + "mlp.shared_expert_gate.weight"] + [p + "mlp.shared_expert.%s.weight" % q for q in ("gate_proj", "up_proj", "down_proj")]
    if full:
        names += [p + n for n in FULL_PROJECTIONS] + [p + "self_attn.o_proj.weight", p + "self_attn.q_norm.weight",
                                                       p + "self_attn.k_norm.weight"]
    else:
        names += [p + n for n in LINEAR_PROJECTIONS] + [p + "linear_attn.out_proj.weight", p + "linear_attn.conv1d.weight",
                                                         p + "linear_attn.A_log", p + "linear_attn.dt_bias", p + "linear_attn.norm.weight"]
    return names


def write_hybrid_model(directory, cfg, weights, model_id="nvmai-amd-synthetic"):
    """A decoder.HybridWeights instance (config decoder.HybridConfig) as a model directory under the reference's
    tensor names: what the repack tool would write for this model (sources/NVMAIRepack), reduced to what the format
    requires.  Rows of a fused projection group are split back into the reference's separate matrices."""
    D, F, E = cfg.hidden, cfg.moe_intermediate, cfg.num_experts
    host = lambda t: t.detach().cpu().numpy()
    raw = lambda t: np.ascontiguousarray(host(t)).view(np.uint8).reshape(-1).tobytes()
    resident = []

    def affine(name, t3, rows, cols, r0=0, r1=None):
        r1 = rows if r1 is None else r1
        w, s, b = t3
        w2, s2, b2 = w.reshape(rows, -1), s.reshape(rows, -1), b.reshape(rows, -1)
        resident.append((name, 0, (r1 - r0, cols), raw(w2[r0:r1]), raw(s2[r0:r1]), raw(b2[r0:r1])))

    def bf16(name, t, shape):
        resident.append((name, 1, tuple(shape), raw(t), None, None))

    affine("language_model.model.embed_tokens.weight", weights.embed, cfg.vocab, D)
    if cfg.head_bits == 16:
        bf16("language_model.lm_head.weight", weights.lm_head[0], (cfg.vocab, D))
    else:
        affine("language_model.lm_head.weight", weights.lm_head, cfg.vocab, D)
    bf16("language_model.model.norm.weight", weights.final_norm, (D,))
    off, used = _cpu_expert_offsets(D, F, cfg.expert_bits)
    sizes = [F * D * cfg.expert_bits // 8, F * (D // 64) * 2, F * (D // 64) * 2] * 2 + \
            [D * F * cfg.expert_bits // 8, D * (F // 64) * 2, D * (F // 64) * 2]
    shapes = [(F, D), (F, D // 64), (F, D // 64)] * 2 + [(D, F), (D, F // 64), (D, F // 64)]
    tensors = {r: SubTensorEntry(off[i], sizes[i], "BF16" if "_" in r else "U32", shapes[i], None if "_" in r else cfg.expert_bits)
               for i, r in enumerate(_ROLES)}
    stride = (used + ALIGNMENT_BYTES - 1) // ALIGNMENT_BYTES * ALIGNMENT_BYTES
    lays = []
    kh, vh, dk, dv, taps = cfg.gdn
    for L, w in enumerate(weights.layers):
        p = LAYER_PREFIX % L
        bf16(p + "input_layernorm.weight", w["in_norm"], (D,))
        bf16(p + "post_attention_layernorm.weight", w["post_norm"], (D,))
        bf16(p + "mlp.gate.weight", w["router"], (E, D))
        affine(p + "mlp.shared_expert_gate.weight", w["gate"], 1, D)
        pool = host(w["pool"])
        blobs = np.zeros((E, stride), np.uint8)
        blobs[:, :used] = pool[:E, :used]
        lays.append({"blobs": blobs, "tensors": tensors, "ranks": None})
        if w.get("shared") is not None:          # a shared expert of another width than the routed ones: its own blob
            shared, sb = host(w["shared"]["blob"]), w["shared"]["bits"]
            s_off, _ = _cpu_expert_offsets(D, F, sb)
            s_sizes = [F * D * sb // 8, F * (D // 64) * 2, F * (D // 64) * 2] * 2 + [D * F * sb // 8, D * (F // 64) * 2, D * (F // 64) * 2]
        else:
            shared, s_off, s_sizes = pool[E], off, sizes
        for i, (proj, rows, cols) in enumerate((("gate_proj", F, D), ("up_proj", F, D), ("down_proj", D, F))):
            cut = lambda j: shared[s_off[3 * i + j]:s_off[3 * i + j] + s_sizes[3 * i + j]].tobytes()
            resident.append((p + "mlp.shared_expert.%s.weight" % proj, 0, (rows, cols), cut(0), cut(1), cut(2)))
        if cfg.is_linear(L):
            rows_of = (cfg.gdn_qkv_dim, cfg.gdn_value_dim, vh, vh)
            total, at = sum(rows_of), 0
            for name, n in zip(LINEAR_PROJECTIONS, rows_of):
                affine(p + name, w["in_proj"], total, D, at, at + n)
                at += n
            affine(p + "linear_attn.out_proj.weight", w["out_proj"], D, cfg.gdn_value_dim)
            bf16(p + "linear_attn.conv1d.weight", w["conv_w"], (cfg.gdn_qkv_dim, taps))
            bf16(p + "linear_attn.A_log", w["a_log"], (vh,))
            bf16(p + "linear_attn.dt_bias", w["dt_bias"], (vh,))
            bf16(p + "linear_attn.norm.weight", w["gdn_norm"], (dv,))
        else:
            rows_of = (2 * cfg.q_dim, cfg.kv_dim, cfg.kv_dim)
            total, at = sum(rows_of), 0
            for name, n in zip(FULL_PROJECTIONS, rows_of):
                affine(p + name, w["qkv"], total, D, at, at + n)
                at += n
            affine(p + "self_attn.o_proj.weight", w["o_proj"], D, cfg.q_dim)
            bf16(p + "self_attn.q_norm.weight", w["q_norm"], (cfg.head_dim,))
            bf16(p + "self_attn.k_norm.weight", w["k_norm"], (cfg.head_dim,))
    slot = lambda b: {"weightBits": b, "scheme": "affine", "scaleType": "bf16", "biasType": "bf16", "groupSize": 64}
    quant = {"embedding": slot(cfg.embed_bits), "attention": slot(cfg.attn_bits), "router": slot(8),
             "sharedExpert": slot(cfg.shared_bits), "routedExpert": slot(cfg.expert_bits)}
    arch = {"hiddenSize": D, "ffnIntermediate": F, "moeIntermediateSize": F, "numHeads": cfg.num_heads,
            "numKVHeads": cfg.num_kv_heads, "numFullKVHeads": cfg.num_kv_heads, "headDim": cfg.head_dim,
            "fullHeadDim": cfg.head_dim, "vocabSize": cfg.vocab, "slidingWindow": 0,
            "finalLogitSoftcap": float(cfg.logit_softcap), "ropeTheta": float(cfg.rope_theta),
            "fullRopeTheta": float(cfg.rope_theta), "partialRotaryFactor": cfg.rotary_dim / cfg.head_dim,
            "numLayers": cfg.layers, "numExperts": E, "topKExperts": cfg.top_k, "tieWordEmbeddings": False,
            "attentionKEqV": False, "hiddenActivation": "silu",
            "fullAttentionLayerMask": [2 if cfg.is_linear(L) else 1 for L in range(cfg.layers)]}
    return write_model(directory, arch, quant, lays, resident, model_id=model_id)


def _cpu_expert_offsets(d, f, bits):
    """CPUExpertFFN.Offsets(d:f:) (CPUExpertFFN.swift:42-59): (nine offsets, blob bytes)."""
    sizes = [f * d * bits // 8, f * (d // 64) * 2, f * (d // 64) * 2] * 2 + [d * f * bits // 8, d * (f // 64) * 2, d * (f // 64) * 2]
    off, at = [], 0
    for n in sizes:
        off.append(at)
        at += n
    return off, at


# ------------------------------------------------------------------------------------ writer (tests, tools)
def write_model(directory, arch, quant, layers, resident, model_id="toy", flags=None):
    """Writes a model directory the readers above accept: `layers` = list of dicts
    {"blobs": uint8 [experts, stride], "tensors": {role: SubTensorEntry}, "ranks": optional
    permutation (physical rank of logical expert e)}; `resident` = list of (name, dtype code, shape,
    weights bytes, scales bytes or None, biases bytes or None).  The counterpart of the reference's
    repack tool (sources/NVMAIRepack), reduced to what the format requires."""
    import hashlib
    os.makedirs(os.path.join(directory, "packed_experts"), exist_ok=True)
    files = {}

    def put(rel, data):
        with open(os.path.join(directory, rel), "wb") as f:
            f.write(data)
        files[rel] = {"size": len(data), "sha256": hashlib.sha256(data).hexdigest()}

    stride = int(layers[0]["blobs"].shape[1])
    n_exp = int(layers[0]["blobs"].shape[0])
    lay_json = []
    for L, lay in enumerate(layers):
        ranks = list(lay.get("ranks") or range(n_exp))
        data = np.zeros((n_exp, stride), np.uint8)
        experts = []
        for e in range(n_exp):
            data[ranks[e]] = lay["blobs"][e]
            experts.append({"expert": e, "physicalRank": ranks[e], "offset": ranks[e] * stride, "size": stride,
                            "tensors": {k: dict(offset=t.offset, size=t.size, dtype=t.dtype, shape=list(t.shape),
                                                **({"bits": t.bits} if t.bits is not None else {}))
                                        for k, t in lay["tensors"].items()}})
        name = "layer_%02d.bin" % L
        put("packed_experts/" + name, data.tobytes())
        lay_json.append({"layer": L, "file": name, "experts": experts})
    layout = {"expertStride": stride, "numLayers": len(layers), "expertsPerLayer": n_exp, "layers": lay_json}
    put("packed_experts/layout.json", json.dumps(layout, sort_keys=True).encode())
    payload, entries = bytearray(), []
    for name, dtype, shape, w, s, b in resident:
        def add(blob):
            while len(payload) % 64:
                payload.append(0)
            at = len(payload)
            payload.extend(blob)
            return at, len(blob)
        wo, wn = add(w)
        so, sn = add(s) if s is not None else (0, 0)
        bo, bn = add(b) if b is not None else (0, 0)
        entries.append(ResidentEntry(name, dtype, wo, wn, tuple(shape), so, sn, bo, bn))
    index, _ = encode_resident_index(entries, len(payload))
    put("model_weights.bin", index + bytes(payload))
    manifest = {"magic": MAGIC, "versionMajor": VERSION_MAJOR, "versionMinor": VERSION_MINOR, "flags": flags or {},
                "modelID": model_id, "arch": arch, "quant": quant, "files": files, "expertsPerLayer": n_exp,
                "numLayers": len(layers), "expertStride": stride}
    with open(os.path.join(directory, "manifest.json"), "w") as f:
        json.dump(manifest, f, sort_keys=True)
    return manifest
