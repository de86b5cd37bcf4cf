"""The .gturbo readers (nvmai_amd/gturbo.py) against the reference's own format tests
(PackedExpertsLayoutTests.swift, ResidentIndexTests.swift, ManifestReaderTests.swift) and the
rules of its validators.  Host logic only: no GPU, no HIP library call."""
import importlib.util
import json
import os
import struct
import sys

import numpy as np
import pytest

# the module itself needs neither torch nor the HIP library: load it without the package's __init__
_spec = importlib.util.spec_from_file_location(
    "nvmai_gturbo", os.path.join(os.path.dirname(__file__), "..", "nvmai_amd", "gturbo.py"))
G = importlib.util.module_from_spec(_spec)
sys.modules["nvmai_gturbo"] = G
_spec.loader.exec_module(G)


def _toy_layout():
    """PackedExpertsLayoutTests.writeToyLayout (PackedExpertsLayoutTests.swift:9-72)."""
    tensors = {"gate": {"offset": 0, "size": 4096, "dtype": "U32", "shape": [64, 64], "bits": 4},
               "gate_scales": {"offset": 4096, "size": 256, "dtype": "BF16", "shape": [64, 1]}}
    return {"expertStride": 16384, "numLayers": 1, "expertsPerLayer": 2,
            "layers": [{"layer": 0, "file": "layer_00.bin",
                        "experts": [{"expert": 0, "offset": 0, "size": 16384, "tensors": tensors},
                                    {"expert": 1, "physicalRank": 1, "offset": 16384, "size": 16384, "tensors": tensors}]}]}


def _write_layout(tmp_path, root):
    d = tmp_path / "packed_experts"
    d.mkdir(parents=True, exist_ok=True)
    (d / "layout.json").write_text(json.dumps(root, sort_keys=True))
    return str(tmp_path)


def test_decodes_toy_layout(tmp_path):
    # PackedExpertsLayoutTests.swift:74-91
    layout = G.load_layout(_write_layout(tmp_path, _toy_layout()))
    assert (layout.expertStride, layout.numLayers, layout.expertsPerLayer, len(layout.layers)) == (16384, 1, 2, 1)
    e0 = layout.expert(0, 0)
    assert (e0.offset, e0.size) == (0, 16384)
    assert e0.subTensors["gate"].offset == 0 and e0.subTensors["gate_scales"].offset == 4096
    e1 = layout.expert(0, 1)
    assert e1.offset == 16384 and e1.expert == 1
    with pytest.raises(G.ModelError) as e:              # PackedExpertsLayout.swift:58-70
        layout.expert(0, 2)
    assert e.value.kind == "indexCorrupt" and "expert 2 is out of range" in e.value.detail
    with pytest.raises(G.ModelError):
        layout.expert(1, 0)


def test_missing_and_oversized_layout(tmp_path):
    # PackedExpertsLayoutTests.swift:93-126
    (tmp_path / "packed_experts").mkdir()
    with pytest.raises(G.ModelError) as e:
        G.load_layout(str(tmp_path))
    assert e.value.kind == "missingFile"
    (tmp_path / "packed_experts" / "layout.json").write_bytes(b" " * 64)
    with pytest.raises(G.ModelError) as e:
        G.load_layout(str(tmp_path), max_bytes=16)
    assert e.value.kind == "indexCorrupt" and "metadata cap" in e.value.detail


def _bad(root, reason):
    with pytest.raises(G.ModelError) as e:
        G.decode_layout(json.dumps(root).encode())
    assert e.value.kind == "indexCorrupt" and reason in e.value.detail, e.value.detail


def test_layout_structural_rules():
    # GTurboV1StructuralValidator.validate, GTurboPackedExpertsLayoutV1.swift:75-160, rule by rule
    r = _toy_layout(); r["expertStride"] = 16000
    _bad(r, "invalid dimensions or stride")
    r = _toy_layout(); r["numLayers"] = 2
    _bad(r, "invalid dimensions or stride")
    r = _toy_layout(); r["layers"][0]["layer"] = 1
    _bad(r, "duplicate or invalid layer")
    r = _toy_layout(); r["layers"][0]["file"] = "sub/layer.bin"
    _bad(r, "expected basename")
    r = _toy_layout(); r["layers"][0]["file"] = "../layer.bin"
    _bad(r, "non-canonical path")
    r = _toy_layout(); r["layers"][0]["file"] = "Layout.JSON"
    _bad(r, "reserved packed-expert filename")
    r = _toy_layout(); r["layers"][0]["experts"].pop()
    _bad(r, "wrong expert count")
    r = _toy_layout(); del r["layers"][0]["experts"][1]["expert"]
    _bad(r, "either all explicit or all positional")
    r = _toy_layout(); r["layers"][0]["experts"][1]["expert"] = 0
    _bad(r, "duplicate or invalid expert mapping")
    r = _toy_layout(); r["layers"][0]["experts"][1]["offset"] = 32768
    _bad(r, "does not match physical rank")
    r = _toy_layout(); r["layers"][0]["experts"][0]["size"] = 8192
    _bad(r, "does not match physical rank")
    r = _toy_layout(); r["layers"][0]["experts"][0]["tensors"]["gate"]["dtype"] = "FP16"
    _bad(r, "invalid dtype or shape")
    r = _toy_layout(); r["layers"][0]["experts"][0]["tensors"]["gate"]["shape"] = [64, 0]
    _bad(r, "invalid dtype or shape")
    r = _toy_layout(); r["layers"][0]["experts"][0]["tensors"]["gate_scales"]["offset"] = 16300
    _bad(r, "range exceeds expert blob")
    r = _toy_layout(); r["layers"][0]["experts"][0]["tensors"]["gate_scales"]["offset"] = 4000
    _bad(r, "overlapping ranges")
    r = _toy_layout(); del r["layers"][0]["experts"][0]["tensors"]["gate"]["size"]
    _bad(r, "packed_experts/layout.json")               # a missing key fails the decode itself
    r = _toy_layout(); r["layers"][0]["experts"][0]["offset"] = -1
    _bad(r, "packed_experts/layout.json")
    # positional ids and a permuted physical order are fine; experts come back in logical order
    r = _toy_layout()
    for e in r["layers"][0]["experts"]:
        e.pop("expert", None); e.pop("physicalRank", None)
    assert [e.expert for e in G.decode_layout(json.dumps(r).encode()).layers[0].experts] == [0, 1]
    r = _toy_layout()
    r["layers"][0]["experts"][0].update(physicalRank=1, offset=16384)
    r["layers"][0]["experts"][1].update(physicalRank=0, offset=0)
    lay = G.decode_layout(json.dumps(r).encode()).layers[0]
    assert [(e.expert, e.physicalRank, e.offset) for e in lay.experts] == [(0, 1, 16384), (1, 0, 0)]


def _index_file(names, entries_rel, resident_bytes):
    index, absolute = G.encode_resident_index(entries_rel, resident_bytes)
    return index + bytes(resident_bytes), absolute


def test_resident_index_roundtrip(tmp_path):
    # ResidentIndexTests.swift:14-100: two entries with distinct shapes, sizes and bias offsets
    names = ["embedding.weight", "layer.0.q_proj.weight"]
    rel = [G.ResidentEntry(names[0], 0, 0, 32, (1024, 64, 0, 0), 32, 16, 48, 16),
           G.ResidentEntry(names[1], 0, 64, 32, (256, 64, 0, 0))]
    data, absolute = _index_file(names, rel, 96)
    # the bytes themselves, field by field (GTurboEncoders.swift:12-45): header, then 72-byte records
    aligned = 16384
    assert struct.unpack_from("<QQQ", data, 0) == (aligned, 96, 2)
    table = 24 + 2 * 72
    assert struct.unpack_from("<IHBB", data, 24) == (table, len(names[0]), 0, 0)
    assert struct.unpack_from("<QQ", data, 24 + 8) == (aligned, 32)
    assert struct.unpack_from("<IIII", data, 24 + 24) == (1024, 64, 0, 0)
    assert struct.unpack_from("<QQQQ", data, 24 + 40) == (aligned + 32, 16, aligned + 48, 16)
    assert struct.unpack_from("<IH", data, 24 + 72) == (table + len(names[0]), len(names[1]))
    assert data[table:table + len(names[0])] == names[0].encode()
    path = tmp_path / "model_weights.bin"
    path.write_bytes(data)
    header, entries = G.load_resident_index(str(path))
    assert header == (aligned, 96, 2)
    e0, e1 = entries[names[0]], entries[names[1]]
    assert e0.shape[:2] == (1024, 64) and (e0.fileOffset, e0.sizeBytes) == (aligned, 32)
    assert (e0.scaleOffset, e0.scaleSize, e0.biasOffset, e0.biasSize) == (aligned + 32, 16, aligned + 48, 16)
    assert e1.shape[:2] == (256, 64) and (e1.fileOffset, e1.sizeBytes) == (aligned + 64, 32)
    assert e1.scaleSize == 0 and e1.biasSize == 0
    assert [entries[n] for n in names] == absolute
    # ResidentIndexTests.swift:102-113
    short = tmp_path / "short.bin"
    short.write_bytes(bytes(8))
    with pytest.raises(G.ModelError) as e:
        G.load_resident_index(str(short))
    assert e.value.kind == "indexCorrupt"


def test_resident_index_rules():
    # GTurboResidentIndexCodec.decodeRegion, GTurboResidentIndexV1.swift:53-150
    rel = [G.ResidentEntry("a", 0, 0, 32, (4, 8, 0, 0), 32, 16, 48, 16), G.ResidentEntry("b", 1, 64, 32, (4, 0, 0, 0))]
    good, _ = _index_file(None, rel, 96)

    def bad(mutate, kind, text):
        buf = bytearray(good)
        mutate(buf)
        with pytest.raises(G.FormatError) as e:
            G.decode_resident_region(bytes(buf), G.decode_resident_header(bytes(buf)))
        assert e.value.kind == kind and text in str(e.value), str(e.value)

    assert len(G.decode_resident_region(good, G.decode_resident_header(good))) == 2
    bad(lambda b: struct.pack_into("<Q", b, 0, 16000), "truncated", "resident.index")              # not 16 KB aligned
    bad(lambda b: struct.pack_into("<Q", b, 0, 64 << 20), "invalid", "metadata cap")
    bad(lambda b: struct.pack_into("<Q", b, 16, 1000), "invalid", "outside index")                 # entry table too long
    bad(lambda b: struct.pack_into("<B", b, 24 + 7, 1), "invalid", "reserved")
    bad(lambda b: struct.pack_into("<I", b, 24, 30), "invalid", "string table")                    # name inside the table
    bad(lambda b: struct.pack_into("<B", b, 24 + 6, 9), "invalid", "unknown dtype")
    bad(lambda b: struct.pack_into("<I", b, 24 + 24, 0), "invalid", "first dimension")
    bad(lambda b: struct.pack_into("<II", b, 24 + 28, 0, 5), "invalid", "trailing")
    bad(lambda b: struct.pack_into("<Q", b, 24 + 16, 0), "invalid", "primary payload is empty")
    bad(lambda b: struct.pack_into("<Q", b, 24 + 8, 100), "invalid", "outside resident payload")   # before the payload
    bad(lambda b: struct.pack_into("<Q", b, 24 + 16, 4096), "invalid", "outside resident payload")  # past its end
    bad(lambda b: struct.pack_into("<Q", b, 24 + 72 + 40, 7), "invalid", "absent payload offset")   # scales absent, offset set
    bad(lambda b: struct.pack_into("<Q", b, 24 + 72 + 8, 16384 + 40), "invalid", "overlaps")
    bad(lambda b: b.__setitem__(slice(24 + 2 * 72 + 1, 24 + 2 * 72 + 2), b"a"), "invalid", "duplicate")
    with pytest.raises(G.FormatError) as e:
        G.decode_resident_header(bytes(8))
    assert e.value.kind == "truncated"


def _arch(layers=2, experts=4):
    return {"hiddenSize": 128, "ffnIntermediate": 256, "moeIntermediateSize": 64, "numHeads": 4, "numKVHeads": 2,
            "numFullKVHeads": 2, "headDim": 32, "fullHeadDim": 32, "vocabSize": 100, "slidingWindow": 0,
            "finalLogitSoftcap": 0.0, "ropeTheta": 10000.0, "fullRopeTheta": 1e7, "partialRotaryFactor": 0.25,
            "numLayers": layers, "numExperts": experts, "topKExperts": 2, "tieWordEmbeddings": False,
            "attentionKEqV": False, "hiddenActivation": "silu", "fullAttentionLayerMask": [0, 1][:layers]}


def _slot(bits):
    return {"weightBits": bits, "scheme": "affine", "scaleType": "bf16", "biasType": "bf16", "groupSize": 64}


def _manifest(**over):
    m = {"magic": "GTURBO", "versionMajor": 1, "versionMinor": 0, "flags": {"streamingPresent": True}, "modelID": "toy",
         "arch": _arch(), "quant": {k: _slot(4) for k in ("embedding", "attention", "router", "sharedExpert", "routedExpert")},
         "files": {"model_weights.bin": {"size": 10, "sha256": "ab" * 32},
                   "packed_experts/layout.json": {"size": 10, "sha256": "00" * 32}},
         "expertsPerLayer": 4, "numLayers": 2, "expertStride": 32768}
    m.update(over)
    return m


def test_manifest_rules():
    # GTurboManifestCodec.validate (GTurboManifestV1.swift:159-255) with ManifestReaderTests.swift's cases
    good = G.decode_manifest(json.dumps(_manifest()).encode())
    assert good.modelID == "toy" and good.quant["routedExpert"].weightBits == 4 and good.arch["hiddenSize"] == 128

    def bad(text, **over):
        with pytest.raises(G.FormatError) as e:
            G.decode_manifest(json.dumps(_manifest(**over)).encode())
        assert text in str(e.value), str(e.value)

    bad("expected GTURBO", magic="GTURB0")                                  # wrongMagic
    bad("unsupported version", versionMajor=2)                              # versionTwo
    bad("unknown v1 flag", flags={"turboQuant": True})                      # unknownFlag / removed flag
    bad("invalid dimensions or stride", expertStride=32000)                 # nonPageAlignedExpertStride
    bad("invalid dimensions or stride", modelID="")
    bad("disagree with streaming metadata", numLayers=3)                    # archMismatch
    a = _arch(); a["topKExperts"] = 9
    bad("invalid architecture values", arch=a)
    a = _arch(); a["fullAttentionLayerMask"] = [0, 3]
    bad("invalid architecture values", arch=a)
    a = _arch(); a["partialRotaryFactor"] = 1.5
    bad("invalid architecture values", arch=a)
    q = {k: _slot(4) for k in ("embedding", "attention", "router", "sharedExpert", "routedExpert")}
    q["router"] = _slot(0)
    bad("manifest.quant.router", quant=q)
    bad("expected 64 hexadecimal", files={"model_weights.bin": {"size": 1, "sha256": "xyz"}})
    bad("reserved artifact filename", files={"manifest.json": {"size": 1, "sha256": "0" * 64}})
    bad("unsafe relative path", files={"/etc/passwd": {"size": 1, "sha256": "0" * 64}})
    bad("filesystem-equivalent duplicate", files={"A.bin": {"size": 1, "sha256": "0" * 64}, "a.bin": {"size": 1, "sha256": "0" * 64}})
    bad("collides with a directory prefix", files={"a": {"size": 1, "sha256": "0" * 64}, "a/b": {"size": 1, "sha256": "0" * 64}})
    a = _arch(); del a["vocabSize"]
    bad("manifest.json", arch=a)                                            # a missing key fails the decode
    # quant may be absent (GTurboManifestV1.swift:108); the codec accepts it
    assert G.decode_manifest(json.dumps(_manifest(quant=None)).encode()).quant is None


def test_cross_validation_against_the_manifest():
    # GTurboV1StructuralValidator.crossValidate, GTurboPackedExpertsLayoutV1.swift:172-196
    lay = _toy_layout()
    files = {"packed_experts/layer_00.bin": {"size": 32768, "sha256": "0" * 64}}
    a = _arch(1, 2); a["topKExperts"] = 1
    m = G.decode_manifest(json.dumps(_manifest(arch=a, files=files, expertsPerLayer=2, numLayers=1, expertStride=16384)).encode())
    assert G.decode_layout(json.dumps(lay).encode(), m).numLayers == 1
    files["packed_experts/layer_00.bin"]["size"] = 16384
    m2 = G.decode_manifest(json.dumps(_manifest(arch=a, files=files, expertsPerLayer=2, numLayers=1, expertStride=16384)).encode())
    with pytest.raises(G.ModelError) as e:
        G.decode_layout(json.dumps(lay).encode(), m2)
    assert "missing or wrong layer size" in e.value.detail
    a3 = _arch(1, 2); a3["topKExperts"] = 1
    m3 = G.decode_manifest(json.dumps(_manifest(arch=a3, files=files, expertsPerLayer=2, numLayers=1, expertStride=32768)).encode())
    with pytest.raises(G.ModelError) as e:
        G.decode_layout(json.dumps(lay).encode(), m3)
    assert "dimension mismatch" in e.value.detail


def _toy_model(tmp_path, rng, bits=4, layers=2, experts=4, d=128, f=64, ranks=None, shared_bits=None, shared_store_bits=None):
    """A complete directory: routed experts (random bytes in the nine roles at the layout of
    CPUExpertFFN.Offsets), router / shared expert / shared gate rows in the resident file."""
    wg, aux_g = f * d * bits // 8, f * (d // 64) * 2
    wd, aux_d = d * f * bits // 8, d * (f // 64) * 2
    sizes = [wg, aux_g, aux_g, wg, aux_g, aux_g, wd, aux_d, aux_d]
    shapes = [(f, d), (f, d // 64), (f, d // 64)] * 2 + [(d, f), (d, f // 64), (d, f // 64)]
    roles = ["gate", "gate_scales", "gate_biases", "up", "up_scales", "up_biases", "down", "down_scales", "down_biases"]
    tensors, at = {}, 0
    for role, size, shape in zip(roles, sizes, shapes):
        packed = not role.endswith(("scales", "biases"))
        tensors[role] = G.SubTensorEntry(at, size, "U32" if packed else "BF16", shape, bits if packed else None)
        at += size
    stride = (at + 16383) // 16384 * 16384
    lays = []
    for _ in range(layers):
        blobs = np.zeros((experts, stride), np.uint8)
        blobs[:, :at] = rng.integers(0, 256, (experts, at), dtype=np.uint8)
        lays.append({"blobs": blobs, "tensors": tensors, "ranks": ranks})
    resident = []
    sbits = shared_bits or bits                         # what the manifest says about the shared expert
    wbits = shared_store_bits or sbits                  # what its arrays were really written at
    for L in range(layers):
        p = "language_model.model.layers.%d.mlp." % L
        resident.append((p + "gate.weight", 1, (experts, d), rng.integers(0, 256, experts * d * 2, dtype=np.uint8).tobytes(), None, None))
        for proj, (rows, cols) in (("gate_proj", (f, d)), ("up_proj", (f, d)), ("down_proj", (d, f))):
            resident.append((p + "shared_expert.%s.weight" % proj, 0, (rows, cols),
                             rng.integers(0, 256, rows * cols * wbits // 8, dtype=np.uint8).tobytes(),
                             rng.integers(0, 256, rows * (cols // 64) * 2, dtype=np.uint8).tobytes(),
                             rng.integers(0, 256, rows * (cols // 64) * 2, dtype=np.uint8).tobytes()))
        resident.append((p + "shared_expert_gate.weight", 1, (1, d), rng.integers(0, 256, d * 2, dtype=np.uint8).tobytes(), None, None))
    quant = {k: _slot(bits) for k in ("embedding", "attention", "router", "sharedExpert", "routedExpert")}
    quant["sharedExpert"] = _slot(sbits)
    a = _arch(layers, experts)
    a.update(hiddenSize=d, moeIntermediateSize=f)
    G.write_model(str(tmp_path), a, quant, lays, resident)
    return lays, resident, tensors, stride


def test_model_directory_roundtrip(tmp_path):
    rng = np.random.default_rng(5)
    ranks = [2, 0, 3, 1]                                # physical rank of logical expert e
    lays, resident, tensors, stride = _toy_model(tmp_path, rng, ranks=ranks)
    m = G.GTurboModel(str(tmp_path))
    assert m.layout.expertStride == stride and m.manifest.files["model_weights.bin"]["size"] == sum(m.header[:2])
    for L in range(2):
        blobs = m.expert_blobs(L)
        assert np.array_equal(np.asarray(blobs), lays[L]["blobs"])          # logical order restored
        raw = np.fromfile(os.path.join(str(tmp_path), "packed_experts", "layer_%02d.bin" % L), np.uint8).reshape(4, stride)
        for e in range(4):
            assert np.array_equal(raw[ranks[e]], lays[L]["blobs"][e])       # and the file holds them by rank
        assert G.routed_expert_offsets(m.layout, L) == tuple(tensors[r].offset for r in G._ROLES)
    for name, dtype, shape, w, s, b in resident:
        gw, gs, gb, e = m.resident(name)
        assert bytes(gw) == w and e.dtype == dtype and e.shape[:len(shape)] == tuple(shape)
        assert (gs is None) == (s is None) and (s is None or gs.tobytes() == s) and (b is None or gb.tobytes() == b)
    blob = m.shared_expert_blob(1)
    gw = m.resident("language_model.model.layers.1.mlp.shared_expert.down_proj.weight")[0]
    assert bytes(blob[tensors["down"].offset:tensors["down"].offset + tensors["down"].size]) == bytes(gw)
    # the schema check of Model.validateRoutedExpertLayout (Model.swift:845-905)
    G.validate_routed_expert_layout(m.layout, 128, 64, 4, 64)
    with pytest.raises(G.ModelError) as e:
        G.validate_routed_expert_layout(m.layout, 128, 64, 8, 64)
    assert "does not match the required schema" in e.value.detail
    with pytest.raises(G.ModelError) as e:
        G.validate_routed_expert_layout(m.layout, 128, 64, 4, 48)
    assert "invalid quant layout" in e.value.detail
    # a layer file that went missing, a weights file that was cut short (Model.swift:640-650)
    os.rename(os.path.join(str(tmp_path), "packed_experts", "layer_01.bin"), os.path.join(str(tmp_path), "x.bin"))
    with pytest.raises(G.ModelError) as e:
        G.GTurboModel(str(tmp_path))
    assert e.value.kind == "missingFile"
    os.rename(os.path.join(str(tmp_path), "x.bin"), os.path.join(str(tmp_path), "packed_experts", "layer_01.bin"))
    with open(os.path.join(str(tmp_path), "model_weights.bin"), "ab") as f:
        f.write(b"\0")
    with pytest.raises(G.ModelError) as e:
        G.GTurboModel(str(tmp_path))
    assert e.value.kind == "indexCorrupt" and "indexSize" in e.value.detail
    os.remove(os.path.join(str(tmp_path), "manifest.json"))
    with pytest.raises(G.ModelError) as e:              # ManifestReaderTests.swift:214-225
        G.GTurboModel(str(tmp_path))
    assert e.value.kind == "partialInstall"


def test_shared_expert_of_another_width_than_the_routed_experts(tmp_path):
    # the reference keeps separate quant slots for the two (Model.swift:59-60) and its repacker's default
    # profile is sharedExpert = 8, routedExpert = 4 (RemoteStreamingRepacker.swift:678-683): the shared
    # expert's blob is then laid out at its own width, never squeezed into the routed sub-tensor regions
    rng = np.random.default_rng(6)
    d, f = 128, 64
    lays, resident, tensors, stride = _toy_model(tmp_path / "mixed", rng, bits=4, shared_bits=8, d=d, f=f)
    m = G.GTurboModel(str(tmp_path / "mixed"))
    assert not m.shared_matches_routed()
    off, size, bits = m.shared_expert_offsets(0)
    wg, aux_g, wd, aux_d = f * d, f * (d // 64) * 2, d * f, d * (f // 64) * 2
    assert bits == 8 and size == 2 * (wg + 2 * aux_g) + wd + 2 * aux_d          # CPUExpertFFN.Offsets at 8 bits
    assert off == (0, wg, wg + aux_g, wg + 2 * aux_g, 2 * wg + 2 * aux_g, 2 * wg + 3 * aux_g,
                   2 * wg + 4 * aux_g, 2 * wg + 4 * aux_g + wd, 2 * wg + 4 * aux_g + wd + aux_d)
    blob = m.shared_expert_blob(1)
    assert blob.size == size
    for i, proj in enumerate(("gate_proj", "up_proj", "down_proj")):
        w, s, b, _ = m.resident("language_model.model.layers.1.mlp.shared_expert.%s.weight" % proj)
        for arr, at in ((w, off[3 * i]), (s.view(np.uint8), off[3 * i + 1]), (b.view(np.uint8), off[3 * i + 2])):
            assert bytes(blob[at:at + arr.size]) == bytes(arr)                  # every array whole, none overlapping
    with pytest.raises(G.ModelError) as e:              # it cannot be a row of the routed pool
        m.expert_pool(0, device="cpu")
    assert e.value.kind == "unsupportedArch"
    # same width: the routed offsets, as before
    _toy_model(tmp_path / "same", rng, bits=4, d=d, f=f)
    m2 = G.GTurboModel(str(tmp_path / "same"))
    assert m2.shared_matches_routed() and m2.shared_expert_offsets(0)[:2] == (G.routed_expert_offsets(m2.layout, 0), stride)
    # arrays that are not of the width the manifest states are refused, not copied over their neighbours
    _toy_model(tmp_path / "lying", rng, bits=4, shared_bits=4, shared_store_bits=8, d=d, f=f)
    m3 = G.GTurboModel(str(tmp_path / "lying"))
    with pytest.raises(G.ModelError) as e:
        m3.shared_expert_blob(0)
    assert e.value.kind == "indexCorrupt" and "needs" in e.value.detail
