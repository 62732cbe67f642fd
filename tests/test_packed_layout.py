"""packed_experts/layout.json: the library's decoder, validator and expert-offset look-up against the
oracle's restatement and the reference's own test vectors
(tests/Shrike/Core/Infrastructure/ModelIO/PackedExpertsLayoutTests.swift,
tests/ShrikeRepack/Core/Planning/DenseLayerLayoutTests.swift)."""
import copy
import errno
import json
import os

import numpy as np
import pytest

from oracle import host_logic as HL
from shrike_amd import host, synth as S

STRIDE = 16384


def toy_layout():
    """PackedExpertsLayoutTests.swift:10-70: one layer, two experts, two sub-tensors each."""
    def tensors():
        return {"gate": {"offset": 0, "size": 4096, "dtype": "U32", "shape": [64, 64], "bits": 4},
                "gate_scales": {"offset": 4096, "size": 256, "dtype": "BF16", "shape": [64, 1]}}
    return {"expertStride": STRIDE, "numLayers": 1, "expertsPerLayer": 2,
            "layers": [{"layer": 0, "file": "layer_00.bin",
                        "experts": [{"expert": 0, "offset": 0, "size": STRIDE, "tensors": tensors()},
                                    {"expert": 1, "physicalRank": 1, "offset": STRIDE, "size": STRIDE,
                                     "tensors": tensors()}]}]}


def dense_layout(empty_layer):
    """DenseLayerLayoutTests.swift:18-35: three layers of two experts, one of them dense."""
    layers = []
    for l in range(3):
        experts = [] if l == empty_layer else [
            {"expert": e, "physicalRank": e, "offset": e * STRIDE, "size": STRIDE,
             "tensors": {"gate": {"offset": 0, "size": 64, "dtype": "U32", "shape": [8, 4], "bits": 4}}}
            for e in range(2)]
        layers.append({"layer": l, "file": f"layer_0{l}.bin", "experts": experts})
    return {"expertStride": STRIDE, "numLayers": 3, "expertsPerLayer": 2, "layers": layers}


def encode(layout) -> bytes:
    return json.dumps(layout, sort_keys=True).encode()


def view_of(lay: host.PackedExpertsLayout) -> dict:
    """The library's runtime view in the oracle's shape."""
    layers = []
    for i in range(lay.num_layers):
        info = lay.layer(i)
        experts = []
        for e in range(info["expert_count"]):
            x = lay.expert(i, e)
            experts.append(x)
        layers.append({"layer": info["layer"], "file": info["file"], "experts": experts})
    return {"expertStride": lay.expert_stride, "numLayers": lay.num_layers, "expertsPerLayer": lay.experts_per_layer,
            "layers": layers}


def assert_same_view(lay, ref):
    got = view_of(lay)
    assert (got["expertStride"], got["numLayers"], got["expertsPerLayer"]) == (
        ref["expertStride"], ref["numLayers"], ref["expertsPerLayer"])
    for i, (gl, rl) in enumerate(zip(got["layers"], ref["layers"])):
        assert (gl["layer"], gl["file"], len(gl["experts"])) == (rl["layer"], rl["file"], len(rl["experts"]))
        for e, (ge, re_) in enumerate(zip(gl["experts"], rl["experts"])):
            assert (ge["expert"], ge["physical_rank"], ge["offset"], ge["size"], ge["tensor_count"]) == (
                re_["logical"], re_["physical"], re_["offset"], re_["size"], len(re_["tensors"]))
            for name, t in re_["tensors"].items():
                assert lay.tensor(i, e, name) == {"offset": t["offset"], "size": t["size"], "dtype": t["dtype"],
                                                  "shape": t["shape"][:4], "bits": t["bits"]}
            assert lay.tensor(i, e, "no_such_role") is None


# ------------------------------------------------------------------ reference vectors

def test_decodes_the_reference_toy_layout(tmp_path):
    """PackedExpertsLayoutTests.decodesToyLayout (:72-90), through the file reader."""
    d = tmp_path / "packed_experts"
    d.mkdir()
    (d / "layout.json").write_bytes(encode(toy_layout()))
    lay = host.PackedExpertsLayout.load(str(tmp_path))
    assert (lay.expert_stride, lay.num_layers, lay.experts_per_layer) == (16384, 1, 2)
    e0, e1 = lay.expert(0, 0), lay.expert(0, 1)
    assert (e0["offset"], e0["size"]) == (0, 16384)
    assert lay.tensor(0, 0, "gate")["offset"] == 0
    assert lay.tensor(0, 0, "gate_scales")["offset"] == 4096
    assert (e1["offset"], e1["expert"]) == (16384, 1)
    assert_same_view(lay, HL.decode_packed_layout(encode(toy_layout())))


def test_missing_layout_is_a_missing_file(tmp_path):
    """PackedExpertsLayoutTests.missingLayoutJsonThrowsMissingFile (:92-107)."""
    (tmp_path / "packed_experts").mkdir()
    with pytest.raises(host.LayoutError, match="missing file") as e:
        host.PackedExpertsLayout.load(str(tmp_path))
    assert e.value.errno == errno.ENOENT


def test_oversized_layout_is_rejected_before_decoding(tmp_path):
    """PackedExpertsLayoutTests.oversizedLayoutRejectsBeforeDecode (:109-127): 64 blanks, cap 16."""
    d = tmp_path / "packed_experts"
    d.mkdir()
    (d / "layout.json").write_bytes(b" " * 64)
    with pytest.raises(host.LayoutError, match="metadata cap") as e:
        host.PackedExpertsLayout.load(str(tmp_path), max_bytes=16)
    assert e.value.errno == errno.EFBIG


def test_dense_layer_validates_and_partial_layer_does_not():
    """DenseLayerLayoutTests.emptyLayerValidatesStructurally / partialExpertCountStillRejected (:37-52)."""
    lay = host.PackedExpertsLayout.decode(encode(dense_layout(0)))
    assert lay.layer(0)["expert_count"] == 0 and lay.layer(1)["expert_count"] == 2
    assert_same_view(lay, HL.decode_packed_layout(encode(dense_layout(0))))
    bad = dense_layout(None)
    bad["numLayers"], bad["layers"] = 1, bad["layers"][:1]
    bad["layers"][0]["experts"] = bad["layers"][0]["experts"][:1]
    with pytest.raises(host.LayoutError, match="wrong expert count"):
        host.PackedExpertsLayout.decode(encode(bad))
    with pytest.raises(HL.LayoutInvalid, match="wrong expert count"):
        HL.decode_packed_layout(encode(bad))


def test_cross_validation_skips_a_dense_layers_file_only():
    """DenseLayerLayoutTests.crossValidateSkipsEmptyLayerFile / ...StillRequiresPopulatedLayerFiles (:54-79)."""
    lay = host.PackedExpertsLayout.decode(encode(dense_layout(0)))
    ref = HL.decode_packed_layout(encode(dense_layout(0)))
    sizes = {"packed_experts/layer_01.bin": 2 * STRIDE, "packed_experts/layer_02.bin": 2 * STRIDE}
    lay.cross_validate(3, 2, STRIDE, sizes)
    HL.cross_validate_layout(ref, 3, 2, STRIDE, sizes)
    del sizes["packed_experts/layer_02.bin"]
    with pytest.raises(host.LayoutError, match="missing or wrong layer size"):
        lay.cross_validate(3, 2, STRIDE, sizes)
    with pytest.raises(HL.LayoutInvalid, match="missing or wrong layer size"):
        HL.cross_validate_layout(ref, 3, 2, STRIDE, sizes)
    for dims in ((2, 2, STRIDE), (3, 4, STRIDE), (3, 2, 2 * STRIDE)):
        with pytest.raises(host.LayoutError, match="dimension mismatch"):
            lay.cross_validate(*dims, {})
    sizes = {"packed_experts/layer_01.bin": 2 * STRIDE, "packed_experts/layer_02.bin": STRIDE}
    with pytest.raises(host.LayoutError, match="missing or wrong layer size"):
        lay.cross_validate(3, 2, STRIDE, sizes)


# ------------------------------------------------------------------ every validator rule

def _mutations():
    """(name, mutate(layout), reason the reference's validator gives) — one per guard of
    GTurboV1StructuralValidator.validate (GTurboPackedExpertsLayoutV1.swift:76-163)."""
    def set_(path, value):
        def go(l):
            node = l
            for key in path[:-1]:
                node = node[key]
            node[path[-1]] = value
        return go
    E0 = ("layers", 0, "experts", 0)
    E1 = ("layers", 0, "experts", 1)
    G = E0 + ("tensors", "gate")
    dims = "invalid dimensions or stride"
    mapping = "duplicate or invalid expert mapping"
    shape = "invalid dtype or shape"
    return [
        ("zero layers", set_(("numLayers",), 0), dims),
        ("negative experts per layer", set_(("expertsPerLayer",), -1), dims),
        ("zero stride", set_(("expertStride",), 0), dims),
        ("unaligned stride", set_(("expertStride",), 16384 + 4096), dims),
        ("layer count mismatch", set_(("numLayers",), 2), dims),
        ("layer id out of range", set_(("layers", 0, "layer"), 1), "duplicate or invalid layer"),
        ("negative layer id", set_(("layers", 0, "layer"), -1), "duplicate or invalid layer"),
        ("empty file name", set_(("layers", 0, "file"), ""), "unsafe relative path"),
        ("absolute file name", set_(("layers", 0, "file"), "/layer.bin"), "unsafe relative path"),
        ("dot file name", set_(("layers", 0, "file"), ".."), "non-canonical path"),
        ("nested file name", set_(("layers", 0, "file"), "a/layer.bin"), "expected basename"),
        ("trailing slash", set_(("layers", 0, "file"), "layer.bin/"), "non-canonical path"),
        ("reserved file name", set_(("layers", 0, "file"), "Layout.JSON"), "reserved packed-expert filename"),
        ("mixed explicit ids", lambda l: l["layers"][0]["experts"][1].pop("expert"),
         "expert ids must be either all explicit or all positional"),
        ("expert id out of range", set_(E1 + ("expert",), 2), mapping),
        ("duplicate expert id", set_(E1 + ("expert",), 0), mapping),
        ("rank out of range", set_(E1 + ("physicalRank",), 2), mapping),
        ("duplicate rank", set_(E1 + ("physicalRank",), 0), mapping),
        ("duplicate offset", set_(E1 + ("offset",), 0), mapping),
        ("offset off its rank", set_(E1 + ("offset",), 2 * STRIDE), "offset or size does not match physical rank"),
        ("size off the stride", set_(E0 + ("size",), STRIDE - 1), "offset or size does not match physical rank"),
        ("unknown dtype", set_(G + ("dtype",), "F16"), shape),
        ("empty tensor", set_(G + ("size",), 0), shape),
        ("empty shape", set_(G + ("shape",), []), shape),
        ("zero dimension", set_(G + ("shape",), [64, 0]), shape),
        ("zero bits", set_(G + ("bits",), 0), shape),
        ("wide bits", set_(G + ("bits",), 33), shape),
        ("empty role name", lambda l: l["layers"][0]["experts"][0]["tensors"].update(
            {"": {"offset": 8192, "size": 16, "dtype": "U32", "shape": [4]}}), shape),
        ("range past the blob", set_(G + ("size",), STRIDE + 1), "range exceeds expert blob"),
        ("overlap", set_(E0 + ("tensors", "gate_scales", "offset"), 4095), "overlapping ranges gate and gate_scales"),
    ]


@pytest.mark.parametrize("name,mutate,reason", _mutations(), ids=[m[0] for m in _mutations()])
def test_validator_rules(name, mutate, reason):
    layout = toy_layout()
    mutate(layout)
    with pytest.raises(HL.LayoutInvalid) as ref:
        HL.decode_packed_layout(encode(layout))
    assert ref.value.reason == reason
    with pytest.raises(host.LayoutError) as got:
        host.PackedExpertsLayout.decode(encode(layout))
    assert got.value.errno == errno.EINVAL
    assert str(got.value) == f"layout.json: invalid {ref.value.field}: {reason}"


def test_duplicate_layers_and_file_names():
    layout = dense_layout(None)
    layout["layers"][2]["layer"] = 1
    with pytest.raises(host.LayoutError, match="duplicate or invalid layer"):
        host.PackedExpertsLayout.decode(encode(layout))
    layout = dense_layout(None)
    layout["layers"][2]["file"] = "LAYER_01.bin"  # the same name on a case-insensitive volume
    for decode, exc in ((host.PackedExpertsLayout.decode, host.LayoutError), (HL.decode_packed_layout, HL.LayoutInvalid)):
        with pytest.raises(exc, match="duplicate layer filename"):
            decode(encode(layout))


@pytest.mark.parametrize("text", [b"", b"{", b"[1, 2]", b'{"expertStride": 16384}', b'{"expertStride": "x"}',
                                  encode(toy_layout()) + b"x", encode(toy_layout()).replace(b"16384", b"16384.5", 1),
                                  encode(toy_layout()).replace(b'"layer": 0', b'"layer": null')])
def test_malformed_documents_are_decoding_errors(text):
    with pytest.raises(host.LayoutError, match="invalid packed_experts/layout.json") as e:
        host.PackedExpertsLayout.decode(text)
    assert e.value.errno == errno.EINVAL
    with pytest.raises(HL.LayoutInvalid):
        HL.decode_packed_layout(text)


def test_json_escapes_unknown_keys_and_null_optionals():
    layout = toy_layout()
    layout["comment"] = {"nested": [1, 2.5, True, None, "é\\\"\n"]}
    layout["layers"][0]["file"] = "läyer_00.bin"
    for e in layout["layers"][0]["experts"]:
        e["physicalRank"] = None
        e["tensors"]["gate_scales"]["bits"] = None
    for ensure_ascii in (True, False):
        text = json.dumps(layout, ensure_ascii=ensure_ascii).encode()
        lay = host.PackedExpertsLayout.decode(text)
        assert lay.layer(0)["file"] == "läyer_00.bin"
        assert_same_view(lay, HL.decode_packed_layout(text))


def test_positional_ids_and_permuted_physical_ranks():
    rng = np.random.default_rng(5)
    for trial in range(20):
        n_layers, per_layer = int(rng.integers(1, 5)), int(rng.integers(1, 9))
        stride = STRIDE * int(rng.integers(1, 4))
        positional = bool(rng.integers(0, 2))
        layers = []
        for l in rng.permutation(n_layers):
            ranks = rng.permutation(per_layer)
            ids = np.arange(per_layer) if positional else rng.permutation(per_layer)
            experts = []
            for pos in range(per_layer):
                logical = int(ids[pos])
                rank = int(ranks[logical])
                e = {"offset": rank * stride, "size": stride,
                     "tensors": {"down": {"offset": 1024, "size": 512, "dtype": "U32", "shape": [16, 8], "bits": 8},
                                 "gate": {"offset": 0, "size": 1024, "dtype": "U32", "shape": [16, 16], "bits": 4},
                                 "down_scales": {"offset": 1536 + 32 * logical, "size": 32, "dtype": "BF16", "shape": [16]}}}
                if not positional:
                    e["expert"] = logical
                e["physicalRank"] = rank
                experts.append(e)
            if rng.integers(0, 5) == 0:
                experts = []
            layers.append({"layer": int(l), "file": f"layer_{int(l):02d}.bin", "experts": experts})
        text = encode({"expertStride": stride, "numLayers": n_layers, "expertsPerLayer": per_layer, "layers": layers})
        lay = host.PackedExpertsLayout.decode(text)
        ref = HL.decode_packed_layout(text)
        assert_same_view(lay, ref)
        with pytest.raises(host.LayoutError, match=f"expert layout has {n_layers} layers; layer {n_layers} is out of range"):
            lay.expert(n_layers, 0)
        populated = [i for i in range(n_layers) if ref["layers"][i]["experts"]]
        for i in populated:
            with pytest.raises(host.LayoutError, match=f"layer {i} has {per_layer} experts; expert {per_layer} is out of range"):
                lay.expert(i, per_layer)


# ------------------------------------------------------------------ offsets for the kernels

@pytest.mark.parametrize("d,f,bits,additive", [(2048, 512, 4, False), (2880, 2880, 4, True), (2304, 1024, 8, False)])
def test_expert_offsets_come_from_expert_zero(tmp_path, d, f, bits, additive):
    """Model.routedExpertOffsets (ModelExpertIO.swift:69-94) on a written model directory: the offsets equal
    the packer's (CPUExpertFFN.Offsets), and the 4-bit 35B-A3B stride is the reference's 1,769,472."""
    written = S.write_packed_experts(str(tmp_path), [[], [np.zeros(1, np.uint8)] * 2], d, f, bits, additive)
    os.remove(tmp_path / "packed_experts" / "layer_01.bin")  # only the layout is read here
    lay = host.PackedExpertsLayout.load(str(tmp_path))
    off, blob_bytes = S.expert_offsets(d, f, bits, additive)
    assert lay.expert_stride == (blob_bytes + 16383) // 16384 * 16384
    if (d, f, bits) == (2048, 512, 4):
        assert lay.expert_stride == 1_769_472  # CPUExpertFFNTests.swift:56-67
    got = lay.expert_offsets(1, additive)
    names = ["gate_w", "gate_s", "gate_b", "up_w", "up_s", "up_b", "down_w", "down_s", "down_b", "gate_ab", "up_ab", "down_ab"]
    assert [getattr(got, n + "_off") for n in names] == [off[n] for n in names]
    ref = HL.decode_packed_layout(json.dumps(written).encode())
    assert [getattr(got, n + "_off") for n in names] == HL.routed_expert_offsets(ref, 1, additive)
    with pytest.raises(host.LayoutError, match="layer 0 has 0 experts; expert 0 is out of range"):
        lay.expert_offsets(0)
    if not additive:
        with pytest.raises(host.LayoutError, match="layer 1 expert blob is missing gate_bias"):
            lay.expert_offsets(1, True)
        with pytest.raises(HL.LayoutInvalid, match="missing gate_bias"):
            HL.routed_expert_offsets(ref, 1, True)


def test_missing_roles_read_as_offset_zero():
    lay = host.PackedExpertsLayout.decode(encode(toy_layout()))
    got = lay.expert_offsets(0)
    assert (got.gate_w_off, got.gate_s_off, got.gate_b_off, got.up_w_off, got.down_b_off) == (0, 4096, 0, 0, 0)
