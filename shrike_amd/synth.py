"""Seeded synthetic tensors for the routed-expert path.

One generator serves the parity tests, the smoke run and the benchmark: SplitMix64
streams derived from a root seed by an FNV-1a hash of a label, the scheme of the
reference's test support (sources/ShrikeValidation/Support/PRNG/SplitMix64.swift:4-25,
SeedTree.swift:4-20), vectorised with numpy (SplitMix64 is counter-based: the i-th
output depends only on seed + i * gamma).

Distributions follow the benchmark definition: weight codes uniform over the code
range, scale = |N(0, 0.02)| rounded to the metadata dtype, bias = -(range/2) * scale,
activations N(0, 1) in fp16, router weights N(0, 0.02) in fp16; normals by Box-Muller
on 24-bit uniforms.
"""
from __future__ import annotations

import numpy as np

GROUP = 64
META_BF16, META_F16 = 0, 1
_GAMMA = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_MASK64 = (1 << 64) - 1


def fnv1a(label: str) -> int:
    h = 0xCBF29CE484222325
    for byte in label.encode("utf-8"):
        h ^= byte
        h = (h * 0x100000001B3) & _MASK64
    return h


class SplitMix64:
    """Vectorised SplitMix64; `next(n)` returns the next n outputs as uint64."""

    def __init__(self, seed: int):
        self.state = seed & _MASK64

    def next(self, n: int) -> np.ndarray:
        with np.errstate(over="ignore"):
            idx = np.arange(1, n + 1, dtype=np.uint64)
            z = np.uint64(self.state) + idx * _GAMMA
            self.state = (self.state + n * int(_GAMMA)) & _MASK64
            z = (z ^ (z >> np.uint64(30))) * _M1
            z = (z ^ (z >> np.uint64(27))) * _M2
            return z ^ (z >> np.uint64(31))

    def uniform(self, lo: float, hi: float, n: int) -> np.ndarray:
        """Uniform float32 in [lo, hi) with 24-bit resolution (SplitMix64.swift:20-23)."""
        u = (self.next(n) >> np.uint64(40)).astype(np.float32) / np.float32(1 << 24)
        return (np.float32(lo) + (np.float32(hi) - np.float32(lo)) * u).astype(np.float32)

    def bytes(self, n: int) -> np.ndarray:
        words = self.next((n + 7) // 8)
        return words.view(np.uint8)[:n].copy()

    def normal(self, n: int, std: float = 1.0) -> np.ndarray:
        """Box-Muller on 24-bit uniforms; float32."""
        m = (n + 1) // 2
        raw = self.next(2 * m)
        u1 = ((raw[:m] >> np.uint64(40)).astype(np.float64) + 1.0) / float(1 << 24)
        u2 = (raw[m:] >> np.uint64(40)).astype(np.float64) / float(1 << 24)
        r = np.sqrt(-2.0 * np.log(u1))
        z = np.concatenate([r * np.cos(2.0 * np.pi * u2), r * np.sin(2.0 * np.pi * u2)])[:n]
        return (z * std).astype(np.float32)


class SeedTree:
    def __init__(self, root: int):
        self.root = root & _MASK64

    def key(self, label: str) -> SplitMix64:
        return SplitMix64(self.root ^ fnv1a(label))


# ----------------------------------------------------------------- dtype helpers

def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    with np.errstate(over="ignore"):
        r = (u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)
    return r.astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_f16_bits(x: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(x, np.float32).astype(np.float16).view(np.uint16)


def f16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(b, np.uint16).view(np.float16).astype(np.float32)


def meta_bits(x: np.ndarray, meta: int) -> np.ndarray:
    return f32_to_f16_bits(x) if meta == META_F16 else f32_to_bf16_bits(x)


def meta_to_f32(b: np.ndarray, meta: int) -> np.ndarray:
    return f16_bits_to_f32(b) if meta == META_F16 else bf16_bits_to_f32(b)


# ------------------------------------------------------------------- blob layout

def expert_offsets(d: int, f: int, bits: int = 4, additive_biases: bool = False):
    """Byte offsets of the sub-tensors in one packed expert blob, in the packer's order
    gate W,S,B, up W,S,B, down W,S,B (sources/Shrike/Kernels/CPU/CPUExpertFFN.swift:43-60),
    generalised to 8-bit codes; optional additive biases follow. Returns (dict, stride)."""
    assert d % GROUP == 0 and f % GROUP == 0
    gw, gm = f * d * bits // 8, f * (d // GROUP) * 2
    dw, dm = d * f * bits // 8, d * (f // GROUP) * 2
    names = ["gate_w", "gate_s", "gate_b", "up_w", "up_s", "up_b", "down_w", "down_s", "down_b"]
    sizes = [gw, gm, gm, gw, gm, gm, dw, dm, dm]
    off, at = {}, 0
    for name, size in zip(names, sizes):
        off[name] = at
        at += size
    off["gate_ab"] = off["up_ab"] = off["down_ab"] = 0
    if additive_biases:
        for name, size in (("gate_ab", f * 2), ("up_ab", f * 2), ("down_ab", d * 2)):
            off[name] = at
            at += size
    return off, at


def affine_matrix(rng: SplitMix64, rows: int, n: int, bits: int, meta: int):
    """Random group-affine matrix: (codes uint8[rows, n*bits/8], scales u16[rows, n/64],
    biases u16[rows, n/64])."""
    codes = rng.bytes(rows * n * bits // 8).reshape(rows, n * bits // 8)
    # 8-bit codes span 16x the range of 4-bit ones: the scale shrinks by 16 so both widths
    # describe weights of the same spread (std 0.02 scales at 8 bits overflow fp16 outputs).
    std = 0.02 if bits == 4 else 0.02 / 16.0
    scale = np.abs(rng.normal(rows * (n // GROUP), std=std)).astype(np.float32)
    sbits = meta_bits(scale, meta)
    srounded = meta_to_f32(sbits, meta)
    half_range = np.float32(8.0 if bits == 4 else 128.0)
    bbits = meta_bits(-half_range * srounded, meta)  # exact: a power-of-two multiple
    return codes, sbits.reshape(rows, n // GROUP), bbits.reshape(rows, n // GROUP)


def expert_blob(tree: SeedTree, label: str, d: int, f: int, bits: int = 4,
                meta: int = META_BF16, additive_biases: bool = False) -> np.ndarray:
    off, stride = expert_offsets(d, f, bits, additive_biases)
    blob = np.zeros(stride, np.uint8)
    for name, rows, n in (("gate", f, d), ("up", f, d), ("down", d, f)):
        w, s, b = affine_matrix(tree.key(f"{label}.{name}"), rows, n, bits, meta)
        blob[off[f"{name}_w"]:off[f"{name}_w"] + w.size] = w.reshape(-1)
        blob[off[f"{name}_s"]:off[f"{name}_s"] + s.size * 2] = s.reshape(-1).view(np.uint8)
        blob[off[f"{name}_b"]:off[f"{name}_b"] + b.size * 2] = b.reshape(-1).view(np.uint8)
    if additive_biases:
        for name, n in (("gate_ab", f), ("up_ab", f), ("down_ab", d)):
            v = f32_to_bf16_bits(tree.key(f"{label}.{name}").normal(n, std=0.1))
            blob[off[name]:off[name] + n * 2] = v.view(np.uint8)
    return blob


def blob_views(blob: np.ndarray, d: int, f: int, bits: int = 4, additive_biases: bool = False):
    """Sub-tensor views of a blob as (w, s, b) triples keyed gate/up/down."""
    off, _ = expert_offsets(d, f, bits, additive_biases)
    out = {}
    for name, rows, n in (("gate", f, d), ("up", f, d), ("down", d, f)):
        wb, mb = rows * n * bits // 8, rows * (n // GROUP) * 2
        out[name] = (blob[off[f"{name}_w"]:off[f"{name}_w"] + wb],
                     blob[off[f"{name}_s"]:off[f"{name}_s"] + mb].view(np.uint16),
                     blob[off[f"{name}_b"]:off[f"{name}_b"] + mb].view(np.uint16))
    return out


def activations_f16(tree: SeedTree, label: str, n: int) -> np.ndarray:
    return f32_to_f16_bits(tree.key(label).normal(n, std=1.0))


def router_f16(tree: SeedTree, label: str, num_experts: int, d: int) -> np.ndarray:
    return f32_to_f16_bits(tree.key(label).normal(num_experts * d, std=0.02)).reshape(num_experts, d)


def quantize_affine(rows_f32: np.ndarray, bits: int, meta: int = META_BF16):
    """Min/max group-affine quantiser, the reference's fixture quantiser
    (sources/Shrike/Infrastructure/ModelIO/Quantization.swift:47-102, :135-177)."""
    rows, n = rows_f32.shape
    levels = np.float32((1 << bits) - 1)
    g = rows_f32.reshape(rows, n // GROUP, GROUP).astype(np.float32)
    lo, hi = g.min(axis=2), g.max(axis=2)
    const = hi == lo
    scale = np.where(const, np.float32(1), (hi - lo) / levels).astype(np.float32)
    sb, bb = meta_bits(scale, meta), meta_bits(lo, meta)
    s, b = meta_to_f32(sb, meta), meta_to_f32(bb, meta)
    inv = np.where(s == 0, np.float32(0), np.float32(1) / s).astype(np.float32)
    q = (g - b[..., None]) * inv[..., None]
    # Swift's .rounded() is round-half-away-from-zero
    q = np.clip(np.where(q >= 0, np.floor(q + np.float32(0.5)), np.ceil(q - np.float32(0.5))),
                0, levels).astype(np.uint8).reshape(rows, n)
    if bits == 4:
        q = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)
    return np.ascontiguousarray(q), sb, bb


# ------------------------------------------------------------------- packed experts directory

_ROLE_OF = {"gate_w": "gate", "gate_s": "gate_scales", "gate_b": "gate_biases", "up_w": "up", "up_s": "up_scales",
            "up_b": "up_biases", "down_w": "down", "down_s": "down_scales", "down_b": "down_biases",
            "gate_ab": "gate_bias", "up_ab": "up_bias", "down_ab": "down_bias"}


def packed_layout_tensors(d: int, f: int, bits: int = 4, additive_biases: bool = False) -> dict:
    """The `tensors` object of one expert in packed_experts/layout.json for a synthetic blob: role names as
    the runtime looks them up (sources/Shrike/Runtime/Inference/ModelExpertIO.swift:69-94), codes as "U32"
    words with their bit width, metadata as "BF16" (the file format has no other 16-bit type)."""
    off, _ = expert_offsets(d, f, bits, additive_biases)
    out = {}
    for name, rows, n in (("gate", f, d), ("up", f, d), ("down", d, f)):
        out[_ROLE_OF[f"{name}_w"]] = {"offset": off[f"{name}_w"], "size": rows * n * bits // 8, "dtype": "U32",
                                      "shape": [rows, n * bits // 32], "bits": bits}
        for part in ("s", "b"):
            out[_ROLE_OF[f"{name}_{part}"]] = {"offset": off[f"{name}_{part}"], "size": rows * (n // GROUP) * 2,
                                               "dtype": "BF16", "shape": [rows, n // GROUP]}
    if additive_biases:
        for name, n in (("gate_ab", f), ("up_ab", f), ("down_ab", d)):
            out[_ROLE_OF[name]] = {"offset": off[name], "size": n * 2, "dtype": "BF16", "shape": [n]}
    return out


def write_packed_experts(model_dir: str, layers: list, d: int, f: int, bits: int = 4, additive_biases: bool = False,
                         physical_rank=None, alignment: int = 16384) -> dict:
    """Writes <model_dir>/packed_experts/layout.json and one layer_NN.bin per populated layer
    (sources/ShrikeFormat/GTurboPackedExpertsLayoutV1.swift:3-62). layers[l] is the list of that layer's
    expert blobs by logical id, or [] for a dense layer. physical_rank(l, e) places expert e in the file
    (identity by default). The file stride is the blob size rounded up to `alignment`. Returns the
    layout as a dict."""
    import json
    import os
    _, blob_bytes = expert_offsets(d, f, bits, additive_biases)
    stride = (blob_bytes + alignment - 1) // alignment * alignment
    per_layer = max(len(blobs) for blobs in layers)
    root = os.path.join(model_dir, "packed_experts")
    os.makedirs(root, exist_ok=True)
    tensors = packed_layout_tensors(d, f, bits, additive_biases)
    out_layers = []
    for l, blobs in enumerate(layers):
        name = f"layer_{l:02d}.bin"
        experts = []
        if blobs:
            image = np.zeros(per_layer * stride, np.uint8)
            for e, blob in enumerate(blobs):
                rank = physical_rank(l, e) if physical_rank else e
                image[rank * stride:rank * stride + blob.size] = blob
                experts.append({"expert": e, "physicalRank": rank, "offset": rank * stride, "size": stride,
                                "tensors": tensors})
            image.tofile(os.path.join(root, name))
        out_layers.append({"layer": l, "file": name, "experts": experts})
    layout = {"expertStride": stride, "numLayers": len(layers), "expertsPerLayer": per_layer, "layers": out_layers}
    with open(os.path.join(root, "layout.json"), "w") as fh:
        json.dump(layout, fh, sort_keys=True)
    return layout
