"""Shared fixtures for the parity tests: seeded layers, the tolerance of the
benchmark definition, and device/oracle runners over the same bytes."""
from __future__ import annotations

import ctypes as C

import numpy as np

from oracle import oracle as O
from shrike_amd import synth as S

ABS_TOL, REL_TOL = 2e-3, 1e-3   # FFN outputs: max-abs 2e-3 / relative 1e-3 (benchmark definition)


def f16(bits: np.ndarray) -> np.ndarray:
    return S.f16_bits_to_f32(bits)


def assert_ffn_close(dev_bits: np.ndarray, ref_bits: np.ndarray, what: str = "", rel: float = REL_TOL):
    a, b = f16(dev_bits).astype(np.float64), f16(ref_bits).astype(np.float64)
    assert np.all(np.isfinite(b)), f"{what}: the oracle's output is not finite; the fixture is unusable"
    err = np.abs(a - b)
    bound = ABS_TOL + rel * np.abs(b)
    worst = int(np.argmax(err - bound))
    assert np.all(err <= bound), (
        f"{what}: element {worst}: device {a[worst]} vs oracle {b[worst]} "
        f"(|diff| {err[worst]:.3e} > {bound[worst]:.3e}); {int(np.sum(err > bound))} of {a.size} out of tolerance")


def assert_rel_close(dev_bits: np.ndarray, ref_bits: np.ndarray, what: str = "", tol: float = REL_TOL):
    """The reference's own metric (sources/ShrikeValidation/Support/Tolerance/RelError.swift:7-19):
    max |a - b| / max(max |b|, 1e-6). Used end to end, where fp16 roundings between the stages
    (gate/up -> act -> down) make single elements of a cancelling sum move by more than 2e-3."""
    a, b = f16(dev_bits).astype(np.float64), f16(ref_bits).astype(np.float64)
    assert np.all(np.isfinite(b)), f"{what}: the oracle's output is not finite"
    rel = np.max(np.abs(a - b)) / max(np.max(np.abs(b)), 1e-6)
    assert rel <= tol, f"{what}: relative error {rel:.3e} > {tol:.1e}"


class Layer:
    """One synthetic MoE layer: E routed expert blobs, router, optional shared expert."""

    def __init__(self, seed, d, f, num_experts, top_k, bits=4, meta=S.META_BF16, router_bits=0,
                 shared_f=0, shared_bits=None, additive_biases=False, label="layer.0"):
        self.d, self.f, self.ne, self.k = d, f, num_experts, top_k
        self.bits, self.meta, self.router_bits = bits, meta, router_bits
        self.additive = additive_biases
        tree = S.SeedTree(seed)
        self.tree = tree
        self.off, self.stride = S.expert_offsets(d, f, bits, additive_biases)
        self.blobs = [S.expert_blob(tree, f"{label}.expert.{e}", d, f, bits, meta, additive_biases)
                      for e in range(num_experts)]
        # router
        if router_bits == 0:
            self.router_w = S.router_f16(tree, f"{label}.router.w", num_experts, d)
            self.router_s = self.router_b = None
        else:
            dense = tree.key(f"{label}.router.w").normal(num_experts * d, std=0.02).reshape(num_experts, d)
            self.router_w, self.router_s, self.router_b = S.quantize_affine(dense, router_bits, meta)
        self.eff_scale = S.f32_to_bf16_bits(np.ones(d, np.float32))
        self.expert_scale = S.f32_to_bf16_bits(np.ones(num_experts, np.float32))
        self.logit_bias = S.f32_to_bf16_bits(np.zeros(num_experts, np.float32))
        self.x = S.activations_f16(tree, f"{label}.x", d)
        self.hidden = S.activations_f16(tree, f"{label}.hidden", d)
        # shared expert as separate resident tensors
        self.shared_f = shared_f
        self.shared_bits = shared_bits or bits
        if shared_f:
            sb = self.shared_bits
            self.shared = {name: S.affine_matrix(tree.key(f"{label}.shared.{name}"), rows, n, sb, meta)
                           for name, rows, n in (("gate", shared_f, d), ("up", shared_f, d), ("down", d, shared_f))}

    def oracle_offsets(self):
        off, stride = O.expert_offsets(self.d, self.f, self.bits, self.additive)
        assert stride == self.stride
        return off

    def router_dict(self):
        return dict(weights=self.router_w, scales=self.router_s, biases=self.router_b,
                    kind=self.router_bits, eff_scale=self.eff_scale, expert_scale=self.expert_scale,
                    bias=self.logit_bias, meta=self.meta)
