"""The C-ABI library loads without a GPU and exports exactly what include/*.h declare."""
import glob
import os
import re
import subprocess

from shrike_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    names = set()
    for path in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = re.sub(r"/\*.*?\*/", "", open(path).read(), flags=re.S)
        names |= set(re.findall(r"\b(shrike_[a-z0-9_]+)\s*\(", text))
    return names


def test_every_declared_symbol_is_exported_and_bound():
    lib = capi.load()
    declared = declared_functions()
    assert len(declared) > 60
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} is declared in include/ but not exported"
    assert declared == set(capi.SIGNATURES), (declared ^ set(capi.SIGNATURES))


def test_no_undeclared_exports():
    out = subprocess.run(["nm", "-D", "--defined-only", capi.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line}
    extra = {n for n in exported if n.startswith("shrike_")} - declared_functions()
    assert not extra, f"exported but not declared: {sorted(extra)}"


def test_pure_helpers_run_without_a_gpu():
    lib = capi.load()
    off = capi.ExpertOffsets()
    assert lib.shrike_expert_offsets_make(2048, 512, 4, 0, off) == 1_769_472
    assert (off.gate_s_off, off.up_w_off, off.down_w_off) == (524_288, 589_824, 1_179_648)
    assert lib.shrike_expert_offsets_make(2048, 512, 8, 0, off) == 3_342_336
    assert lib.shrike_expert_offsets_make(2048, 100, 4, 0, off) == 0  # not a multiple of the group size
    # ExpertCacheBudgetTests.swift:20-29, :85-89, :117-153
    assert lib.shrike_expert_cache_slots(1_769_472, 40, 8 << 30) == 128
    assert lib.shrike_expert_cache_slots(3_342_336, 40, 8 << 30) == 64
    assert lib.shrike_expert_cache_slots(1_769_472, 40, 11_324_620_800) == 160
    assert [lib.shrike_expert_cache_slots(1_769_472, 40, g << 30) for g in (1, 4, 8)] == [16, 64, 128]
    assert lib.shrike_expert_cache_slots(0, 40, 8 << 30) == 8 and lib.shrike_expert_cache_slots(1_769_472, 0, 8 << 30) == 8
    ok = {"8G": 8 << 30, "2g": 2 << 30, "512M": 512 << 20, "8GiB": 8 << 30, "1024KB": 1024 << 10, " 4G ": 4 << 30,
          "1073741824": 1 << 30, "1.5G": int(1.5 * (1 << 30)), "0.5G": 1 << 29}
    for text, want in ok.items():
        assert lib.shrike_parse_budget_bytes(text.encode()) == want, text
    for bad in ["", " ", "bogus", "G", "-2G", "0", "0G", "abcG", "2X", "2GG"]:
        assert lib.shrike_parse_budget_bytes(bad.encode()) == -1, bad


def test_budget_helpers_agree_with_the_restatement():
    from oracle import host_logic as H
    lib = capi.load()
    for stride in (1_769_472, 2_555_904, 3_342_336, 7_520_256, 13_996_800):
        for layers in (1, 24, 40, 48):
            for budget in (1 << 27, 1 << 30, 3 << 30, 8 << 30, 64 << 30, 11_324_620_800):
                assert lib.shrike_expert_cache_slots(stride, layers, budget) == H.expert_cache_slots(stride, layers, budget)
    for text in ["7G", "7.25gib", "12mb", "1e3K", " 3 M", "3 M ", "+5G", ".5G", "5.G", "1_0G", "٣G", "0x10G", "infG", "nanG", "9223372036854775807", "9223372036854775808"]:
        want = H.parse_budget_bytes(text)
        assert lib.shrike_parse_budget_bytes(text.encode()) == (-1 if want is None else want), text


def test_product_never_imports_the_oracle():
    for path in glob.glob(os.path.join(ROOT, "shrike_amd", "**", "*.py"), recursive=True):
        text = open(path).read()
        assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), path
