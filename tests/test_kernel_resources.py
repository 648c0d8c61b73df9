"""Build-time guard of the register budgets the kernels' speed depends on (CPU only: hipcc cross-compiles for gfx950).

The d = 64 kernels are tuned to the register counts at which one more wave fits a SIMD (128 VGPRs: four waves, 168: three).
One extra live register in a main loop silently costs a wave per SIMD or turns into scratch traffic, so the counts the
compiler reports (-Rpass-analysis=kernel-resource-usage) are pinned here for the variants the headline workloads run.
"""
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "flash-attention_amd"))
import build as fa_build  # noqa: E402


def _resources(src):
    cmd = [fa_build.HIPCC] + fa_build.FLAGS + ["-Rpass-analysis=kernel-resource-usage", "-c",
                                               os.path.join(fa_build.CSRC, src), "-o", os.devnull]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout[-2000:]
    out, name = {}, None
    for line in r.stdout.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            out[name] = {}
            continue
        m = re.search(r"remark:\s+([A-Za-z ]+?)(?: \[[^\]]*\])?: (\d+)", line)
        if m and name:
            out[name][m.group(1).strip()] = int(m.group(2))
    return out


def _pick(res, *parts):
    hits = [v for k, v in res.items() if all(p in k for p in parts)]
    assert len(hits) == 1, (parts, [k for k in res if parts[0] in k])
    return hits[0]


@pytest.mark.timeout(600)
def test_d64_kernels_keep_their_waves_per_simd():
    fwd = _resources("fa_fwd_d64.hip")
    bwd = _resources("fa_bwd_d64.hip")
    # <f16, 64, ..., causal, dropout, sparse, alibi, key split> mangled as ...IDF16_Li64E...Lb{0,1}E x3, Li{0,1,2}E for the score bias, Li{1,2}E
    # (the dK/dV kernel has no key-split parameter)
    plain, causal, dropout = "Lb0ELb0ELb0ELi0E", "Lb1ELb0ELb0ELi0E", "Lb0ELb1ELb0ELi0E"
    full = "Li1EEEv"
    # (the forward's last parameter: the dropout variant that also leaves its keep decisions for the backward)
    for flags, want in ((plain, 4), (causal, 4), (dropout, 3)):
        k = _pick(fwd, "fa_fwd_kernelIDF16_Li64E", flags + "Li1ELb0EEEv")
        # (the plain variant parks one register pair in scratch across its main loop: stored before, reloaded after)
        assert k["Occupancy"] >= want and k["VGPRs Spill"] <= (2 if flags == plain else 0), ("forward", flags, k)
        k = _pick(fwd, "fa_fwd_kernelIDF16_Li64E", flags + "Li2ELb0EEEv")  # half-size tiles
        assert k["Occupancy"] >= 4 and k["VGPRs Spill"] == 0, ("forward, key split", flags, k)
    k = _pick(fwd, "fa_fwd_kernelIDF16_Li64E", dropout + "Li1ELb1EEEv")
    assert k["Occupancy"] >= 3 and k["VGPRs Spill"] == 0, ("forward, keep words", k)
    k = _pick(fwd, "fa_fwd_kernelIDF16_Li64E", dropout + "Li2ELb1EEEv")
    # (scalar registers that do not fit are parked in lanes of a vector register, outside the main loop: a handful is fine)
    assert k["Occupancy"] >= 4 and k["VGPRs Spill"] == 0 and k["SGPRs Spill"] <= 8, ("forward, keep words, key split", k)
    # backward kernels: <..., causal, dropout mode (0 none, 1 drawn with Philox, 2 read from the forward's keep words),
    # sparse, alibi, ...>
    bplain, bcausal, bdrawn, bread = "Lb0ELi0ELb0ELi0E", "Lb1ELi0ELb0ELi0E", "Lb0ELi1ELb0ELi0E", "Lb0ELi2ELb0ELi0E"
    for flags, want in ((bplain, 3), (bcausal, 3), (bdrawn, 3), (bread, 3)):
        k = _pick(bwd, "fa_bwd_dq_kernelIDF16_Li64E", flags + full)
        assert k["Occupancy"] >= want and k["VGPRs Spill"] == 0, ("dq", flags, k)
        k = _pick(bwd, "fa_bwd_dq_kernelIDF16_Li64E", flags + "Li2EEEv")
        assert k["Occupancy"] >= 3 and k["VGPRs Spill"] == 0, ("dq, key split", flags, k)
    for flags, want, spill in ((bplain, 3, 2), (bcausal, 3, 2), (bdrawn, 2, 0), (bread, 2, 0)):
        k = _pick(bwd, "fa_bwd_dkdv_kernelIDF16_Li64E", flags + "Lb0EEEv")  # (last flag: the variant that turns dK back, rotary)
        assert k["Occupancy"] >= want and k["VGPRs Spill"] <= spill, ("dkdv", flags, k)
    # the ALiBi variants (fourth flag set) keep the waves per SIMD of their plain counterparts in the backward
    for flags, bflags in (("Lb0ELb0ELb0ELi1E", "Lb0ELi0ELb0ELi1E"), ("Lb1ELb0ELb0ELi1E", "Lb1ELi0ELb0ELi1E")):
        assert _pick(fwd, "fa_fwd_kernelIDF16_Li64E", flags + "Li1ELb0EEEv")["Occupancy"] >= 3, flags  # (the bias costs the fourth)
        assert _pick(bwd, "fa_bwd_dq_kernelIDF16_Li64E", bflags + full)["Occupancy"] >= 3, bflags
        k = _pick(bwd, "fa_bwd_dkdv_kernelIDF16_Li64E", bflags + "Lb0EEEv")
        assert k["Occupancy"] >= 3 and k["VGPRs Spill"] <= 4, (bflags, k)


@pytest.mark.timeout(600)
def test_d64_bias_tensor_and_one_kernel_backward_variants():
    """The variants that read a bias tensor run at three (forward without dropout) and two waves per SIMD; the dK/dV variant
    that also draws dropout decisions is at the register limit and may spill a few registers, the others must not.  The
    one-kernel backward runs two workgroups per compute unit: two waves per SIMD, nothing spilled, at most 80 KB of LDS."""
    fwd = _resources("fa_fwd_d64.hip")
    bwd = _resources("fa_bwd_d64.hip")
    for causal in ("Lb0E", "Lb1E"):
        k = _pick(fwd, "fa_fwd_kernelIDF16_Li64E", causal + "Lb0ELb0ELi2ELi1ELb0EEEv")
        assert k["Occupancy"] >= 3 and k["VGPRs Spill"] <= 3, ("forward, bias tensor", causal, k)
        for drop, words in (("Lb1E", "Lb0E"), ("Lb1E", "Lb1E")):
            k = _pick(fwd, "fa_fwd_kernelIDF16_Li64E", causal + drop + "Lb0ELi2ELi1E" + words + "EEv")
            assert k["Occupancy"] >= 2 and k["VGPRs Spill"] == 0, ("forward, bias tensor, dropout", causal, words, k)
        for drop, spill in (("Li0E", 0), ("Li2E", 4), ("Li1E", 16)):
            k = _pick(bwd, "fa_bwd_dq_kernelIDF16_Li64E", causal + drop + "Lb0ELi2ELi1EEEv")
            assert k["Occupancy"] >= 2 and k["VGPRs Spill"] == 0, ("dq, bias tensor", causal, drop, k)
            k = _pick(bwd, "fa_bwd_dkdv_kernelIDF16_Li64E", causal + drop + "Lb0ELi2ELb0EEEv")
            assert k["Occupancy"] >= 2 and k["VGPRs Spill"] <= spill, ("dkdv, bias tensor", causal, drop, k)
    # dQ and dK/dV in one launch (short launches): the register count of the dK/dV part, two waves per SIMD, nothing spilled
    for dt in ("IDF16_", "IDF16b"):
        for flags in ("Lb0ELi0E", "Lb0ELi2E", "Lb1ELi0E", "Lb1ELi2E"):
            k = _pick(bwd, "fa_bwd_merged_kernel" + dt, flags + "EEv")
            assert k["Occupancy"] >= 2 and k["VGPRs Spill"] == 0 and k["LDS Size"] <= 80 * 1024, ("merged backward", dt, flags, k)
    fused = _resources("fa_bwd_fused.hip")
    for dt in ("IDF16_", "IDF16b"):
        k = _pick(fused, "fa_bwd_fused_kernel%sLi64ELi0E" % dt)
        assert k["Occupancy"] >= 2 and k["VGPRs Spill"] == 0 and k["LDS Size"] <= 80 * 1024, ("one-kernel backward", dt, k)


@pytest.mark.timeout(600)
def test_d128_backward_keeps_two_waves_per_simd():
    """d = 128: the dK/dV kernel holds its V tile in LDS so that K, the two accumulators and the scores fit 256 registers
    (two waves per SIMD, nothing spilled: a spill's scratch load would wait behind the tile prefetch on every step)."""
    bwd = _resources("fa_bwd_d128.hip")
    for dt in ("IDF16_", "IDF16b"):
        # plain, causal, both with a block layout, and the two without that read the dropout decisions from keep words
        for flags in ("Lb0ELi0ELb0ELi0E", "Lb1ELi0ELb0ELi0E", "Lb0ELi0ELb1ELi0E", "Lb1ELi0ELb1ELi0E", "Lb0ELi2ELb0ELi0E",
                      "Lb1ELi2ELb0ELi0E"):
            k = _pick(bwd, "fa_bwd_dkdv_kernel%sLi128E" % dt, flags + "Lb0EEEv")
            assert k["Occupancy"] >= 2 and k["VGPRs Spill"] == 0 and k["LDS Size"] <= 80 * 1024, (dt, flags, k)
            k = _pick(bwd, "fa_bwd_dq_kernel%sLi128E" % dt, flags + "Li1EEEv")
            assert k["Occupancy"] >= 2 and k["VGPRs Spill"] <= (1 if "Lb1ELi0E" in flags[8:] else 0), ("dq", dt, flags, k)
        # the dK/dV kernel of wave pairs (launch policy 0x40) is built for three waves per SIMD and three workgroups' LDS
        for flags in ("Lb0ELb0E", "Lb1ELb0E", "Lb0ELb1E", "Lb1ELb1E"):
            k = _pick(bwd, "fa_bwd_dkdv_pair_kernel%s" % dt, flags + "EEv")
            assert k["Occupancy"] >= 3 and k["VGPRs Spill"] <= 2 and k["LDS Size"] <= 160 * 1024 // 3, (dt, flags, k)
