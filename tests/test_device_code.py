"""Properties of the compiled gfx950 device code that the arithmetic contract and the target
machine rely on, checked on the assembly hipcc emits for the package's own kernels (no GPU needed).
"""
import os
import re
import shutil
import subprocess

import pytest

from ramtorch_amd import build as B


@pytest.fixture(scope="module")
def device_asm(tmp_path_factory):
    if shutil.which(B.hipcc()) is None and not os.path.exists(B.hipcc()):
        pytest.skip("hipcc not available")
    out = tmp_path_factory.mktemp("asm") / "api.s"
    flags = [f for f in B.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    cmd = [B.hipcc(), *flags, "-S", "--cuda-device-only", "-o", str(out)] + [os.path.join(B.CSRC, s) for s in B.SOURCES]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    return out.read_text()


def _mnemonics(asm):
    return set(re.findall(r"^\s+([a-z][a-z0-9_]+)\s", asm, flags=re.M))


def test_no_mixed_precision_fma_and_no_packed_fp32(device_asm):
    """Every rounding is part of the contract: an fp32 result that is stored as fp16 must be rounded
    to fp32 first (a v_fma_mix* instruction rounds once, straight to fp16), and no packed-fp32
    arithmetic may be formed."""
    ops = _mnemonics(device_asm)
    bad = sorted(o for o in ops if o.startswith(("v_fma_mix", "v_mad_mix")) or
                 re.fullmatch(r"v_pk_(add|mul|fma)_f32(_e64)?", o))
    assert not bad, bad


def test_division_and_sqrt_are_the_correctly_rounded_sequences(device_asm):
    ops = _mnemonics(device_asm)
    assert any(o.startswith("v_div_fixup_f32") for o in ops) and any(o.startswith("v_div_scale_f32") for o in ops)
    assert any(o.startswith("v_fma_f32") for o in ops)


def test_kernels_use_no_scratch_memory_and_no_scalar_stores(device_asm):
    ops = _mnemonics(device_asm)
    bad = sorted(o for o in ops if o.startswith(("scratch_", "s_store", "s_atomic", "s_buffer_store", "s_dcache_wb",
                                                 "s_dcache_inv")))
    assert not bad, bad
    sizes = [int(x) for x in re.findall(r"\.private_segment_fixed_size:\s*(\d+)", device_asm)]
    assert sizes and max(sizes) == 0, max(sizes)


def test_update_kernels_keep_their_occupancy(device_asm):
    """The all-bf16 Philox instance of the fast kernel keeps all 16 loads of a unit in flight (64 vector
    registers of raw data) and still fits 4 waves per SIMD: at most 104 of the 512 vector registers a
    SIMD lane has (99 with the launch tables read through scalar loads; a build that read them with
    vector loads kept the records in 20 more vector registers)."""
    for cen, limit in (("Lb0", 104), ("Lb1", 120)):   # plain instance; the one that centralizes gradients
        m = re.search(r"\.name:\s+(_ZN2rt20sr_adamw_fast_kernelILi0ELi0ELi0ELi0ELi0E" + cen +
                      r"EE\w+)\n(?:.*\n)*?\s+\.vgpr_count:\s+(\d+)", device_asm)
        assert m, "kernel metadata not found"
        print(cen, "vgpr_count", m.group(2))
        assert int(m.group(2)) <= limit, m.group(2)
    # the row-wise centralizing kernel: four waves per SIMD for rows that are read twice, three for the
    # instance that keeps a row's gradient in registers
    for short, limit in (("Lb0", 128), ("Lb1", 168)):
        m = re.search(r"\.name:\s+(_ZN2rt23sr_adamw_rowwise_kernelILi0ELi0ELi0ELi0E" + short +
                      r"EE\w+)\n(?:.*\n)*?\s+\.vgpr_count:\s+(\d+)", device_asm)
        assert m, "kernel metadata not found"
        print("row-wise", short, "vgpr_count", m.group(2))
        assert int(m.group(2)) <= limit, m.group(2)
