"""Properties of the compiled kernels that no run-time test sees fail loudly: they only get slower, or round differently
on one element in hundreds.  Checked on the device assembly that the Makefile's own flags produce (needs hipcc, no GPU)."""

import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "heavyball_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


@pytest.fixture(scope="module")
def ns5_asm(tmp_path_factory):
    if not (os.path.exists(HIPCC) and shutil.which("make")):
        pytest.skip("needs hipcc and make")
    out = str(tmp_path_factory.mktemp("asm") / "ns5.s")
    subprocess.run(["make", "-C", CSRC, "asm-ns5", f"ASM_OUT={out}"], check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    with open(out) as f:
        return f.read()


def test_newton_schulz_accumulators_stay_in_registers(ns5_asm):
    """The product kernels keep their accumulator tiles in registers.  The 256 x 256 kernel's epilogue is a fully unrolled walk
    over 16 sub-tiles; when it outgrows the compiler's size limit for ``#pragma unroll`` the walk stays a loop, the accumulator is
    indexed at run time and moves to scratch memory (1088 bytes per lane), silently, and the product takes five times as long."""
    kernels = re.findall(r"\.name:\s+(\S*ns_gemm\S*)\n(.*?)\.wavefront_size", ns5_asm, re.S)
    assert len(kernels) >= 10
    for name, meta in kernels:
        scratch = int(re.search(r"\.private_segment_fixed_size:\s+(\d+)", meta).group(1))
        assert scratch <= 128, (name, scratch)  # a few spilled registers at most


def test_float16_conversions_round_twice(ns5_asm):
    """A product that is converted to float16 is rounded to fp32 first and to float16 second, as torch computes float16 tensors;
    v_fma_mixlo_f16 / v_mad_mixlo_f16 would round the exact product once (different on float16 ties, one element in a few
    hundred of a bf16 value times a constant).  hb_device.h keeps the product in a register to rule that out."""
    assert not re.search(r"v_(fma|mad)_mixlo_f16", ns5_asm)
