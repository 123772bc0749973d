"""Build-level checks of the hand-written kernels that need no GPU.

The four-wave GEMM issues its v_mfma_f32_16x16x32 instructions as assembly
statements with the accumulator tied to the result (zdraw_amd/csrc/gemm_half.hip,
mfma16). The compiler adds no wait states around assembly, so anything it places
on its own between such an MFMA and the `s_nop 15` that ends the run (a copy or a
spill of an accumulator) would read the register before the MFMA has written it.
The check compiles the file to gfx950 assembly and fails on any such instruction.
"""
import os
import shutil

import pytest

from zdraw_amd import build


@pytest.mark.skipif(not (os.path.exists("/opt/rocm/bin/hipcc") or shutil.which("hipcc")), reason="needs hipcc")
def test_nothing_reads_an_accumulator_inside_a_run_of_tied_mfmas():
    bad = build.tied_mfma_hazards()
    assert not bad, "\n".join(bad[:20])


@pytest.mark.skipif(not (os.path.exists("/opt/rocm/bin/hipcc") or shutil.which("hipcc")), reason="needs hipcc")
def test_only_the_source_writes_m0_in_the_four_wave_gemm():
    # its slab loads come in runs of four that share one M0 (attn_device.hpp, lds_dma_base): the
    # compiler does not know M0 is live between them, so it must not have put a write of its own there
    bad = build.m0_writes()
    assert not bad, "\n".join(bad[:20])


@pytest.mark.skipif(not (os.path.exists("/opt/rocm/bin/hipcc") or shutil.which("hipcc")), reason="needs hipcc")
def test_wide_head_kernel_keeps_its_accumulators_in_place_and_its_loop_free_of_spills():
    # attn_wide.hip: every MFMA of attn_wide_kernel is an assembly statement with the accumulator
    # tied to the result; nothing else may touch the accumulation file before the wait that ends a
    # step, and the blocks that hold the MFMAs may not use scratch memory
    bad = build.wide_mfma_hazards()
    assert not bad, "\n".join(bad[:20])
