"""Builds the gfx950 shared libraries in-tree with hipcc / g++.

`python -m zdraw_amd.build` compiles
  zdraw_amd/lib/libzdraw_hip.so   the C-ABI library (HIP kernels + bridge)
  zdraw_amd/lib/libzdraw_host.so  the C++ host layer above the C ABI
hipcc cross-compiles for gfx950 without a GPU present.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
LIBDIR = os.path.join(HERE, "lib")

HIP_LIB = os.path.join(LIBDIR, "libzdraw_hip.so")
HOST_LIB = os.path.join(LIBDIR, "libzdraw_host.so")

# Packed-FP32 VALU forms are disabled for every device translation unit.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("build failed: " + " ".join(cmd))
    return proc


def build_hip(verbose: bool = False, out: str | None = None, extra_flags=()) -> str:
    """Compile the C-ABI library. `out` / `extra_flags` build an experimental
    copy elsewhere (kernel tuning defines) without touching the shipped one."""
    os.makedirs(LIBDIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    target = out or HIP_LIB
    tag = "" if out is None else "." + os.path.basename(out)
    srcs = [os.path.join(CSRC, f) for f in ("attn_fwd.hip", "attn_wide.hip", "qk_prepass.hip", "gemm_half.hip", "bridge.hip")]
    from concurrent.futures import ThreadPoolExecutor
    objs = [os.path.join(LIBDIR, os.path.basename(src) + tag + ".o") for src in srcs]
    with ThreadPoolExecutor(max_workers=min(len(srcs), os.cpu_count() or 1)) as pool:  # one hipcc per source file
        list(pool.map(lambda so: _run([hipcc, *HIPCC_FLAGS, *extra_flags, "-c", so[0], "-o", so[1]]), zip(srcs, objs)))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", target, *objs])
    if verbose:
        print("built", target)
    return target


_ASM_CACHE: dict = {}


def _device_asm(src: str, extra_flags=()) -> list[str]:
    import tempfile
    key = (src, tuple(extra_flags), os.path.getmtime(src))
    if key in _ASM_CACHE:
        return _ASM_CACHE[key]
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    with tempfile.TemporaryDirectory() as tmp:
        asm = os.path.join(tmp, "out.s")
        _run([hipcc, *HIPCC_FLAGS, *extra_flags, "-S", "--cuda-device-only", "-o", asm, src])
        with open(asm) as f:
            _ASM_CACHE[key] = f.read().split("\n")
    return _ASM_CACHE[key]


def m0_writes(src: str = os.path.join(CSRC, "gemm_half.hip"), kernel_substr: str = "gemm_ring_kernel", extra_flags=()) -> list[str]:
    """Compiles `src` to gfx950 assembly and lists, for the kernels whose symbol contains
    `kernel_substr`, every instruction that writes M0 other than the source's own
    `s_mov_b32 m0, <sgpr>` + `s_nop 0` pair (attn_device.hpp, lds_dma_base). The four-wave GEMM
    keeps M0 live across several loads without the compiler knowing; a write of the compiler's
    own in between would send those loads elsewhere in LDS."""
    import re
    lines = [l.split(";")[0].strip() for l in _device_asm(src, extra_flags)]
    lines = [l for l in lines if l]
    bad = []
    kernel = ""
    writes = re.compile(r"^s_\w+\s+m0\s*,")
    for i, text in enumerate(lines):
        if text.endswith(":") and not text.startswith("."):
            kernel = text[:-1]
            continue
        if kernel_substr not in kernel or not writes.match(text):
            continue
        own = re.match(r"^s_mov_b32\s+m0\s*,\s*s\d+$", text) and i + 1 < len(lines) and lines[i + 1] == "s_nop 0"
        if not own:
            bad.append(f"{kernel}: {text}")
    return bad


def tied_mfma_hazards(src: str = os.path.join(CSRC, "gemm_half.hip"), extra_flags=(),
                      mfma_prefix: str = "v_mfma_f32_16x16x32", kernel_substr: str = "") -> list[str]:
    """Compiles `src` to gfx950 assembly and lists every place (in the kernels whose symbol
    contains `kernel_substr`) where something other than an MFMA touches an accumulation
    register while a hand-written MFMA (`mfma_prefix`) may still be writing it. Those MFMAs are assembly statements, so the compiler adds none of
    the wait states it adds after the builtin; the source instead ends every run of them
    with `s_nop 15` before control leaves the block. A copy or spill of an accumulator that
    the register allocator places inside such a run would read a stale value: this check
    (run by the CPU tests) fails the build that contains one."""
    import re
    lines = _device_asm(src, extra_flags)
    bad = []
    agpr = re.compile(r"\ba(\[\d+:\d+\]|\d+)\b")
    kernel, hot = "", False
    for no, line in enumerate(lines, 1):
        text = line.split(";")[0].strip()
        if not text:
            continue
        if text.endswith(":") and not text.startswith("."):
            kernel, hot = text[:-1], False
            continue
        if kernel_substr not in kernel:
            continue
        op = text.split()[0]
        if op.startswith(mfma_prefix):
            hot = True
        elif op == "s_nop" and text.split()[1] == "15":
            hot = False
        elif hot and agpr.search(text):
            bad.append(f"{kernel}: line {no}: {text}")
    return bad


def wide_mfma_hazards(extra_flags=()) -> list[str]:
    """The same check for the wide-head kernel (attn_wide.hip, attn_wide_kernel): all of its MFMAs
    are assembly statements, its 256 accumulation registers hold O^T for the whole walk, and every
    step ends with the wait (`s_nop 15` ...) before anything else may read them. Also lists any
    use of scratch memory inside a block that holds such MFMAs: the loop is written to fit the
    register file exactly, and a spill there waits on every load in flight."""
    import re
    src = os.path.join(CSRC, "attn_wide.hip")
    bad = tied_mfma_hazards(src, extra_flags, mfma_prefix="v_mfma_f32_32x32x16", kernel_substr="attn_wide_kernel")
    lines = _device_asm(src, extra_flags)
    kernel, block, mfmas, scratch = "", "", 0, []
    label = re.compile(r"^([.\w$]+):")

    def close():
        if "attn_wide_kernel" in kernel and mfmas >= 32 and scratch:
            bad.append(f"{kernel}: {len(scratch)} scratch accesses in {block} beside {mfmas} MFMAs, e.g. {scratch[0]}")

    for line in lines:
        text = line.split(";")[0].strip()
        if not text:
            continue
        m = label.match(text)
        if m:
            close()
            if not text.startswith("."):
                kernel = m.group(1)
            block, mfmas, scratch = m.group(1), 0, []
            continue
        if text.startswith("v_mfma"):
            mfmas += 1
        elif text.startswith("scratch_"):
            scratch.append(text)
    close()
    return bad


def build_host(verbose: bool = False) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    srcs = [os.path.join(HOST, f) for f in sorted(os.listdir(HOST)) if f.endswith(".cc")]
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra",
          "-I", os.path.join(ROOT, "include"), "-o", HOST_LIB, *srcs,
          "-L", LIBDIR, "-lzdraw_hip", "-Wl,-rpath,$ORIGIN"])
    if verbose:
        print("built", HOST_LIB)
    return HOST_LIB


def check_hand_scheduled_kernels(verbose: bool = False):
    """The GEMM's hand-placed MFMAs and its M0 held across loads are safe only as long as the
    compiler puts nothing of its own in between: a toolchain that does fails the build here."""
    bad = m0_writes() + tied_mfma_hazards() + wide_mfma_hazards()
    if bad:
        raise RuntimeError("a kernel compiled to code that breaks its hand-written schedule:\n  " + "\n  ".join(bad))
    if verbose:
        print("hand-scheduled kernels: no foreign M0 write, no accumulator touched inside an MFMA run")


def build_all(verbose: bool = False):
    build_hip(verbose)
    build_host(verbose)
    check_hand_scheduled_kernels(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
