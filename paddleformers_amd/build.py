"""Builds libpf8.so (the HIP kernels + C ABI) in-tree with hipcc for gfx950.

Usage: python -m paddleformers_amd.build [--force]
hipcc cross-compiles without a GPU; the resulting .so sits next to this file so that it travels
with the source tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libpf8.so")
SOURCES = ["pf8_api.hip", "pf8_quant.hip", "pf8_gemm.hip", "pf8_gemm_fm.hip", "pf8_gemm_e8.hip", "pf8_wgrad_e8.hip", "pf8_permute.hip", "pf8_norm.hip"]
HEADERS = ["pf8_device.h", "pf8_host.h", "pf8_gemm_common.h", "pf8_e8_common.h", os.path.join("..", "..", "include", "pf8.h"),
           os.path.join("..", "..", "include", "pf8_selftest.h")]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # bit-exactness against the CPU checker: no implicit fused multiply-adds, IEEE divide/sqrt,
    # fp32 denormals kept
    "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-fno-gpu-flush-denormals-to-zero",
    # packed fp32 arithmetic stays off on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    # per-kernel register, LDS and scratch usage as compiler remarks: build() refuses a kernel that spills to scratch
    "-Rpass-analysis=kernel-resource-usage",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; cannot build libpf8.so")


def up_to_date() -> bool:
    if not os.path.exists(LIB):
        return False
    t = os.path.getmtime(LIB)
    deps = [os.path.join(CSRC, f) for f in SOURCES + HEADERS]
    return all(os.path.getmtime(d) <= t for d in deps)


def kernels_with_scratch(remarks):
    """(kernels seen, [(kernel, bytes per lane)] of those that report scratch memory) from the compiler's
    kernel-resource-usage remarks.  The hand-scheduled kernels are written to fit the register file: a spill there
    is a performance bug, and scratch makes every launch depend on a per-queue scratch allocation."""
    seen, found, name = [], [], None
    for l in remarks:
        if "Function Name:" in l:
            name = l.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in l and name:
            n = int(l.split("ScratchSize [bytes/lane]:")[1].split("[")[0].strip())
            seen.append(name)
            if n > 0:
                found.append((name, n))
            name = None
    return seen, found


# kernels whose register budget was fitted by hand: each must show up in the remarks, or the check has gone blind
EXPECTED_KERNELS = ("k_gemm_fm", "k_gemm_fwd_deep", "k_gemm_fwd128", "k_gemm_wgrad", "k_gemm_e8", "k_quant_rowcol", "k_quant_1x128")


def check_scratch(remarks) -> str:
    """Raises when a kernel spills to scratch (PF8_ALLOW_SCRATCH=1 turns that into the returned warning text, for a
    compiler release that spills a few bytes where this one does not) and when the remarks the check reads are not
    there at all (a changed wording must not let it pass vacuously)."""
    seen, spilling = kernels_with_scratch(remarks)
    missing = [k for k in EXPECTED_KERNELS if not any(k in name for name in seen)]
    if missing:
        raise RuntimeError("resource remarks not found for: " + ", ".join(missing) +
                           " (the -Rpass-analysis=kernel-resource-usage output has changed; the scratch check cannot run)")
    if not spilling:
        return ""
    msg = "kernels that spill registers to scratch memory (bytes per lane): " + ", ".join(f"{k}: {v}" for k, v in spilling)
    if os.environ.get("PF8_ALLOW_SCRATCH") == "1":
        return "warning: " + msg
    raise RuntimeError(msg + " (set PF8_ALLOW_SCRATCH=1 to build anyway)")


def check_fragment_ring(flags) -> None:
    """pf8_gemm_fm.hip keeps its weight-fragment ring in AGPRs that only its inline assembly names; the compiler, which
    sees them as free, must not have put anything of its own there.  It does so only through v_accvgpr_* copies, so the
    device assembly of that file must hold none."""
    import tempfile

    src = os.path.join(CSRC, "pf8_gemm_fm.hip")
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "pf8_gemm_fm.s")
        cmd = [hipcc()] + [f for f in flags if f not in ("-shared", "-fPIC") and not f.startswith("-Rpass")] + \
              ["--offload-device-only", "-S", src, "-o", out]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise RuntimeError("hipcc -S failed on pf8_gemm_fm.hip:\n" + proc.stdout)
        text = open(out).read()
    if "k_gemm_fm" not in text or "v_mfma_f32_32x32x64_f8f6f4" not in text:
        raise RuntimeError("the device assembly of pf8_gemm_fm.hip does not look as expected; the AGPR check cannot run")
    hz = sgpr_address_hazards(text)
    if hz:
        raise RuntimeError(f"pf8_gemm_fm.hip: {len(hz)} memory instructions read a scalar address register too soon after the vector "
                           f"unit wrote it, e.g. line {hz[0][0]}: {hz[0][1]}")
    n = text.count("v_accvgpr")
    if n:
        raise RuntimeError(f"pf8_gemm_fm.hip: the compiler placed {n} accumulation-register copies of its own; they would "
                           "overwrite the weight-fragment ring (lower the register pressure of k_gemm_fm)")


def sgpr_address_hazards(asm_text: str, need: int = 5):
    """[(line, instruction, sgpr, wait states)] where a vector-memory instruction reads, as its scalar address, a register
    the vector unit wrote (v_readlane / v_readfirstlane: restored spills, uniform values computed on the vector unit)
    fewer than `need` wait states earlier.  The hardware needs five; the compiler pads its own instructions with s_nop
    but not the text of inline assembly, so a kernel whose memory instructions are written by hand can be handed an
    address register that is not yet readable.  Every instruction counts as one wait state, s_nop N as N + 1."""
    import re

    bad, last, n = [], {}, 0
    for ln, l in enumerate(asm_text.splitlines(), 1):
        t = l.strip()
        if not l.startswith("\t") or not t or t.startswith((".", ";")):
            continue
        op = t.split()[0]
        if op == "s_nop":
            n += int(t.split()[1]) + 1
            continue
        n += 1
        m = re.match(r"v_(?:readlane|readfirstlane)_b32 s(\d+)", t)
        if m:
            last[int(m.group(1))] = n
        if op.startswith(("global_", "buffer_", "flat_", "scratch_")):
            for a, b in re.findall(r"s\[(\d+):(\d+)\]", t):
                for r in range(int(a), int(b) + 1):
                    if r in last and n - last[r] - 1 < need:
                        bad.append((ln, t, r, n - last[r] - 1))
    return bad


def check_accumulator_tiles(flags) -> None:
    """pf8_gemm_e8.hip and pf8_wgrad_e8.hip keep a 256x256 accumulator tile in the whole AGPR file, named only by their
    inline assembly.  The compiler sees those registers as free and, under register pressure, parks values of its own
    there (v_accvgpr_write_b32 aN, vM), which would overwrite accumulators.  The kernels' own accesses are writes of the
    constant 0 and reads by the epilogues (256 per copy of the epilogue): anything else fails the build."""
    import re
    import tempfile

    for name, reads in (("pf8_gemm_e8.hip", None), ("pf8_wgrad_e8.hip", 1024)):
        src = os.path.join(CSRC, name)
        with tempfile.TemporaryDirectory() as tmp:
            out = os.path.join(tmp, name + ".s")
            cmd = [hipcc()] + [f for f in flags if f not in ("-shared", "-fPIC") and not f.startswith("-Rpass")] + \
                  ["--offload-device-only", "-S", src, "-o", out]
            proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
            if proc.returncode != 0:
                raise RuntimeError(f"hipcc -S failed on {name}:\n" + proc.stdout)
            text = open(out).read()
        if "v_mfma_scale_f32_16x16x128_f8f6f4" not in text:
            raise RuntimeError(f"the device assembly of {name} does not look as expected; the AGPR check cannot run")
        hz = sgpr_address_hazards(text)
        if hz:
            raise RuntimeError(f"{name}: {len(hz)} memory instructions read a scalar address register too soon after the vector unit "
                               f"wrote it, e.g. line {hz[0][0]}: {hz[0][1]} (s{hz[0][2]} after {hz[0][3]} wait states; put an s_nop in "
                               "front of the instruction in its inline assembly)")
        parked = [l.strip() for l in text.splitlines() if re.search(r"v_accvgpr_write_b32 a\d+, [vs]", l) or "v_accvgpr_mov" in l]
        n_reads = text.count("v_accvgpr_read_b32")
        if parked or (reads is not None and n_reads != reads):
            raise RuntimeError(f"{name}: the compiler uses accumulation registers of its own ({len(parked)} copies in, {n_reads} reads"
                               f"{'' if reads is None else ' where the epilogues make ' + str(reads)}); they would overwrite the "
                               "accumulator tile (lower the kernel's register pressure)")


def build(force: bool = False, verbose: bool = False) -> str:
    if not force and up_to_date():
        return LIB
    cmd = [hipcc()] + FLAGS + [os.path.join(CSRC, f) for f in SOURCES] + ["-o", LIB]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    lines = proc.stdout.splitlines()
    # drop the feature warning of the host pass and the resource-usage remarks with the source lines they quote
    kept, skip = [], 0
    for l in lines:
        if "kernel-resource-usage" in l:
            skip = 2
        elif skip and (l.lstrip().startswith("|") or l.lstrip().split(" |")[0].isdigit()):
            skip -= 1
        elif "packed-fp32-ops" not in l:
            kept.append(l)
            skip = 0
    out = "\n".join(kept)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    try:
        warning = check_scratch(lines)
        check_fragment_ring(FLAGS)
        check_accumulator_tiles(FLAGS)
    except RuntimeError:
        os.remove(LIB)
        raise
    if warning:
        print(warning, file=sys.stderr)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
