"""Builds the HIP kernels and the C-ABI shared library for gfx950.

    python -m megafold_amd.build            # compile every source, link lib/libmegafold_amd.so

hipcc cross-compiles without a GPU.  Objects go to ``megafold_amd/_build`` and the library to
``megafold_amd/lib`` (both git-ignored); nothing is installed outside the source tree.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OBJ = PKG / "_build"
LIB = PKG / "lib" / "libmegafold_amd.so"

# -packed-fp32-ops: keep the compiler from forming packed fp32 VALU instructions.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# Per-source flags.  evoattn_bwd_pw.hip keeps its running sums in accumulation registers through inline
# assembly and wants every MFMA builtin (the score products, whose results the vector ALU reads) to write
# ordinary vector registers; with up to 512 registers per lane the compiler would otherwise choose the
# accumulation-register form for all of them and copy each score out one register at a time.
PER_SOURCE_FLAGS = {
    "evoattn_bwd_pw": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        sys.stderr.write(out + "\n")


# sources whose MFMAs are inline assembly: the compiler does not see their hazards
ASM_MFMA_SOURCES = ("evoattn_bwd_pw", "evoattn_bwd_dbias_ring")


def _check_generated_code(hipcc: str, extra: list[str]) -> None:
    """evoattn_bwd_pw.hip and evoattn_bwd_dbias_ring.hip issue their MFMAs as inline assembly, which hides them
    from the compiler's hazard handling; csrc/check_pw_hazards.py verifies the required distances on the
    generated assembly text."""
    sys.path.insert(0, str(CSRC))
    try:
        import check_pw_hazards
    finally:
        sys.path.pop(0)
    for stem in ASM_MFMA_SOURCES:
        src = CSRC / (stem + ".hip")
        asm = OBJ / (stem + ".s")
        _run([hipcc, *HIPCC_FLAGS, *PER_SOURCE_FLAGS.get(src.stem, []), *extra, "-S", "--cuda-device-only", str(src),
              "-o", str(asm)])
        errs = check_pw_hazards.check(str(asm))
        if errs:
            raise RuntimeError("hazards in the generated code of %s:\n%s" % (src.name, "\n".join(errs[:20])))


def build(verbose: bool = False, jobs: int | None = None) -> Path:
    """Compile every ``csrc/*.hip`` and link the shared library.  Always recompiles."""
    OBJ.mkdir(exist_ok=True)
    LIB.parent.mkdir(exist_ok=True)
    hipcc = _hipcc()
    srcs = sources()
    if not srcs:
        raise RuntimeError("no HIP sources under %s" % CSRC)
    objs = [OBJ / (s.stem + ".o") for s in srcs]
    extra = os.environ.get("MF_HIPCC_EXTRA", "").split()   # e.g. -DMF_TIMELINE (development builds)
    cmds = [[hipcc, *HIPCC_FLAGS, *PER_SOURCE_FLAGS.get(s.stem, []), *extra, "-c", str(s), "-o", str(o)]
            for s, o in zip(srcs, objs)]
    jobs = jobs or min(8, len(cmds))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for cmd, _ in zip(cmds, ex.map(_run, cmds)):
            if verbose:
                print(" ".join(cmd))
    _check_generated_code(hipcc, extra)
    tmp = LIB.with_suffix(".so.tmp")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *map(str, objs), "-o", str(tmp)])
    os.replace(tmp, LIB)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
