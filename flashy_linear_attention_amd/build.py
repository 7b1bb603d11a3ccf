"""Builds ``libfla_gfx950.so`` in-tree with hipcc (gfx950 only).

Run as ``python -m flashy_linear_attention_amd.build``.  hipcc cross-compiles
without a GPU.  One object per (dtype, DC, DO) kernel instantiation, compiled in
parallel, then linked with the C ABI into the package directory.
"""

from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from typing import List

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(REPO_ROOT, "include")
OBJ_DIR = os.path.join(PKG_DIR, "csrc", "_obj")
LIB_NAME = "libfla_gfx950.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)

DIMS = (32, 64, 128, 256)
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # hipcc may not form packed fp32 VALU ops on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results in architectural VGPRs (operands may still sit in AGPRs): the S
    # accumulators are read by VALU right away, and the AGPR form costs 32 copies per sub-tile
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    "-Wno-unused-command-line-argument",
    "-I" + INCLUDE,
    "-I" + CSRC,
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP kernels cannot be built")
    return exe


def _run(cmd: List[str]) -> str:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + proc.stdout)
    return proc.stdout


def _check_no_scratch(report: str, kernel: str) -> None:
    """Fail the build if an instantiation of `kernel` spills registers.  The reverse walk keeps its
    running sums in accumulation registers through MFMAs issued from inline assembly, with the wait
    states they need placed by hand; a spill or reload the register allocator put between two of them
    would get none and read stale values without any error.  `report`: the compiler's
    -Rpass-analysis=kernel-resource-usage remarks."""
    name, seen = None, 0
    for line in report.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
        elif "ScratchSize" in line and name and kernel in name:
            seen += 1
            size = int(line.split("ScratchSize [bytes/lane]:")[1].split()[0])
            if size != 0:
                raise RuntimeError(f"{name} uses {size} bytes of scratch per lane: its hand-placed MFMA wait states "
                                   "assume that no spill code sits between its MFMAs")
    if seen == 0:
        raise RuntimeError(f"no resource report for {kernel}: the spill check did not run")


def _compile_inst(args) -> str:
    dtype, dc, do = args
    obj = os.path.join(OBJ_DIR, f"inst_t{dtype}_c{dc}_o{do}.o")
    _run([_hipcc(), *HIPCC_FLAGS, f"-DFLA_INST_DTYPE={dtype}", f"-DFLA_INST_DC={dc}", f"-DFLA_INST_DO={do}",
          "-c", os.path.join(CSRC, "fla_inst.hip"), "-o", obj])
    return obj


def build(jobs: int | None = None, verbose: bool = True) -> str:
    """Compile every kernel instantiation and link the shared library.  Always recompiles."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    work = [(t, dc, do) for t in (0, 1) for dc in DIMS for do in DIMS]
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile_inst, work))
    capi = os.path.join(OBJ_DIR, "fla_capi.o")
    _run([_hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, "fla_capi.hip"), "-o", capi])
    walk = os.path.join(OBJ_DIR, "fla_walk_inst.o")
    report = _run([_hipcc(), *HIPCC_FLAGS, "-Rpass-analysis=kernel-resource-usage", "-c",
                   os.path.join(CSRC, "fla_walk_inst.hip"), "-o", walk])
    _check_no_scratch(report, "walk_bwd_rev_kernel")
    _check_no_scratch(report, "walk_bwd_rev_wide_kernel")
    # (this one without the VGPR form of MFMA: see the file's header)
    pair = os.path.join(OBJ_DIR, "fla_pair_inst.o")
    pair_flags = [f for f in HIPCC_FLAGS if f not in ("-mllvm", "-amdgpu-mfma-vgpr-form")]
    _run([_hipcc(), *pair_flags, "-c", os.path.join(CSRC, "fla_pair_inst.hip"), "-o", pair])
    tmp = LIB_PATH + ".tmp"
    _run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, capi, walk, pair, *objs])
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} ({os.path.getsize(LIB_PATH) / 1e6:.1f} MB, {len(objs)} kernel objects)")
    return LIB_PATH


TRACE_LIB_PATH = os.path.join(OBJ_DIR, "trace", "libfla_trace.so")


def build_trace(jobs: int | None = None) -> str:
    """The host-only trace build of the same sources (``-DFLA_TRACE_LAUNCHES``): a library with the
    same C ABI that makes no launch and writes every launch down instead (kernel, grid, LDS, every
    argument), plus ``fla_trace_take``.  Runs without a GPU; the launch-plan tests load it."""
    out_dir = os.path.dirname(TRACE_LIB_PATH)
    os.makedirs(out_dir, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    flags = ["--offload-arch=gfx950", "--offload-host-only", "-O1", "-std=c++17", "-fPIC", "-DFLA_TRACE_LAUNCHES",
             "-Wno-unused-command-line-argument", "-I" + INCLUDE, "-I" + CSRC]

    def one(args) -> str:
        src, obj, defs = args
        _run([_hipcc(), *flags, *defs, "-c", os.path.join(CSRC, src), "-o", os.path.join(out_dir, obj)])
        return os.path.join(out_dir, obj)

    work = [("fla_inst.hip", f"inst_t{t}_c{dc}_o{do}.o",
             [f"-DFLA_INST_DTYPE={t}", f"-DFLA_INST_DC={dc}", f"-DFLA_INST_DO={do}"])
            for t in (0, 1) for dc in DIMS for do in DIMS]
    work += [("fla_capi.hip", "fla_capi.o", []), ("fla_walk_inst.hip", "fla_walk_inst.o", []),
             ("fla_pair_inst.hip", "fla_pair_inst.o", []),
             ("fla_trace.cc", "fla_trace.o", ["-x", "c++"])]
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(one, work))
    # A host-only object still registers its (absent) device code with the HIP runtime when it is
    # loaded: it refers to a code-object symbol that the device link would have made, and calls the
    # runtime's registration hooks.  The trace library brings both itself -- empty code objects and
    # hooks that do nothing, bound inside the library -- so that loading it touches no HIP runtime.
    names = set()
    for obj in objs:
        out = subprocess.run(["nm", "-u", obj], stdout=subprocess.PIPE, text=True, check=True).stdout
        names.update(tok for tok in out.split() if tok.startswith("__hip_fatbin_"))
    stubs = os.path.join(out_dir, "registration_stubs.c")
    with open(stubs, "w") as f:
        for name in sorted(names):
            f.write(f"const char {name}[64] = {{0}};\n")
        f.write("void **__hipRegisterFatBinary(const void *d) { static void *h; (void)d; return &h; }\n"
                "void __hipUnregisterFatBinary(void **h) { (void)h; }\n"
                "void __hipRegisterFunction(void **m, const void *f, char *a, const char *b, unsigned c, void *d,\n"
                "                           void *e, void *g, void *h, int *i) {}\n"
                "void __hipRegisterVar(void **m, void *v, char *a, const char *b, int c, unsigned long d, int e,\n"
                "                      int g) {}\n")
    stubs_obj = os.path.join(out_dir, "registration_stubs.o")
    _run(["gcc", "-O1", "-fPIC", "-c", stubs, "-o", stubs_obj])
    tmp = TRACE_LIB_PATH + ".tmp"
    _run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-Bsymbolic", "-o", tmp, *objs, stubs_obj])
    os.replace(tmp, TRACE_LIB_PATH)
    return TRACE_LIB_PATH


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "trace":
        print(build_trace())
    else:
        build()
    sys.exit(0)
