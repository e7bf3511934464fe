"""Build recipes for the native libraries (run on a CPU-only machine too).

    liboxhip.so    HIP kernels + C host layer (hipcc cross-compiles gfx950)
    liboxsynth.so  synthetic tensor generator (gcc)

Everything is built in-tree next to this file so that the shared objects
travel with the source tree.
"""
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
CC = os.environ.get("CC", "gcc")

# -ffp-contract=off: the block terms must round exactly like the reference's
# C code.  -packed-fp32-ops is switched off on purpose for this target.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wall", "-Wno-unused-command-line-argument"]
C_FLAGS = ["-std=c11", "-O2", "-fPIC", "-Wall", "-Wextra", "-ffp-contract=off"]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    return proc.stdout


HIP_UNITS = ("oxh_kernels", "oxh_plan")


def exported_names():
    """The functions the public headers declare: exactly what liboxhip.so exports."""
    import re
    names = set()
    for header in ("oxhip.h", "oxhip_lab.h"):
        text = open(os.path.join(INCLUDE, header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b((?:oxh|oc)_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def write_export_map(path):
    """A linker version script: the declared functions are global, everything else (the kernels' host
    stubs, the symbols the two translation units and the C host layer share, the lab functions behind
    oxh_lab's table) stays inside the library."""
    with open(path, "w") as f:
        f.write("{\n  global:\n")
        for n in exported_names():
            f.write("    %s;\n" % n)
        f.write("  local:\n    *;\n};\n")


def build_oxhip(verbose=False, only=None):
    """`only`: names of HIP translation units to recompile (the others' objects are reused)."""
    from concurrent.futures import ThreadPoolExecutor
    obj_c = os.path.join(CSRC, "oc_matvec.o")
    obj_g = os.path.join(CSRC, "oxh_gguf.o")
    out = os.path.join(HERE, "liboxhip.so")
    units = [u for u in HIP_UNITS if only is None or u in only or not os.path.exists(os.path.join(CSRC, u + ".o"))]

    def compile_unit(u):
        return _run([HIPCC] + HIP_FLAGS + ["-I", INCLUDE, "-I", CSRC, "-c", os.path.join(CSRC, u + ".hip"),
                                          "-o", os.path.join(CSRC, u + ".o")])

    with ThreadPoolExecutor(max_workers=len(HIP_UNITS)) as pool:
        log = "".join(pool.map(compile_unit, units))
    hip_objs = [os.path.join(CSRC, u + ".o") for u in HIP_UNITS]
    log += _run([CC] + C_FLAGS + ["-I", INCLUDE, "-I", CSRC, "-c",
                                  os.path.join(CSRC, "oc_matvec.c"), "-o", obj_c])
    log += _run([CC] + C_FLAGS + ["-I", INCLUDE, "-I", CSRC, "-c",
                                  os.path.join(CSRC, "oxh_gguf.c"), "-o", obj_g])
    export_map = os.path.join(CSRC, "liboxhip.map")
    write_export_map(export_map)
    log += _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + hip_objs + [obj_c, obj_g,
                 "-lpthread", "-Wl,--version-script=" + export_map, "-Wno-unused-command-line-argument"])
    if verbose and log.strip():
        print(log)
    return out


def build_synth():
    out = os.path.join(HERE, "liboxsynth.so")
    _run([CC] + C_FLAGS + ["-fopenmp", "-shared", "-o", out, os.path.join(CSRC, "synth.c")])
    return out


def build_all(verbose=False):
    return [build_oxhip(verbose), build_synth()]


if __name__ == "__main__":
    for path in build_all(verbose=True):
        print("built", path)
