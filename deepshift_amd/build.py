"""Builds ``lib/libdeepshift_hip.so`` (gfx950) from ``csrc/*.hip`` with hipcc.

    python -m deepshift_amd.build            # rebuild unconditionally
    python -m deepshift_amd.build --if-stale # only when a source is newer than the library
    python -m deepshift_amd.build --incremental  # recompile only the units that changed
"""
import glob
import os
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_DIR = os.path.join(_HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libdeepshift_hip.so")
ARCH = "gfx950"

# -packed-fp32-ops is switched off: this library has no business with packed fp32 and the
# conversions in the quantise kernels must stay scalar.
HIPCC_FLAGS = [
    "--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def hipcc():
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    path = os.path.join(rocm, "bin", "hipcc")
    return path if os.path.exists(path) else "hipcc"


def sources():
    """The HIP translation units and the host-only ones (the CPU twins of the kernels)."""
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.cpp")))


def is_stale():
    if not os.path.exists(LIB_PATH):
        return True
    built = os.path.getmtime(LIB_PATH)
    deps = sources() + glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(CSRC, "*.py")) + \
        glob.glob(os.path.join(_HERE, "..", "include", "*.h"))
    return any(os.path.getmtime(p) > built for p in deps)


def _deps(src):
    return [src] + glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(CSRC, "*.inc")) + \
        glob.glob(os.path.join(_HERE, "..", "include", "*.h"))


def build(verbose=True, incremental=False):
    """Compile every translation unit (in parallel) and link the shared library.  ``incremental``
    skips the units whose object file is newer than the source and every header."""
    os.makedirs(LIB_DIR, exist_ok=True)
    # the asm main loop of the shift-plane kernel is generated text (csrc/ds_planes_asm.inc)
    subprocess.check_call([sys.executable, os.path.join(CSRC, "gen_planes_asm.py")])
    obj_dir = os.path.join(_HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    procs = []
    objs = []
    for src in sources():
        obj = os.path.join(obj_dir, os.path.splitext(os.path.basename(src))[0] + ".o")
        objs.append(obj)
        if incremental and os.path.exists(obj) and \
                all(os.path.getmtime(d) <= os.path.getmtime(obj) for d in _deps(src)):
            continue
        if src.endswith(".cpp"):
            cmd = [hipcc(), "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-pthread", "-Wall",
                   "-c", src, "-o", obj]
        else:
            cmd = [hipcc()] + HIPCC_FLAGS + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
    failed = False
    for src, proc in procs:
        out = proc.communicate()[0].decode(errors="replace")
        out = "\n".join(line for line in out.splitlines()
                        if "packed-fp32-ops" not in line and line.strip())
        if out and verbose:
            print(out, flush=True)
        if proc.returncode != 0:
            print("hipcc failed on %s\n%s" % (src, out), file=sys.stderr)
            failed = True
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc(), "--offload-arch=" + ARCH, "-shared", "-fPIC", "-pthread", "-o", LIB_PATH] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB_PATH


if __name__ == "__main__":
    if "--if-stale" in sys.argv and not is_stale():
        print("up to date:", LIB_PATH)
    else:
        print(build(incremental="--incremental" in sys.argv))
