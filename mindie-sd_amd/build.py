"""Build the HIP library of this package for gfx950 (MI355X).

    python mindie-sd_amd/build.py

compiles every ``csrc/*.hip`` with hipcc into one shared object,
``mindiesd/plugin/libmindiesd_hip.so`` (the location mirrors the reference's
``<package>/plugin/libPTAExtensionOPS.so``, mindiesd/layers/register_ops.py:24-44).
hipcc cross-compiles without a GPU present.  The library has a plain C ABI
(``include/mindiesd_hip.h``) and links against nothing but the HIP runtime.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "mindiesd", "plugin", "libmindiesd_hip.so")

# -packed-fp32-ops is switched OFF on purpose (target feature with a leading minus).
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def build(verbose=False, extra=()):
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    objs = []
    procs = []
    for src in sources():
        obj = os.path.join(CSRC, os.path.basename(src)[:-4] + ".o")
        cmd = ["hipcc", *[f for f in FLAGS if f != "-shared"], "-c", src, "-o", obj, "-I", CSRC, *extra]
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for cmd, pr in procs:
        out, _ = pr.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if pr.returncode != 0:
            raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), out))
        if verbose and out.strip():
            print(out)
    link = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", OUT]
    subprocess.run(link, check=True)
    return OUT


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
