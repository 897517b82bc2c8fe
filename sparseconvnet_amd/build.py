"""Compiles sparseconvnet_amd/csrc/*.hip into sparseconvnet_amd/libscn_hip.so with hipcc
for gfx950.  hipcc cross-compiles without a GPU.  Run as `python -m sparseconvnet_amd.build`."""
import glob
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libscn_hip.so")

FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
         # keep the compiler from forming packed-fp32 VALU instructions
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def sources():
    return sorted(glob.glob(os.path.join(HERE, "csrc", "*.hip")))


def build_library(verbose=False, incremental=False):
    """incremental: translation units whose object file is newer than the source and every header
    are not compiled again (for work on one kernel file; the default compiles everything)."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = sources()
    objs = []
    procs = []
    objdir = os.path.join(HERE, "csrc", "build")
    os.makedirs(objdir, exist_ok=True)
    headers = glob.glob(os.path.join(HERE, "csrc", "*.h")) + glob.glob(os.path.join(HERE, "..", "include", "*.h"))
    newest_header = max(os.path.getmtime(h) for h in headers)
    for s in srcs:  # one hipcc per translation unit, in parallel
        o = os.path.join(objdir, os.path.basename(s)[:-4] + ".o")
        objs.append(o)
        if incremental and os.path.exists(o) and os.path.getmtime(o) > max(os.path.getmtime(s), newest_header):
            continue
        cmd = [hipcc] + [f for f in FLAGS if f != "-shared"] + os.environ.get("SCN_EXTRA_FLAGS", "").split() + ["-c", s, "-o", o]
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
    for cmd, p in procs:
        out = p.communicate()[0].decode()
        if p.returncode != 0:
            raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), out))
        if verbose:
            print(out)
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB]
    subprocess.check_call(link)
    return LIB


if __name__ == "__main__":
    import sys
    print(build_library(incremental="--incremental" in sys.argv))
