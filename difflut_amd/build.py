"""Compile difflut_amd/csrc/*.hip into difflut_amd/lib/libdifflut_hip.so for gfx950."""
import glob
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libdifflut_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-munsafe-fp-atomics",  # float atomics as single hardware instructions
    # packed-fp32 instruction forms are kept out of every code object
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose=False, jobs=None):
    """Always recompiles (the sources in parallel, one hipcc per file), then links; returns the path of the library."""
    from concurrent.futures import ThreadPoolExecutor

    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(LIB_DIR, "_obj")
    os.makedirs(obj_dir, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"] + ["-c"]

    def compile_one(src):
        obj = os.path.join(obj_dir, os.path.basename(src) + ".o")
        cmd = [hipcc] + compile_flags + ["-o", obj, src]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("hipcc failed on " + src + ":\n" + res.stdout + res.stderr)
        if verbose:
            print(" ".join(cmd))
        return obj

    srcs = sources()
    with ThreadPoolExecutor(max_workers=jobs or min(8, len(srcs))) as pool:
        objs = list(pool.map(compile_one, srcs))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc (link) failed:\n" + res.stdout + res.stderr)
    if verbose:
        print(" ".join(cmd))
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
