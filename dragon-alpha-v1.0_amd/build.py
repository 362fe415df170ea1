"""Builds libalpha_conv_hip.so (HIP kernels + C ABI + JNI shim) for gfx950 with hipcc, in-tree.

Usage: python build.py [--jobs N]. hipcc cross-compiles without a GPU present.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libalpha_conv_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",  # no packed-fp32 VALU forms
    "-Wall", "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp")))


def _compile(src):
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + FLAGS + (["-x", "hip"] if src.endswith(".cpp") else []) + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj, out


def build(jobs=8, verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    # jni_shim.cpp is generated from the method table in gen_jni_shim.py and the C ABI header: regenerate it on every
    # build so that the committed file cannot drift from its generator
    subprocess.check_call([sys.executable, os.path.join(CSRC, "gen_jni_shim.py")], stdout=subprocess.DEVNULL)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, sources()))
    for _, out in results:
        if verbose and out.strip():
            print(out)
    objs = [o for o, _ in results]
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    jobs = 8
    if "--jobs" in sys.argv:
        jobs = int(sys.argv[sys.argv.index("--jobs") + 1])
    print(build(jobs=jobs, verbose=True))
