"""Builds cubert_amd/libcuBERT.so in-tree with hipcc for gfx950.

    python -m cubert_amd.build          # or cubert_amd.build.build()

Device code: csrc/kernels/*.hip and csrc/runtime.hip; host code: csrc/host/*.cpp.
Objects go to cubert_amd/build/ (git-ignored), the library next to this file.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libcuBERT.so")

ARCH = "gfx950"
INCLUDES = ["-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(CSRC, "kernels"), "-I" + os.path.join(CSRC, "host")]
# -packed-fp32-ops is switched off: hipcc must not form v_pk_*_f32 from scalar float code.
# -amdgpu-mfma-vgpr-form: matrix-core accumulators stay in ordinary vector registers.  The default puts them in the
# accumulation registers and copies every result out before the first ordinary instruction can touch it (96 copies
# per wavefront in the one-launch attention kernel) and, with both files in use, holds fewer wavefronts per SIMD.
DEVICE_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
                "-packed-fp32-ops", "-mllvm", "-amdgpu-mfma-vgpr-form=1", "-Wno-unused-command-line-argument"]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-command-line-argument"]

DEVICE_SOURCES = ["kernels/layernorm.hip", "kernels/softmax.hip", "kernels/elementwise.hip", "kernels/attention.hip", "kernels/gemm_skinny.hip", "kernels/gemm_batch.hip", "kernels/split.hip",
                  "runtime.hip"]
HOST_SOURCES = ["host/Transformer.cpp", "host/Bert.cpp", "host/BertM.cpp", "host/Graph.cpp", "host/tokenization.cpp",
                "host/api.cpp"]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _compile(job):
    src, obj, flags = job
    cmd = [hipcc()] + flags + INCLUDES + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("compile failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(verbose=False, jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    work = []
    for rel in DEVICE_SOURCES:
        work.append((os.path.join(CSRC, rel), os.path.join(OBJ, os.path.basename(rel) + ".o"), DEVICE_FLAGS))
    for rel in HOST_SOURCES:
        work.append((os.path.join(CSRC, rel), os.path.join(OBJ, os.path.basename(rel) + ".o"), HOST_FLAGS))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        for out in pool.map(_compile, work):
            if verbose and out.strip():
                print(out)
    link = [hipcc(), "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB] + [w[1] for w in work] + \
           ["-L/opt/rocm/lib", "-lhipblaslt", "-Wl,-rpath,/opt/rocm/lib"]
    r = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed: %s\n%s" % (" ".join(link), r.stdout))
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
