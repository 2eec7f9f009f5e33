"""Builds libcust_opapi.so (the aclnn C-ABI over the gfx950 HIP kernels) in-tree with hipcc.

    python ops-transformer_amd/build.py [--force]

hipcc cross-compiles for gfx950 without a GPU.  Objects go to ops-transformer_amd/build/, the library to
ops-transformer_amd/lib/libcust_opapi.so — the file name the reference's dlsym-based binder searches first
(common/include/fallback/fallback.h:79-135 in the reference).
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libcust_opapi.so")

SOURCES = [
    "acl_runtime.cpp",
    "moe_gating_top_k_softmax_v2.hip",
    "moe_init_routing.hip",
    "grouped_gemm_i8.hip",
    "grouped_matmul_swiglu_quant.hip",
    "grouped_matmul_v4.hip",
    "grouped_matmul_finalize_routing.hip",
    "moe_finalize_routing_v2.hip",
    "calibration_copy.hip",
]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

COMMON_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "--offload-arch=gfx950",
    "-ffp-contract=off",
    # packed-fp32 instructions stay off for all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


def _headers():
    out = []
    for base in (CSRC, os.path.join(ROOT, "include")):
        for d, _, files in os.walk(base):
            out += [os.path.join(d, f) for f in files if f.endswith(".h")]
    return out


def _compile(src, force):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    src_path = os.path.join(CSRC, src)
    deps = [src_path] + _headers()
    if not force and os.path.exists(obj) and all(os.path.getmtime(obj) >= os.path.getmtime(d) for d in deps):
        return obj, False
    cmd = [HIPCC] + COMMON_FLAGS + (["-x", "hip"] if src.endswith(".cpp") else []) + ["-c", src_path, "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    log = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
    if log.strip():
        sys.stderr.write(log + "\n")
    return obj, True


def build(force=False, jobs=None):
    """Compile every source for gfx950 and link the shared library.  Returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    jobs = jobs or min(len(SOURCES), os.cpu_count() or 1)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(lambda s: _compile(s, force), SOURCES))
    objs = [o for o, _ in results]
    rebuilt = any(r for _, r in results)
    if rebuilt or not os.path.exists(LIB_PATH):
        cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB_PATH] + objs
        subprocess.check_call(cmd)
    return LIB_PATH


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
