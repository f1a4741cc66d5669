"""Builds libmegray_vrank.so (the gfx950 kernels, the planner, the MegRay C++ API and the C ABI)
with hipcc, in tree.  Run as ``python -m megray_amd.build``."""
import json
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(HERE, "libmegray_vrank.so")
RESOURCES_PATH = os.path.join(HERE, "kernel_resources.json")  # registers, scratch, LDS of every kernel built

ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.environ.get("HIPCC", os.path.join(ROCM, "bin", "hipcc"))
ARCH = "gfx950"

COMMON_FLAGS = [
    "-std=c++17", "-O3", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter",
    "-ffp-contract=off",  # a fold is a chain of single IEEE operations; never fuse
    f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}",
]
# device code: gfx950 only; packed fp32 instructions (v_pk_add_f32 / v_pk_mul_f32 / v_pk_fma_f32) are kept out of
# the generated code.  The feature flag acts on the DEVICE pass; hipcc's host pass does not know it and prints
# "'-packed-fp32-ops' is not a recognized feature for this target (ignoring feature)", which _diagnostics() drops
# from the log.  tests/test_build_flags.py compiles a float2 kernel both ways and checks the device assembly.
DEVICE_FLAGS = [f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def sources():
    out = []
    for name in sorted(os.listdir(CSRC)):
        if name.endswith(".cpp") or name.endswith(".hip"):
            out.append(os.path.join(CSRC, name))
    return out


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
    cmd = [HIPCC] + COMMON_FLAGS
    if src.endswith(".hip"):
        cmd += ["-x", "hip", "-Rpass-analysis=kernel-resource-usage"] + DEVICE_FLAGS
    else:  # host-only translation units: plain C++ against the HIP runtime API headers
        cmd += ["-x", "c++", "-D__HIP_PLATFORM_AMD__=1", "-pthread", f"-I{ROCM}/include"]
    cmd += ["-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    return src, obj, proc


def _kernel_resources(stderr):
    """{kernel symbol: {"vgprs", "agprs", "sgprs", "scratch", "lds", "occupancy"}} from the compiler's
    kernel-resource-usage remarks."""
    out, cur = {}, None
    keys = {"VGPRs": "vgprs", "AGPRs": "agprs", "TotalSGPRs": "sgprs", "ScratchSize [bytes/lane]": "scratch",
            "LDS Size [bytes/block]": "lds", "Occupancy [waves/SIMD]": "occupancy"}
    for line in stderr.splitlines():
        m = re.search(r"remark: (?:\s*)([^:]+): (\S+) \[-Rpass-analysis=kernel-resource-usage\]", line)
        if not m:
            continue
        key, value = m.group(1).strip(), m.group(2)
        if key == "Function Name":
            cur = out.setdefault(value, {})
        elif cur is not None and key in keys:
            cur[keys[key]] = int(value)
    return out


def _diagnostics(stderr, noise):
    """The compiler's output without the resource-usage remarks (and the source excerpts under them)."""
    kept, in_remark = [], False
    for line in stderr.splitlines():
        if "[-Rpass-analysis=kernel-resource-usage]" in line:
            in_remark = True
            continue
        if in_remark and (re.match(r"^\s*\d*\s*\|", line) or line.startswith("In file included from")):
            continue
        in_remark = False
        if noise in line or re.match(r"^\d+ warnings? generated", line):
            continue
        kept.append(line)
    # "In file included from" headers whose remark followed them
    return "\n".join(l for i, l in enumerate(kept)
                     if not (l.startswith("In file included from") and (i + 1 == len(kept) or kept[i + 1].startswith("In file included from") or not kept[i + 1].strip())))


def build_library(verbose=True):
    """Compile every source and link the shared library.  Always recompiles."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        results = list(pool.map(_compile, srcs))
    objs = []
    resources = {}
    for src, obj, proc in results:
        noise = "'-packed-fp32-ops' is not a recognized feature"
        resources.update(_kernel_resources(proc.stderr))
        err = _diagnostics(proc.stderr, noise)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}\n{proc.stderr}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
        objs.append(obj)
    with open(RESOURCES_PATH, "w") as f:
        json.dump(resources, f, indent=1, sort_keys=True)
    link = [HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB_PATH] + objs + ["-lpthread"]
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    return LIB_PATH


CPP_TEST_SRC = os.path.join(ROOT, "tests", "cpp", "test_vrank_opr.cpp")
CPP_TEST_BIN = os.path.join(ROOT, "tests", "cpp", "test_vrank_opr")


def build_cpp_test():
    """Compile the thread-per-rank C++ API test against the library just built."""
    cmd = [HIPCC, "-std=c++17", "-O2", "-x", "c++", "-D__HIP_PLATFORM_AMD__=1", f"-I{os.path.join(ROOT, 'include')}",
           f"-I{ROCM}/include", CPP_TEST_SRC, "-o", CPP_TEST_BIN, f"-L{HERE}", "-lmegray_vrank", f"-L{ROCM}/lib",
           "-lamdhip64", "-pthread", "-Wl,-rpath,$ORIGIN/../../megray_amd", f"-Wl,-rpath,{ROCM}/lib"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"building {CPP_TEST_SRC} failed:\n{proc.stdout}\n{proc.stderr}")
    return CPP_TEST_BIN


PERF_SRC = os.path.join(HERE, "apps", "performance.cpp")
PERF_BIN = os.path.join(HERE, "apps", "megray_performance")


def build_performance():
    """Compile the performance CLI (the MegRay benchmark harness for this backend)."""
    # compiled as HIP: the tool has one kernel of its own (the random fill of -R)
    cmd = [HIPCC, "-std=c++17", "-O2", "-x", "hip", "-ffp-contract=off"] + DEVICE_FLAGS + [
           f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}", PERF_SRC, "-o", PERF_BIN, f"-L{HERE}", "-lmegray_vrank",
           "-pthread", "-Wl,-rpath,$ORIGIN/..", f"-Wl,-rpath,{ROCM}/lib"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"building {PERF_SRC} failed:\n{proc.stdout}\n{proc.stderr}")
    return PERF_BIN


if __name__ == "__main__":
    print(build_library())
    print(build_cpp_test())
    print(build_performance())
