"""Builds libpskv.so (hand-written HIP for gfx950) in-tree with hipcc.

The library is the product: tests, the smoke check and the benchmark load the
built file and never fall back to anything else.
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libpskv.so")
SOURCES = ["table.hip", "slice.hip", "hostmem.hip", "stager.hip", "match.hip", "meta_codec.cc"]
HEADERS = ["device_common.h", "host_common.h", "scan.h", "stager.h", "table_kernels.h"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",  # float sums must round exactly like the CPU's `+=`
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-I" + os.path.join(REPO, "include"),
]


def lib_path():
    return LIB


def is_built():
    return os.path.exists(LIB)


def build_lib(verbose=False):
    """Compiles every HIP source and links libpskv.so. Always compiles."""
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
        cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if verbose and out.strip():
            print(out, flush=True)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB]
    subprocess.run(cmd, check=True)
    return LIB


HOST_TEST = os.path.join(REPO, "tests", "test_kv_app_gpu")


def build_host_test():
    """Compiles the test program tests/test_kv_app_gpu.cc, which drives the adapters of
    include/pskv/ps_adapters.h the way tests/test_kv_app.cc of the reference drives ps-lite
    (test infrastructure: it uses the in-process ps:: surface of tests/include/pskv/ps_min.h)."""
    cmd = ["g++", "-std=c++11", "-O2", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
           "-I" + os.path.join(REPO, "include"), "-I" + os.path.join(REPO, "tests", "include"),
           os.path.join(REPO, "tests", "test_kv_app_gpu.cc"), "-L" + HERE, "-lpskv",
           "-Wl,-rpath,$ORIGIN/../ps-lite_amd", "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib", "-lamdhip64",
           "-o", HOST_TEST]
    subprocess.run(cmd, check=True)
    # the same program for a ps-lite built with 32-bit keys (USE_KEY32, include/ps/base.h:10-16)
    subprocess.run(cmd[:-1] + [HOST_TEST + "32", "-DUSE_KEY32=1"], check=True)
    return HOST_TEST


def build_oracle():
    """Compiles the CPU oracle (test infrastructure) and, when the reference tree is
    present, the reference's own slicer into oracle/_ref/."""
    # (-B: compiled on every call, like the library, so that a call says whether it still builds)
    subprocess.run(["make", "-B", "-C", os.path.join(REPO, "oracle")], check=True,
                   stdout=subprocess.DEVNULL)


if __name__ == "__main__":
    print(build_lib(verbose=True))
