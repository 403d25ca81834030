"""The drop-in boundary WITHOUT a GPU: libpskv.so loads and exports every function that
include/pskv/capi.h declares, its signatures are plain C, and the C++ adapters compile both
against the in-process ps:: surface and against the real ps-lite headers."""
import ctypes
import os
import re
import subprocess

import pytest

from conftest import REPO

HEADER = os.path.join(REPO, "include", "pskv", "capi.h")
REFERENCE = "/root/reference"


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pskv_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(capi):
    lib = capi.load()
    names = declared_functions()
    assert len(names) >= 15
    for name in names:
        assert hasattr(lib, name), "libpskv.so does not export %s" % name
    assert sorted(capi.SYMBOLS) == names, "the ctypes binding and the header disagree"


def test_header_is_plain_c(tmp_path):
    """The boundary is a C ABI: the header compiles as C99 and mentions no C++ or torch type."""
    src = tmp_path / "use.c"
    src.write_text('#include "pskv/capi.h"\nint main(void){ pskv_opts o; (void)o; return PSKV_OK; }\n')
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I" + os.path.join(REPO, "include"), "-c", str(src),
                    "-o", str(tmp_path / "use.o")], check=True)
    code = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)  # comments may cite C++ names
    assert "torch" not in code and "std::" not in code and "at::" not in code


def test_errors_without_a_device(capi):
    """No compute here: only that misuse is reported through status codes and not by crashing."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("covered by the GPU tests")
    with pytest.raises(capi.PskvError) as e:
        capi.Table()
    assert e.value.code == capi.EHIP
    b, e_ = capi.server_ranges(4)
    assert int(e_[-1]) == ((1 << 64) - 1) // 4 * 4
    assert capi.version().startswith("pskv")
    # the recorded-request entry points refuse what they can refuse without a table
    import ctypes
    lib = capi.load()
    h = ctypes.c_void_p()
    assert lib.pskv_replay_record(ctypes.byref(h), None, 0, capi.REPLAY_PUSH, None, None, None, None, None, None,
                                  None, None) == capi.EINVAL
    assert lib.pskv_replay_record(None, None, 0, capi.REPLAY_PUSH, None, None, None, None, None, None, None,
                                  None) == capi.EINVAL
    assert lib.pskv_replay_run(None) == capi.EINVAL
    assert lib.pskv_replay_destroy(None) == capi.OK


def test_adapters_compile_with_in_process_surface(tmp_path):
    subprocess.run(["g++", "-std=c++11", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__", "-isystem", "/opt/rocm/include",
                    "-I" + os.path.join(REPO, "include"), "-I" + os.path.join(REPO, "tests", "include"), "-c",
                    os.path.join(REPO, "tests", "test_kv_app_gpu.cc"), "-o",
                    str(tmp_path / "t.o")], check=True)


@pytest.mark.parametrize("key32", [0, 1])
def test_adapters_fit_real_pslite_headers(tmp_path, key32):
    """KVWorker::set_slicer / KVServer::set_request_handle of the real library accept the adapters,
    with its 64-bit keys and in a USE_KEY32 build (include/ps/base.h:10-16)."""
    if not os.path.exists(os.path.join(REFERENCE, "include", "ps", "ps.h")):
        pytest.skip("the reference tree is not present on this machine")
    subprocess.run(["g++", "-std=c++11", "-DUSE_KEY32=%d" % key32, "-I" + os.path.join(REFERENCE, "include"),
                    "-I" + os.path.join(REPO, "include"), "-c",
                    os.path.join(REPO, "tests", "adapters_real_pslite_check.cc"), "-o", str(tmp_path / "c.o")],
                   check=True)


def test_product_never_touches_the_oracle():
    """The shipped path must not import, link or call anything under oracle/."""
    for root in ("ps-lite_amd", "include"):
        for dirpath, _, files in os.walk(os.path.join(REPO, root)):
            for f in files:
                if f.endswith((".py", ".h", ".hip", ".cc", ".cpp")):
                    text = open(os.path.join(dirpath, f), errors="replace").read()
                    assert "pskv_oracle" not in text and "liboracle" not in text, os.path.join(dirpath, f)
                    if f != "build.py":
                        assert "oracle" not in text.lower() or f == "build.py", os.path.join(dirpath, f)


def test_bench_measures_one_gpu_only():
    """A table lives on one device; asked for more GPUs the benchmark says so and stops."""
    import sys
    p = subprocess.run([sys.executable, os.path.join(REPO, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert p.returncode != 0
    assert "ONE GPU" in (p.stdout + p.stderr)
    assert not p.stdout.strip().startswith("{")  # no result line


def test_bench_reads_its_traffic_figures_from_the_profiles():
    """roofline.traffic is not typed into bench.py: it comes from the `traffic_per_launch:` lines of the
    rocprofv3 summaries under profiles/, for the launch shapes the default commands run."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_for_test", os.path.join(REPO, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    table = bench.traffic_table()
    for kind, units in [("push_scalar", 1000000), ("rows_acc_fixed", 268435456), ("rows_gather_fixed", 268435456),
                        ("rows_acc_varlen", 99077384), ("rows_gather_varlen", 99077384),
                        ("push_scalar_cached", 16000000), ("same_keys", 16000000)]:
        assert (kind, units) in table, (kind, units)
        nbytes, source = table[(kind, units)]
        assert nbytes > 0 and source.startswith("profiles/")
        assert os.path.exists(os.path.join(REPO, source))
    # every figure is at least the algorithmic traffic of its kernel and within 2x of it, except the
    # random-probe kernel, which moves whole lines
    assert 0.99 * 12 * 268435456 <= table[("rows_acc_fixed", 268435456)][0] <= 1.05 * 12 * 268435456
    assert 0.99 * 12 * 99077384 <= table[("rows_acc_varlen", 99077384)][0] <= 1.1 * 12 * 99077384
    assert 0.99 * 12 * 16000000 <= table[("push_scalar_cached", 16000000)][0] <= 1.05 * 12 * 16000000
    assert bench.traffic("push_scalar", 123) is None  # another launch shape: no figure
