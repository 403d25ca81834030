"""Runs the C++ program that drives the GPU slicer and the GPU request handle through the
ps::KVWorker / ps::KVServer interface the way tests/test_kv_app.cc of the reference does."""
import os
import subprocess

import pytest

from conftest import REPO, announce

pytestmark = pytest.mark.gpu

BIN = os.path.join(REPO, "tests", "test_kv_app_gpu")


@pytest.mark.parametrize("num_servers", [1, 2, 4])
def test_kv_app_through_adapters(num_servers):
    announce("kv_app_through_adapters", num_servers)
    assert os.path.exists(BIN), "build() compiles tests/test_kv_app_gpu"
    r = subprocess.run([BIN, str(num_servers)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True, timeout=100)
    print(r.stdout)
    assert r.returncode == 0, r.stdout
    assert "test_kv_app_gpu: ok" in r.stdout
    # the two workers of tests/test_kv_app_multi_workers.cc ran, each on its own thread
    assert "two workers, customer 0: error 0, 0" in r.stdout and "two workers, customer 1: error 0, 0" in r.stdout
    # the reference test's 50 pushes of one key set, recorded once and replayed through the C ABI alone
    assert "ranges replayed, 0 + 0 floats differ" in r.stdout


def test_kv_app_with_32_bit_keys():
    """The same program compiled as against a ps-lite with USE_KEY32 (include/ps/base.h:10-16): the adapters
    widen the keys for the C ABI; slices, sums and failure cases are those of the 64-bit run."""
    announce("kv_app_32_bit_keys")
    assert os.path.exists(BIN + "32"), "build() compiles tests/test_kv_app_gpu32"
    r = subprocess.run([BIN + "32", "2"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    print(r.stdout)
    assert r.returncode == 0, r.stdout
    assert "test_kv_app_gpu: ok" in r.stdout


def test_dense_chunks_from_host_memory_through_adapters():
    """Configuration 3 (64 keys x 4,194,304 floats, 1 GiB per request) from ordinary host memory through
    GpuSlicer + GpuKVHandle and through the C ABI alone; the program checks the sums against their closed
    form and prints the PCIe-inclusive rates (they are not the benchmark's `value`)."""
    announce("dense_from_host_through_adapters")
    assert os.path.exists(BIN), "build() compiles tests/test_kv_app_gpu"
    r = subprocess.run([BIN, "1", "4194304"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=280)
    print(r.stdout)
    assert r.returncode == 0, r.stdout
    assert "dense from host memory" in r.stdout and "test_kv_app_gpu: ok" in r.stdout
