"""The library from a host program in plain C: loaded with dlopen(RTLD_LAZY | RTLD_LOCAL) and resolved
name by name with dlsym, which is how ZLUDA's tracing interposer reaches the library it wraps
(zluda_trace_common/src/lib.rs:67-71, zluda_trace_blaslt/src/lib.rs:6-11 and :24) and how a CUDA
application's dynamic linker does; no Python, torch or initialised HIP runtime in that process."""
import os
import subprocess

import pytest

from zluda_amd.cublaslt import SIGNATURES

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST_DIR = os.path.join(ROOT, "tests", "host_c")
HOST = os.path.join(HOST_DIR, "plain_c_host")


@pytest.fixture(scope="module")
def host():
    if not os.path.exists(HOST):
        subprocess.run(["make", "-C", HOST_DIR, "plain_c_host"], check=True)
    return HOST


def run(host, api, *args, timeout=120):
    # the versioned name a CUDA 12 application asks for (zluda_blaslt/Cargo.toml:21-23)
    lib = os.path.join(os.path.dirname(api.path), "libcublasLt.so.12")
    env = {k: v for k, v in os.environ.items() if k != "LD_LIBRARY_PATH"}   # the library's own RUNPATH must do
    r = subprocess.run([host, lib, *args], capture_output=True, text=True, timeout=timeout, env=env)
    print(r.stdout, r.stderr, flush=True)
    return r


def test_every_export_resolves_for_a_local_dlopen(host, api):
    r = run(host, api, "symbols", *sorted(SIGNATURES))
    assert r.returncode == 0, r.stderr
    assert r.stdout.strip() == "45 names, 0 missing"


def test_a_missing_name_is_reported(host, api):
    r = run(host, api, "symbols", "cublasLtMatmul", "cublasLtShutdownCtx")   # cuda_macros/src/cublaslt_internal.rs:4
    assert r.returncode == 1 and "missing export cublasLtShutdownCtx" in r.stderr


@pytest.mark.gpu
def test_int8_problems_from_plain_c(host, gpu_api):
    r = run(host, gpu_api, "matmul")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "plain C host ok" in r.stdout
    assert r.stdout.count("0 of ") == 4
