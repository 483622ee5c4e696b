"""The C ABI from a host that is neither Python nor PyTorch: tests/cabi_host/host_check.cpp links the library
through include/dg_attn.h with the system's HIP runtime, the way the reference's Rust side would through its FFI
(src/metal/step_kernel/enc.rs:2102-2220 is the call site a src/hip backend replaces), runs four attention cases and
one producer + attention layer step and compares each with the CPU oracle.  The program is built by __graft_entry__.build() (tests/cabi_host/Makefile);
this test runs it as a child process and reads its verdict."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "cabi_host", "host_check")


def test_c_host_program_passes_against_the_oracle(gpu_ready):
    assert os.path.exists(BINARY), f"{BINARY} is missing: __graft_entry__.build() (or make -C tests/cabi_host) builds it"
    res = subprocess.run([BINARY], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(res.stdout, flush=True)
    assert res.returncode == 0, res.stdout[-3000:]
    assert res.stdout.count("PASS ") == 5 and "all cases passed" in res.stdout
