"""The C ABI used from plain C99 (tests/c/abi_client.c), the way a cinterop / Panama binding uses it: the header
compiles as strict C, the client links against the built library, the host-only leg runs here and the device leg
(one Q8_0 matvec with a closed-form answer, bit-exact) on the GPU box."""
import os
import subprocess

import pytest

from skainet_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def client(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("abi") / "abi_client")
    libdir = os.path.dirname(runtime.LIB_PATH)
    cmd = ["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "c", "abi_client.c"), "-o", exe, "-L", libdir, "-lskainet_hip",
           f"-Wl,-rpath,{libdir}"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    return exe


def test_c_client_host_leg(client):
    r = subprocess.run([client, "host"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0 and r.stdout.strip() == "ok", r.stderr


@pytest.mark.gpu
def test_c_client_device_leg(client):
    r = subprocess.run([client, "device"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and r.stdout.strip() == "ok", r.stderr
