"""Runs the host-only native tests of the GGUF reader and the Pack v3 builder / adopter (tests/native/test_pack_v3.cpp):
files, hashing and the byte-exact inverse proof need no GPU."""
import importlib
import os
import subprocess

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "bin", "test_pack_v3")


def test_pack_v3_host():
    if not os.path.exists(BIN):  # nothing built yet: build the host library and the native tests
        build = importlib.import_module("tokspur-public_amd.build")
        if not os.path.exists(build.LIB):
            build.build()
        build.build_host()
        build.build_native_tests()
    proc = subprocess.run([BIN], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout[-4000:]
