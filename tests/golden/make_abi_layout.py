"""Writes tests/golden/art_abi_layout.txt: sizes, offsets and constants of the art C API as the REFERENCE
headers define them (compiled with the definitions of a normal NART build).  Needs /root/reference."""
import os
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [os.path.dirname(HERE), os.path.dirname(os.path.dirname(HERE))]
from test_engine_cpu import REF_TREE, _probe_source  # noqa: E402

with tempfile.TemporaryDirectory() as d:
    src, exe = os.path.join(d, "probe.c"), os.path.join(d, "probe")
    open(src, "w").write(_probe_source())
    subprocess.check_call(["gcc", "-std=gnu11", "-w", "-DUSE_REF", "-DART_CONSTRAINT_WITH_NAME", "-DNART_LOG_LEVEL=1",
                           "-I" + os.path.join(REF_TREE, "art", "include"), src, "-o", exe])
    out = subprocess.check_output([exe]).decode()
open(os.path.join(HERE, "art_abi_layout.txt"), "w").write(out)
print(out)
