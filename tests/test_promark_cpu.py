"""nart_promark (nart_amd/csrc/tools/promark.cpp): argument and configuration handling, no GPU needed.
The reference's runner (tools/promark.cpp) prints the usage line and returns 1 without arguments (:214-228), and
refuses a configuration without "workspaces" / "input_workspace" or with an unknown module (:136-190)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOOL = os.path.join(ROOT, "nart_amd", "lib", "nart_promark")


def run(args, cwd=None):
    return subprocess.run([TOOL] + args, cwd=cwd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)


def test_usage():
    r = run([])
    assert r.returncode == 1 and "Usage" in r.stderr and "-m model" in r.stderr
    r = run(["-n", "3"])  # no model file
    assert r.returncode == 1 and "Usage" in r.stderr


def test_configuration_errors(tmp_path):
    cfg = tmp_path / "c.json"
    for text, msg in (('{"workspaces": {"nope": {}}, "input_workspace": "nope"}', "module not found"),
                      ('{"workspaces": 3}', "[workspaces] required"),
                      ('{"workspaces": {}, "input_workspace": 7}', "\"input_workspace\" required"),
                      ('{"workspaces": {}, "input_workspace": "hip"}', "has not been registered"),
                      ('{"workspaces": {"a": {}', "Parse config error"),
                      ('[1, 2]', "Parse config error")):
        cfg.write_text(text)
        r = run(["-m", str(tmp_path / "missing.bin"), "-c", str(cfg)])
        assert r.returncode == 1, text
        assert msg in r.stderr and "init module failed" in r.stderr, (text, r.stderr)
