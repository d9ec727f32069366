"""The C ABI from a C program (tests/c_client/kv_client.c): the public header compiled as C99
with warnings as errors, the library linked the way a foreign-function binding links it, and
results checked against double-precision arithmetic done in C, not against the Python oracle."""
import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "c_client"))
import build_client  # noqa: E402


def run(mode, directory, timeout):
    binary = build_client.BINARY
    if not os.path.exists(binary) or mode == "host":
        binary = build_client.build()
    env = dict(os.environ)
    # The run-time search path compiled in is this tree's; a copied tree finds the library here.
    env["LD_LIBRARY_PATH"] = build_client.LIB_DIR + os.pathsep + env.get("LD_LIBRARY_PATH", "")
    res = subprocess.run([binary, mode, str(directory)], capture_output=True, text=True,
                         timeout=timeout, env=env)
    assert res.returncode == 0, res.stderr + res.stdout
    assert res.stdout.strip() == f"{mode} ok"


def test_hashes_codec_and_store_from_c(tmp_path):
    run("host", tmp_path, 60)


@pytest.mark.gpu
def test_pool_attention_round_snapshot_and_store_from_c(tmp_path):
    run("device", tmp_path, 110)
