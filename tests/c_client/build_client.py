"""Builds tests/c_client/kv_client.c with gcc as plain C99 against the public header and the
in-tree shared library (run-time search path set to the library's directory)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB_DIR = os.path.join(ROOT, "itak-torch-rebuild_amd", "lib")
BINARY = os.path.join(HERE, "kv_client")


def build(force: bool = False) -> str:
    src = os.path.join(HERE, "kv_client.c")
    lib = os.path.join(LIB_DIR, "libitak_hip_kv.so")
    if not os.path.exists(lib):
        raise RuntimeError(f"{lib} is missing: build the library first")
    newest = max(os.path.getmtime(p) for p in (src, lib, os.path.join(ROOT, "include", "itak_hip_kv.h")))
    if not force and os.path.exists(BINARY) and os.path.getmtime(BINARY) >= newest:
        return BINARY
    cmd = ["gcc", "-std=c99", "-O1", "-Wall", "-Wextra", "-pedantic", "-Werror",
           "-I", os.path.join(ROOT, "include"), src, "-o", BINARY,
           "-L", LIB_DIR, "-litak_hip_kv", "-lm",
           "-Wl,-rpath," + LIB_DIR, "-Wl,-rpath-link,/opt/rocm/lib", "-Wl,--allow-shlib-undefined"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("gcc failed on kv_client.c:\n" + res.stderr)
    return BINARY


if __name__ == "__main__":
    print(build(force=True))
