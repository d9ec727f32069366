"""CPU-only checks of the C ABI: the library loads, exports exactly what the header
declares, and refuses bad construction arguments by name without touching a GPU."""
import ctypes as C
import os
import subprocess
import sys

import pytest

from helpers import HEADER, ROOT, declared_symbols, pkg


def test_library_exports_every_declared_symbol():
    N = pkg()._native
    lib = N.load()
    declared = declared_symbols()
    assert len(declared) >= 30
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    assert sorted(N.PROTOTYPES) == declared, "binding table and header disagree"
    out = subprocess.check_output(["nm", "-D", "--defined-only", N.LIB_PATH], text=True)
    exported = sorted(l.split()[-1] for l in out.splitlines() if " T itak_" in l)
    assert exported == declared
    assert lib.itak_abi_version() == 1


def test_library_does_not_link_the_oracle():
    N = pkg()._native
    out = subprocess.check_output(["ldd", N.LIB_PATH], text=True)
    assert "oracle" not in out
    syms = subprocess.check_output(["nm", "-D", N.LIB_PATH], text=True)
    assert "orc_" not in syms


def _create(**kw):
    N = pkg()._native
    lib = N.load()
    cfg = N.PoolConfig()
    cfg.layer_count = kw.get("layers", 1)
    cfg.num_kv_heads = kw.get("kv_heads", 2)
    cfg.head_dim = kw.get("head_dim", 128)
    cfg.elem = kw.get("elem", N.ELEM_F32)
    cfg.max_slots = kw.get("max_slots", 1)
    cfg.capacity_rows = kw.get("capacity", 16)
    kinds = kw.get("kinds")
    windows = kw.get("windows")
    keep = []
    if kinds is not None:
        arr = (C.c_uint8 * len(kinds))(*kinds)
        keep.append(arr)
        cfg.layer_kinds = C.cast(arr, C.c_void_p)
    if windows is not None:
        arr = (C.c_uint64 * len(windows))(*windows)
        keep.append(arr)
        cfg.windows = C.cast(arr, C.c_void_p)
    handle = C.c_void_p()
    status = lib.itak_pool_create(C.byref(cfg), C.byref(handle))
    info = N.ErrorInfo()
    lib.itak_last_error_info(None, C.byref(info))
    return status, info, (lib.itak_last_error(None) or b"").decode(), handle


def test_construction_refusals_need_no_gpu():
    # The refusals of KvCache::new (crates/attention/tests/cache_tests.rs:133-183).
    status, info, msg, _ = _create(layers=0)
    assert (status, info.what) == (1, b"layer pattern")
    assert msg == "layer pattern must be positive, got 0"
    status, info, _, _ = _create(kv_heads=0)
    assert (status, info.what) == (1, b"num_kv_heads")
    status, info, _, _ = _create(head_dim=0)
    assert (status, info.what) == (1, b"head_dim")
    status, info, msg, _ = _create(kinds=[1], windows=[0])
    assert status == 2 and msg == "sliding window must be positive, got 0"
    status, info, _, _ = _create(kinds=[1], windows=[2**64 - 1])
    assert (status, info.what) == (3, b"windowed layer storage")
    status, info, _, _ = _create(kv_heads=2**64 - 1, head_dim=2)
    assert (status, info.what) == (3, b"kv row length")
    # A valid windowed pattern passes every check and goes on to the device (absent here: a
    # HIP error, not a refusal of the pattern).
    status, info, msg, handle = _create(kinds=[1], windows=[4])
    assert status in (0, 16), msg
    if status == 0:
        N.load().itak_pool_destroy(handle)
    status, _, msg, _ = _create(elem=7)
    assert status == 17


def test_debug_channel_is_off_by_default_and_says_why_a_call_was_refused(capfd):
    # attention::diag (crates/attention/src/diag.rs:13-33 and its two tests, :108-131): silent
    # unless switched on; a line per event with a fixed prefix when it is.
    lib = pkg()._native.load()
    os.environ.pop("ITAK_HIP_KV_DEBUG", None)
    lib.itak_set_debug_enabled(0)
    assert lib.itak_debug_enabled() == 0
    _create(layers=0)
    assert "[itak_hip_kv::diag]" not in capfd.readouterr().err
    lib.itak_set_debug_enabled(1)
    try:
        assert lib.itak_debug_enabled() == 1
        _create(layers=0)
        err = capfd.readouterr().err
        assert "[itak_hip_kv::diag] refused code=1: layer pattern must be positive, got 0" in err
    finally:
        lib.itak_set_debug_enabled(0)
    # The environment variable is looked up at every event: any value but "0" or empty.
    for value, on in (("1", True), ("yes", True), ("0", False), ("", False)):
        os.environ["ITAK_HIP_KV_DEBUG"] = value
        try:
            assert lib.itak_debug_enabled() == int(on), value
            _create(kv_heads=0)
            assert ("refused code=1: num_kv_heads" in capfd.readouterr().err) == on, value
        finally:
            del os.environ["ITAK_HIP_KV_DEBUG"]


def test_python_front_end_raises_named_errors_without_a_gpu():
    P = pkg()
    with pytest.raises(P.AttentionError) as e:
        P.KvPool([], 2, 128)
    assert e.value == P.AttentionError("ZeroDimension", what="layer pattern")
    with pytest.raises(P.AttentionError) as e:
        P.LayerKind.windowed(0)
    assert e.value == P.AttentionError("InvalidWindow", window=0)
    with pytest.raises(P.AttentionError) as e:
        P.kv_head_for_query_head(0, 3, 2)
    assert e.value == P.AttentionError("NonDivisibleHeads", num_q_heads=3, num_kv_heads=2)
    for h in range(32):
        assert P.kv_head_for_query_head(h, 32, 2) == (0 if h < 16 else 1)
    assert abs(float(P.AttentionParams.new().scale_for(128)) - 0.08838835) < 1e-7
    cache = P.PositionCache()
    cache.advance(5)
    cache.rewind_to(3)
    assert cache.position() == 3


def test_product_sources_never_reference_the_oracle():
    import os

    root = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                        "itak-torch-rebuild_amd")
    for dirpath, _, files in os.walk(root):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "itak_oracle" not in text, f


def _rust_externs():
    """name -> argument count of every `pub fn` in the extern block of itak-hip-sys."""
    import re
    path = os.path.join(ROOT, "crates", "itak-hip-sys", "src", "lib.rs")
    text = open(path).read()
    block = text[text.index('extern "C" {'):]
    block = block[:block.index("\n}")]
    out = {}
    for name, args in re.findall(r"pub fn (itak_[a-z0-9_]+)\((.*?)\)(?: -> [^;]+)?;", block):
        out[name] = 0 if not args.strip() else len([a for a in args.split(",") if a.strip()])
    return out


def _header_functions():
    import re
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    out = {}
    for name, args in re.findall(r"\b(itak_[a-z0-9_]+)\s*\(([^;{}]*?)\)\s*;", text, flags=re.S):
        args = " ".join(args.split())
        out[name] = 0 if args in ("", "void") else len(args.split(","))
    return out


def test_rust_binding_declares_the_header_symbol_for_symbol():
    # crates/itak-hip-sys/src/lib.rs is written from the header by gen_bindings.py: the same
    # functions with the same number of arguments, the ctypes table too, and the file is current.
    N = pkg()._native
    rust, header = _rust_externs(), _header_functions()
    assert sorted(rust) == sorted(header) == declared_symbols()
    assert rust == header
    table = {name: len(proto[1]) for name, proto in N.PROTOTYPES.items()}
    assert table == header
    gen = os.path.join(ROOT, "crates", "itak-hip-sys", "gen_bindings.py")
    assert subprocess.run([sys.executable, gen, "--check"]).returncode == 0
    # Every struct the header declares has a #[repr(C)] twin.
    import re
    text = open(os.path.join(ROOT, "crates", "itak-hip-sys", "src", "lib.rs")).read()
    header_text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    for name in re.findall(r"typedef\s+struct\s+(\w+)", header_text):
        assert f"pub struct {name} " in text, name


def _rust_calls(path):
    """(name, argument count, line) of every call of an `itak_*` function in a Rust source:
    arguments are counted by the commas at the call's own nesting depth."""
    import re
    text = re.sub(r"//[^\n]*", "", open(path).read())
    calls = []
    for m in re.finditer(r"\b(itak_[a-z0-9_]+)\s*\(", text):
        if re.search(r"\bfn\s+$", text[:m.start()]):
            continue  # a declaration, not a call
        depth, commas, i, seen = 1, 0, m.end(), False
        while depth:
            c = text[i]
            depth += c in "([{"
            depth -= c in ")]}"
            commas += c == "," and depth == 1
            seen = seen or (depth >= 1 and not c.isspace())
            trailing = c == "," and depth == 1 and text[i + 1:].lstrip().startswith(")")
            commas -= trailing
            i += 1
        calls.append((m.group(1), commas + 1 if seen else 0, text.count("\n", 0, m.start()) + 1))
    return calls


def test_the_safe_rust_layer_calls_the_header_with_the_headers_arity():
    # The crates are source only here (no Rust toolchain): what a compiler would check of the
    # safe layer's calls into the extern block is checked as text, so that a function renamed or
    # given another argument in the header does not leave the wrappers behind.
    header = _header_functions()
    seen = set()
    for rel in (("itak-hip-sys", "src", "safe.rs"), ("hip-compute", "src", "lib.rs"),
                ("hip-compute", "src", "target.rs")):
        path = os.path.join(ROOT, "crates", *rel)
        for name, count, line in _rust_calls(path):
            assert name in header, f"{'/'.join(rel)}:{line} calls {name}, which the header does not declare"
            assert count == header[name], \
                f"{'/'.join(rel)}:{line} calls {name} with {count} arguments, the header declares {header[name]}"
            seen.add(name)
    assert {"itak_pool_create", "itak_compute_attention", "itak_kv_truncate",
            "itak_store_restore_prefix", "itak_store_capture_and_put"} <= seen
