"""CPU-only checks of the host side: the C ABI library loads and exports every
symbol the header declares, and the engine's host logic (kv_bits switch, cache
sizing, rotation matrix) behaves like the reference's.  No kernel is launched."""
import ctypes
import re
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "triebwerk_kv.h"


def declared_functions():
    text = HEADER.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b((?:launch|tw)_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_header_declares_the_reference_launchers():
    names = declared_functions()
    for fn in ("launch_kv_cache_write_batch", "launch_turbo_kv_quantize", "launch_turbo_kv_quantize_batch",
               "launch_gqa_attention", "launch_gqa_attention_batch", "launch_turbo_gqa_attention",
               "launch_turbo_gqa_attention_batch", "launch_gqa_prefill_attention",
               "launch_turbo_gqa_prefill_attention", "launch_increment_positions"):
        assert fn in names


def test_library_exports_every_declared_symbol():
    from triebwerk_amd import _lib
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, missing
    # and the Python binding table covers the same set
    assert sorted(_lib.SIGNATURES) == declared_functions()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from triebwerk_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(_lib.LibraryMissing):
        _lib.load()


def test_engine_kv_bits_switch(capfd):
    """engine.cpp:300-317: 0, 2, 4 are kept; anything else warns and falls back to fp16."""
    from triebwerk_amd import Engine
    assert Engine().kv_bits() == 0 and Engine().max_seq_len() == 1024  # engine_py.cpp:22 defaults
    assert Engine(512, 2).kv_bits() == 2
    assert Engine(max_seq_len=64, kv_bits=4).kv_bits() == 4
    capfd.readouterr()
    assert Engine(64, 3).kv_bits() == 0
    assert "kv_bits=3 not supported" in capfd.readouterr().err
    assert Engine(64, 8).kv_bits() == 0


def test_cache_sizes_match_the_reference_readme():
    """README.md:163-165: G=4, 28 layers, 1,024 tokens: fp16 448 MB, TQ4 116 MB.  The table's longer
    rows are not 8x those (8,192 tokens: 3,893 / 1,005 MB), so beyond the first row the test checks the
    arithmetic the layout fixes: 4096 | 1056 | 544 bytes per token and layer."""
    from triebwerk_amd import _lib
    lib = _lib.load()

    def cache_bytes(bits, G, msl):
        e = lib.tw_engine_create(1024, bits)
        total = lib.tw_engine_arena_bytes_needed(e, G, msl)
        lib.tw_engine_destroy(e)
        scratch = G * 16 * msl * 4
        return total - scratch

    mib = 1024 * 1024
    assert abs(cache_bytes(0, 4, 1024) / mib - 448) < 0.1
    assert abs(cache_bytes(4, 4, 1024) / mib - 115.5) < 0.1
    assert abs(cache_bytes(4, 4, 8192) / mib - 924) < 0.1      # 4*8192*28*1056 B
    assert abs(cache_bytes(2, 4, 1024) / mib - 59.5) < 0.1     # 544 B per token per layer


def test_set_shape_rejects_what_the_kernels_cannot_run():
    from triebwerk_amd import Engine
    e = Engine(64, 4)
    e.set_shape(36, 32, 8, 128)
    with pytest.raises(ValueError):
        e.set_shape(2, 16, 8, 64)
    with pytest.raises(ValueError):
        e.set_shape(2, 15, 8, 128)


def test_host_rotation_is_the_fixture(rotation_fixture):
    """The matrix the library builds on the host (engine.cpp:366-392) is the committed one."""
    from triebwerk_amd import kvcache
    r = kvcache.make_rotation(128, 42).numpy()
    assert np.array_equal(r.view(np.uint16), rotation_fixture.view(np.uint16))


def test_decode_step_plan_is_the_documented_rule():
    """Which decode-step form mode 0 picks, from host knowledge alone (no GPU needed: without a device the
    library assumes 256 compute units, the MI355X's number)."""
    from triebwerk_amd import _lib
    lib = _lib.load()
    plan = lib.tw_kv_decode_step_plan
    # the benchmark's target: 64 sequences of 8192 tokens, lengths known and equal -> one launch at 4 and at 2 bit
    # (2 bit: 73.7 against 76.8 us per layer); at 2 bit the three-kernel path is ahead for 96 sequences of that length
    # (110 against 114 us) and for small batches of long contexts
    assert plan(64, 16, 8, 4, 8448, 8192, 8192) == 1
    assert plan(64, 16, 8, 2, 8448, 8192, 8192) == 1
    assert plan(64, 16, 8, 2, 8448, 6000, 6000) == 1
    assert plan(96, 16, 8, 2, 8448, 8192, 8192) == 0
    assert plan(96, 16, 8, 2, 8448, 4096, 4096) == 1
    assert plan(128, 16, 8, 2, 8448, 4096, 4096) == 1
    assert plan(32, 16, 8, 2, 8448, 8192, 8192) == 0
    assert plan(128, 16, 8, 4, 8448, 4096, 4096) == 1
    # the same batch with nothing known about the lengths, or known to be ragged: three launches
    assert plan(64, 16, 8, 4, 8448, 0, 0) == 0
    assert plan(64, 16, 8, 4, 8448, 512, 8192) == 0
    # short contexts by max_seq_len alone: at most 8 tiles per wave (2 heads per workgroup -> 8 parts of 256 tokens)
    assert plan(64, 16, 8, 4, 2048, 0, 0) == 1
    assert plan(64, 16, 8, 4, 2049, 0, 0) == 0
    # a rollout: 128 sequences a few hundred tokens long, at either width
    assert plan(128, 16, 8, 4, 1536, 300, 300) == 1
    assert plan(128, 16, 8, 2, 1536, 300, 300) == 1
    # small batches: one head per workgroup, 16 parts; long contexts of few sequences do not fill the GPU with one
    # workgroup per (sequence, head) -- 63 us per layer against 45 at batch 16, 8192 tokens -- shorter ones do
    assert plan(4, 16, 8, 4, 640, 0, 0) == 1
    assert plan(4, 16, 8, 4, 16384, 16000, 16000) == 0
    assert plan(16, 16, 8, 4, 8448, 8192, 8192) == 0
    assert plan(32, 16, 8, 4, 8448, 8192, 8192) == 0
    assert plan(16, 16, 8, 4, 8448, 2048, 2048) == 1
    # a caller with tickets (the engine): the one launch may share a sequence's context between workgroups, which makes
    # it the choice for small batches of long sequences too; nothing changes where the batch fills the GPU or is ragged
    plan2 = lib.tw_kv_decode_step_plan2
    assert plan2(16, 32, 8, 2, 4352, 4097, 4097, 1) == 1          # BASELINE config 4
    assert plan2(4, 16, 8, 4, 16384, 16000, 16000, 1) == 1
    assert plan2(16, 16, 8, 4, 8448, 8192, 8192, 1) == 1
    assert plan2(32, 16, 8, 4, 8448, 8192, 8192, 1) == 1
    assert plan2(16, 16, 8, 4, 8448, 8192, 8192, 0) == 0
    assert plan2(64, 16, 8, 4, 8448, 8192, 8192, 1) == 1 and plan2(96, 16, 8, 2, 8448, 8192, 8192, 1) == 0
    assert plan2(64, 16, 8, 4, 8448, 512, 8192, 1) == 0
    assert plan2(16, 16, 8, 4, 400, 0, 0, 1) == 1                 # too little scratch for shares: as without
    assert plan(16, 32, 8, 2, 4352, 4097, 4097) == 1          # 2 bit, GQA 4, 65k tokens
    # batches that fill three quarters of the CUs with two or four heads per workgroup
    assert plan(48, 16, 8, 4, 8448, 8192, 8192) == 1
    assert plan(96, 16, 8, 4, 8448, 4096, 4096) == 1
    # large launches: the three-kernel path has caught up
    assert plan(256, 16, 8, 4, 8448, 8192, 8192) == 0
    assert plan(128, 16, 8, 4, 8448, 8192, 8192) == 1          # 183 against 188 us per layer
    # shapes the one-launch kernel does not take
    assert plan(64, 64, 8, 4, 1024, 0, 0) == 0                # GQA group 8
    assert plan(64, 16, 8, 3, 1024, 0, 0) == 0
    assert plan(0, 16, 8, 4, 1024, 0, 0) == 0


def header_prototypes():
    """name -> (return kind, [parameter kinds]) for every function the header declares; a kind is 'ptr', 'int',
    'uint', 'llong', 'size', 'float', 'double', 'bool', 'void' or 'cstr'."""
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    text = re.sub(r"typedef\s+struct\s+\w+\s*\{.*?\}\s*\w+\s*;", "", text, flags=re.S)   # struct bodies hold no prototypes

    def kind(decl: str) -> str:
        decl = decl.strip()
        if "*" in decl:
            return "cstr" if re.match(r"const\s+char\s*\*", decl) else "ptr"
        base = re.sub(r"\b(const|struct)\b", "", decl).split()
        if len(base) > 1 and re.match(r"^[A-Za-z_]\w*$", base[-1]) and base[-1] not in ("int", "long", "char", "unsigned"):
            base = base[:-1]                                       # drop the parameter's name
        t = " ".join(base)
        return {"int": "int", "unsigned": "uint", "unsigned int": "uint", "long long": "llong", "size_t": "size",
                "float": "float", "double": "double", "bool": "bool", "void": "void", "hipStream_t": "ptr"}[t]

    protos = {}
    for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b((?:launch|tw)_[a-z0-9_]+)\s*\(([^()]*)\)\s*;", text):
        ret, name, params = m.group(1), m.group(2), m.group(3).strip()
        plist = [] if params in ("", "void") else [kind(p) for p in params.split(",")]
        protos[name] = (kind(ret + " x") if "*" not in ret else kind(ret), plist)
    return protos


def test_ctypes_table_matches_the_header_prototypes():
    """Parameter count and kind (pointer / int / float / ...) of every prototype in the header against the ctypes
    table the Python mirror binds, return types included: a parameter added, dropped or retyped on one side fails."""
    from triebwerk_amd import _lib
    C = ctypes
    kinds = {C.c_void_p: "ptr", C.c_int: "int", C.c_uint: "uint", C.c_longlong: "llong", C.c_size_t: "size",
             C.c_float: "float", C.c_double: "double", C.c_bool: "bool", C.c_char_p: "cstr", None: "void"}

    def ckind(t):
        if t in kinds:
            return kinds[t]
        assert issubclass(t, C._Pointer), t          # POINTER(struct) / POINTER(c_int) / POINTER(POINTER(c_int))
        return "ptr"
    protos = header_prototypes()
    assert sorted(protos) == sorted(_lib.SIGNATURES)
    for name, (restype, argtypes) in _lib.SIGNATURES.items():
        want_ret, want_args = protos[name]
        got_ret = ckind(restype)
        # size_t and unsigned long long share a ctypes type on this platform; pointers returned as void*
        assert got_ret == want_ret or {got_ret, want_ret} <= {"ptr", "cstr"} or (got_ret, want_ret) == ("size", "size"), \
            f"{name}: returns {want_ret} in the header, {got_ret} in the table"
        got_args = [ckind(t) for t in argtypes]
        assert got_args == want_args, f"{name}: header {want_args}, table {got_args}"
    # the struct the layer-step calls take: same number of fields as the header's
    body = re.search(r"typedef\s+struct\s+tw_layer_step_args\s*\{(.*?)\}\s*tw_layer_step_args\s*;", HEADER.read_text(), flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    nfields = sum(len(stmt.split(",")) for stmt in body.split(";") if stmt.strip())
    assert nfields == len(_lib.LayerStepArgs._fields_)


def test_pybind_module_by_the_reference_name(capfd):
    """engine_py.cpp:18-26, 44-45 and triebwerk/engine.py:23: `jetson_engine.Engine(1024, kv_bits)`, `.kv_bits()`,
    `.reset()`.  The module is built beside the library; no GPU work happens before a batch is allocated."""
    import importlib
    import sys
    from triebwerk_amd import build
    path = build.pybind_module_path()
    assert path.exists(), f"{path} is not built (python -m triebwerk_amd.build)"
    sys.path.insert(0, str(path.parent))
    try:
        je = importlib.import_module("jetson_engine")
    finally:
        sys.path.pop(0)
    e = je.Engine()
    assert e.kv_bits() == 0 and e.max_seq_len() == 1024
    assert je.Engine(1024, 4).kv_bits() == 4
    assert je.Engine(max_seq_len=512, kv_bits=2).kv_bits() == 2
    capfd.readouterr()
    assert je.Engine(1024, kv_bits=5).kv_bits() == 0
    assert "kv_bits=5 not supported" in capfd.readouterr().err
    e.reset()                                   # nothing allocated yet: a no-op, as before any load in the reference
    assert not e.is_allocated()
    with pytest.raises(RuntimeError):
        e.decode_step(0, 0, 0, 0)               # no arena: the C call's error becomes RuntimeError
    with pytest.raises(RuntimeError):
        e.set_shape(2, 16, 8, 64)               # head_dim must be 128
