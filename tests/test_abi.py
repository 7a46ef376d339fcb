"""The shared library loads without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "retro_mi355.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ri_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from retrievalattention_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python -m retrievalattention_amd.build"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared()
    assert len(names) >= 30
    missing = [n for n in names if not hasattr(handle, n)]
    assert not missing, f"declared in the header but not exported: {missing}"


def test_python_binding_covers_the_header():
    from retrievalattention_amd import _lib
    assert sorted(_lib.SIGNATURES) == _declared()


def test_status_strings_and_version():
    from retrievalattention_amd import _lib
    l = _lib.lib()
    assert l.ri_abi_version() >= 1
    assert l.ri_status_string(0) == b"ok"
    assert b"workspace" in l.ri_status_string(-3)
    # two fp32 tile partials per (group, 256-centroid tile, head) and one 16-bit sort key per centroid
    assert l.ri_score_select_workspace_bytes(32, 4, 8192) == 2 * 32 * 32 * 4 * 4 + 32 * 8192 * 2
    assert l.ri_flash_decoding_workspace_bytes(0, 4) == 0


def test_missing_library_is_a_loud_error(monkeypatch, tmp_path):
    from retrievalattention_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    import pytest
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.lib()


def test_header_is_plain_c_and_cxx(tmp_path):
    """What a cgo / JNI / ctypes binding would include: the header compiles as C99 and as C++11 on its own."""
    import shutil
    import subprocess
    src = '#include "retro_mi355.h"\nint main(void) { return (int)sizeof(ri_stream_t) * 0; }\n'
    for cc, name, std in (("gcc", "t.c", "-std=c99"), ("g++", "t.cpp", "-std=c++11")):
        if shutil.which(cc) is None:
            continue
        f = tmp_path / name
        f.write_text(src)
        r = subprocess.run([cc, std, "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
                            "-fsyntax-only", str(f)], capture_output=True, text=True)
        assert r.returncode == 0, r.stderr


def test_binding_arguments_match_the_header():
    """Every prototype of the header has as many parameters, of the same kinds, as the ctypes signature that binds it."""
    from retrievalattention_amd import _lib
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    protos = dict(re.findall(r"\b(ri_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S))
    assert sorted(protos) == sorted(_lib.SIGNATURES)
    def kind(decl):
        decl = decl.strip()
        if "*" in decl or re.match(r"(const\s+)?ri_stream_t\b", decl):
            return ctypes.c_void_p
        base = re.sub(r"\b(const|unsigned)\b", "", decl).split()[0]
        return {"int": ctypes.c_int, "int32_t": ctypes.c_int, "int64_t": ctypes.c_int64, "float": ctypes.c_float,
                "size_t": ctypes.c_size_t}[base]

    for name, params in protos.items():
        params = params.strip()
        kinds = [] if params in ("", "void") else [kind(x) for x in params.split(",")]
        bound = _lib.SIGNATURES[name][1]
        assert len(kinds) == len(bound), (name, len(kinds), len(bound))
        # and of the same kind: a 64-bit stride or a size bound as int would be cut in half without any error
        for i, (a, b) in enumerate(zip(kinds, bound)):
            assert a is b, (name, i, a, b)
    rets = dict((n, r.strip()) for r, n in re.findall(r"([A-Za-z_][\w \*]*?)\s*\b(ri_[a-z0-9_]+)\s*\(", text))
    for name, (restype, _) in _lib.SIGNATURES.items():
        r = rets[name]
        want = ctypes.c_char_p if r == "const char*" else ctypes.c_void_p if "*" in r else \
            {"int": ctypes.c_int, "size_t": ctypes.c_size_t, "int64_t": ctypes.c_int64, "void": None}[r]
        assert restype is want, (name, r, restype)
