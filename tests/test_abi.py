"""The C-ABI library loads without a GPU and exports exactly what include/prad_hip.h declares.
No compute entry point is called here."""
import ctypes
import os
import re
import subprocess

import pytest

from parallelreverseautodiff_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "prad_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(prad_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_functions():
    names = declared_functions()
    assert "prad_init" in names and "prad_matmul_fwd" in names and "prad_matmul_bwd" in names
    assert len(names) >= 40


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in declared_functions():
        assert hasattr(lib, name), "libprad_hip.so does not export %s" % name


def test_binding_table_covers_header():
    assert sorted(_lib.SIGNATURES) == declared_functions()


def test_exported_prad_symbols_are_all_declared():
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], stdout=subprocess.PIPE, text=True, check=True).stdout
    exported = sorted(set(re.findall(r" T (prad_[a-z0-9_]+)$", out, flags=re.M)))
    assert exported == declared_functions()


def test_header_compiles_as_c(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "prad_hip.h"\nint main(void) { return PRAD_OK; }\n')
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", str(src), "-o",
                    str(tmp_path / "t.o")], check=True)


def test_calls_before_init_report_not_initialized():
    lib = _lib.load()
    if lib.prad_is_initialized():
        pytest.skip("library already initialised in this process")
    h = ctypes.c_void_p()
    assert lib.prad_buf_alloc(_lib.PRAD_F64, 4, 4, ctypes.byref(h)) == _lib.PRAD_ERR_NOT_INITIALIZED
    assert lib.prad_stream_sync() == _lib.PRAD_ERR_NOT_INITIALIZED
    assert lib.prad_matmul_fwd(None, None, None) == _lib.PRAD_ERR_NOT_INITIALIZED
    assert b"prad_init" in lib.prad_last_error()
    assert lib.prad_device_id() == -1


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libprad_hip.so")
    with pytest.raises(ImportError, match="no CPU fallback"):
        _lib.load()


def test_integration_notes_declare_every_function_for_pinvoke():
    """The C# block of the integration notes is the output of parallelreverseautodiff_amd.pinvoke and lists every
    function the header declares, with a C# type for every parameter."""
    from parallelreverseautodiff_amd import pinvoke
    decls = pinvoke.declarations()
    protos = pinvoke.prototypes()
    assert len(decls) == len(protos) > 80
    notes = os.path.join(ROOT, "INTEGRATION.md")
    text = open(notes).read()
    for d in decls:
        assert d in text, "%s lacks: %s" % (os.path.basename(notes), d)
    header_names = {p[1] for p in protos}
    from parallelreverseautodiff_amd import _lib
    assert header_names == set(_lib.SIGNATURES)


def test_pinvoke_device_pointers_are_not_out_parameters():
    """Device memory travels as IntPtr in the generated C# declarations, for float as for double: `out` is only for
    host variables that a call fills in (handles, shapes, counters, an event's elapsed time)."""
    import re
    from parallelreverseautodiff_amd import pinvoke
    protos = {p[1]: p for p in pinvoke.prototypes()}
    for name, (_, _, params) in protos.items():
        decl = pinvoke.declaration(*protos[name])
        for ctype, pname in params:
            cs = pinvoke.csharp_type(ctype, name, pname)
            if name.startswith("prad_gemm") and pname in ("A", "B", "C"):
                assert cs == "IntPtr", (name, pname, cs)
            if re.fullmatch(r"(const )?(double|float)\s*\*", ctype) and (name, pname) not in pinvoke._HOST_OUT:
                assert cs == "IntPtr", (name, pname, cs)
        if name.endswith("_f32") and name[:-4] + "_f64" in protos:   # the two precisions differ in nothing but the name
            twin = pinvoke.declaration(*protos[name[:-4] + "_f64"])
            assert decl.replace("_f32(", "_f64(") == twin
    assert "out float ms" in pinvoke.declaration(*protos["prad_event_elapsed_ms"])
