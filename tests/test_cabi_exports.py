"""CPU-side checks of the C-ABI: the library loads and exports every symbol the header declares."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols(header="torsh_hipq.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    return sorted(set(re.findall(r"HIPQ_API[^;()]*?\b(hipq_[a-z0-9_]+)\s*\(", text)))


def _test_hooks():
    """The hooks of include/torsh_hipq_testing.h: exported, bound by the Python tests, not part of the binding
    surface (the generated Rust declarations leave them out)."""
    return _declared_symbols("torsh_hipq_testing.h")


def test_header_declares_entry_points():
    names = _declared_symbols()
    assert "hipq_ctx_create" in names and "hipq_linear_i8_f32" in names and len(names) >= 30


def test_library_exports_every_declared_symbol():
    from torsh_amd import hipq

    assert os.path.exists(hipq.lib_path()), "build with `python -m torsh_amd.build`"
    lib = ctypes.CDLL(hipq.lib_path())
    missing = [n for n in _declared_symbols() + _test_hooks() if not hasattr(lib, n)]
    assert not missing, missing


def test_python_binding_covers_the_header():
    from torsh_amd import hipq

    assert sorted(hipq.exported_symbols()) == sorted(_declared_symbols() + _test_hooks())
    assert _test_hooks() == ["hipq_ctx_set_trace_buffer", "hipq_ctx_set_wait_spin_limit",
                             "hipq_probe_buffer_range_check", "hipq_probe_vector_memory_path",
                             "hipq_set_gemm_kernel_variant"]
    assert not set(_test_hooks()) & set(_declared_symbols())


def test_error_string_api_without_gpu():
    from torsh_amd import hipq

    lib = hipq.load()
    lib.hipq_clear_last_error()
    assert lib.hipq_has_error() == 0
    assert lib.hipq_version().startswith(b"torsh_hipq")
    # null out-pointer is rejected before any device call
    rc = lib.hipq_ctx_create(0, None)
    assert rc == hipq.INVALID_ARGUMENT
    assert lib.hipq_has_error() == 1 and b"null pointer" in lib.hipq_get_last_error()
    lib.hipq_clear_last_error()
    assert lib.hipq_has_error() == 0


def test_no_silent_fallback_when_library_missing(monkeypatch):
    from torsh_amd import hipq

    monkeypatch.setattr(hipq, "_lib", None)
    monkeypatch.setattr(hipq, "_LIB_PATH", "/nonexistent/libtorsh_hipq.so")
    with pytest.raises(FileNotFoundError):
        hipq.load()


def test_generated_rust_declarations_are_in_sync_with_the_header():
    """include/torsh_hipq_sys.rs (the extern "C" block for a torsh-hipq-sys crate) is generated from the header."""
    import importlib.util

    spec = importlib.util.spec_from_file_location("gen_rust_bindings", os.path.join(ROOT, "include", "gen_rust_bindings.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    text = gen.generate()
    assert open(os.path.join(ROOT, "include", "torsh_hipq_sys.rs")).read() == text, \
        "run `python include/gen_rust_bindings.py` after changing include/torsh_hipq.h"
    declared = re.findall(r"pub fn (hipq_\w+)\(", text)
    assert sorted(declared) == _declared_symbols()
    # spot checks of the type mapping
    assert "pub fn hipq_ctx_create(device: i32, out_ctx: *mut *mut hipq_ctx) -> i32;" in text
    assert "pub fn hipq_version() -> *const c_char;" in text
    assert "pub nonfinite: u64," in text and "pub reserved: [i32; 3]," in text
