"""The C-ABI library loads without a GPU and exports every entry point the
header declares (the flat-C counterpart of the `caml_llmopt_metal_*` externals,
lib/metal_native.ml:8-124).  No compute call is made here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "llmopt_hip.h")
LIBRARY = os.path.join(ROOT, "llmopt_amd", "libllmopt_hip.so")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(llmopt_hip_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def library():
    if not os.path.exists(LIBRARY):
        pytest.fail(f"{LIBRARY} is not built: run `python -m llmopt_amd.build`")
    return ctypes.CDLL(LIBRARY)


def test_header_declares_the_boundary():
    names = declared_symbols()
    assert len(names) >= 35
    # one per reference external that the hot path uses (lib/metal_native.ml:8-124)
    for stem in ("create_context", "device_name", "load_library", "has_function", "preload_pipeline",
                 "buffer_of_bytes", "create_buffer", "map_file", "buffer_view", "buffer_contents",
                 "buffer_argmax_f16", "buffer_length", "buffer_copy", "buffer_set_int64",
                 "buffer_set_u32_array", "dispatch", "begin_batch", "batch_dispatch",
                 "batch_dispatch_all", "batch_copy", "batch_barrier", "commit_batch",
                 "commit_batch_async", "abort_batch", "prebaked_create", "prebaked_execute"):
        assert "llmopt_hip_" + stem in names, stem


def test_library_exports_every_declared_symbol(library):
    missing = [name for name in declared_symbols() if not hasattr(library, name)]
    assert not missing, missing


def test_python_binding_lists_the_same_symbols():
    from llmopt_amd import native
    assert sorted(native.EXPORTED_SYMBOLS) == declared_symbols()


def test_last_error_is_a_c_string(library):
    library.llmopt_hip_last_error.restype = ctypes.c_char_p
    assert isinstance(library.llmopt_hip_last_error(), bytes)


def test_null_handles_are_rejected_not_dereferenced(library):
    """Error behaviour of finalized / absent handles (native/ocaml_metal_stubs.m:174-227):
    a status and a message, never a crash."""
    library.llmopt_hip_last_error.restype = ctypes.c_char_p
    library.llmopt_hip_has_function.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
    status = library.llmopt_hip_has_function(None, b"llmopt_w4a16_linear_f16_g64")
    assert status < 0
    assert b"finalized" in library.llmopt_hip_last_error() or b"null" in library.llmopt_hip_last_error().lower()
    library.llmopt_hip_buffer_length.argtypes = [ctypes.c_void_p]
    library.llmopt_hip_buffer_length.restype = ctypes.c_int64
    assert library.llmopt_hip_buffer_length(None) < 0
    library.llmopt_hip_commit_batch.argtypes = [ctypes.c_void_p]
    assert library.llmopt_hip_commit_batch(None) < 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    """There is no CPU fallback: without the HIP library the host mirror raises."""
    from llmopt_amd import native
    monkeypatch.setattr(native, "_lib", None)
    monkeypatch.setattr(native, "LIBRARY_PATH", str(tmp_path / "absent.so"))
    with pytest.raises((OSError, native.LlmoptError)):
        native.lib()
